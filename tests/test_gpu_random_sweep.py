"""Seeded random sweeps over shapes, expert counts and operand formats.

GEMMs run on exactly representable operands (small multiples of 1/2 with power-of-two scales: every
product and partial sum is exact in fp32), so every output element must equal the reference bit for
bit whatever the accumulation order: small shapes against the CPU oracle, larger ones (several tiles
per workgroup, up to [20000, 4096] x [4096, 4096]) against the fp32 library matmul of the dequantised
operands, which is exact for these inputs.  Quantisers run on random bf16 data with wide dynamic range,
zeros and non-finite values, against the oracle byte for byte."""

import numpy as np
import pytest
import torch

from oracle import mx_oracle as o

pytestmark = pytest.mark.gpu
E8 = torch.float8_e8m0fnu


def _dt(fmt):
    return torch.float8_e4m3fn if fmt == 0 else torch.float4_e2m1fn_x2


def _dev(a, gpu, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).to(gpu).view(dtype)


def _exact_np(rng, rows, k, fmt):
    if fmt == 0:
        vals = np.array([0x00, 0x38, 0x40, 0x44, 0x48, 0xB8, 0xC0, 0xC4], dtype=np.uint8)      # 0, +-1, +-2, +-3, 4
        q = vals[rng.integers(0, 8, size=(rows, k))]
    else:
        q = o.pack_fp4(rng.integers(0, 16, size=(rows, k)).astype(np.uint8))
    return q, rng.integers(125, 130, size=(rows, k // 32)).astype(np.uint8)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_small_shapes_against_the_oracle(gpu, seed):
    from primus_amd.pytorch import kernels as K

    rng = np.random.default_rng(seed)
    for _ in range(40):
        G = int(rng.choice([1, 2, 3, 5, 8, 17, 40]))
        lens = [int(v) for v in rng.choice([0, 1, 7, 31, 32, 33, 100, 128, 129, 255, 256, 257, 300, 511, 513], size=G)]
        if rng.random() < 0.15:
            lens = [0] * G
        m = sum(lens)
        n = int(rng.choice([32, 64, 96, 128, 160, 256, 288, 320, 512, 544]))
        k = int(rng.choice([128, 256, 384, 512, 640]))
        afmt, bfmt = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        case = f"G={G} lens={lens} n={n} k={k} formats=({afmt},{bfmt})"
        gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
        if m:
            aq, as_ = _exact_np(rng, m, k, afmt)
            bq, bs = _exact_np(rng, G * n, k, bfmt)
            bq, bs = bq.reshape(G, n, -1), bs.reshape(G, n, k // 32)
            want = o.grouped_gemm_nt_ref(aq, as_, bq, bs, lens, afmt, bfmt)
            got = K.grouped_gemm_mx_nt_impl(_dev(aq, gpu, _dt(afmt)), _dev(as_, gpu, E8), _dev(bq, gpu, _dt(bfmt)),
                                            _dev(bs, gpu, E8), gl)
            assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), want), "forward " + case
        W = o.padded_width(m, G)
        if W:
            _, poffs = o.segment_layout(lens)
            live = np.zeros(W, dtype=bool)
            for g, ln in enumerate(lens):
                live[poffs[g] : poffs[g] + ln] = True

            def operand(rows, fmt):
                q, s = _exact_np(rng, rows, W, fmt)
                if fmt == 1:
                    nib = o.unpack_fp4(q)
                    nib[:, ~live] = 0
                    q = o.pack_fp4(nib)
                else:
                    q[:, ~live] = 0
                return q, s

            nn, kk = int(rng.choice([32, 96, 256, 288])), int(rng.choice([32, 160, 256, 320]))
            (a2, s2), (b2, t2) = operand(nn, afmt), operand(kk, bfmt)
            want = o.grouped_gemm_wgrad_ref(a2, s2, b2, t2, lens, afmt, bfmt)
            got = K.grouped_gemm_mx_wgrad_impl(_dev(a2, gpu, _dt(afmt)), _dev(s2, gpu, E8), _dev(b2, gpu, _dt(bfmt)),
                                               _dev(t2, gpu, E8), gl, m)
            assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), want), "wgrad " + case


@pytest.mark.parametrize("seed", [4, 5])
def test_quantisers_against_the_oracle(gpu, seed):
    from primus_amd.pytorch import kernels as K

    rng = np.random.default_rng(seed)
    torch.manual_seed(seed)
    u8 = lambda t: t.view(torch.uint8).cpu().numpy()   # noqa: E731
    for _ in range(40):
        G = int(rng.choice([0, 1, 2, 3, 6, 20]))
        lens = [int(v) for v in rng.choice([0, 1, 5, 31, 32, 33, 127, 128, 129, 200, 384], size=max(G, 1))]
        m = sum(lens)
        cols = int(rng.choice([32, 64, 96, 128, 160, 224, 256, 288, 1024]))
        fmt, smode, pad = int(rng.integers(0, 2)), int(rng.integers(0, 3)), int(rng.choice([1, 128]))
        per = 2 if fmt == 1 else 1
        case = f"G={G} lens={lens} cols={cols} fmt={fmt} scale_mode={smode} pad_to={pad}"
        x = torch.randn(m, cols)
        kind = int(rng.integers(0, 4))
        if kind == 1:
            x = x * torch.logspace(-6, 6, cols)[None, :]
        elif kind == 2:
            x = x * (torch.rand(m, 1) < 0.3) * 100
        elif kind == 3 and m:
            x[int(rng.integers(0, m)), int(rng.integers(0, cols))] = float("inf")
            x[int(rng.integers(0, m)), int(rng.integers(0, cols))] = float("nan")
        x = x.bfloat16()
        gl = None if G == 0 else torch.tensor(lens, dtype=torch.int64, device=gpu)
        q = K.quantize_mx_impl(x.to(gpu), fmt, smode, rowwise=True, colwise=True, group_lens=gl, pad_to=pad)
        if m:
            oq, os_ = o.quantize_mx_rowwise(x, fmt, smode)
            assert np.array_equal(u8(q[0])[:, : cols // per], oq) and np.array_equal(u8(q[1])[:, : cols // 32], os_), case
            assert not u8(q[0])[:, cols // per:].any() and not u8(q[1])[:, cols // 32:].any(), case
        oqT, osT = o.quantize_mx_colwise_segmented(x, lens, fmt, smode)
        assert np.array_equal(u8(q[2]), oqT) and np.array_equal(u8(q[3]), osT), "transposed " + case
        if fmt == 1 and kind != 3:
            s_seed, signs = int(rng.integers(0, 2**62)), int(rng.integers(0, 65536))
            e = K.quantize_mx_impl(x.to(gpu), 1, smode, rowwise=True, colwise=True, group_lens=gl, pad_to=pad,
                                   sr_seed=s_seed, rht_signs=signs)
            if m:
                assert np.array_equal(u8(e[0])[:, : cols // 2], o.quantize_mx_rowwise_sr(x, s_seed, smode)[0]), "sr " + case
            oqT, osT = o.quantize_mx_colwise_segmented_fp4(x, lens, smode, sr_seed=s_seed, rht_signs=signs)
            assert np.array_equal(u8(e[2]), oqT) and np.array_equal(u8(e[3]), osT), "sr + hadamard " + case
        B, n, k = int(rng.choice([1, 1, 2, 5])), int(rng.choice([32, 64, 96, 128, 160, 256, 416])), int(rng.choice([32, 64, 128, 160, 288, 512]))
        w = (torch.randn(B, n, k) * 0.05).bfloat16()
        wq = K.quantize_mx_weight_2d_impl(w.to(gpu), fmt, smode, rowwise=True, colwise=True, pad_to=pad)
        oq, os_, oqT, osT = o.quantize_mx_2d(w, fmt, smode)
        wcase = case + f" weights [{B},{n},{k}]"
        assert np.array_equal(u8(wq[0])[:, :, : k // per], oq) and np.array_equal(u8(wq[1])[:, :, : k // 32], os_), wcase
        assert np.array_equal(u8(wq[2])[:, :, : n // per], oqT) and np.array_equal(u8(wq[3])[:, :, : n // 32], osT), wcase


def test_large_shapes_every_output_element(gpu):
    from primus_amd.pytorch import kernels as K

    rng = np.random.default_rng(6)
    gen = torch.Generator(device=gpu).manual_seed(6)

    def exact(rows, k, fmt):
        if fmt == 0:
            vals = torch.tensor([0x00, 0x38, 0x40, 0x44, 0x48, 0xB8, 0xC0, 0xC4], dtype=torch.uint8, device=gpu)
            q = vals[torch.randint(0, 8, (rows, k), generator=gen, device=gpu)]
        else:   # E2M1 values 0 .. +-3: exact sums up to k = 8192
            table = torch.tensor([0, 1, 2, 3, 4, 5, 9, 10, 11, 12, 13, 8], dtype=torch.uint8, device=gpu)
            nib = table[torch.randint(0, 12, (rows, k), generator=gen, device=gpu)]
            q = (nib[:, 0::2] | (nib[:, 1::2] << 4)).contiguous()
        s = torch.randint(126, 129, (rows, k // 32), generator=gen, device=gpu, dtype=torch.uint8)
        return q.view(_dt(fmt)), s.view(E8)

    done = 0
    while done < 24:
        G = int(rng.choice([1, 2, 4, 8, 32]))
        lens = [int(v) for v in rng.choice([0, 100, 256, 300, 512, 700, 1024, 1500, 2048], size=G)]
        m = sum(lens)
        if m == 0 or m > 20000:
            continue
        n, k = int(rng.choice([256, 512, 1024, 2048, 4096])), int(rng.choice([128, 256, 1024, 2048, 4096]))
        afmt, bfmt = done % 2, (done // 2) % 2                      # all four format pairs in turn
        case = f"G={G} lens={lens} n={n} k={k} formats=({afmt},{bfmt})"
        gl = torch.tensor(lens, dtype=torch.int64, device=gpu)
        offs = np.concatenate([[0], np.cumsum(lens)])
        aq, as_ = exact(m, k, afmt)
        bq, bs = exact(G * n, k, bfmt)
        y = K.grouped_gemm_mx_nt_impl(aq, as_, bq.view(G, n, -1), bs.view(G, n, k // 32), gl)
        af, bf = K.dequantize_mx_impl(aq, as_).float(), K.dequantize_mx_impl(bq, bs).float().view(G, n, k)
        for g in range(G):
            a, b = int(offs[g]), int(offs[g + 1])
            if b > a:
                assert torch.equal(y[a:b], (af[a:b] @ bf[g].T).bfloat16()), f"expert {g} " + case
        done += 1

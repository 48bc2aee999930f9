/*
 * C restatement of the CPU oracle (oracle/mx_oracle.py) for the MX linear path.
 *
 * TEST INFRASTRUCTURE ONLY: used by tests/ as a second, independent
 * implementation of the oracle and by bench.py as the timed CPU baseline
 * ("port").  Nothing under primus_amd/ links or loads it.
 *
 * The algorithm is the published OCP MX v1.0 one; the reference tree holds only
 * its call sites because the arithmetic lives in the un-vendored package
 * primus_turbo (pinned by /root/reference/.github/workflows/ci.yaml:43):
 *   block 32 / E8M0 / E4M3, E2M1:  primus/backends/megatron/core/fp8_utils.py:162-168,
 *                                  primus/backends/megatron/core/fp4_utils.py:144-150
 *   row-wise (axis=-1) and transposed col-wise (axis=-2) copies:
 *                                  primus/backends/megatron/core/extensions/primus_turbo.py:321-354
 *   2-D 32x32 weight blocks:       primus_turbo.py:313-317, core/optimizer/weight_deosc.py:29-33
 *   NT GEMM operand table:         core/extensions/primus_turbo_mxfp4_local.py:316-331,432-459
 * Parity status is the one stated in mx_oracle.py's header; this file is
 * checked against it bit for bit in tests/test_oracle_c.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define BLOCK 32
enum { FMT_E4M3 = 0, FMT_E2M1 = 1 };
enum { SCALE_OCP_FLOOR = 0, SCALE_RCEIL = 1, SCALE_EVEN = 2 };

static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bf16_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }
static inline uint16_t f32_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

/* E8M0 byte from the largest 15-bit bf16 magnitude of a block. */
static inline uint8_t scale_byte(uint32_t amax16, int fmt, int mode) {
    if (amax16 >= 0x7F80u) return 255;
    const int emax = fmt == FMT_E4M3 ? 8 : 2;
    const uint32_t maxman = fmt == FMT_E4M3 ? 0x600000u : 0x400000u;
    const int mbits = fmt == FMT_E4M3 ? 3 : 1;
    uint32_t b = amax16 << 16;
    if (mode == SCALE_EVEN) b += 1u << (23 - mbits - 1);
    int e = (int)(b >> 23);
    if (mode == SCALE_RCEIL && (b & 0x7FFFFFu) > maxman) e += 1;
    e -= emax;
    if (e < 0) e = 0;
    if (e > 254) e = 254;
    return (uint8_t)e;
}

/* saturating round-to-nearest-even casts of x * 2^(127 - byte) */
static inline uint8_t cast_e4m3(uint16_t xb, uint8_t byte) {
    const uint8_t sign = (uint8_t)((xb >> 8) & 0x80);
    if ((xb & 0x7FFF) >= 0x7F80) return sign | 0x7F;
    if (byte == 255) return sign;
    float a = fabsf(bf16_f32(xb)) * bits_f32((uint32_t)(254 - byte) << 23);
    if (a > 448.f) a = 448.f;
    uint32_t code;
    if (a >= 0.015625f) {
        uint32_t ab = f32_bits(a);
        code = ((ab + 0x7FFFFu + ((ab >> 20) & 1u)) >> 20) - ((127 - 7) << 3);
    } else {
        code = (uint32_t)lrintf(a * 512.f); /* default rounding mode: nearest even */
    }
    if (code > 0x7E) code = 0x7E;
    return sign | (uint8_t)code;
}
static inline uint8_t cast_e2m1(uint16_t xb, uint8_t byte) {
    const uint8_t sign = (uint8_t)((xb >> 12) & 0x8);
    if ((xb & 0x7FFF) >= 0x7F80) return sign | 0x7;
    if (byte == 255) return sign;
    float a = fabsf(bf16_f32(xb)) * bits_f32((uint32_t)(254 - byte) << 23);
    if (a > 6.f) a = 6.f;
    uint32_t code;
    if (a >= 1.f) {
        uint32_t ab = f32_bits(a);
        code = ((ab + 0x1FFFFFu + ((ab >> 22) & 1u)) >> 22) - ((127 - 1) << 1);
    } else {
        code = (uint32_t)lrintf(a * 2.f);
    }
    if (code > 7) code = 7;
    return sign | (uint8_t)code;
}
static inline float dec_e4m3(uint8_t c) {
    const int e = (c >> 3) & 0xF, m = c & 7;
    float v;
    if ((c & 0x7F) == 0x7F) v = NAN;
    else if (e == 0) v = (float)m * 0.001953125f;
    else v = ldexpf((float)(8 + m), e - 10);
    return (c & 0x80) ? -v : v;
}
static inline float dec_e2m1(uint8_t c) {
    static const float tab[8] = {0.f, 0.5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f};
    const float v = tab[c & 7];
    return (c & 8) ? -v : v;
}
static inline float scale_val(uint8_t byte) { return byte == 255 ? NAN : ldexpf(1.f, (int)byte - 127); }

/* Row-wise quantise x[rows, cols] (bf16 bits).  codes: [rows, cols] or packed [rows, cols/2]. */
void mxo_quantize_rowwise(const uint16_t* x, int64_t rows, int64_t cols, int fmt, int mode, uint8_t* codes,
                          uint8_t* scales) {
    const int64_t nb = cols / BLOCK;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t b = 0; b < nb; ++b) {
            const uint16_t* p = x + r * cols + b * BLOCK;
            uint32_t amax = 0;
            for (int i = 0; i < BLOCK; ++i) {
                uint32_t m = p[i] & 0x7FFF;
                if (m > amax) amax = m;
            }
            const uint8_t byte = scale_byte(amax, fmt, mode);
            scales[r * nb + b] = byte;
            if (fmt == FMT_E4M3) {
                for (int i = 0; i < BLOCK; ++i) codes[r * cols + b * BLOCK + i] = cast_e4m3(p[i], byte);
            } else {
                for (int i = 0; i < BLOCK; i += 2)
                    codes[(r * cols + b * BLOCK + i) / 2] =
                        (uint8_t)(cast_e2m1(p[i], byte) | (cast_e2m1(p[i + 1], byte) << 4));
            }
        }
    }
}

/* Column-wise, transposed, segment-padded: x[rows, cols] -> codesT[cols, W], scalesT[cols, W/32];
 * poffs[g] = padded start of group g, offs[g] = source start (host arrays of G+1 entries). */
void mxo_quantize_colwise_segmented(const uint16_t* x, int64_t rows, int64_t cols, int fmt, int mode,
                                    const int64_t* offs, const int64_t* poffs, int G, int64_t W, uint8_t* codesT,
                                    uint8_t* scalesT) {
    const int per = fmt == FMT_E2M1 ? 2 : 1;
    memset(codesT, 0, (size_t)(cols * W / per));
    memset(scalesT, 0, (size_t)(cols * W / BLOCK));
    (void)rows;
#pragma omp parallel for schedule(static)
    for (int64_t c = 0; c < cols; ++c) {
        for (int g = 0; g < G; ++g) {
            const int64_t len = offs[g + 1] - offs[g];
            for (int64_t b0 = 0; b0 < len; b0 += BLOCK) {
                uint16_t blk[BLOCK];
                uint32_t amax = 0;
                for (int i = 0; i < BLOCK; ++i) {
                    blk[i] = (b0 + i < len) ? x[(offs[g] + b0 + i) * cols + c] : 0;
                    uint32_t m = blk[i] & 0x7FFF;
                    if (m > amax) amax = m;
                }
                const uint8_t byte = scale_byte(amax, fmt, mode);
                const int64_t pos = poffs[g] + b0;
                scalesT[c * (W / BLOCK) + pos / BLOCK] = byte;
                if (fmt == FMT_E4M3) {
                    for (int i = 0; i < BLOCK; ++i) codesT[c * W + pos + i] = cast_e4m3(blk[i], byte);
                } else {
                    for (int i = 0; i < BLOCK; i += 2)
                        codesT[(c * W + pos + i) / 2] =
                            (uint8_t)(cast_e2m1(blk[i], byte) | (cast_e2m1(blk[i + 1], byte) << 4));
                }
            }
        }
    }
}

/* 2-D 32x32 block quantisation of `batch` matrices w[n, k]; either output pair may be NULL. */
void mxo_quantize_2d(const uint16_t* w, int64_t batch, int64_t n, int64_t k, int fmt, int mode, uint8_t* q_row,
                     uint8_t* s_row, uint8_t* q_colT, uint8_t* s_colT) {
    const int per = fmt == FMT_E2M1 ? 2 : 1;
    const int64_t nbn = n / BLOCK, nbk = k / BLOCK;
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t m = 0; m < batch; ++m) {
        for (int64_t bn = 0; bn < nbn; ++bn) {
            for (int64_t bk = 0; bk < nbk; ++bk) {
                const uint16_t* base = w + (m * n + bn * BLOCK) * k + bk * BLOCK;
                uint32_t amax = 0;
                for (int i = 0; i < BLOCK; ++i)
                    for (int j = 0; j < BLOCK; ++j) {
                        uint32_t v = base[i * k + j] & 0x7FFF;
                        if (v > amax) amax = v;
                    }
                const uint8_t byte = scale_byte(amax, fmt, mode);
                uint8_t c[BLOCK][BLOCK];
                for (int i = 0; i < BLOCK; ++i)
                    for (int j = 0; j < BLOCK; ++j)
                        c[i][j] = fmt == FMT_E4M3 ? cast_e4m3(base[i * k + j], byte) : cast_e2m1(base[i * k + j], byte);
                for (int i = 0; i < BLOCK; ++i) {
                    const int64_t row = m * n + bn * BLOCK + i;
                    if (q_row) {
                        s_row[row * nbk + bk] = byte;
                        if (per == 1)
                            for (int j = 0; j < BLOCK; ++j) q_row[row * k + bk * BLOCK + j] = c[i][j];
                        else
                            for (int j = 0; j < BLOCK; j += 2)
                                q_row[(row * k + bk * BLOCK + j) / 2] = (uint8_t)(c[i][j] | (c[i][j + 1] << 4));
                    }
                }
                if (q_colT) {
                    for (int j = 0; j < BLOCK; ++j) {
                        const int64_t trow = m * k + bk * BLOCK + j;
                        s_colT[trow * nbn + bn] = byte;
                        if (per == 1)
                            for (int i = 0; i < BLOCK; ++i) q_colT[trow * n + bn * BLOCK + i] = c[i][j];
                        else
                            for (int i = 0; i < BLOCK; i += 2)
                                q_colT[(trow * n + bn * BLOCK + i) / 2] = (uint8_t)(c[i][j] | (c[i + 1][j] << 4));
                    }
                }
            }
        }
    }
}

/* Row-wise dequantise to fp32: out[rows, k]. */
void mxo_dequantize(const uint8_t* codes, const uint8_t* scales, int64_t rows, int64_t k, int fmt, float* out) {
    const int64_t nb = k / BLOCK;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t b = 0; b < nb; ++b) {
            const float s = scale_val(scales[r * nb + b]);
            for (int i = 0; i < BLOCK; ++i) {
                const int64_t e = r * k + b * BLOCK + i;
                const float v = fmt == FMT_E4M3 ? dec_e4m3(codes[e]) : dec_e2m1((codes[e / 2] >> (4 * (e & 1))) & 0xF);
                out[e] = v * s;
            }
        }
}

/* c[m, n] (bf16 bits) = a[m, k] . b[n, k]^T on fp32 inputs, fp32 accumulation. */
void mxo_matmul_nt_bf16(const float* a, const float* b, int64_t m, int64_t n, int64_t k, uint16_t* c) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j) {
            float acc = 0.f;
            for (int64_t p = 0; p < k; ++p) acc += a[i * k + p] * b[j * k + p];
            c[i * n + j] = f32_bf16(acc);
        }
}

// Host-side bounds check of the GEMM kernels' operand requests.  It includes the header the kernels take their
// address arithmetic from (primus_amd/csrc/mx_gemm_addr.h) and walks every request a tile can issue -- every
// thread, every load round, every K slot including the look-ahead slots past the contraction range, tiles that
// start anywhere in the operand -- applying the hardware's range check (per dword, on the sum of the per-lane and the
// scalar offset, as measured on gfx950 and pinned by tests/test_gpu_range_check.py).
// Claim checked: a dword that is not dropped lies inside the operand; and no dword of a row that exists, in a K
// slot that exists, is dropped.  Built and run by tests/test_gemm_bounds.py with g++ (no GPU involved).
#include <cstdint>
#include <cstdio>
#include <initializer_list>

#include "../primus_amd/csrc/mx_gemm_addr.h"

using namespace mxl::addr;

static long long n_checked = 0, n_dropped = 0;
static int failures = 0;

static void fail(const char* what, long long a, long long b, long long c, long long d) {
    if (failures < 20) std::printf("FAIL %s: %lld %lld %lld %lld\n", what, a, b, c, d);
    ++failures;
}

// one 16-byte request: descriptor d, per-lane offset voff, scalar offset soff, operand of `bytes` bytes.
// must_hold: the request addresses data that exists, so nothing of it may be dropped.
static void request(const Desc& d, uint32_t voff, uint32_t soff, int64_t bytes, bool must_hold, const char* what) {
    for (int c = 0; c < 4; ++c) {
        ++n_checked;
        if (!accepted(d, voff, soff, c)) {
            ++n_dropped;
            if (must_hold) fail(what, d.base, d.records, voff, c);
            continue;
        }
        const int64_t a = d.base + (int64_t)voff + (int64_t)soff + 4 * c;
        if (a < 0 || a + 4 > bytes) fail(what, a, bytes, voff, soff);
    }
}

static void check_slot2(int layout, int kb_row /* bytes of a row per K slot: 128 FP8, 64 FP4 */, int64_t rows_total, int64_t k_slots,
                        int64_t row0) {
    const int cpr = kb_row / 16, rows_per_ld = 256 / cpr, rounds = cpr;   // cpr rounds cover 256 rows
    const int64_t ld = k_slots * kb_row, bytes = rows_total * ld;
    const uint32_t cstride = (uint32_t)(rows_total * kb_row);
    const Desc d = slot2_code_desc(layout, rows_total, row0, ld, kb_row);
    // contraction ranges: the whole row (forward / dgrad) and every sub-range (a group's segment in wgrad)
    for (int64_t s0 = 0; s0 < k_slots; ++s0)
        for (int64_t np = 1; s0 + np <= k_slots; np += (s0 == 0 ? 1 : k_slots)) {
            const uint32_t k0 = layout ? (uint32_t)s0 : (uint32_t)(s0 * kb_row);
            for (int kp = 0; kp < np + 2; ++kp)       // the kernel requests up to two K slots past the range
                for (int r = 0; r < rounds; ++r)
                    for (int t = 0; t < 256; ++t) {
                        const int row = t / cpr;
                        const int swz = kb_row == 64 ? ((row >> 2) & 3) : ((row >> 1) & 7);
                        const uint32_t voff = slot2_code_lane(layout, t, cpr, swz, ld, kb_row);
                        const uint32_t soff = slot2_code_round(layout, r, rows_per_ld, ld, kb_row) +
                                              slot2_code_k(layout, k0, kp, kb_row, cstride);
                        const bool exists = row0 + r * rows_per_ld + row < rows_total && kp < np;
                        request(d, voff, soff, bytes, exists, layout ? "slot2 codes chunked" : "slot2 codes row-major");
                    }
        }
    // scales: row-major [rows_total, 4 * k_slots]; panels of 16 bytes, requested up to one panel past the range
    const int64_t ld_s = 4 * k_slots, sbytes = rows_total * ld_s;
    const Desc ds = slot2_scale_desc(rows_total, row0, ld_s);
    for (int64_t s0 = 0; s0 < k_slots; s0 += 3)
        for (int pn = 0; pn <= (k_slots - s0 + 3) / 4; ++pn)
            for (int t = 0; t < 256; ++t) {
                const uint32_t voff = slot2_scale_off(t, ld_s, 0u, 0), soff = slot2_scale_off(0, ld_s, (uint32_t)(4 * s0), pn);
                request(ds, voff, soff, sbytes, false, "slot2 scales");
                // the bytes of the range that exist must come through
                if (row0 + t < rows_total)
                    for (int c = 0; c < 4; ++c)
                        if (4 * s0 + 16 * pn + 4 * c + 4 <= ld_s && !accepted(ds, voff, soff, c)) fail("slot2 scales dropped", voff, c, ld_s, pn);
            }
}

static void check_ring(int row_bytes, int64_t rows_total, int64_t steps, int64_t row0) {
    const bool half = row_bytes == 32;
    const int rounds = half ? 2 : 4;
    const int64_t bytes = steps * rows_total * row_bytes;
    const Desc d = ring_code_desc(rows_total, steps, row0, row_bytes);
    for (int64_t st = 0; st < steps + 2; ++st)      // (the kernel clamps the step to the contraction range; two more here)
        for (int e = 0; e < rounds; ++e)
            for (int t = 0; t < 256; ++t) {
                const uint32_t voff = ring_code_lane(t, e, half);
                const int row = half ? (t >> 1) + 128 * e : (t >> 2) + 64 * e;
                request(d, voff, (uint32_t)(st * rows_total * row_bytes), bytes, row0 + row < rows_total && st < steps, "ring codes");
            }
    const int64_t panels = (steps * 64 + 511) / 512, pbytes = panels * rows_total * 16;
    const Desc dp = ring_panel_desc(rows_total, panels, row0);
    for (int64_t pn = 0; pn < panels + 1; ++pn)
        for (int t = 0; t < 256; ++t)
            request(dp, ring_panel_lane(t), (uint32_t)(pn * rows_total * 16), pbytes, row0 + t < rows_total && pn < panels, "ring panels");
}

// packed FP4 codes in the pre-shuffled order (64-byte K slots, 4 rounds of 64 rows): rows_total a multiple of 16
static void check_slot2_shuffled(int64_t rows_total, int64_t k_slots, int64_t row0) {
    const int cpr = 4, rows_per_ld = 64;
    const int64_t ld = k_slots * 64, bytes = rows_total * ld;
    const Desc d = slot2_code_desc(0, rows_total, row0, ld, 64);
    for (int kp = 0; kp < k_slots + 2; ++kp)
        for (int r = 0; r < 4; ++r)
            for (int t = 0; t < 256; ++t) {
                const int row = t / cpr;
                const uint32_t voff = slot2_code_lane_shuffled(t, cpr, (row >> 2) & 3, ld);
                const uint32_t soff = slot2_code_round(0, r, rows_per_ld, ld, 64) + slot2_code_k_shuffled(kp);
                request(d, voff, soff, bytes, row0 + r * rows_per_ld + row < rows_total && kp < k_slots, "slot2 codes pre-shuffled");
            }
}

// the ring kernel reading b transposed: planes of [rows_total][64], descriptor at (plane0, row0), round e = e planes
// further on per lane, K step = 64 rows further on in the scalar offset
static void check_ring_bt(int64_t groups, int64_t kc, int64_t planes, int64_t grp, int64_t plane0) {
    const int64_t rows_total = groups * kc, bytes = planes * rows_total * 64;
    const Desc d = ring_bt_desc(rows_total, planes, grp * kc, plane0);
    const int64_t steps = kc / 64;
    for (int64_t st = 0; st < steps; ++st)           // the kernel clamps the step to the contraction range
        for (int e = 0; e < 4; ++e)
            for (int t = 0; t < 256; ++t)
                request(d, ring_bt_lane(t, e, rows_total), (uint32_t)(st * 64 * 64), bytes, plane0 + e < planes, "ring codes transposed");
}

// the same for E2M1 codes in 128-element steps: planes of 128 output columns, a K step = 128 rows, round e = plane e / 2,
// rows 64 (e % 2) .. + 63 of the step
static void check_ring_bt4(int64_t groups, int64_t kc, int64_t planes, int64_t grp, int64_t plane0) {
    const int64_t rows_total = groups * kc, bytes = planes * rows_total * 64;
    const Desc d = ring_bt_desc(rows_total, planes, grp * kc, plane0);
    const int64_t steps = kc / 128;
    for (int64_t st = 0; st < steps; ++st)
        for (int e = 0; e < 4; ++e)
            for (int t = 0; t < 256; ++t)
                request(d, ring_bt4_lane(t, e, rows_total), (uint32_t)(st * 128 * 64), bytes, plane0 + (e >> 1) < planes, "ring E2M1 codes transposed");
}

int main() {
    for (int64_t groups : {1, 3})
        for (int64_t kc : {128, 384})
            for (int64_t planes : {1, 2, 3, 5})
                for (int64_t grp = 0; grp < groups; ++grp)
                    for (int64_t plane0 = 0; plane0 < planes; plane0 += 2) check_ring_bt4(groups, kc, planes, grp, plane0);
    for (int64_t rows_total : {16, 48, 256, 272, 1008})
        for (int64_t row0 = 0; row0 < rows_total; row0 += 16)
            for (int64_t k_slots : {2, 6}) check_slot2_shuffled(rows_total, k_slots, row0);
    for (int64_t groups : {1, 3})
        for (int64_t kc : {128, 384})
            for (int64_t planes : {2, 4, 6, 10})
                for (int64_t grp = 0; grp < groups; ++grp)
                    for (int64_t plane0 = 0; plane0 < planes; plane0 += 4) check_ring_bt(groups, kc, planes, grp, plane0);
    for (int64_t rows_total : {1, 31, 37, 255, 256, 257, 300, 511, 513, 1000})
        for (int64_t row0 = 0; row0 < rows_total; row0 += (rows_total > 300 ? 97 : 1) + (row0 % 7 == 0 ? 0 : 12)) {
            for (int64_t k_slots : {1, 2, 5})
                for (int layout = 0; layout < 2; ++layout)
                    for (int kb_row : {128, 64}) check_slot2(layout, kb_row, rows_total, k_slots, row0);
            for (int64_t steps : {2, 4, 9})
                for (int row_bytes : {64, 32}) check_ring(row_bytes, rows_total, steps, row0);
        }
    // the last rows of a large operand (descriptor fields near their limits; nothing is dereferenced)
    check_ring(64, (1ll << 31) / 64 / 16 + 3, 16, (1ll << 31) / 64 / 16 - 200);
    check_slot2(1, 128, (1ll << 24) - 5, 1, (1ll << 24) - 250);
    check_slot2(0, 128, (1ll << 24) - 5, 2, (1ll << 24) - 250);
    std::printf("%lld dwords checked, %lld dropped by the range check, %d failures\n", n_checked, n_dropped, failures);
    return failures ? 1 : 0;
}

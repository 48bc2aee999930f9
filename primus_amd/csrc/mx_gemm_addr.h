// Address arithmetic of the GEMM kernels' operand requests, shared between the device code and a host-side
// bounds check (tests/test_gemm_bounds.py compiles this header with g++ and walks every request of a launch).
//
// An operand request is an LDS-direct buffer load of 16 bytes per lane:
//     address = descriptor base + per-lane offset (voffset) + scalar offset (soffset).
// On gfx950 a raw buffer descriptor's range check covers BOTH offsets, dword by dword: dword c of a request is
// fetched iff  voffset + soffset + 4 c + 4 <= num_records,  otherwise nothing is read and zeros arrive (in the
// register or, for an LDS-direct load, in LDS); there is no wrap-around when soffset alone exceeds num_records.
// (Measured on the device; tests/test_gpu_range_check.py pins it through mxl_calibrate_range_check.)
// The rule of these kernels: the descriptor of a tile starts at the tile's first row and its num_records ends with
// the OPERAND.  Whatever a request adds -- the row of a ragged last tile, a load round, a K slot beyond the
// contraction range -- a dword that is fetched lies inside the operand, whatever follows the operand in memory.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define MXL_HD __host__ __device__ __forceinline__
#else
#define MXL_HD inline
#endif

namespace mxl {
namespace addr {

// A buffer descriptor in operand-relative terms: `base` = byte offset of the descriptor's first byte from the
// operand's first byte; `records` = num_records (bytes; the hardware field saturates at 2^32 - 1).
struct Desc {
    int64_t base;
    int64_t records;
};

// ---------------- 2-slot kernel (mx_gemm_kernel) ----------------
// Codes, LAYOUT 0: row-major [rows_total, ld] (ld = bytes per row).  LAYOUT 1: K-chunk-major [ld / kb][rows_total][kb]
// (kb = bytes of a row in one K slot of 128 elements).  row0 = the tile's first row.
MXL_HD Desc slot2_code_desc(int layout, int64_t rows_total, int64_t row0, int64_t ld, int kb) {
    if (layout) return Desc{row0 * kb, rows_total * ld - row0 * kb};   // up to the end of the last chunk plane
    return Desc{row0 * ld, (rows_total - row0) * ld};
}
// thread t of the workgroup fetches 16-byte piece (t % cpr) ^ swz of tile row t / cpr in load round 0
MXL_HD uint32_t slot2_code_lane(int layout, int t, int cpr, int swz, int64_t ld, int kb) {
    return (uint32_t)((t / cpr) * (layout ? (int64_t)kb : ld) + 16 * ((t % cpr) ^ swz));
}
// load round r covers tile rows [r * rows_per_ld, (r + 1) * rows_per_ld)
MXL_HD uint32_t slot2_code_round(int layout, int r, int rows_per_ld, int64_t ld, int kb) {
    return (uint32_t)((int64_t)(r * rows_per_ld) * (layout ? (int64_t)kb : ld));
}
// K slot kp of a contraction range that starts at k0 (LAYOUT 0: byte offset inside a row; LAYOUT 1: chunk index);
// cstride = bytes of a chunk plane (rows_total * kb)
MXL_HD uint32_t slot2_code_k(int layout, uint32_t k0, int kp, int kb, uint32_t cstride) {
    return layout ? (k0 + (uint32_t)kp) * cstride : k0 + (uint32_t)kp * (uint32_t)kb;
}
// Packed FP4 codes in the pre-shuffled byte order (mxl_shuffle_codes): every block of 16 rows x 32 bytes is 512
// consecutive bytes, [16-byte half][row][16 bytes], blocks row-major.  Byte (row R, column byte c) sits at
//   ((R / 16) * (ld / 32) + c / 32) * 512 + ((c / 16) % 2) * 256 + (R % 16) * 16 + c % 16.
// A tile starts at a multiple of 16 rows, so its descriptor is the row-major one (16 rows of ld bytes are 16 * ld bytes
// in both orders); what changes is the per-lane offset of a 16-byte piece and the advance per K slot of 64 bytes
// (two 32-byte block columns = 1024 bytes).
MXL_HD uint32_t slot2_code_lane_shuffled(int t, int cpr, int swz, int64_t ld) {
    const int row = t / cpr, piece = (t % cpr) ^ swz;
    return (uint32_t)((int64_t)(row / 16) * (16 * ld) + (piece >> 1) * 512 + (piece & 1) * 256 + (row % 16) * 16);
}
MXL_HD uint32_t slot2_code_k_shuffled(int kp) { return (uint32_t)kp * 1024u; }

// Scales are row-major [rows_total, ld_s] bytes; thread t fetches the 16 bytes of panel pn (K slots 4 pn .. 4 pn + 3)
// of tile row t.  ks0 = first scale byte of the contraction range inside a row.
MXL_HD Desc slot2_scale_desc(int64_t rows_total, int64_t row0, int64_t ld_s) {
    return Desc{row0 * ld_s, (rows_total - row0) * ld_s};
}
MXL_HD uint32_t slot2_scale_off(int t, int64_t ld_s, uint32_t ks0, int pn) {
    return (uint32_t)(t * ld_s) + ks0 + 16u * (uint32_t)pn;
}

// ---------------- ring kernel (mx_gemm_ring_kernel) ----------------
// Codes are K-step-major [steps][rows_total][row_bytes] (row_bytes = 64, or 32 for E2M1 weights against FP8 rows);
// the step plane is chosen by the scalar offset step * rows_total * row_bytes.
MXL_HD Desc ring_code_desc(int64_t rows_total, int64_t steps, int64_t row0, int row_bytes) {
    return Desc{row0 * row_bytes, rows_total * steps * row_bytes - row0 * row_bytes};
}
// load round e of an operand: 4 KiB further on (64 rows of 64 bytes, or 128 rows of 32)
MXL_HD uint32_t ring_code_lane(int t, int e, bool half_rows) {
    if (half_rows) return (uint32_t)((t >> 1) * 32 + 16 * ((t & 1) ^ ((t >> 4) & 1)) + e * 4096);
    const int row = t >> 2;
    return (uint32_t)(row * 64 + 16 * ((t & 3) ^ ((row >> 2) & 3)) + e * 4096);
}
// The same operand read TRANSPOSED (the ring kernel's BT mode): the code array is [planes][rows_total][64] with
// rows_total = groups * contraction length; a tile's descriptor starts at plane `plane0` (its first 64 output columns),
// row `row0` (the group's first contraction row); load round e adds e planes per lane, the K step adds
// step * 64 rows * 64 bytes as the scalar offset (clamped to the contraction range by the kernel).
MXL_HD Desc ring_bt_desc(int64_t rows_total, int64_t planes, int64_t row0, int64_t plane0) {
    const int64_t base = (plane0 * rows_total + row0) * 64;
    return Desc{base, planes * rows_total * 64 - base};
}
MXL_HD uint32_t ring_bt_lane(int t, int e, int64_t rows_total) {
    return ring_code_lane(t, 0, false) + (uint32_t)e * (uint32_t)(rows_total * 64);
}
// The transposed read of E2M1 codes stored in 128-element steps (64-byte rows): [planes][rows_total][64] with 128
// output columns per plane; a K step is 128 contraction rows, so a tile's 256 output columns take two planes and a
// step's four load rounds are (plane e / 2, rows 64 (e % 2) .. + 63); the K step adds 128 rows * 64 bytes.
MXL_HD uint32_t ring_bt4_lane(int t, int e, int64_t rows_total) {
    return ring_code_lane(t, 0, false) + (uint32_t)(e >> 1) * (uint32_t)(rows_total * 64) + (uint32_t)(e & 1) * 4096u;
}
// Scale panels [panels][rows_total][16]: thread t fetches the 16 bytes of tile row t; the panel is chosen by the
// scalar offset panel * rows_total * 16.
MXL_HD Desc ring_panel_desc(int64_t rows_total, int64_t panels, int64_t row0) {
    return Desc{row0 * 16, rows_total * panels * 16 - row0 * 16};
}
MXL_HD uint32_t ring_panel_lane(int t) { return (uint32_t)(t * 16); }

// The hardware's decision for dword c (0 .. 3) of a 16-byte request
MXL_HD bool accepted(const Desc& d, uint32_t voff, uint32_t soff, int c) {
    const uint64_t rec = d.records <= 0 ? 0u : (d.records > 0xFFFFFFFFll ? 0xFFFFFFFFull : (uint64_t)d.records);
    return (uint64_t)voff + (uint64_t)soff + 4u * (uint32_t)c + 4u <= rec;
}

}  // namespace addr
}  // namespace mxl

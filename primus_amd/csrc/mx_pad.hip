// Padding of expert groups to the quantisation alignment, on the device.  The reference's expert MLP reads
// tokens_per_expert back to the host, splits the permuted tokens per expert and appends zero rows up to a
// multiple of the alignment (primus/backends/megatron/core/transformer/experts.py:196-209, undone at :262-264;
// the alignment is 32 for the MX recipes, 16 otherwise: primus/backends/megatron/core/extensions/
// primus_turbo.py:2344-2353).  Here the counts never leave the device:
//
//   padded[g]  = ceil(lens[g] / align) * align
//   out[dst_off[g] + i] = x[src_off[g] + i]   for i < lens[g],   zero rows for lens[g] <= i < padded[g]
//
// with src_off / dst_off the exclusive prefix sums of lens / padded.  The host cannot know sum(padded) without
// reading the counts, so `out` is sized for the worst case by the caller; the rows behind the last group's
// padding are zero rows too and are counted into the last group (padded_lens always sums to out_rows), which
// keeps "the group lengths cover the buffer" true for the kernels that consume it.  Zero rows change neither
// the other rows of a linear's output nor its weight gradient.
//
// Index work and copies only: each row is moved 16 bytes per lane where alignment allows.
#include "mx_device.h"

namespace mxl {

constexpr int PTHREADS = 256;
constexpr int PAD_MAX_GROUPS = 1024;

typedef uint32_t pu32x4 __attribute__((ext_vector_type(4)));

// exclusive prefix sums of the group lengths (negative counts read as 0) and of their padded values, by wave 0
__device__ __forceinline__ void pad_offsets(const int64_t* lens, int groups, int64_t align, int64_t* len_off,
                                            int64_t* pad_off) {
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x, per = (groups + 63) / 64, g0 = lane * per;
        int64_t a = 0, b = 0;
        for (int i = 0; i < per; ++i) {
            if (g0 + i < groups) {
                const int64_t l = lens[g0 + i] > 0 ? lens[g0 + i] : 0;
                a += l;
                b += (l + align - 1) / align * align;
            }
        }
        int64_t sa = a, sb = b;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int64_t ta = __shfl_up(sa, d), tb = __shfl_up(sb, d);
            if (lane >= d) {
                sa += ta;
                sb += tb;
            }
        }
        int64_t ea = sa - a, eb = sb - b;
        for (int i = 0; i < per; ++i) {
            if (g0 + i < groups) {
                const int64_t l = lens[g0 + i] > 0 ? lens[g0 + i] : 0;
                len_off[g0 + i] = ea;
                pad_off[g0 + i] = eb;
                ea += l;
                eb += (l + align - 1) / align * align;
            }
        }
        if (lane == 63) {
            len_off[groups] = sa;
            pad_off[groups] = sb;
        }
    }
    __syncthreads();
}

// the last group whose offset is <= row (offsets ascending, off[0] = 0): rows behind the last group map to it
__device__ __forceinline__ int group_of(const int64_t* off, int groups, int64_t row) {
    int lo = 0, hi = groups;   // first g in (0, groups] with off[g] > row, or groups
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (off[mid] > row) hi = mid;
        else lo = mid + 1;
    }
    return lo > 0 ? lo - 1 : 0;
}

// UNPAD = 0: rows of `out` are indexed in the padded space, rows of `in` in the packed one; 1: the reverse.
// ROWS_PER_LANE: rows narrower than a vector are handled one per lane, wider rows one per wave.
template <typename V, int UNPAD, int ROW_PER_LANE>
__global__ __launch_bounds__(PTHREADS) void pad_groups_kernel(const unsigned char* in, int64_t in_rows,
                                                              const int64_t* lens, int groups, int64_t align,
                                                              int64_t row_bytes, unsigned char* out, int64_t out_rows,
                                                              int64_t* padded_lens) {
    __shared__ int64_t len_off[PAD_MAX_GROUPS + 1], pad_off[PAD_MAX_GROUPS + 1];
    pad_offsets(lens, groups, align, len_off, pad_off);
    const int64_t* to_off = UNPAD ? len_off : pad_off;
    const int64_t* from_off = UNPAD ? pad_off : len_off;
    if (padded_lens != nullptr && blockIdx.x == 0) {
        for (int g = threadIdx.x; g < groups; g += PTHREADS) {
            const int64_t lo = pad_off[g] < out_rows ? pad_off[g] : out_rows;
            int64_t hi = pad_off[g + 1] < out_rows ? pad_off[g + 1] : out_rows;
            if (g == groups - 1) hi = out_rows;
            padded_lens[g] = hi - lo;
        }
    }
    const int64_t vecs = row_bytes / (int64_t)sizeof(V);
    V zero;
    __builtin_memset(&zero, 0, sizeof(V));
    if (ROW_PER_LANE) {
        for (int64_t j = (int64_t)blockIdx.x * PTHREADS + threadIdx.x; j < out_rows; j += (int64_t)gridDim.x * PTHREADS) {
            const int g = group_of(to_off, groups, j);
            const int64_t local = j - to_off[g], src = from_off[g] + local;
            const bool live = local < len_off[g + 1] - len_off[g] && src < in_rows;
            for (int64_t v = 0; v < vecs; ++v)
                ((V*)(out + j * row_bytes))[v] = live ? ((const V*)(in + src * row_bytes))[v] : zero;
        }
    } else {
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
        for (int64_t j = (int64_t)blockIdx.x * 4 + wave; j < out_rows; j += (int64_t)gridDim.x * 4) {
            const int g = group_of(to_off, groups, j);
            const int64_t local = j - to_off[g], src = from_off[g] + local;
            const bool live = local < len_off[g + 1] - len_off[g] && src < in_rows;
            V* o = (V*)(out + j * row_bytes);
            const V* s = (const V*)(in + src * row_bytes);
            if (live) {
                for (int64_t v = lane; v < vecs; v += 64) __builtin_nontemporal_store(__builtin_nontemporal_load(s + v), o + v);
            } else {
                for (int64_t v = lane; v < vecs; v += 64) __builtin_nontemporal_store(zero, o + v);
            }
        }
    }
}

template <typename V, int UNPAD>
static void launch_pad(const void* in, int64_t in_rows, const int64_t* lens, int groups, int64_t align, int64_t row_bytes,
                       void* out, int64_t out_rows, int64_t* padded_lens, hipStream_t st) {
    const bool per_lane = row_bytes <= 16;
    const int64_t per_block = per_lane ? PTHREADS : 4;
    int64_t blocks = (out_rows + per_block - 1) / per_block;
    if (blocks > 256 * 8) blocks = 256 * 8;
    if (blocks < 1) blocks = 1;   // padded_lens is written even when there is no row to move
    if (per_lane)
        hipLaunchKernelGGL((pad_groups_kernel<V, UNPAD, 1>), dim3((unsigned)blocks), dim3(PTHREADS), 0, st,
                           (const unsigned char*)in, in_rows, lens, groups, align, row_bytes, (unsigned char*)out,
                           out_rows, padded_lens);
    else
        hipLaunchKernelGGL((pad_groups_kernel<V, UNPAD, 0>), dim3((unsigned)blocks), dim3(PTHREADS), 0, st,
                           (const unsigned char*)in, in_rows, lens, groups, align, row_bytes, (unsigned char*)out,
                           out_rows, padded_lens);
}

template <int UNPAD>
static int pad_dispatch(const void* in, int64_t in_rows, const int64_t* lens, int groups, int64_t align, int64_t row_bytes,
                        void* out, int64_t out_rows, int64_t* padded_lens, void* stream) {
    if (groups < 1 || groups > PAD_MAX_GROUPS || align < 1 || align > (1 << 20) || row_bytes < 1 || in_rows < 0 ||
        out_rows < 0 || in_rows > (int64_t(1) << 40) || out_rows > (int64_t(1) << 40) || !lens)
        return MXL_EINVAL;
    if ((in_rows > 0 && !in) || (out_rows > 0 && !out)) return MXL_EINVAL;
    if (out_rows == 0 && padded_lens == nullptr) return MXL_OK;
    if (!device_is_gfx950()) return MXL_ENODEV;
    hipStream_t st = (hipStream_t)stream;
    const uintptr_t bits = (uintptr_t)in | (uintptr_t)out | (uintptr_t)row_bytes;
    if ((bits & 15) == 0) launch_pad<pu32x4, UNPAD>(in, in_rows, lens, groups, align, row_bytes, out, out_rows, padded_lens, st);
    else if ((bits & 3) == 0) launch_pad<uint32_t, UNPAD>(in, in_rows, lens, groups, align, row_bytes, out, out_rows, padded_lens, st);
    else if ((bits & 1) == 0) launch_pad<uint16_t, UNPAD>(in, in_rows, lens, groups, align, row_bytes, out, out_rows, padded_lens, st);
    else launch_pad<uint8_t, UNPAD>(in, in_rows, lens, groups, align, row_bytes, out, out_rows, padded_lens, st);
    return hipGetLastError() == hipSuccess ? MXL_OK : MXL_ELAUNCH;
}

}  // namespace mxl

using namespace mxl;

extern "C" int64_t mxl_padded_rows_bound(int64_t rows, int num_groups, int align) {
    if (rows < 0 || num_groups < 1 || align < 1) return -1;
    return (rows + (int64_t)num_groups * (align - 1)) / align * align;
}

extern "C" int mxl_pad_groups(const void* x, int64_t rows, int64_t row_bytes, const int64_t* group_lens, int num_groups,
                              int align, void* out, int64_t out_rows, int64_t* padded_lens, void* stream) {
    if (num_groups >= 1 && align >= 1 && rows >= 0 && out_rows < mxl_padded_rows_bound(rows, num_groups, align))
        return MXL_EINVAL;
    return pad_dispatch<0>(x, rows, group_lens, num_groups, align, row_bytes, out, out_rows, padded_lens, stream);
}

extern "C" int mxl_unpad_groups(const void* y, int64_t padded_rows, int64_t row_bytes, const int64_t* group_lens,
                                int num_groups, int align, void* out, int64_t rows, void* stream) {
    return pad_dispatch<1>(y, padded_rows, group_lens, num_groups, align, row_bytes, out, rows, nullptr, stream);
}

// Transposes that put the contraction dimension innermost for the backward GEMMs (gfx950).
// The grouped GEMM kernels multiply operands that are both contiguous along K ("NT").  The
// backward pass needs   dX = dY . W   (contraction over W's rows)  and  dW = dY^T . X
// (contraction over the token rows), so weights and activations are transposed once per step by
// these HBM-bound kernels: 64 x 64 tiles through LDS, 16-byte global accesses on both sides.
//
//   ats_transpose_batched      : E matrices [R, C] -> [C, R] (expert weights)
//   ats_wgrad_plan             : per expert, the padded K extent and its first column
//   ats_transpose_grouped_rows : rows [A, C] (optionally gathered) -> [C, ld_out]; the rows of expert
//                                e become columns k_start[e] .. k_start[e] + k_count[e] - 1, zero padded
#include "ats_common.hpp"

namespace ats {

constexpr int kTile = 64;
constexpr int kKPad = 64;  // K granularity of the pipelined GEMM kernels (128 bytes of bf16)

// One 64 x 64 tile.  Fast path (aligned operands, full 16-byte groups): 16-byte global loads along the
// source rows, element-wise LDS writes into the transposed tile (row pitch padded so that the
// 8 / 4 writes of a lane and the 16-byte reads afterwards spread over the banks), 16-byte LDS reads and
// 16-byte global stores along the destination rows.  Otherwise: element-wise accesses.
// in: tile origin, unless gather != nullptr: then in = matrix base + column offset and
// gather[i] / gather_div is the source row of tile row i.  Tile rows >= rows_valid read as zero;
// destination columns < out_cols_store are written (zero padding included).
template <typename T>
__device__ __forceinline__ void transpose_tile(const T* __restrict__ in, int64_t ld_in, int rows_valid, int cols_valid,
                                               const int32_t* __restrict__ gather, int gather_div,
                                               T* __restrict__ out, int64_t ld_out, int out_cols_store, T* tile,
                                               bool vec) {
    constexpr int V = Elem<T>::kVec;
    constexpr int P = kTile + V;   // pitch of the transposed tile [c][r], in elements (16-byte aligned rows)
    const int tid = threadIdx.x;
    if (vec) {
        constexpr int VPR = kTile / V;                 // vectors per tile row
        for (int i = tid; i < kTile * VPR; i += blockDim.x) {
            const int r = i / VPR, c0 = (i % VPR) * V;
            uint4 raw = make_uint4(0u, 0u, 0u, 0u);
            if (r < rows_valid && c0 < cols_valid) {
                const int64_t src = gather ? (int64_t)(gather[r] / gather_div) : (int64_t)r;
                raw = *reinterpret_cast<const uint4*>(in + src * ld_in + c0);
            }
            const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
            for (int j = 0; j < V; ++j) tile[(c0 + j) * P + r] = e[j];
        }
        __syncthreads();
        for (int i = tid; i < kTile * VPR; i += blockDim.x) {
            const int c = i / VPR, r0 = (i % VPR) * V;
            if (c < cols_valid && r0 < out_cols_store)
                *reinterpret_cast<uint4*>(out + (int64_t)c * ld_out + r0) = *reinterpret_cast<const uint4*>(tile + c * P + r0);
        }
    } else {
        for (int i = tid; i < kTile * kTile; i += blockDim.x) {
            const int r = i / kTile, c = i % kTile;
            float v = 0.f;
            if (r < rows_valid && c < cols_valid) {
                const int64_t src = gather ? (int64_t)(gather[r] / gather_div) : (int64_t)r;
                v = Elem<T>::load(in + src * ld_in + c);
            }
            Elem<T>::store(tile + c * P + r, v);
        }
        __syncthreads();
        for (int i = tid; i < kTile * kTile; i += blockDim.x) {
            const int c = i / kTile, r = i % kTile;
            if (c < cols_valid && r < out_cols_store) out[(int64_t)c * ld_out + r] = tile[c * P + r];
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void transpose_batched_kernel(const void* const* __restrict__ in_ptrs,
                                                                void* const* __restrict__ out_ptrs, int R, int C,
                                                                bool vec) {
    __shared__ __align__(16) T tile[kTile * (kTile + Elem<T>::kVec)];
    const int e = blockIdx.z;
    const int r0 = blockIdx.y * kTile, c0 = blockIdx.x * kTile;
    const T* in = static_cast<const T*>(in_ptrs[e]) + (int64_t)r0 * C + c0;
    T* out = static_cast<T*>(out_ptrs[e]) + (int64_t)c0 * R + r0;
    const int rv = R - r0 < kTile ? R - r0 : kTile;
    const int cv = C - c0 < kTile ? C - c0 : kTile;
    transpose_tile<T>(in, C, rv, cv, nullptr, 1, out, R, rv, tile, vec);
}

__global__ void wgrad_plan_kernel(const int32_t* __restrict__ row_count, int E, int32_t* __restrict__ k_start,
                                  int32_t* __restrict__ k_count) {
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    int acc = 0;
    for (int e = 0; e < E; ++e) {
        const int c = row_count[e];
        const int kp = c <= 0 ? kKPad : (c + kKPad - 1) / kKPad * kKPad;
        k_start[e] = acc;
        k_count[e] = kp;
        acc += kp;
    }
}

// grid.x walks the padded row tiles of all experts (upper bound from max_rows), grid.y the column tiles.
template <typename T>
__global__ __launch_bounds__(256) void transpose_grouped_kernel(const T* __restrict__ in, int64_t ld_in, int C,
                                                                const int32_t* __restrict__ gather, int gather_div,
                                                                const int32_t* __restrict__ row_start,
                                                                const int32_t* __restrict__ row_count, int E,
                                                                T* __restrict__ out, int64_t ld_out, bool vec) {
    __shared__ __align__(16) T tile[kTile * (kTile + Elem<T>::kVec)];
    int tile_id = blockIdx.x;
    int e = 0, kstart = 0, kp = 0;
    for (; e < E; ++e) {
        const int c = row_count[e];
        kp = c <= 0 ? kKPad : (c + kKPad - 1) / kKPad * kKPad;
        const int nt = kp / kTile;
        if (tile_id < nt) break;
        tile_id -= nt;
        kstart += kp;
    }
    if (e >= E) return;
    const int i0 = tile_id * kTile;              // first local row of this tile inside expert e
    const int count = row_count[e] > 0 ? row_count[e] : 0;
    const int rv = count - i0 < 0 ? 0 : (count - i0 < kTile ? count - i0 : kTile);
    const int c0 = blockIdx.y * kTile;
    const int cv = C - c0 < kTile ? C - c0 : kTile;
    const int64_t r0 = (int64_t)row_start[e] + i0;
    const T* src = gather ? in + c0 : in + r0 * ld_in + c0;
    transpose_tile<T>(src, ld_in, rv, cv, gather ? gather + r0 : nullptr, gather_div,
                      out + (int64_t)c0 * ld_out + kstart + i0, ld_out, kTile, tile, vec);
}

// The 64 columns of every group without rows, zeroed (the kernels that write a transposed copy from their
// epilogue never visit such a group).  grid.x: groups, grid.y: blocks of 32 rows of the transposed matrix.
template <typename T>
__global__ __launch_bounds__(256) void zero_empty_groups_kernel(T* __restrict__ out, int64_t ld, int C,
                                                                const int32_t* __restrict__ row_count,
                                                                const int32_t* __restrict__ k_start) {
    const int e = blockIdx.x;
    if (row_count[e] > 0) return;
    constexpr int V = Elem<T>::kVec;               // elements per 16 bytes
    constexpr int LPR = kKPad / V;                 // lanes per row of 64 zero columns
    const int c = blockIdx.y * (256 / LPR) + (int)threadIdx.x / LPR;
    if (c >= C) return;
    T* dst = out + (int64_t)c * ld + k_start[e] + ((int)threadIdx.x % LPR) * V;
    *reinterpret_cast<uint4*>(dst) = make_uint4(0u, 0u, 0u, 0u);
}

}  // namespace ats

extern "C" int ats_transposed_zero_empty_groups(void* out, int64_t ld, int C, const int32_t* row_count,
                                                const int32_t* k_start, int E, int dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(E > 0 && C > 0 && out && row_count && k_start && ld % kKPad == 0 && aligned16(out), ATS_ERR_INVALID_ARG,
                "ats_transposed_zero_empty_groups: E=%d C=%d ld=%lld (a multiple of %d, 16-byte aligned buffer)", E, C,
                (long long)ld, kKPad);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED,
                "ats_transposed_zero_empty_groups: dtype tag %d", dtype);
    const int rows_per_block = dtype == ATS_F32 ? 256 / (kKPad / 4) : 256 / (kKPad / 8);
    const dim3 grid((unsigned)E, (unsigned)((C + rows_per_block - 1) / rows_per_block));
    ATS_REQUIRE(grid.y <= 65535, ATS_ERR_UNSUPPORTED, "ats_transposed_zero_empty_groups: grid");
    if (dtype == ATS_F32)
        hipLaunchKernelGGL((zero_empty_groups_kernel<float>), grid, dim3(256), 0, as_stream(stream),
                           static_cast<float*>(out), ld, C, row_count, k_start);
    else
        hipLaunchKernelGGL((zero_empty_groups_kernel<bf16_t>), grid, dim3(256), 0, as_stream(stream),
                           static_cast<bf16_t*>(out), ld, C, row_count, k_start);
    ATS_CHECK_LAUNCH("ats_transposed_zero_empty_groups");
    return ATS_OK;
}

extern "C" int ats_transpose_batched(const void* const* in_ptrs, void* const* out_ptrs, int E, int R, int C, int dtype,
                                     int aligned_bases, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(E >= 0 && E <= 65535 && R > 0 && C > 0, ATS_ERR_INVALID_ARG, "ats_transpose_batched: E=%d R=%d C=%d", E, R, C);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_transpose_batched: dtype tag %d", dtype);
    if (E == 0) return ATS_OK;
    ATS_REQUIRE(in_ptrs && out_ptrs, ATS_ERR_INVALID_ARG, "ats_transpose_batched: null pointer");
    const dim3 grid((unsigned)((C + kTile - 1) / kTile), (unsigned)((R + kTile - 1) / kTile), (unsigned)E);
    ATS_REQUIRE(grid.y <= 65535, ATS_ERR_UNSUPPORTED, "ats_transpose_batched: R=%d", R);
    // 16-byte accesses need whole vector groups in both directions; the matrix bases are checked on
    // the device side only through this promise: callers pass 16-byte aligned matrices.
    const int V = dtype == ATS_F32 ? 4 : 8;
    const bool vec = R % V == 0 && C % V == 0 && aligned_bases != 0;
    if (dtype == ATS_F32)
        hipLaunchKernelGGL((transpose_batched_kernel<float>), grid, dim3(256), 0, as_stream(stream), in_ptrs, out_ptrs, R, C, vec);
    else
        hipLaunchKernelGGL((transpose_batched_kernel<bf16_t>), grid, dim3(256), 0, as_stream(stream), in_ptrs, out_ptrs, R, C, vec);
    ATS_CHECK_LAUNCH("ats_transpose_batched");
    return ATS_OK;
}

extern "C" int64_t ats_wgrad_padded_rows(int64_t max_rows, int E) {
    // upper bound of sum_e max(64, roundup(count_e, 64)) given sum_e count_e <= max_rows
    return (max_rows + (int64_t)ats::kKPad * E + ats::kKPad - 1) / ats::kKPad * ats::kKPad;
}

extern "C" int ats_wgrad_plan(const int32_t* row_count, int E, int32_t* k_start, int32_t* k_count, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(E > 0 && row_count && k_start && k_count, ATS_ERR_INVALID_ARG, "ats_wgrad_plan: E=%d or null pointer", E);
    hipLaunchKernelGGL(wgrad_plan_kernel, dim3(1), dim3(64), 0, as_stream(stream), row_count, E, k_start, k_count);
    ATS_CHECK_LAUNCH("ats_wgrad_plan");
    return ATS_OK;
}

extern "C" int ats_transpose_grouped_rows(const void* in, int64_t ld_in, int C, const int32_t* gather, int gather_div,
                                          const int32_t* row_start, const int32_t* row_count, int E, int64_t max_rows,
                                          void* out, int64_t ld_out, int dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(E > 0 && C > 0 && max_rows >= 0 && ld_in >= C && ld_out >= ats_wgrad_padded_rows(max_rows, E),
                ATS_ERR_INVALID_ARG, "ats_transpose_grouped_rows: E=%d C=%d max_rows=%lld ld_in=%lld ld_out=%lld", E, C,
                (long long)max_rows, (long long)ld_in, (long long)ld_out);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_transpose_grouped_rows: dtype tag %d", dtype);
    ATS_REQUIRE(in && row_start && row_count && out && (!gather || gather_div > 0), ATS_ERR_INVALID_ARG,
                "ats_transpose_grouped_rows: null pointer");
    const int64_t tiles = ats_wgrad_padded_rows(max_rows, E) / kTile;
    const dim3 grid((unsigned)tiles, (unsigned)((C + kTile - 1) / kTile));
    ATS_REQUIRE(tiles <= 0x7fffffffLL && grid.y <= 65535, ATS_ERR_UNSUPPORTED, "ats_transpose_grouped_rows: grid");
    const int V = dtype == ATS_F32 ? 4 : 8;
    const bool vec = C % V == 0 && ld_in % V == 0 && ld_out % V == 0 && aligned16(in) && aligned16(out);
    if (dtype == ATS_F32)
        hipLaunchKernelGGL((transpose_grouped_kernel<float>), grid, dim3(256), 0, as_stream(stream),
                           static_cast<const float*>(in), ld_in, C, gather, gather_div, row_start, row_count, E,
                           static_cast<float*>(out), ld_out, vec);
    else
        hipLaunchKernelGGL((transpose_grouped_kernel<bf16_t>), grid, dim3(256), 0, as_stream(stream),
                           static_cast<const bf16_t*>(in), ld_in, C, gather, gather_div, row_start, row_count, E,
                           static_cast<bf16_t*>(out), ld_out, vec);
    ATS_CHECK_LAUNCH("ats_transpose_grouped_rows");
    return ATS_OK;
}

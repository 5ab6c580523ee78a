// Capacity dispatch plan, row gather, token-map inversion and token-major
// combine for gfx950.
//
// The plan is a stable counting sort of the T*k assignments by expert id, in
// (token, choice) order, so that the slot of an assignment equals the number of
// earlier assignments to the same expert - exactly what a sequential
// first-come-first-served loop produces, but without ordered atomics:
//   1. per-chunk histograms (chunk = kPlanChunk consecutive assignments),
//   2. an exclusive scan over chunks per expert (+ totals, kept, offsets),
//   3. per-chunk ranking: inside a wave the rank among equal ids comes from
//      ballots; across the steps of a wave and the waves of a block from small
//      LDS counters that are only ever advanced in program order.
// Small plans (T*k <= kPlanSingle) run all three steps in one block, one launch; plans of up to kPlanFused
// assignments run in one launch of many blocks that each count the chunks before their own themselves.
#include <limits.h>

#include "ats_common.hpp"

// Products and sums below must round separately (the reference computes them as separate
// tensor ops); the HIP default would contract a*b+c into one fused multiply-add.
#pragma clang fp contract(off)

namespace ats {

constexpr int kPlanChunk = 256;      // assignments per block of the multi-block plan (64 per wave: one step)
constexpr int kPlanSingle = 1024;    // largest plan done by one block alone (256 per wave: four steps)
constexpr int kPlanMaxE = 1024;

template <typename IdxT>
__device__ __forceinline__ int load_expert(const IdxT* idx, int64_t a, int64_t n, int E, bool* bad) {
    if (a >= n) return -1;
    const long long e = (long long)idx[a];
    if (e < 0 || e >= E) {
        *bad = true;
        return -1;
    }
    return (int)e;
}

// step 1: counts of one chunk into LDS (s_cnt[w*E + e] per wave), returns via LDS
template <typename IdxT, int PERWAVE>
__device__ void chunk_wave_counts(const IdxT* idx, int64_t n, int E, int64_t chunk_base, int* s_cnt, bool* bad) {
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < 4 * E; i += 256) s_cnt[i] = 0;
    __syncthreads();
    for (int step = 0; step < PERWAVE / kWave; ++step) {
        const int64_t a = chunk_base + wave * PERWAVE + step * kWave + lane;
        const int e = load_expert(idx, a, n, E, bad);
        if (e >= 0) atomicAdd(&s_cnt[wave * E + e], 1);
    }
    __syncthreads();
}

template <typename IdxT>
__global__ __launch_bounds__(256) void plan_hist_kernel(const IdxT* __restrict__ idx, int64_t n, int E,
                                                        int32_t* __restrict__ chunk_hist,
                                                        int32_t* __restrict__ status) {
    extern __shared__ int s_cnt[];
    bool bad = false;
    chunk_wave_counts<IdxT, kPlanChunk / 4>(idx, n, E, (int64_t)blockIdx.x * kPlanChunk, s_cnt, &bad);
    for (int e = threadIdx.x; e < E; e += 256)
        chunk_hist[(int64_t)e * gridDim.x + blockIdx.x] = s_cnt[e] + s_cnt[E + e] + s_cnt[2 * E + e] + s_cnt[3 * E + e];
    // the status word is cleared here and raised by the ranking kernel, which runs after this one
    if (blockIdx.x == 0 && threadIdx.x == 0) status[0] = 0;
}

// step 2 (one block): chunk_hist -> exclusive chunk bases (in place), hist, kept, offsets.  chunk_hist is
// [E, nchunks]: an expert's chunk counts lie side by side, so the lanes of a scanning wave read one line.
// A wave scans four experts at a time: 64 chunks per pass with a prefix sum over the wave, the carry
// runs across passes.
__device__ void scan_totals(int32_t* chunk_hist, int nchunks, int E, int C, int32_t* hist, int32_t* kept,
                            int32_t* offsets, int* s_tot) {
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    constexpr int U = 4;   // experts scanned together by a wave (their loads are issued back to back)
    constexpr int P = 2;   // passes of 64 chunks whose loads are issued together
    for (int e0 = wave * U; e0 < E; e0 += nwaves * U) {
        int carry[U];
#pragma unroll
        for (int u = 0; u < U; ++u) carry[u] = 0;
        for (int base = 0; base < nchunks; base += P * kWave) {
            int v[P][U];
#pragma unroll
            for (int q = 0; q < P; ++q) {
                const int c = base + q * kWave + lane;
#pragma unroll
                for (int u = 0; u < U; ++u)
                    v[q][u] = (c < nchunks && e0 + u < E) ? chunk_hist[(int64_t)(e0 + u) * nchunks + c] : 0;
            }
#pragma unroll
            for (int q = 0; q < P; ++q) {
                const int c = base + q * kWave + lane;
                if (base + q * kWave >= nchunks) break;      // wave-uniform
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int incl = wave_inclusive_scan(v[q][u]);
                    if (c < nchunks && e0 + u < E) chunk_hist[(int64_t)(e0 + u) * nchunks + c] = carry[u] + incl - v[q][u];
                    carry[u] += __builtin_amdgcn_readlane(incl, kWave - 1);
                }
            }
        }
        if (lane == 0) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (e0 + u < E) {
                    hist[e0 + u] = carry[u];
                    const int kp = carry[u] < C ? carry[u] : C;
                    kept[e0 + u] = kp;
                    s_tot[e0 + u] = kp;
                }
            }
        }
    }
    __syncthreads();
    // offsets = exclusive prefix sums of the kept counts: the first wave, 64 experts per step
    if (wave == 0) {
        int run = 0;
        for (int e0 = 0; e0 < E; e0 += kWave) {
            const int e = e0 + lane;
            const int kp = e < E ? s_tot[e] : 0;
            const int incl = wave_inclusive_scan(kp);
            if (e < E) offsets[e] = run + incl - kp;
            run += __builtin_amdgcn_readlane(incl, kWave - 1);
        }
        if (lane == 0) offsets[E] = run;
    }
    __syncthreads();
}

__global__ __launch_bounds__(1024) void plan_scan_kernel(int32_t* __restrict__ chunk_hist, int nchunks, int E, int C,
                                                        int32_t* __restrict__ hist, int32_t* __restrict__ kept,
                                                        int32_t* __restrict__ offsets) {
    extern __shared__ int s_tot[];
    scan_totals(chunk_hist, nchunks, E, C, hist, kept, offsets, s_tot);
}

// step 3: ranks of one chunk.  s_cnt holds the per-wave counts of this chunk
// (from chunk_wave_counts); they are turned into per-wave running bases.
template <typename IdxT, int PERWAVE>
__device__ void chunk_rank_and_write(const IdxT* idx, int64_t n, int k, int E, int C, int64_t chunk_base,
                                     const int32_t* chunk_excl /* this chunk's entry of expert 0 */, int chunk_pitch,
                                     const int32_t* offsets, int* s_cnt, int32_t* slot, int32_t* token_map,
                                     int32_t* row_src, int32_t* row_of) {
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    // per-wave running base = chunk base + counts of the earlier waves
    for (int e = threadIdx.x; e < E; e += 256) {
        int run = chunk_excl[(int64_t)e * chunk_pitch];
        for (int w = 0; w < 4; ++w) {
            const int v = s_cnt[w * E + e];
            s_cnt[w * E + e] = run;
            run += v;
        }
    }
    __syncthreads();
    int* my_base = s_cnt + wave * E;
    const unsigned long long lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    // up to 64 experts: lane l keeps the running base of expert l in a register, so the loop below touches no LDS
    const bool in_regs = E <= kWave;
    int base_reg = (in_regs && lane < E) ? my_base[lane] : 0;
    for (int step = 0; step < PERWAVE / kWave; ++step) {
        const int64_t a = chunk_base + wave * PERWAVE + step * kWave + lane;
        bool bad = false;
        const int e = load_expert(idx, a, n, E, &bad);
        int rank = -1;
        unsigned long long remaining = __ballot(e >= 0);
        while (remaining) {
            // the leader and its expert are the same in all lanes: scalar reads instead of shuffles
            const int leader = __builtin_amdgcn_readfirstlane(__ffsll((long long)remaining) - 1);
            const int le = __builtin_amdgcn_readlane(e, leader);
            const unsigned long long same = __ballot(e == le);
            const int n_same = __popcll(same);
            if (in_regs) {
                const int b = __builtin_amdgcn_readlane(base_reg, le);
                if (e == le) rank = b + __popcll(same & lt_mask);
                if (lane == le) base_reg += n_same;
            } else {
                if (e == le) rank = my_base[le] + __popcll(same & lt_mask);
                // all lanes have read my_base[le]; the leader advances it for the next step
                if (lane == leader) my_base[le] += n_same;
            }
            remaining &= ~same;
        }
        if (a < n) {
            if (e >= 0 && rank < C) {
                const int row = offsets[e] + rank;
                slot[a] = rank;
                token_map[(int64_t)e * C + rank] = (int32_t)a;
                row_src[row] = (int32_t)a;
                row_of[a] = row;
            } else {
                slot[a] = -1;
                row_of[a] = -1;
            }
        }
    }
}

template <typename IdxT>
__global__ __launch_bounds__(256) void plan_rank_kernel(const IdxT* __restrict__ idx, int64_t n, int k, int E, int C,
                                                        const int32_t* __restrict__ chunk_excl,
                                                        const int32_t* __restrict__ kept,
                                                        const int32_t* __restrict__ offsets,
                                                        int32_t* __restrict__ slot, int32_t* __restrict__ token_map,
                                                        int32_t* __restrict__ row_src, int32_t* __restrict__ row_of,
                                                        int64_t row_src_len, int32_t* __restrict__ status) {
    extern __shared__ int s_cnt[];
    bool bad = false;
    const int64_t chunk_base = (int64_t)blockIdx.x * kPlanChunk;
    chunk_wave_counts<IdxT, kPlanChunk / 4>(idx, n, E, chunk_base, s_cnt, &bad);
    if (bad) status[0] = 1;
    chunk_rank_and_write<IdxT, kPlanChunk / 4>(idx, n, k, E, C, chunk_base, chunk_excl + blockIdx.x, (int)gridDim.x, offsets, s_cnt, slot,
                         token_map, row_src, row_of);
    // empty slots and unused compact rows
    const int64_t stride = (int64_t)gridDim.x * 256;
    const int64_t ec = (int64_t)E * C;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < ec; i += stride) {
        const int e = (int)(i / C);
        const int pos = (int)(i - (int64_t)e * C);
        if (pos >= kept[e]) token_map[i] = -1;
    }
    const int total = offsets[E];
    for (int64_t i = total + (int64_t)blockIdx.x * 256 + threadIdx.x; i < row_src_len; i += stride) row_src[i] = -1;
}

// Plans of up to kPlanFused assignments in ONE launch of many blocks and no workspace: a block does not wait
// for the histograms of the chunks before its own, it counts them itself.  Every block walks the whole
// index list once (at most 128 KiB from L2; 16-byte loads when the list is int32): the assignments before
// its chunk give the chunk's exclusive bases, all of them give the totals, from which every block forms
// kept / offsets for itself; then it ranks its chunk as the third kernel of the long form does.  Three
// dependent launches (4.5 + 4.7 + 7.7 us at 24576 assignments over 64 experts) become one.  Same integers
// by construction: the bases are counts of the same sets.
constexpr int kPlanFused = 32768;

// Replicas of a wave's counters in the counting pass: with few experts most lanes of a wave hit the same
// counter and the LDS atomics of an instruction run one after the other (with Zipf-skewed routing over 8
// experts two fifths of the lanes hit expert 0's).
__host__ __device__ inline int plan_count_replicas(int E) { return E <= 16 ? 8 : (E <= 64 ? 2 : 1); }

// One pass over all n indices into two counter sets: assignments before `split` (a multiple of 4) into
// cnt, the others into cnt + set_stride.  cnt: [4 waves][E][R] counters per set.
template <typename IdxT>
__device__ __forceinline__ void count_split(const IdxT* __restrict__ idx, int64_t n, int64_t split, int E, int R,
                                            int* cnt, int set_stride, bool* bad) {
    int* mine = cnt + (threadIdx.x >> 6) * E * R + (threadIdx.x & (R - 1));
    int64_t tail_from = 0;
    if (sizeof(IdxT) == 4 && (reinterpret_cast<uintptr_t>(idx) & 15) == 0) {
        // sixteen 16-byte loads in flight per thread: one at a time, the L2 round trips of the 24-32 loads a
        // thread makes were the whole cost of the pass
        const int4* v = reinterpret_cast<const int4*>(idx);
        constexpr int U = 16;
        const int64_t qend = n / 4, qsplit = split / 4;
        for (int64_t q0 = threadIdx.x; q0 < qend; q0 += 256 * U) {
            int4 w[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t q = q0 + (int64_t)u * 256;
                w[u] = v[q < qend ? q : q0];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t q = q0 + (int64_t)u * 256;
                if (q >= qend) break;
                int* set = mine + (q >= qsplit ? set_stride : 0);
                const int ids[4] = {w[u].x, w[u].y, w[u].z, w[u].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (ids[j] < 0 || ids[j] >= E) *bad = true;
                    else atomicAdd(&set[ids[j] * R], 1);
                }
            }
        }
        tail_from = qend * 4;
    }
    for (int64_t a = tail_from + threadIdx.x; a < n; a += 256) {
        const int e = load_expert(idx, a, n, E, bad);
        if (e >= 0) atomicAdd(&mine[(a >= split ? set_stride : 0) + e * R], 1);
    }
}

__device__ __forceinline__ int count_total(const int* cnt, int E, int R, int e) {
    int t = 0;
    for (int w = 0; w < 4; ++w)
        for (int r = 0; r < R; ++r) t += cnt[(w * E + e) * R + r];
    return t;
}

template <typename IdxT>
__global__ __launch_bounds__(256) void plan_fused_kernel(const IdxT* __restrict__ idx, int64_t n, int k, int E, int C,
                                                         int32_t* __restrict__ hist, int32_t* __restrict__ kept,
                                                         int32_t* __restrict__ offsets, int32_t* __restrict__ slot,
                                                         int32_t* __restrict__ token_map, int32_t* __restrict__ row_src,
                                                         int32_t* __restrict__ row_of, int64_t row_src_len,
                                                         int32_t* __restrict__ status) {
    extern __shared__ int s_all[];
    const int R = plan_count_replicas(E);
    int* s_cnt = s_all;               // [4 * E] per-wave counters of the chunk
    int* s_pre = s_all + 4 * E;       // [E] assignments before this chunk
    int* s_kept = s_all + 5 * E;      // [E]
    int* s_off = s_all + 6 * E;       // [E + 1]
    int* s_rep = s_all + 7 * E + 1;   // [2][4 * E * R] counters of the counting pass
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int64_t chunk_base = (int64_t)blockIdx.x * kPlanChunk;
    bool bad = false;
    // one pass over the whole list: assignments before the chunk into the first counter set (the chunk's
    // exclusive bases), the chunk and everything after it into the second (with the first: the totals)
    const int set = 4 * E * R;
    for (int i = threadIdx.x; i < 2 * set; i += 256) s_rep[i] = 0;
    __syncthreads();
    count_split<IdxT>(idx, n, chunk_base, E, R, s_rep, set, &bad);
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += 256) {
        const int pre = count_total(s_rep, E, R, e);
        const int tot = pre + count_total(s_rep + set, E, R, e);
        const int kp = tot < C ? tot : C;
        s_pre[e] = pre;
        s_kept[e] = kp;
        if (blockIdx.x == 0) {
            hist[e] = tot;
            kept[e] = kp;
        }
    }
    __syncthreads();
    if (wave == 0) {
        int run = 0;
        for (int e0 = 0; e0 < E; e0 += kWave) {
            const int e = e0 + lane;
            const int kp = e < E ? s_kept[e] : 0;
            const int incl = wave_inclusive_scan(kp);
            if (e < E) s_off[e] = run + incl - kp;
            run += __builtin_amdgcn_readlane(incl, kWave - 1);
        }
        if (lane == 0) s_off[E] = run;
    }
    __syncthreads();
    if (blockIdx.x == 0) {
        for (int e = threadIdx.x; e <= E; e += 256) offsets[e] = s_off[e];
        // block 0 has seen every index: it alone writes the status word
        const int any_bad = __syncthreads_or(bad ? 1 : 0);
        if (threadIdx.x == 0) status[0] = any_bad;
    }
    // ranks of the chunk
    chunk_wave_counts<IdxT, kPlanChunk / 4>(idx, n, E, chunk_base, s_cnt, &bad);
    chunk_rank_and_write<IdxT, kPlanChunk / 4>(idx, n, k, E, C, chunk_base, s_pre, 1, s_off, s_cnt, slot, token_map,
                                               row_src, row_of);
    const int64_t stride = (int64_t)gridDim.x * 256;
    const int64_t ec = (int64_t)E * C;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < ec; i += stride) {
        const int e = (int)(i / C);
        const int pos = (int)(i - (int64_t)e * C);
        if (pos >= s_kept[e]) token_map[i] = -1;
    }
    const int total = s_off[E];
    for (int64_t i = total + (int64_t)blockIdx.x * 256 + threadIdx.x; i < row_src_len; i += stride) row_src[i] = -1;
}

// Whole plan in one block (n <= kPlanSingle).
template <typename IdxT>
__global__ __launch_bounds__(256) void plan_single_kernel(const IdxT* idx, int64_t n, int k, int E,
                                                          int C, int32_t* chunk_hist,
                                                          int32_t* hist, int32_t* kept,
                                                          int32_t* offsets, int32_t* slot,
                                                          int32_t* token_map,
                                                          int32_t* row_src, int32_t* row_of,
                                                          int64_t row_src_len, int32_t* status) {
    extern __shared__ int s_all[];
    int* s_cnt = s_all;          // [4*E]
    int* s_tot = s_all + 4 * E;  // [E]
    bool bad = false;
    chunk_wave_counts<IdxT, kPlanSingle / 4>(idx, n, E, 0, s_cnt, &bad);
    if (threadIdx.x == 0) status[0] = 0;
    __syncthreads();
    if (bad) status[0] = 1;
    for (int e = threadIdx.x; e < E; e += 256)
        chunk_hist[e] = s_cnt[e] + s_cnt[E + e] + s_cnt[2 * E + e] + s_cnt[3 * E + e];
    __syncthreads();
    scan_totals(chunk_hist, 1, E, C, hist, kept, offsets, s_tot);
    __threadfence_block();
    chunk_rank_and_write<IdxT, kPlanSingle / 4>(idx, n, k, E, C, 0, chunk_hist, 1, offsets, s_cnt, slot, token_map, row_src,
                                                row_of);
    const int64_t ec = (int64_t)E * C;
    for (int64_t i = threadIdx.x; i < ec; i += 256) {
        const int e = (int)(i / C);
        const int pos = (int)(i - (int64_t)e * C);
        if (pos >= kept[e]) token_map[i] = -1;
    }
    const int total = offsets[E];
    for (int64_t i = total + threadIdx.x; i < row_src_len; i += 256) row_src[i] = -1;
}

// ------------------------------------------------------------------ row gather
// One wave per output row; 16-byte accesses; zero rows for negative map entries.
template <typename T>
__global__ __launch_bounds__(256) void gather_rows_kernel(const T* __restrict__ src, const int32_t* __restrict__ map,
                                                          int div, T* __restrict__ out, int64_t n_rows, int H,
                                                          bool vec) {
    constexpr int V = Elem<T>::kVec;
    const int lane = lane_id();
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
    for (int64_t r = wave; r < n_rows; r += nwaves) {
        const int m = map[r];
        const int64_t srow = m < 0 ? -1 : (int64_t)(m / div);
        if (vec) {
            const int nvec = H / V;
            uint4* o = reinterpret_cast<uint4*>(out + r * H);
            if (srow < 0) {
                for (int v = lane; v < nvec; v += kWave) o[v] = make_uint4(0, 0, 0, 0);
            } else {
                const uint4* s = reinterpret_cast<const uint4*>(src + srow * H);
                for (int v = lane; v < nvec; v += kWave) o[v] = s[v];
            }
        } else {
            for (int h = lane; h < H; h += kWave) {
                if (srow < 0) Elem<T>::store(out + r * H + h, 0.f);
                else out[r * H + h] = src[srow * H + h];
            }
        }
    }
}

__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        p[i] = v;
}
__global__ __launch_bounds__(256) void invert_map_kernel(const int32_t* __restrict__ token_map, int64_t n_slots,
                                                         int32_t* __restrict__ row_of, int64_t n_assign) {
    for (int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; r < n_slots;
         r += (int64_t)gridDim.x * blockDim.x) {
        const int m = token_map[r];
        if (m >= 0 && m < n_assign) row_of[m] = (int32_t)r;
    }
}

// ------------------------------------------------------------------ combine
// One wave per token.  Lanes 0..k-1 hold (row, weight) of the k choices and
// rank them by row; rows then come out in ascending order as wave-uniform
// values, and every lane accumulates its 16-byte column slices in float32 with
// separately rounded product and sum.
template <typename TY, typename TO>
__global__ __launch_bounds__(256) void combine_kernel(const TY* __restrict__ y, const int32_t* __restrict__ row_of,
                                                      const float* __restrict__ w, const TO* __restrict__ residual,
                                                      TO* __restrict__ out, int64_t T, int k, int H) {
    const int lane = lane_id();
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
    for (int64_t t = wave; t < T; t += nwaves) {
        int my_row = -1;
        float my_w = 0.f;
        if (lane < k) {
            my_row = row_of[t * k + lane];
            my_w = w[t * k + lane];
        }
        // position of this lane's row among the kept rows of the token
        int my_rank = 0;
        for (int j = 0; j < k; ++j) {
            const int rj = __shfl(my_row, j, 64);
            if (rj >= 0 && (rj < my_row || (rj == my_row && j < lane))) ++my_rank;
        }
        const int n_kept = __popcll(__ballot(my_row >= 0));
        // the column loop is wave-uniform (every lane makes every trip, lanes past the end with nh = 0): the
        // ballots and shuffles inside need lanes 0..k-1 active on the last, partial trip as well
        for (int hb = 0; hb < H; hb += kWave * 4) {
            const int h0 = hb + lane * 4;
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            const int nh = max(0, min(4, H - h0));
            for (int n = 0; n < n_kept; ++n) {
                const unsigned long long who = __ballot(my_row >= 0 && my_rank == n);
                const int src = who ? __ffsll((long long)who) - 1 : 0;
                const int64_t row = __shfl(my_row, src, 64);
                const float wt = __shfl(my_w, src, 64);
                const TY* yr = y + row * H + h0;
                for (int j = 0; j < nh; ++j) acc[j] = ((acc[j]) + (((wt) * (Elem<TY>::load(yr + j)))));
            }
            for (int j = 0; j < nh; ++j) {
                float v = acc[j];
                if (residual) v = ((Elem<TO>::load(residual + t * H + h0 + j)) + (v));
                Elem<TO>::store(out + t * H + h0 + j, v);
            }
        }
    }
}

// Vector form: H multiple of the 16-byte vector width of both types, aligned.
// PARTS: y is n_parts float32 partial results part_stride elements apart (a down projection split
// along K); an expert row is their sum in slice order, rounded to the output type like the unsplit
// projection's result, before the weighting.
// out_rows (optional): token t's sum is rounded to the output type and added onto row out_rows[t] of `out`
// (skipped where negative) instead of being written to row t: the combine followed by a scatter-add of the
// token-major result, without the intermediate tensor.
template <typename TY, typename TO, int MAXK, bool PARTS = false>
__global__ __launch_bounds__(256) void combine_vec_kernel(const TY* __restrict__ y, const int32_t* __restrict__ row_of,
                                                          const float* __restrict__ w,
                                                          const TO* __restrict__ residual, TO* __restrict__ out,
                                                          int64_t T, int k, int H, int cols_per_wave,
                                                          int n_parts = 1, int64_t part_stride = 0,
                                                          const int32_t* __restrict__ out_rows = nullptr) {
    constexpr int V = 8;  // columns per lane per step (one 16-byte bf16 vector or two float vectors)
    const int lane = lane_id();
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
    // a wave owns cols_per_wave columns of one token (combine_cols_per_wave below)
    const int pieces = (H + cols_per_wave - 1) / cols_per_wave;
    for (int64_t item = wave; item < T * pieces; item += nwaves) {
        const int64_t t = item / pieces;
        const int h_first = (int)(item - t * pieces) * cols_per_wave;
        const int h_end = min(H, h_first + cols_per_wave);
        const int64_t t_out = out_rows ? (int64_t)out_rows[t] : t;
        if (t_out < 0) continue;
        int my_row = -1;
        float my_w = 0.f;
        if (lane < k) {
            my_row = row_of[t * k + lane];
            my_w = w[t * k + lane];
        }
        // the source lanes below are the same for the whole wave: scalar reads, no shuffles through LDS
        int my_rank = 0;
        for (int j = 0; j < k; ++j) {
            const int rj = __builtin_amdgcn_readlane(my_row, j);
            if (rj >= 0 && (rj < my_row || (rj == my_row && j < lane))) ++my_rank;
        }
        const int n_kept = __popcll(__ballot(my_row >= 0));
        int64_t rows[MAXK];
        float wts[MAXK];
#pragma unroll
        for (int n = 0; n < MAXK; ++n) {
            const unsigned long long who = __ballot(my_row >= 0 && my_rank == n);
            const int src = __builtin_amdgcn_readfirstlane(who ? __ffsll((long long)who) - 1 : 0);
            rows[n] = __builtin_amdgcn_readlane(my_row, src);
            wts[n] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_w), src));
        }
#pragma unroll 4
        for (int h0 = h_first + lane * V; h0 < h_end; h0 += kWave * V) {
            float acc[V];
#pragma unroll
            for (int j = 0; j < V; ++j) acc[j] = 0.f;
            float yv[MAXK][V];
#pragma unroll
            for (int n = 0; n < MAXK; ++n) {
                if (n < n_kept) {
                    const TY* yr = y + rows[n] * H + h0;
                    if constexpr (PARTS) {
                        static_assert(sizeof(TY) == 4, "partial results are float32");
#pragma unroll
                        for (int j = 0; j < V; ++j) yv[n][j] = 0.f;
                        for (int s2 = 0; s2 < n_parts; ++s2) {
                            float pv[V];
                            Elem<TY>::unpack(*reinterpret_cast<const uint4*>(yr + s2 * part_stride), pv);
                            Elem<TY>::unpack(*reinterpret_cast<const uint4*>(yr + s2 * part_stride + 4), pv + 4);
#pragma unroll
                            for (int j = 0; j < V; ++j) yv[n][j] += pv[j];
                        }
                        if constexpr (sizeof(TO) == 2) {
#pragma unroll
                            for (int j = 0; j < V; ++j) yv[n][j] = bf16_bits_to_float(float_to_bf16_bits(yv[n][j]));
                        }
                    } else if constexpr (sizeof(TY) == 2) {
                        Elem<TY>::unpack(*reinterpret_cast<const uint4*>(yr), yv[n]);
                    } else {
                        Elem<TY>::unpack(*reinterpret_cast<const uint4*>(yr), yv[n]);
                        Elem<TY>::unpack(*reinterpret_cast<const uint4*>(yr + 4), yv[n] + 4);
                    }
                }
            }
#pragma unroll
            for (int n = 0; n < MAXK; ++n) {
                if (n < n_kept) {
#pragma unroll
                    for (int j = 0; j < V; ++j) acc[j] = ((acc[j]) + (((wts[n]) * (yv[n][j]))));
                }
            }
            if (residual) {
                float rv[V];
                const TO* rr = residual + t * H + h0;
                if constexpr (sizeof(TO) == 2) {
                    Elem<TO>::unpack(*reinterpret_cast<const uint4*>(rr), rv);
                } else {
                    Elem<TO>::unpack(*reinterpret_cast<const uint4*>(rr), rv);
                    Elem<TO>::unpack(*reinterpret_cast<const uint4*>(rr + 4), rv + 4);
                }
#pragma unroll
                for (int j = 0; j < V; ++j) acc[j] = ((rv[j]) + (acc[j]));
            }
            TO* o = out + t_out * H + h0;
            if (out_rows) {
                // the sum as the token-major result would hold it, then the addition a scatter-add performs
                float ov[V];
                if constexpr (sizeof(TO) == 2) {
                    Elem<TO>::unpack(*reinterpret_cast<const uint4*>(o), ov);
#pragma unroll
                    for (int j = 0; j < V; ++j) acc[j] = ((ov[j]) + (bf16_bits_to_float(float_to_bf16_bits(acc[j]))));
                } else {
                    Elem<TO>::unpack(*reinterpret_cast<const uint4*>(o), ov);
                    Elem<TO>::unpack(*reinterpret_cast<const uint4*>(o + 4), ov + 4);
#pragma unroll
                    for (int j = 0; j < V; ++j) acc[j] = ((ov[j]) + (acc[j]));
                }
            }
            if constexpr (sizeof(TO) == 2) {
                *reinterpret_cast<uint4*>(o) = Elem<TO>::pack(acc);
            } else {
                *reinterpret_cast<uint4*>(o) = Elem<TO>::pack(acc);
                *reinterpret_cast<uint4*>(o + 4) = Elem<TO>::pack(acc + 4);
            }
        }
    }
}

// Columns of a token that one wave combines: 1024-column pieces (two steps of 64 lanes x 8 columns) for many
// tokens, 512-column pieces for few, so that a handful of tokens still fills the chip.  Whole rows per wave
// were slower where a token has many choices (4096 tokens x 6 choices x 2048 columns: 39 -> 34 us), the same
// elsewhere: every wave spends its first microseconds on the row and weight look-up, and shorter waves overlap
// that with other waves' loads.
static int combine_cols_per_wave(int64_t T, int H) {
    const int piece = T >= 4096 ? 1024 : 512;
    return H <= piece ? H : piece;
}

template <typename TY, typename TO>
static bool launch_combine(const void* y, const int32_t* row_of, const float* w, const void* residual, void* out,
                           int64_t T, int k, int H, hipStream_t s, const int32_t* out_rows = nullptr) {
    const int cols = combine_cols_per_wave(T, H);
    int64_t blocks = (T * ((H + cols - 1) / cols) + 3) / 4;
    if (blocks > 16384) blocks = 16384;
    const TY* yp = static_cast<const TY*>(y);
    const TO* rp = static_cast<const TO*>(residual);
    TO* op = static_cast<TO*>(out);
    const bool vec = H % 8 == 0 && aligned16(y) && aligned16(out) && (!residual || aligned16(residual)) && k <= 8;
    if (out_rows && !vec) return false;      // the scattering form exists for the vector kernel only
    if (vec && k <= 2)
        hipLaunchKernelGGL((combine_vec_kernel<TY, TO, 2>), dim3((unsigned)blocks), dim3(256), 0, s, yp, row_of, w, rp,
                           op, T, k, H, cols, 1, (int64_t)0, out_rows);
    else if (vec && k <= 4)
        hipLaunchKernelGGL((combine_vec_kernel<TY, TO, 4>), dim3((unsigned)blocks), dim3(256), 0, s, yp, row_of, w, rp,
                           op, T, k, H, cols, 1, (int64_t)0, out_rows);
    else if (vec)
        hipLaunchKernelGGL((combine_vec_kernel<TY, TO, 8>), dim3((unsigned)blocks), dim3(256), 0, s, yp, row_of, w, rp,
                           op, T, k, H, cols, 1, (int64_t)0, out_rows);
    else
        hipLaunchKernelGGL((combine_kernel<TY, TO>), dim3((unsigned)blocks), dim3(256), 0, s, yp, row_of, w, rp, op, T,
                           k, H);
    return true;
}

// out[i] = sum over the n_parts partial results of parts[s * part_stride + i], added in slice order.
template <typename TO>
__global__ __launch_bounds__(256) void sum_partials_kernel(const float* __restrict__ parts, int n_parts,
                                                           int64_t part_stride, TO* __restrict__ out, int64_t n4) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
        float4 acc = *reinterpret_cast<const float4*>(parts + i * 4);
        for (int s = 1; s < n_parts; ++s) {
            const float4 v = *reinterpret_cast<const float4*>(parts + s * part_stride + i * 4);
            acc.x += v.x;
            acc.y += v.y;
            acc.z += v.z;
            acc.w += v.w;
        }
        if constexpr (sizeof(TO) == 2) {
            uint2 u;
            u.x = pack_bf16x2(acc.x, acc.y);
            u.y = pack_bf16x2(acc.z, acc.w);
            *reinterpret_cast<uint2*>(out + i * 4) = u;
        } else {
            *reinterpret_cast<float4*>(out + i * 4) = acc;
        }
    }
}

// Gate/up projection of a few rows cut along K: parts [n_parts][rows][2I] float32 (gate columns first).
// out[r, c] = silu(sum_s gate) * (sum_s up), sums in slice order, one rounding to the output type - the
// arithmetic of the fused gate/up epilogue on the summed accumulators.
template <typename TO>
__global__ __launch_bounds__(256) void swiglu_partials_kernel(const float* __restrict__ parts, int n_parts,
                                                              int64_t part_stride, TO* __restrict__ out, int64_t rows,
                                                              int I) {
    const int64_t n4 = rows * (I / 4);
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / (I / 4);
        const int c = (int)(i - r * (I / 4)) * 4;
        const float* p = parts + r * 2 * I + c;
        float4 g = *reinterpret_cast<const float4*>(p);
        float4 u = *reinterpret_cast<const float4*>(p + I);
        for (int s = 1; s < n_parts; ++s) {
            const float4 gs = *reinterpret_cast<const float4*>(p + s * part_stride);
            const float4 us = *reinterpret_cast<const float4*>(p + s * part_stride + I);
            g.x += gs.x; g.y += gs.y; g.z += gs.z; g.w += gs.w;
            u.x += us.x; u.y += us.y; u.z += us.z; u.w += us.w;
        }
        const float4 h = make_float4(silu_f(g.x) * u.x, silu_f(g.y) * u.y, silu_f(g.z) * u.z, silu_f(g.w) * u.w);
        TO* o = out + r * I + c;
        if constexpr (sizeof(TO) == 2) {
            uint2 w;
            w.x = pack_bf16x2(h.x, h.y);
            w.y = pack_bf16x2(h.z, h.w);
            *reinterpret_cast<uint2*>(o) = w;
        } else {
            *reinterpret_cast<float4*>(o) = h;
        }
    }
}

}  // namespace ats

extern "C" int ats_swiglu_partials(const float* parts, int n_parts, int64_t part_stride, void* out, int64_t rows, int I,
                                   int out_dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(n_parts >= 1 && rows >= 0 && I > 0 && I % 4 == 0 && part_stride % 4 == 0 && part_stride >= rows * 2 * I,
                ATS_ERR_INVALID_ARG, "ats_swiglu_partials: n_parts=%d rows=%lld I=%d part_stride=%lld", n_parts,
                (long long)rows, I, (long long)part_stride);
    ATS_REQUIRE(out_dtype == ATS_F32 || out_dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_swiglu_partials: dtype tag %d",
                out_dtype);
    if (rows == 0) return ATS_OK;
    ATS_REQUIRE(parts && out && aligned16(parts) && (reinterpret_cast<uintptr_t>(out) & 7u) == 0, ATS_ERR_INVALID_ARG,
                "ats_swiglu_partials: null or misaligned pointer");
    int64_t blocks = (rows * (I / 4) + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (out_dtype == ATS_F32)
        hipLaunchKernelGGL((swiglu_partials_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), parts,
                           n_parts, part_stride, static_cast<float*>(out), rows, I);
    else
        hipLaunchKernelGGL((swiglu_partials_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           parts, n_parts, part_stride, static_cast<bf16_t*>(out), rows, I);
    ATS_CHECK_LAUNCH("ats_swiglu_partials");
    return ATS_OK;
}

extern "C" int ats_sum_partials(const float* parts, int n_parts, int64_t part_stride, void* out, int64_t n,
                                int out_dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(n_parts >= 1 && n >= 0 && n % 4 == 0 && part_stride % 4 == 0 && part_stride >= n, ATS_ERR_INVALID_ARG,
                "ats_sum_partials: n_parts=%d n=%lld part_stride=%lld (multiples of 4 elements)", n_parts, (long long)n,
                (long long)part_stride);
    ATS_REQUIRE(out_dtype == ATS_F32 || out_dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_sum_partials: dtype tag %d",
                out_dtype);
    if (n == 0) return ATS_OK;
    ATS_REQUIRE(parts && out && aligned16(parts) && (reinterpret_cast<uintptr_t>(out) & 7u) == 0, ATS_ERR_INVALID_ARG,
                "ats_sum_partials: null or misaligned pointer");
    const int64_t n4 = n / 4;
    int64_t blocks = (n4 + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (out_dtype == ATS_F32)
        hipLaunchKernelGGL((sum_partials_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), parts,
                           n_parts, part_stride, static_cast<float*>(out), n4);
    else
        hipLaunchKernelGGL((sum_partials_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), parts,
                           n_parts, part_stride, static_cast<bf16_t*>(out), n4);
    ATS_CHECK_LAUNCH("ats_sum_partials");
    return ATS_OK;
}

extern "C" int ats_combine_partials(const float* parts, int n_parts, int64_t part_stride, const int32_t* row_of,
                                    const float* w, const void* residual, void* out, int64_t T, int k, int H,
                                    int out_dtype, ats_stream_t stream) {
    using namespace ats;
    const char* name = "ats_combine_partials";
    ATS_REQUIRE(T >= 0 && k > 0 && k <= 8 && H > 0 && H % 8 == 0 && n_parts >= 1 && part_stride % 4 == 0,
                ATS_ERR_INVALID_ARG, "%s: T=%lld k=%d (<= 8) H=%d (multiple of 8) n_parts=%d part_stride=%lld", name,
                (long long)T, k, H, n_parts, (long long)part_stride);
    ATS_REQUIRE(out_dtype == ATS_F32 || out_dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "%s: dtype tag %d", name, out_dtype);
    if (T == 0) return ATS_OK;
    ATS_REQUIRE(parts && row_of && w && out && aligned16(parts) && aligned16(out) && (!residual || aligned16(residual)),
                ATS_ERR_INVALID_ARG, "%s: null or misaligned pointer", name);
    const int cols = combine_cols_per_wave(T, H);
    int64_t blocks = (T * ((H + cols - 1) / cols) + 3) / 4;
    if (blocks > 16384) blocks = 16384;
    hipStream_t s = as_stream(stream);
#define ATS_COMBINE_PARTS(TO_, MAXK_)                                                                              \
    hipLaunchKernelGGL((combine_vec_kernel<float, TO_, MAXK_, true>), dim3((unsigned)blocks), dim3(256), 0, s, parts, \
                       row_of, w, static_cast<const TO_*>(residual), static_cast<TO_*>(out), T, k, H, cols, n_parts, \
                       part_stride)
    if (out_dtype == ATS_F32) {
        if (k <= 2) ATS_COMBINE_PARTS(float, 2);
        else if (k <= 4) ATS_COMBINE_PARTS(float, 4);
        else ATS_COMBINE_PARTS(float, 8);
    } else {
        if (k <= 2) ATS_COMBINE_PARTS(bf16_t, 2);
        else if (k <= 4) ATS_COMBINE_PARTS(bf16_t, 4);
        else ATS_COMBINE_PARTS(bf16_t, 8);
    }
#undef ATS_COMBINE_PARTS
    ATS_CHECK_LAUNCH(name);
    return ATS_OK;
}

extern "C" size_t ats_dispatch_plan_workspace(int64_t T, int k, int E) {
    if (T <= 0 || k <= 0 || E <= 0) return 0;
    const int64_t n = T * k;
    const int64_t nchunks = (n + ats::kPlanChunk - 1) / ats::kPlanChunk;
    return (size_t)nchunks * E * sizeof(int32_t);
}

extern "C" int ats_dispatch_plan(const void* idx, int idx_dtype, int64_t T, int k, int E, int C, int32_t* slot,
                                 int32_t* token_map, int32_t* hist, int32_t* kept, int32_t* offsets, int32_t* row_src,
                                 int32_t* row_of, int32_t* status, void* workspace, size_t workspace_bytes,
                                 ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(T >= 0 && k > 0 && E > 0 && E <= kPlanMaxE && C >= 0, ATS_ERR_INVALID_ARG,
                "ats_dispatch_plan: T=%lld k=%d E=%d C=%d (E <= %d)", (long long)T, k, E, C, kPlanMaxE);
    ATS_REQUIRE(idx_dtype == ATS_IDX_I32 || idx_dtype == ATS_IDX_I64, ATS_ERR_INVALID_ARG,
                "ats_dispatch_plan: idx dtype tag %d", idx_dtype);
    ATS_REQUIRE(T * (int64_t)k < (int64_t)INT_MAX && (int64_t)E * C < (int64_t)INT_MAX, ATS_ERR_UNSUPPORTED,
                "ats_dispatch_plan: T*k and E*C must fit in int32");
    ATS_REQUIRE((token_map || (int64_t)E * C == 0) && (T == 0 || (slot && row_of)) && hist && kept && offsets &&
                    row_src && status,
                ATS_ERR_INVALID_ARG, "ats_dispatch_plan: null output pointer");
    ATS_REQUIRE(T == 0 || idx, ATS_ERR_INVALID_ARG, "ats_dispatch_plan: null idx");
    const int64_t n = T * k;
    const bool single = n <= kPlanSingle;
    const bool fused = !single && n <= kPlanFused;
    const int64_t nchunks = single ? 1 : (n + kPlanChunk - 1) / kPlanChunk;
    const size_t need = fused ? 0 : (size_t)nchunks * E * sizeof(int32_t);
    ATS_REQUIRE(fused || (workspace && workspace_bytes >= need), ATS_ERR_WORKSPACE,
                "ats_dispatch_plan: workspace %zu bytes, need %zu", workspace_bytes, need);
    hipStream_t s = as_stream(stream);
    int32_t* chunk_hist = static_cast<int32_t*>(workspace);
    int64_t row_src_len = n < (int64_t)E * C ? n : (int64_t)E * C;
    if (row_src_len < 1) row_src_len = 1;
    const size_t smem = (size_t)5 * E * sizeof(int);
    if (fused) {
        const size_t smem_fused = ((size_t)7 * E + 1 + (size_t)8 * E * plan_count_replicas(E)) * sizeof(int);
        if (idx_dtype == ATS_IDX_I32)
            hipLaunchKernelGGL((plan_fused_kernel<int32_t>), dim3((unsigned)nchunks), dim3(256), smem_fused, s,
                               static_cast<const int32_t*>(idx), n, k, E, C, hist, kept, offsets, slot, token_map,
                               row_src, row_of, row_src_len, status);
        else
            hipLaunchKernelGGL((plan_fused_kernel<int64_t>), dim3((unsigned)nchunks), dim3(256), smem_fused, s,
                               static_cast<const int64_t*>(idx), n, k, E, C, hist, kept, offsets, slot, token_map,
                               row_src, row_of, row_src_len, status);
        ATS_CHECK_LAUNCH("ats_dispatch_plan(fused)");
        return ATS_OK;
    }
    if (single) {
        if (idx_dtype == ATS_IDX_I32)
            hipLaunchKernelGGL((plan_single_kernel<int32_t>), dim3(1), dim3(256), smem, s,
                               static_cast<const int32_t*>(idx), n, k, E, C, chunk_hist, hist, kept, offsets, slot,
                               token_map, row_src, row_of, row_src_len, status);
        else
            hipLaunchKernelGGL((plan_single_kernel<int64_t>), dim3(1), dim3(256), smem, s,
                               static_cast<const int64_t*>(idx), n, k, E, C, chunk_hist, hist, kept, offsets, slot,
                               token_map, row_src, row_of, row_src_len, status);
        ATS_CHECK_LAUNCH("ats_dispatch_plan(single)");
        return ATS_OK;
    }
    if (idx_dtype == ATS_IDX_I32)
        hipLaunchKernelGGL((plan_hist_kernel<int32_t>), dim3((unsigned)nchunks), dim3(256), smem, s,
                           static_cast<const int32_t*>(idx), n, E, chunk_hist, status);
    else
        hipLaunchKernelGGL((plan_hist_kernel<int64_t>), dim3((unsigned)nchunks), dim3(256), smem, s,
                           static_cast<const int64_t*>(idx), n, E, chunk_hist, status);
    ATS_CHECK_LAUNCH("ats_dispatch_plan(hist)");
    // 16 waves: every wave scans four experts' chunk columns, so 64 experts take one round instead of four
    hipLaunchKernelGGL(plan_scan_kernel, dim3(1), dim3(1024), (size_t)E * sizeof(int), s, chunk_hist, (int)nchunks, E,
                       C, hist, kept, offsets);
    ATS_CHECK_LAUNCH("ats_dispatch_plan(scan)");
    if (idx_dtype == ATS_IDX_I32)
        hipLaunchKernelGGL((plan_rank_kernel<int32_t>), dim3((unsigned)nchunks), dim3(256), smem, s,
                           static_cast<const int32_t*>(idx), n, k, E, C, chunk_hist, kept, offsets, slot, token_map,
                           row_src, row_of, row_src_len, status);
    else
        hipLaunchKernelGGL((plan_rank_kernel<int64_t>), dim3((unsigned)nchunks), dim3(256), smem, s,
                           static_cast<const int64_t*>(idx), n, k, E, C, chunk_hist, kept, offsets, slot, token_map,
                           row_src, row_of, row_src_len, status);
    ATS_CHECK_LAUNCH("ats_dispatch_plan(rank)");
    return ATS_OK;
}

// ------------------------------------------------------------------ plan without a workspace argument
// For callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc): the chunk histograms of the plan live in a fixed array in device memory instead of a
// caller-provided workspace.  Each GPU the library runs on holds its own copy of the array, at its own address,
// until the process ends.  In host code the array's name is only a stand-in for the symbol, never a device
// address: the address is looked up once per device with hipGetSymbolAddress and only that pointer is handed
// to kernels.
namespace ats {
constexpr size_t kPlanScratchInts = (size_t)1 << 20;      // 4 MiB: chunks * E <= 1 048 576
static __device__ __align__(256) int32_t scratch[kPlanScratchInts];
constexpr int kPlanScratchMaxDevices = 64;
static std::atomic<int32_t*> g_plan_scratch_ptr[kPlanScratchMaxDevices];

// Device address of this GPU's copy of `scratch` (looked up on the first call on a device, with that device
// current; racing first calls repeat the same idempotent lookup).
static int plan_scratch_for_current_device(int32_t** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    ATS_REQUIRE(e == hipSuccess, ATS_ERR_LAUNCH, "ats_dispatch_plan_static: hipGetDevice: %s", hipGetErrorString(e));
    ATS_REQUIRE(dev >= 0 && dev < kPlanScratchMaxDevices, ATS_ERR_UNSUPPORTED,
                "ats_dispatch_plan_static: device id %d (at most %d devices)", dev, kPlanScratchMaxDevices);
    int32_t* ptr = g_plan_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
        ATS_REQUIRE(e == hipSuccess && ptr, ATS_ERR_LAUNCH, "ats_dispatch_plan_static: hipGetSymbolAddress: %s",
                    hipGetErrorString(e));
        g_plan_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return ATS_OK;
}
}  // namespace ats

extern "C" int ats_dispatch_plan_static(const void* idx, int idx_dtype, int64_t T, int k, int E, int C, int32_t* slot,
                                        int32_t* token_map, int32_t* hist, int32_t* kept, int32_t* offsets,
                                        int32_t* row_src, int32_t* row_of, int32_t* status, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(T >= 0 && k > 0 && E > 0, ATS_ERR_INVALID_ARG, "ats_dispatch_plan_static: T=%lld k=%d E=%d",
                (long long)T, k, E);
    const size_t need = ats_dispatch_plan_workspace(T, k, E);
    ATS_REQUIRE(need <= kPlanScratchInts * sizeof(int32_t), ATS_ERR_WORKSPACE,
                "ats_dispatch_plan_static: T*k=%lld assignments over %d experts need %zu bytes of chunk histograms, "
                "the fixed scratch array holds %zu (use ats_dispatch_plan with a workspace)",
                (long long)(T * k), E, need, kPlanScratchInts * sizeof(int32_t));
    int32_t* chunk_hist = nullptr;
    const int rc = plan_scratch_for_current_device(&chunk_hist);
    if (rc != ATS_OK) return rc;
    // every chunk histogram the plan reads is written by its first kernel, so nothing has to start at zero
    return ats_dispatch_plan(idx, idx_dtype, T, k, E, C, slot, token_map, hist, kept, offsets, row_src, row_of, status,
                             chunk_hist, kPlanScratchInts * sizeof(int32_t), stream);
}

extern "C" int ats_gather_rows(const void* src, const int32_t* map, int div, void* out, int64_t n_rows, int H,
                               int dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(n_rows >= 0 && H > 0 && div > 0, ATS_ERR_INVALID_ARG, "ats_gather_rows: n_rows=%lld H=%d div=%d",
                (long long)n_rows, H, div);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_gather_rows: dtype tag %d", dtype);
    if (n_rows == 0) return ATS_OK;
    ATS_REQUIRE(src && map && out, ATS_ERR_INVALID_ARG, "ats_gather_rows: null pointer");
    int64_t blocks = (n_rows + 3) / 4;
    if (blocks > 32768) blocks = 32768;
    const int V = dtype == ATS_F32 ? 4 : 8;
    const bool vec = H % V == 0 && aligned16(src) && aligned16(out);
    if (dtype == ATS_F32)
        hipLaunchKernelGGL((gather_rows_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const float*>(src), map, div, static_cast<float*>(out), n_rows, H, vec);
    else
        hipLaunchKernelGGL((gather_rows_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const bf16_t*>(src), map, div, static_cast<bf16_t*>(out), n_rows, H, vec);
    ATS_CHECK_LAUNCH("ats_gather_rows");
    return ATS_OK;
}

extern "C" int ats_invert_token_map(const int32_t* token_map, int64_t n_slots, int32_t* row_of, int64_t n_assign,
                                    ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(n_slots >= 0 && n_assign >= 0 && n_slots < INT_MAX, ATS_ERR_INVALID_ARG,
                "ats_invert_token_map: n_slots=%lld n_assign=%lld", (long long)n_slots, (long long)n_assign);
    if (n_assign == 0) return ATS_OK;
    ATS_REQUIRE(row_of && (n_slots == 0 || token_map), ATS_ERR_INVALID_ARG, "ats_invert_token_map: null pointer");
    hipStream_t s = as_stream(stream);
    int64_t b1 = (n_assign + 255) / 256;
    if (b1 > 4096) b1 = 4096;
    hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)b1), dim3(256), 0, s, row_of, n_assign, -1);
    ATS_CHECK_LAUNCH("ats_invert_token_map(fill)");
    if (n_slots > 0) {
        int64_t b2 = (n_slots + 255) / 256;
        if (b2 > 4096) b2 = 4096;
        hipLaunchKernelGGL(invert_map_kernel, dim3((unsigned)b2), dim3(256), 0, s, token_map, n_slots, row_of,
                           n_assign);
        ATS_CHECK_LAUNCH("ats_invert_token_map");
    }
    return ATS_OK;
}

extern "C" int ats_combine_scatter_add(const void* y, const int32_t* row_of, const float* w, const int32_t* out_rows,
                                       void* out, int64_t T, int k, int H, int y_dtype, int out_dtype,
                                       ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(T >= 0 && k > 0 && H > 0, ATS_ERR_INVALID_ARG, "ats_combine_scatter_add: T=%lld k=%d H=%d", (long long)T,
                k, H);
    ATS_REQUIRE((y_dtype == ATS_F32 || y_dtype == ATS_BF16) && (out_dtype == ATS_F32 || out_dtype == ATS_BF16),
                ATS_ERR_UNSUPPORTED, "ats_combine_scatter_add: dtype tags %d/%d", y_dtype, out_dtype);
    if (T == 0) return ATS_OK;
    ATS_REQUIRE(y && row_of && w && out && out_rows, ATS_ERR_INVALID_ARG, "ats_combine_scatter_add: null pointer");
    ATS_REQUIRE(k <= 8 && H % 8 == 0 && aligned16(y) && aligned16(out), ATS_ERR_UNSUPPORTED,
                "ats_combine_scatter_add: k=%d (at most 8), H=%d (a multiple of 8), 16-byte aligned operands; use "
                "ats_combine and ats_scatter_add_rows", k, H);
    hipStream_t s = as_stream(stream);
    bool ok;
    if (y_dtype == ATS_F32 && out_dtype == ATS_F32)
        ok = launch_combine<float, float>(y, row_of, w, nullptr, out, T, k, H, s, out_rows);
    else if (y_dtype == ATS_BF16 && out_dtype == ATS_BF16)
        ok = launch_combine<bf16_t, bf16_t>(y, row_of, w, nullptr, out, T, k, H, s, out_rows);
    else if (y_dtype == ATS_F32 && out_dtype == ATS_BF16)
        ok = launch_combine<float, bf16_t>(y, row_of, w, nullptr, out, T, k, H, s, out_rows);
    else
        ok = launch_combine<bf16_t, float>(y, row_of, w, nullptr, out, T, k, H, s, out_rows);
    ATS_REQUIRE(ok, ATS_ERR_UNSUPPORTED, "ats_combine_scatter_add: sizes outside the vector kernel");
    ATS_CHECK_LAUNCH("ats_combine_scatter_add");
    return ATS_OK;
}

extern "C" int ats_combine(const void* y, const int32_t* row_of, const float* w, const void* residual, void* out,
                           int64_t T, int k, int H, int y_dtype, int out_dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(T >= 0 && k > 0 && k <= 64 && H > 0, ATS_ERR_INVALID_ARG, "ats_combine: T=%lld k=%d H=%d",
                (long long)T, k, H);
    ATS_REQUIRE((y_dtype == ATS_F32 || y_dtype == ATS_BF16) && (out_dtype == ATS_F32 || out_dtype == ATS_BF16),
                ATS_ERR_UNSUPPORTED, "ats_combine: dtype tags %d/%d", y_dtype, out_dtype);
    if (T == 0) return ATS_OK;
    ATS_REQUIRE(y && row_of && w && out, ATS_ERR_INVALID_ARG, "ats_combine: null pointer");
    hipStream_t s = as_stream(stream);
    if (y_dtype == ATS_F32 && out_dtype == ATS_F32) launch_combine<float, float>(y, row_of, w, residual, out, T, k, H, s);
    else if (y_dtype == ATS_BF16 && out_dtype == ATS_BF16)
        launch_combine<bf16_t, bf16_t>(y, row_of, w, residual, out, T, k, H, s);
    else if (y_dtype == ATS_F32 && out_dtype == ATS_BF16)
        launch_combine<float, bf16_t>(y, row_of, w, residual, out, T, k, H, s);
    else
        launch_combine<bf16_t, float>(y, row_of, w, residual, out, T, k, H, s);
    ATS_CHECK_LAUNCH("ats_combine");
    return ATS_OK;
}

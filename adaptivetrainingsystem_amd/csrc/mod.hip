// Mixture-of-Depths helpers for gfx950: per-token router score (H -> 1 linear,
// HBM-bound: x is read once), per-sequence top-`keep` selection, and the
// scatter-add of the block output onto the residual stream.
#include <limits.h>
#include <math.h>

#include "ats_common.hpp"

// Sums below must not be contracted with a preceding product into a fused multiply-add.
#pragma clang fp contract(off)

namespace ats {

// One wave per token row; 16-byte loads; weight vector re-read from L2.  copy_out (optional): the rows are also
// written there as they pass, which starts a residual output without a second pass over x.
template <typename T>
__global__ __launch_bounds__(256) void row_dot_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                      const float* __restrict__ bias, float* __restrict__ score,
                                                      float* __restrict__ prob, float temperature,
                                                      T* __restrict__ copy_out, int64_t Tn, int H, bool vec) {
    constexpr int V = Elem<T>::kVec;
    const int lane = lane_id();
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
    for (int64_t t = wave; t < Tn; t += nwaves) {
        float acc = 0.f;
        if (vec) {
            const uint4* xr = reinterpret_cast<const uint4*>(x + t * H);
            const uint4* wr = reinterpret_cast<const uint4*>(w);
            uint4* cr = copy_out ? reinterpret_cast<uint4*>(copy_out + t * H) : nullptr;
            for (int v = lane; v < H / V; v += kWave) {
                float a[V], b[V];
                const uint4 xv = xr[v];
                if (cr) cr[v] = xv;
                Elem<T>::unpack(xv, a);
                Elem<T>::unpack(wr[v], b);
#pragma unroll
                for (int j = 0; j < V; ++j) acc += a[j] * b[j];
            }
        } else {
            for (int h = lane; h < H; h += kWave) {
                if (copy_out) copy_out[t * H + h] = x[t * H + h];
                acc += Elem<T>::load(x + t * H + h) * Elem<T>::load(w + h);
            }
        }
        acc = wave_sum(acc);
        if (lane == 0) {
            const float sc = acc + (bias ? bias[0] : 0.f);
            if (score) score[t] = sc;
            if (prob) prob[t] = 1.0f / (1.0f + expf(-__fdiv_rn(sc, temperature)));
        }
    }
}

// One block per sequence.  Bitonic sort of (score desc, position asc) keys in
// LDS, then the first `keep` positions are flagged and compacted in position
// order with a block-wide prefix sum.
__global__ __launch_bounds__(1024) void select_topk_seq_kernel(const float* __restrict__ score, int L, int Lpow2,
                                                               int keep, int32_t* __restrict__ sel) {
    extern __shared__ unsigned char smem_raw[];
    float* s_val = reinterpret_cast<float*>(smem_raw);      // [Lpow2]
    int* s_pos = reinterpret_cast<int*>(s_val + Lpow2);      // [Lpow2]
    int* s_flag = s_pos + Lpow2;                             // [Lpow2] then prefix sums
    const int b = blockIdx.x;
    const int nthr = blockDim.x;
    for (int i = threadIdx.x; i < Lpow2; i += nthr) {
        s_val[i] = i < L ? score[(int64_t)b * L + i] : -INFINITY;
        s_pos[i] = i < L ? i : INT_MAX;
        s_flag[i] = 0;
    }
    __syncthreads();
    // "a before b": larger score first (NaN above all), lower position among equals
    auto before = [](float va, int pa, float vb, int pb) {
        const bool na = va != va, nb = vb != vb;
        if (na != nb) return na;
        if (!na && va != vb) return va > vb;
        return pa < pb;
    };
    for (int size = 2; size <= Lpow2; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int i = threadIdx.x; i < (Lpow2 >> 1); i += nthr) {
                const int lo = 2 * i - (i & (stride - 1));
                const int hi = lo + stride;
                const bool asc_block = ((lo & size) == 0);  // this block sorts "before"-first
                const float va = s_val[lo], vb = s_val[hi];
                const int pa = s_pos[lo], pb = s_pos[hi];
                const bool swap = asc_block ? before(vb, pb, va, pa) : before(va, pa, vb, pb);
                if (swap) {
                    s_val[lo] = vb;
                    s_val[hi] = va;
                    s_pos[lo] = pb;
                    s_pos[hi] = pa;
                }
            }
            __syncthreads();
        }
    }
    for (int i = threadIdx.x; i < keep; i += nthr) s_flag[s_pos[i]] = 1;
    __syncthreads();
    // inclusive prefix sum of the flags (Hillis-Steele over LDS, two buffers folded into s_val as int)
    int* s_a = s_flag;
    int* s_b = reinterpret_cast<int*>(s_val);
    for (int off = 1; off < Lpow2; off <<= 1) {
        for (int i = threadIdx.x; i < Lpow2; i += nthr) s_b[i] = s_a[i] + (i >= off ? s_a[i - off] : 0);
        __syncthreads();
        int* t = s_a;
        s_a = s_b;
        s_b = t;
    }
    for (int i = threadIdx.x; i < L; i += nthr) {
        const int incl = s_a[i];
        const int prev = i > 0 ? s_a[i - 1] : 0;
        if (incl != prev) sel[(int64_t)b * keep + prev] = b * L + i;
    }
}

// The same selection by radix select, for sequences of up to 1024 * PER positions: thread t keeps positions
// [t * PER, (t + 1) * PER) in registers as order-preserving keys (NaN above everything, as torch.topk ranks it).
// Four 8-bit passes from the top byte find the key of the keep-th largest score and how many positions with
// exactly that key are still wanted; those are the ones with the lowest positions (rank among equals by a
// block-wide prefix sum in position order).  A second prefix sum compacts the selected positions in ascending
// order.  No sort: 4 histogram passes + 2 scans instead of 66 compare-exchange passes over LDS.
__device__ __forceinline__ uint32_t topk_key(float f) {
    if (f != f) return 0xffffffffu;
    if (f == 0.f) return 0x80000000u;       // -0 and +0 are equal scores
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Exclusive prefix sum of one int per thread over a 1024-thread block, in thread order.  s_wave: 16 ints of LDS.
__device__ __forceinline__ int block_exclusive_scan_1024(int v, int* s_wave, int* total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int incl = wave_inclusive_scan(v);
    __syncthreads();                       // s_wave may still be read from a previous call
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    int base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
        const int c = s_wave[w];
        if (w < wave) base += c;
        tot += c;
    }
    *total = tot;
    return base + incl - v;
}

template <int PER>
__global__ __launch_bounds__(1024) void select_topk_radix_kernel(const float* __restrict__ score, int L, int keep,
                                                                 int32_t* __restrict__ sel) {
    __shared__ unsigned int s_hist[256];
    __shared__ int s_wave[16];
    __shared__ unsigned int s_pick[2];      // chosen bin, count still wanted inside it
    const int b = blockIdx.x;
    const int t = threadIdx.x;
    uint32_t key[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = t * PER + j;
        key[j] = i < L ? topk_key(score[(int64_t)b * L + i]) : 0u;     // positions past L never match (see valid)
    }
    uint32_t prefix = 0, mask = 0;
    unsigned int want = (unsigned int)keep;
    for (int pass = 3; pass >= 0; --pass) {
        if (t < 256) s_hist[t] = 0;
        __syncthreads();
        const int shift = pass * 8;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int i = t * PER + j;
            if (i < L && (key[j] & mask) == prefix) atomicAdd(&s_hist[(key[j] >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (t < 64) {
            // lane l owns bins 255 - 4l ... 252 - 4l (descending); suffix sums from the top bin down
            unsigned int c[4], sum = 0;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                c[q] = s_hist[255 - 4 * t - q];
                sum += c[q];
            }
            const unsigned int incl = (unsigned int)wave_inclusive_scan((int)sum);
            const unsigned int before = incl - sum;          // keys in higher bins than this lane's
            if (before < want && incl >= want) {
                unsigned int acc = before;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if (acc < want && acc + c[q] >= want) {
                        s_pick[0] = 255u - 4u * t - q;
                        s_pick[1] = want - acc;
                    }
                    acc += c[q];
                }
            }
        }
        __syncthreads();
        prefix |= s_pick[0] << shift;
        mask |= 255u << shift;
        want = s_pick[1];
        __syncthreads();
    }
    // prefix = key of the keep-th largest; `want` positions with exactly that key are taken, lowest positions first
    int eq = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) eq += (t * PER + j < L && key[j] == prefix) ? 1 : 0;
    int tot;
    int eq_rank = block_exclusive_scan_1024(eq, s_wave, &tot);
    bool take[PER];
    int ntake = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const bool valid = t * PER + j < L;
        take[j] = valid && key[j] > prefix;
        if (valid && key[j] == prefix) {
            take[j] = eq_rank < (int)want;
            ++eq_rank;
        }
        ntake += take[j] ? 1 : 0;
    }
    int out = block_exclusive_scan_1024(ntake, s_wave, &tot);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        if (take[j]) sel[(int64_t)b * keep + out++] = b * L + t * PER + j;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void scatter_add_rows_kernel(T* __restrict__ base, const int32_t* __restrict__ rows,
                                                               const T* __restrict__ delta, int64_t n, int H,
                                                               bool vec) {
    constexpr int V = Elem<T>::kVec;
    const int lane = lane_id();
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (blockDim.x >> 6);
    for (int64_t i = wave; i < n; i += nwaves) {
        const int64_t r = rows[i];
        if (r < 0) continue;
        if (vec) {
            uint4* bp = reinterpret_cast<uint4*>(base + r * H);
            const uint4* dp = reinterpret_cast<const uint4*>(delta + i * H);
            for (int v = lane; v < H / V; v += kWave) {
                float a[V], d[V];
                Elem<T>::unpack(bp[v], a);
                Elem<T>::unpack(dp[v], d);
#pragma unroll
                for (int j = 0; j < V; ++j) a[j] = ((a[j]) + (d[j]));
                bp[v] = Elem<T>::pack(a);
            }
        } else {
            for (int h = lane; h < H; h += kWave)
                Elem<T>::store(base + r * H + h, ((Elem<T>::load(base + r * H + h)) + (Elem<T>::load(delta + i * H + h))));
        }
    }
}

// k-th smallest value (1-based) of n floats by a 4-pass, 8-bit radix select in one
// block, then a threshold mask.  Keys are the usual order-preserving unsigned
// image of the float bits.
__device__ __forceinline__ uint32_t order_key(float f) {
    // -0.0 and +0.0 compare equal as floats, so they share a key
    const uint32_t u = f == 0.0f ? 0u : __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// One digit of the radix select, by one wave (all 64 lanes): the bin of `hist` (256 counts, ascending digits)
// in which the running rank falls.  Lane l owns bins 4l .. 4l+3; a prefix sum over the lanes' sums finds the
// lane, a walk over its four bins the bin.  Returns the bin and updates *rank to the rank inside it.
__device__ __forceinline__ int kth_find_bin(const unsigned int* hist, long long* rank, int lane) {
    unsigned int c[4];
    unsigned int sum = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        c[q] = hist[4 * lane + q];
        sum += c[q];
    }
    const long long incl = (long long)(unsigned int)wave_inclusive_scan((int)sum);
    const long long before = incl - sum;
    const long long want = *rank;
    // the first lane whose inclusive count reaches the rank; the last lane takes what is left (bin 255 then)
    unsigned long long hit = __ballot(want <= incl);
    const int owner = hit ? __ffsll((long long)hit) - 1 : 63;
    int bin = 4 * lane + 3;
    long long left = want - before;
    if (lane == owner) {
        if (left <= (long long)c[0]) {
            bin = 4 * lane;
        } else {
            left -= c[0];
            if (left <= (long long)c[1]) {
                bin = 4 * lane + 1;
            } else {
                left -= c[1];
                if (left <= (long long)c[2]) {
                    bin = 4 * lane + 2;
                } else {
                    left -= c[2];
                }
            }
        }
    }
    const int b = __builtin_amdgcn_readlane(bin, owner);
    const int lo = __builtin_amdgcn_readlane((int)(left & 0xffffffffll), owner);
    const int hi = __builtin_amdgcn_readlane((int)(left >> 32), owner);
    *rank = ((long long)hi << 32) | (unsigned int)lo;
    return b;
}

__global__ __launch_bounds__(1024) void kth_value_kernel(const float* __restrict__ v, int64_t n, int64_t kth,
                                                         uint32_t* __restrict__ key_out,
                                                         long long* __restrict__ count_out) {
    __shared__ unsigned int hist[256];
    __shared__ uint32_t s_prefix;
    __shared__ long long s_rank;
    if (threadIdx.x == 0) {
        s_prefix = 0;
        s_rank = kth;
    }
    for (int pass = 3; pass >= 0; --pass) {
        for (int i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0;
        __syncthreads();
        const uint32_t prefix = s_prefix;
        const uint32_t hi_mask = pass == 3 ? 0u : (0xffffffffu << (8 * (pass + 1)));
        for (int64_t i = threadIdx.x; i < n; i += blockDim.x) {
            const uint32_t key = order_key(v[i]);
            if ((key & hi_mask) == prefix) atomicAdd(&hist[(key >> (8 * pass)) & 255u], 1u);
        }
        __syncthreads();
        if (threadIdx.x < 64) {
            long long rank = s_rank;
            const int b = kth_find_bin(hist, &rank, (int)threadIdx.x);
            if (threadIdx.x == 0) {
                s_rank = rank;
                s_prefix = prefix | ((uint32_t)b << (8 * pass));
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        key_out[0] = s_prefix;
        // s_rank is now the 1-based rank of the k-th value among the values equal to it, so kth - s_rank values
        // are strictly smaller and the mask keeps the rest
        if (count_out) count_out[0] = (long long)n - kth + s_rank;
    }
}

// The same select over many workgroups, one launch per digit: every block counts the digit of its share of
// the values that match the prefix found so far into LDS and adds its 256 counts to the pass's histogram in
// `ghist` ([4][256], zeroed by the caller).  The prefix is not stored anywhere: the first wave of every block
// walks the histograms of the passes above its own again (at most three 256-bin searches).
__device__ __forceinline__ void kth_walk(const unsigned int* ghist, int upto, long long kth, int lane, uint32_t* prefix,
                                         long long* rank) {
    uint32_t pre = 0;
    long long r = kth;
    for (int q = 3; q > upto; --q) {
        const int b = kth_find_bin(ghist + q * 256, &r, lane);
        pre |= (uint32_t)b << (8 * q);
    }
    *prefix = pre;
    *rank = r;
}

__global__ __launch_bounds__(256) void kth_digit_hist_kernel(const float* __restrict__ v, int64_t n, int64_t kth, int pass,
                                                             unsigned int* __restrict__ ghist) {
    __shared__ unsigned int hist[256];
    __shared__ uint32_t s_prefix;
    hist[threadIdx.x] = 0;
    if (threadIdx.x < 64) {
        uint32_t prefix;
        long long rank;
        kth_walk(ghist, pass, kth, (int)threadIdx.x, &prefix, &rank);
        if (threadIdx.x == 0) s_prefix = prefix;
    }
    __syncthreads();
    const uint32_t prefix = s_prefix;
    const uint32_t hi_mask = pass == 3 ? 0u : (0xffffffffu << (8 * (pass + 1)));
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const uint32_t key = order_key(v[i]);
        if ((key & hi_mask) == prefix) atomicAdd(&hist[(key >> (8 * pass)) & 255u], 1u);
    }
    __syncthreads();
    const unsigned int c = hist[threadIdx.x];
    if (c) atomicAdd(&ghist[pass * 256 + threadIdx.x], c);
}

__global__ __launch_bounds__(256) void kth_mask_kernel(const float* __restrict__ v, int64_t n, int64_t kth,
                                                       const unsigned int* __restrict__ ghist,
                                                       uint32_t* __restrict__ key_out, long long* __restrict__ count_out,
                                                       float* __restrict__ mask) {
    __shared__ uint32_t s_thr;
    if (threadIdx.x < 64) {
        uint32_t prefix;
        long long rank;
        kth_walk(ghist, -1, kth, (int)threadIdx.x, &prefix, &rank);
        if (threadIdx.x == 0) {
            s_thr = prefix;
            if (blockIdx.x == 0) {
                key_out[0] = prefix;
                if (count_out) count_out[0] = (long long)n - kth + rank;
            }
        }
    }
    __syncthreads();
    const uint32_t thr = s_thr;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        mask[i] = order_key(v[i]) >= thr ? 1.0f : 0.0f;
}

__global__ __launch_bounds__(64) void kth_key_kernel(int64_t n, int64_t kth, const unsigned int* __restrict__ ghist,
                                                     uint32_t* __restrict__ key_out, long long* __restrict__ count_out) {
    uint32_t prefix;
    long long rank;
    kth_walk(ghist, -1, kth, (int)threadIdx.x, &prefix, &rank);
    if (threadIdx.x == 0) {
        key_out[0] = prefix;
        count_out[0] = (long long)n - kth + rank;
    }
}

__global__ __launch_bounds__(256) void kth_zero_kernel(unsigned int* __restrict__ ghist) {
    for (int i = threadIdx.x; i < 4 * 256; i += 256) ghist[i] = 0;
}

__global__ __launch_bounds__(256) void threshold_mask_kernel(const float* __restrict__ v, int64_t n,
                                                             const uint32_t* __restrict__ key, float* __restrict__ mask) {
    const uint32_t thr = key[0];
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        mask[i] = order_key(v[i]) >= thr ? 1.0f : 0.0f;
}

// Training branch of the MoD router (MS/core/model.py:941-965): a 0/1 mask with exactly k ones at the k
// largest values, and the straight-through weights (mask - p) + p formed in float32 in the reference's order.
// `thr` is the order key of the k-th largest value and `count_ge` the number of values >= it (both from the
// radix select).  When count_ge == k every value at the threshold is in; otherwise only the first
// k - (number above) of them in index order are (the lower index wins among equals, the rule of the routing
// kernels), which the second kernel settles in one workgroup that walks the values in order.
__device__ __forceinline__ float ste_weight(float m, float p) { return (m - p) + p; }

__global__ __launch_bounds__(256) void topk_mask_kernel(const float* __restrict__ v, int64_t n, int64_t k,
                                                        const uint32_t* __restrict__ key,
                                                        const long long* __restrict__ count_ge,
                                                        float* __restrict__ mask, float* __restrict__ ste) {
    const uint32_t thr = key[0];
    const bool all_ties_in = count_ge[0] == (long long)k;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const float p = v[i];
        const uint32_t kk = order_key(p);
        const float m = (kk > thr || (kk == thr && all_ties_in)) ? 1.0f : 0.0f;
        mask[i] = m;
        if (ste) ste[i] = ste_weight(m, p);
    }
}

__global__ __launch_bounds__(1024) void topk_ties_kernel(const float* __restrict__ v, int64_t n, int64_t k,
                                                         const uint32_t* __restrict__ key,
                                                         const long long* __restrict__ count_ge,
                                                         float* __restrict__ mask, float* __restrict__ ste) {
    if (count_ge[0] == (long long)k) return;          // uniform: nothing to settle
    __shared__ int wave_cnt[16];
    __shared__ long long s_total;
    const uint32_t thr = key[0];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // values equal to the threshold
    long long mine = 0;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) mine += order_key(v[i]) == thr ? 1 : 0;
    int w = wave_inclusive_scan((int)mine);
    if (lane == 63) wave_cnt[wave] = w;
    __syncthreads();
    if (threadIdx.x == 0) {
        long long t = 0;
        for (int q = 0; q < 16; ++q) t += wave_cnt[q];
        s_total = t;
    }
    __syncthreads();
    // ones still to hand out: k minus the values above the threshold
    long long need = (long long)k - (count_ge[0] - s_total);
    long long base = 0;
    for (int64_t i0 = 0; i0 < n && base < need; i0 += blockDim.x) {
        const int64_t i = i0 + threadIdx.x;
        const bool eq = i < n && order_key(v[i]) == thr;
        const unsigned long long b = __ballot(eq);
        __syncthreads();                              // wave_cnt of the previous chunk has been read
        if (lane == 0) wave_cnt[wave] = __popcll(b);
        __syncthreads();
        int before = 0, chunk = 0;
        for (int q = 0; q < 16; ++q) {
            const int c = wave_cnt[q];
            before += q < wave ? c : 0;
            chunk += c;
        }
        if (eq) {
            const long long rank = base + before + __popcll(b & ((1ull << lane) - 1ull));
            if (rank < need) {
                mask[i] = 1.0f;
                if (ste) ste[i] = ste_weight(1.0f, v[i]);
            }
        }
        base += chunk;
    }
}

__global__ __launch_bounds__(256) void fill_mask_kernel(const float* __restrict__ v, int64_t n, float m,
                                                        float* __restrict__ mask, float* __restrict__ ste) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        mask[i] = m;
        if (ste) ste[i] = ste_weight(m, v[i]);
    }
}

// Gradient of the router's logits: gl = (dL/dweights + dL/dprobs) * p * (1 - p) / temperature (the
// straight-through weights pass their gradient to the probabilities unchanged; sigmoid' = p (1 - p)), and the
// gradient of the bias, their sum, added in a fixed order by one workgroup.
__global__ __launch_bounds__(1024) void mod_route_bwd_kernel(const float* __restrict__ gw, const float* __restrict__ gp,
                                                             const float* __restrict__ prob, float inv_temperature,
                                                             float* __restrict__ gl, float* __restrict__ dbias,
                                                             int64_t n) {
    __shared__ float part[1024];
    float acc = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float p = prob[i];
        const float g = ((gw ? gw[i] : 0.f) + (gp ? gp[i] : 0.f)) * (p * (1.0f - p)) * inv_temperature;
        gl[i] = g;
        acc += g;
    }
    part[threadIdx.x] = acc;
    __syncthreads();
    for (int s2 = 512; s2 > 0; s2 >>= 1) {
        if ((int)threadIdx.x < s2) part[threadIdx.x] += part[threadIdx.x + s2];
        __syncthreads();
    }
    if (threadIdx.x == 0 && dbias) dbias[0] = part[0];
}

// Dense-FFN activation of the fused wrapper: out = gate * silu(up).
template <typename T>
__global__ __launch_bounds__(256) void swiglu_mul_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                                         T* __restrict__ out, int64_t n, bool vec) {
    constexpr int V = Elem<T>::kVec;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec) {
        const int64_t nv = n / V;
        for (int64_t i = tid; i < nv; i += stride) {
            float g[V], u[V];
            Elem<T>::unpack(reinterpret_cast<const uint4*>(gate)[i], g);
            Elem<T>::unpack(reinterpret_cast<const uint4*>(up)[i], u);
#pragma unroll
            for (int j = 0; j < V; ++j) g[j] = g[j] * (u[j] / (1.0f + expf(-u[j])));
            reinterpret_cast<uint4*>(out)[i] = Elem<T>::pack(g);
        }
        for (int64_t i = nv * V + tid; i < n; i += stride) {
            const float u = Elem<T>::load(up + i);
            Elem<T>::store(out + i, Elem<T>::load(gate + i) * (u / (1.0f + expf(-u))));
        }
    } else {
        for (int64_t i = tid; i < n; i += stride) {
            const float u = Elem<T>::load(up + i);
            Elem<T>::store(out + i, Elem<T>::load(gate + i) * (u / (1.0f + expf(-u))));
        }
    }
}

}  // namespace ats

extern "C" int ats_row_dot(const void* x, const void* w, const float* bias, float* score, float* prob,
                           float temperature, int64_t T, int H, int dtype, ats_stream_t stream) {
    return ats_row_dot_copy(x, w, bias, score, prob, temperature, nullptr, T, H, dtype, stream);
}

extern "C" int ats_row_dot_copy(const void* x, const void* w, const float* bias, float* score, float* prob,
                                float temperature, void* copy_out, int64_t T, int H, int dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(T >= 0 && H > 0, ATS_ERR_INVALID_ARG, "ats_row_dot: T=%lld H=%d", (long long)T, H);
    ATS_REQUIRE(!copy_out || copy_out != x, ATS_ERR_INVALID_ARG, "ats_row_dot_copy: the copy must not alias x");
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_row_dot: dtype tag %d", dtype);
    ATS_REQUIRE(!prob || temperature > 0.f, ATS_ERR_INVALID_ARG, "ats_row_dot: temperature %g", temperature);
    if (T == 0) return ATS_OK;
    ATS_REQUIRE(x && w && (score || prob), ATS_ERR_INVALID_ARG, "ats_row_dot: null pointer");
    int64_t blocks = (T + 3) / 4;
    if (blocks > 16384) blocks = 16384;
    const int V = dtype == ATS_F32 ? 4 : 8;
    const bool vec = H % V == 0 && aligned16(x) && aligned16(w) && (!copy_out || aligned16(copy_out));
    if (dtype == ATS_F32)
        hipLaunchKernelGGL((row_dot_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const float*>(x), static_cast<const float*>(w), bias, score, prob, temperature,
                           static_cast<float*>(copy_out), T, H, vec);
    else
        hipLaunchKernelGGL((row_dot_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), bias, score, prob,
                           temperature, static_cast<bf16_t*>(copy_out), T, H, vec);
    ATS_CHECK_LAUNCH("ats_row_dot");
    return ATS_OK;
}

extern "C" int ats_select_topk_per_sequence(const float* score, int B, int L, int keep, int32_t* sel,
                                            ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(B >= 0 && L > 0 && L <= 8192 && keep >= 0 && keep <= L, ATS_ERR_INVALID_ARG,
                "ats_select_topk_per_sequence: B=%d L=%d keep=%d (L <= 8192, keep <= L)", B, L, keep);
    ATS_REQUIRE((int64_t)B * L < INT_MAX, ATS_ERR_UNSUPPORTED, "ats_select_topk_per_sequence: B*L must fit in int32");
    if (B == 0 || keep == 0) return ATS_OK;
    ATS_REQUIRE(score && sel, ATS_ERR_INVALID_ARG, "ats_select_topk_per_sequence: null pointer");
    hipStream_t st = as_stream(stream);
    if (L > 512) {      // long sequences: radix select (short ones are cheap to sort and keep the sort)
        if (L <= 2048) hipLaunchKernelGGL(select_topk_radix_kernel<2>, dim3(B), dim3(1024), 0, st, score, L, keep, sel);
        else if (L <= 4096) hipLaunchKernelGGL(select_topk_radix_kernel<4>, dim3(B), dim3(1024), 0, st, score, L, keep, sel);
        else hipLaunchKernelGGL(select_topk_radix_kernel<8>, dim3(B), dim3(1024), 0, st, score, L, keep, sel);
        ATS_CHECK_LAUNCH("ats_select_topk_per_sequence");
        return ATS_OK;
    }
    int lp2 = 2;
    while (lp2 < L) lp2 <<= 1;
    const int threads = lp2 / 2 < 64 ? 64 : (lp2 / 2 > 1024 ? 1024 : lp2 / 2);
    const size_t smem = (size_t)lp2 * 12;
    if (smem > 64 * 1024) {
        static LdsReservation reserved;
        hipError_t e = reserve_lds(reserved, {reinterpret_cast<const void*>(select_topk_seq_kernel)}, 8192 * 12);
        ATS_REQUIRE(e == hipSuccess, ATS_ERR_LAUNCH, "ats_select_topk_per_sequence: LDS attribute: %s",
                    hipGetErrorString(e));
    }
    hipLaunchKernelGGL(select_topk_seq_kernel, dim3(B), dim3(threads), smem, as_stream(stream), score, L, lp2, keep,
                       sel);
    ATS_CHECK_LAUNCH("ats_select_topk_per_sequence");
    return ATS_OK;
}

extern "C" int ats_scatter_add_rows(void* base, const int32_t* rows, const void* delta, int64_t n, int H, int dtype,
                                    ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(n >= 0 && H > 0, ATS_ERR_INVALID_ARG, "ats_scatter_add_rows: n=%lld H=%d", (long long)n, H);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_scatter_add_rows: dtype tag %d", dtype);
    if (n == 0) return ATS_OK;
    ATS_REQUIRE(base && rows && delta, ATS_ERR_INVALID_ARG, "ats_scatter_add_rows: null pointer");
    int64_t blocks = (n + 3) / 4;
    if (blocks > 16384) blocks = 16384;
    const int V = dtype == ATS_F32 ? 4 : 8;
    const bool vec = H % V == 0 && aligned16(base) && aligned16(delta);
    if (dtype == ATS_F32)
        hipLaunchKernelGGL((scatter_add_rows_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<float*>(base), rows, static_cast<const float*>(delta), n, H, vec);
    else
        hipLaunchKernelGGL((scatter_add_rows_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<bf16_t*>(base), rows, static_cast<const bf16_t*>(delta), n, H, vec);
    ATS_CHECK_LAUNCH("ats_scatter_add_rows");
    return ATS_OK;
}

// Values from which the select runs over many workgroups, and the workspace that takes:
// key (4 bytes), pad, count (8 bytes), then the four digit histograms.
static constexpr int64_t kKthMultiBlockMin = 16384;
static constexpr size_t kKthMultiBlockBytes = 16 + 4 * 256 * sizeof(unsigned int);

extern "C" size_t ats_kth_value_workspace(int64_t n) {
    return n >= kKthMultiBlockMin && n < (int64_t)INT_MAX ? kKthMultiBlockBytes : 16;
}

extern "C" int ats_kth_value_mask(const float* v, int64_t n, int64_t kth, float* mask, void* workspace,
                                  size_t workspace_bytes, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(n >= 0 && (n == 0 || (kth >= 1 && kth <= n)), ATS_ERR_INVALID_ARG,
                "ats_kth_value_mask: n=%lld kth=%lld", (long long)n, (long long)kth);
    if (n == 0) return ATS_OK;
    ATS_REQUIRE(n < (int64_t)INT_MAX, ATS_ERR_UNSUPPORTED, "ats_kth_value_mask: n=%lld (below 2^31)", (long long)n);
    ATS_REQUIRE(v && mask, ATS_ERR_INVALID_ARG, "ats_kth_value_mask: null pointer");
    ATS_REQUIRE(workspace && workspace_bytes >= sizeof(uint32_t), ATS_ERR_WORKSPACE,
                "ats_kth_value_mask: workspace of at least 4 bytes needed");
    hipStream_t s = as_stream(stream);
    uint32_t* key = static_cast<uint32_t*>(workspace);
    long long* count = workspace_bytes >= 16 ? reinterpret_cast<long long*>(static_cast<char*>(workspace) + 8) : nullptr;
    int64_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (n >= kKthMultiBlockMin && n < (int64_t)INT_MAX && workspace_bytes >= kKthMultiBlockBytes) {
        // one launch per digit over many workgroups; a smaller workspace keeps the single-workgroup select
        unsigned int* ghist = reinterpret_cast<unsigned int*>(static_cast<char*>(workspace) + 16);
        int64_t hb = (n + 2047) / 2048;          // eight values per thread
        if (hb > 1024) hb = 1024;
        hipLaunchKernelGGL(kth_zero_kernel, dim3(1), dim3(256), 0, s, ghist);
        for (int pass = 3; pass >= 0; --pass)
            hipLaunchKernelGGL(kth_digit_hist_kernel, dim3((unsigned)hb), dim3(256), 0, s, v, n, kth, pass, ghist);
        hipLaunchKernelGGL(kth_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, s, v, n, kth, ghist, key, count, mask);
        ATS_CHECK_LAUNCH("ats_kth_value_mask(multi)");
        return ATS_OK;
    }
    hipLaunchKernelGGL(kth_value_kernel, dim3(1), dim3(1024), 0, s, v, n, kth, key, count);
    ATS_CHECK_LAUNCH("ats_kth_value_mask(select)");
    hipLaunchKernelGGL(threshold_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, s, v, n, key, mask);
    ATS_CHECK_LAUNCH("ats_kth_value_mask(mask)");
    return ATS_OK;
}

extern "C" int ats_topk_mask_ste(const float* v, int64_t n, int64_t k, float* mask, float* ste, void* workspace,
                                 size_t workspace_bytes, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(n >= 0 && k >= 0, ATS_ERR_INVALID_ARG, "ats_topk_mask_ste: n=%lld k=%lld", (long long)n, (long long)k);
    if (n == 0) return ATS_OK;
    ATS_REQUIRE(n < (int64_t)INT_MAX, ATS_ERR_UNSUPPORTED, "ats_topk_mask_ste: n=%lld (below 2^31)", (long long)n);
    ATS_REQUIRE(v && mask, ATS_ERR_INVALID_ARG, "ats_topk_mask_ste: null pointer");
    hipStream_t s = as_stream(stream);
    int64_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (k == 0 || k >= n) {
        hipLaunchKernelGGL(fill_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, s, v, n, k == 0 ? 0.0f : 1.0f, mask, ste);
        ATS_CHECK_LAUNCH("ats_topk_mask_ste(fill)");
        return ATS_OK;
    }
    ATS_REQUIRE(workspace && workspace_bytes >= ats_kth_value_workspace(n), ATS_ERR_WORKSPACE,
                "ats_topk_mask_ste: workspace of ats_kth_value_workspace(n) = %zu bytes needed, got %zu",
                ats_kth_value_workspace(n), workspace_bytes);
    // the k-th largest is the (n - k + 1)-th smallest; the select leaves its key and the count of values >= it
    const int64_t kth = n - k + 1;
    uint32_t* key = static_cast<uint32_t*>(workspace);
    long long* count = reinterpret_cast<long long*>(static_cast<char*>(workspace) + 8);
    if (n >= kKthMultiBlockMin) {
        unsigned int* ghist = reinterpret_cast<unsigned int*>(static_cast<char*>(workspace) + 16);
        int64_t hb = (n + 2047) / 2048;
        if (hb > 1024) hb = 1024;
        hipLaunchKernelGGL(kth_zero_kernel, dim3(1), dim3(256), 0, s, ghist);
        for (int pass = 3; pass >= 0; --pass)
            hipLaunchKernelGGL(kth_digit_hist_kernel, dim3((unsigned)hb), dim3(256), 0, s, v, n, kth, pass, ghist);
        hipLaunchKernelGGL(kth_key_kernel, dim3(1), dim3(64), 0, s, n, kth, ghist, key, count);
    } else {
        hipLaunchKernelGGL(kth_value_kernel, dim3(1), dim3(1024), 0, s, v, n, kth, key, count);
    }
    ATS_CHECK_LAUNCH("ats_topk_mask_ste(select)");
    hipLaunchKernelGGL(topk_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, s, v, n, k, key, count, mask, ste);
    hipLaunchKernelGGL(topk_ties_kernel, dim3(1), dim3(1024), 0, s, v, n, k, key, count, mask, ste);
    ATS_CHECK_LAUNCH("ats_topk_mask_ste");
    return ATS_OK;
}

extern "C" int ats_mod_route_bwd(const float* grad_weights, const float* grad_probs, const float* prob,
                                 float temperature, float* grad_logits, float* grad_bias, int64_t n,
                                 ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(n >= 0 && temperature > 0.f, ATS_ERR_INVALID_ARG, "ats_mod_route_bwd: n=%lld temperature=%g",
                (long long)n, temperature);
    ATS_REQUIRE(n == 0 || (prob && grad_logits), ATS_ERR_INVALID_ARG, "ats_mod_route_bwd: null pointer");
    hipLaunchKernelGGL(mod_route_bwd_kernel, dim3(1), dim3(1024), 0, as_stream(stream), grad_weights, grad_probs, prob,
                       1.0f / temperature, grad_logits, grad_bias, n);
    ATS_CHECK_LAUNCH("ats_mod_route_bwd");
    return ATS_OK;
}

extern "C" int ats_swiglu_mul(const void* gate, const void* up, void* out, int64_t n, int dtype,
                              ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(n >= 0, ATS_ERR_INVALID_ARG, "ats_swiglu_mul: n=%lld", (long long)n);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "ats_swiglu_mul: dtype tag %d", dtype);
    if (n == 0) return ATS_OK;
    ATS_REQUIRE(gate && up && out, ATS_ERR_INVALID_ARG, "ats_swiglu_mul: null pointer");
    const bool vec = aligned16(gate) && aligned16(up) && aligned16(out);
    int64_t blocks = (n / (dtype == ATS_F32 ? 4 : 8) + 255) / 256 + 1;
    if (blocks > 16384) blocks = 16384;
    if (dtype == ATS_F32)
        hipLaunchKernelGGL((swiglu_mul_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const float*>(gate), static_cast<const float*>(up), static_cast<float*>(out),
                           n, vec);
    else
        hipLaunchKernelGGL((swiglu_mul_kernel<bf16_t>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const bf16_t*>(gate), static_cast<const bf16_t*>(up),
                           static_cast<bf16_t*>(out), n, vec);
    ATS_CHECK_LAUNCH("ats_swiglu_mul");
    return ATS_OK;
}

// Rotary position embedding (rotate-half, grouped-query aware) for gfx950.
// HBM-bound: q and k are read once and written once.  A group of lanes owns one
// (batch, position) and a chunk of heads; lanes of a wave cover consecutive
// positions of one head, i.e. one contiguous span of memory per head, with
// 16-byte accesses per lane.  The waves of a block share one slice of the
// float32 cos/sin table through LDS.
#include <math.h>

#include "ats_common.hpp"

// Products and sums below must round separately (the reference computes them as separate
// tensor ops); the HIP default would contract a*b+c into one fused multiply-add.
#pragma clang fp contract(off)

namespace ats {

// heads per wave: 8 when there are many positions (more loads in flight per wave), 4 for a handful of
// positions (decoding: more waves)
constexpr int kRopeHeadsLong = 8, kRopeHeadsShort = 4;
constexpr int kRopeLongMinPositions = 64;

struct RopeSeg {
    const void* in;
    void* out;
    int64_t sb, sh, sl;  // input element strides: batch, head, position
    int heads;
    int chunks;  // ceil(heads / heads per wave)
    int64_t ob, oh, ol;  // output element strides (the position stride of a contiguous [B, H, L, D] result is D)
    int rotate;          // 0: the rows are copied as they are (values appended to a cache beside the rotated keys)
};

static RopeSeg rope_seg(const void* in, void* out, int64_t sb, int64_t sh, int64_t sl, int heads, int L, int D) {
    const int hp = L >= kRopeLongMinPositions ? kRopeHeadsLong : kRopeHeadsShort;
    return RopeSeg{in, out, sb, sh, sl, heads, (heads + hp - 1) / hp, (int64_t)heads * L * D, (int64_t)L * D, (int64_t)D, 1};
}

// The rotation with the block as the unit: the waves of a block take the head chunks (HP heads each) of ONE
// (batch, position group), so the block needs one slice of the table (pos_per_wave positions x D/2 columns of
// cos and of sin).  It is fetched once per block, behind the rows, into LDS (at most one 16-byte load per
// thread instead of four per lane of every wave), and a barrier later every lane picks up its columns.  With
// a wave per (position group, chunk of 4 heads) that loaded its own table slice, q[4,16,2048,128] +
// k[4,4,2048,128] bf16 took 17.3 us; without any table loads 16.6; this kernel 16.6 with 4 and 16.4 with 8 heads
// per wave (more loads in flight per wave; with 2 heads 18.9).
template <typename T, int HP>
__global__ __launch_bounds__(512) void rope_vec_block_kernel(RopeSeg q, RopeSeg k, RopeSeg v3,
                                                             const float* __restrict__ cos_tab,
                                                             const float* __restrict__ sin_tab, int table_stride, int L,
                                                             int D, int pos_offset, int lanes_per_row, int pos_per_wave,
                                                             int n_pos_groups, int blocks_per_group, bool tab_vec,
                                                             float sin_sign) {
    constexpr int V = Elem<T>::kVec;
    extern __shared__ float tab_lds[];     // [2][pos_per_wave * half]
    const int lane = lane_id();
    const int wpb = blockDim.x >> 6;
    const int bg = (int)(blockIdx.x % blocks_per_group);
    const int64_t r0 = blockIdx.x / blocks_per_group;
    const int pg = (int)(r0 % n_pos_groups);
    const int b = (int)(r0 / n_pos_groups);
    const int total_chunks = q.chunks + k.chunks + v3.chunks;
    int chunk = bg * wpb + (int)(threadIdx.x >> 6);
    const bool wave_on = chunk < total_chunks;
    if (!wave_on) chunk = 0;
    const RopeSeg& seg = chunk < q.chunks ? q : chunk < q.chunks + k.chunks ? k : v3;
    if (chunk >= q.chunks + k.chunks) chunk -= q.chunks + k.chunks;
    else if (chunk >= q.chunks) chunk -= q.chunks;

    const int half = D >> 1;
    const int prow = lane / lanes_per_row;
    const int c = lane - prow * lanes_per_row;
    const int pos0 = pg * pos_per_wave;
    const int pos = pos0 + prow;
    const bool on = wave_on && prow < pos_per_wave && pos < L;

    const int h0 = chunk * HP;
    const T* in = static_cast<const T*>(seg.in);
    T* out = static_cast<T*>(seg.out);
    uint4 lo[HP], hi[HP];
    if (on) {
#pragma unroll
        for (int i = 0; i < HP; ++i) {
            const int h = h0 + i;
            if (h < seg.heads) {
                const T* p = in + b * seg.sb + h * seg.sh + pos * seg.sl + c * V;
                lo[i] = stream_load(reinterpret_cast<const uint4*>(p));
                hi[i] = stream_load(reinterpret_cast<const uint4*>(p + half));
            }
        }
    }
    // the block's table slice
    const int slice = pos_per_wave * half;              // floats per table
    if (tab_vec) {
        const int per_row = half >> 2;                  // float4 per position
        for (int f = threadIdx.x; f < 2 * (slice >> 2); f += blockDim.x) {
            const int which = f >= (slice >> 2);
            const int g = which ? f - (slice >> 2) : f;
            const int row = g / per_row, col4 = g - row * per_row;
            if (pos0 + row < L) {
                const float* src = (which ? sin_tab : cos_tab) + (int64_t)(pos_offset + pos0 + row) * table_stride + col4 * 4;
                *reinterpret_cast<float4*>(tab_lds + which * slice + row * half + col4 * 4) =
                    *reinterpret_cast<const float4*>(src);
            }
        }
    } else {
        for (int f = threadIdx.x; f < 2 * slice; f += blockDim.x) {
            const int which = f >= slice;
            const int g = which ? f - slice : f;
            const int row = g / half, col = g - row * half;
            if (pos0 + row < L)
                tab_lds[which * slice + row * half + col] =
                    (which ? sin_tab : cos_tab)[(int64_t)(pos_offset + pos0 + row) * table_stride + col];
        }
    }
    __syncthreads();
    if (!on) return;
    float cs[V], sn[V];
#pragma unroll
    for (int j = 0; j < V; j += 4) {
        const float4 cv = *reinterpret_cast<const float4*>(tab_lds + prow * half + c * V + j);
        const float4 sv = *reinterpret_cast<const float4*>(tab_lds + slice + prow * half + c * V + j);
        cs[j] = cv.x; cs[j + 1] = cv.y; cs[j + 2] = cv.z; cs[j + 3] = cv.w;
        sn[j] = sv.x * sin_sign; sn[j + 1] = sv.y * sin_sign; sn[j + 2] = sv.z * sin_sign; sn[j + 3] = sv.w * sin_sign;
    }
#pragma unroll
    for (int i = 0; i < HP; ++i) {
        const int h = h0 + i;
        if (h < seg.heads) {
            float a[V], bb[V], o1[V], o2[V];
            Elem<T>::unpack(lo[i], a);
            Elem<T>::unpack(hi[i], bb);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                o1[j] = ((((a[j]) * (cs[j]))) - (((bb[j]) * (sn[j]))));
                o2[j] = ((((a[j]) * (sn[j]))) + (((bb[j]) * (cs[j]))));
            }
            T* p = out + b * seg.ob + h * seg.oh + pos * seg.ol + c * V;
            stream_store(reinterpret_cast<uint4*>(p), seg.rotate ? Elem<T>::pack(o1) : lo[i]);
            stream_store(reinterpret_cast<uint4*>(p + half), seg.rotate ? Elem<T>::pack(o2) : hi[i]);
        }
    }
}

// Any even D / alignment: one thread per rotated pair.
template <typename T>
__global__ __launch_bounds__(256) void rope_scalar_kernel(RopeSeg q, RopeSeg k, RopeSeg v3, const float* __restrict__ cos_tab,
                                                          const float* __restrict__ sin_tab, int table_stride,
                                                          int B, int L, int D, int pos_offset, float sin_sign) {
    const int half = D >> 1;
    const int heads_all = q.heads + k.heads + v3.heads;
    const int64_t per_b = (int64_t)heads_all * L * half;
    const int64_t total = per_b * B;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int d = (int)(i % half);
        int64_t r = i / half;
        const int pos = (int)(r % L);
        r /= L;
        const int hh = (int)(r % heads_all);
        const int b = (int)(r / heads_all);
        const RopeSeg& seg = hh < q.heads ? q : hh < q.heads + k.heads ? k : v3;
        const int h = hh < q.heads ? hh : hh < q.heads + k.heads ? hh - q.heads : hh - q.heads - k.heads;
        const T* p = static_cast<const T*>(seg.in) + b * seg.sb + h * seg.sh + pos * seg.sl + d;
        const float a = Elem<T>::load(p), bb = Elem<T>::load(p + half);
        const float cs = cos_tab[(int64_t)(pos_offset + pos) * table_stride + d];
        const float sn = sin_tab[(int64_t)(pos_offset + pos) * table_stride + d] * sin_sign;
        T* o = static_cast<T*>(seg.out) + b * seg.ob + h * seg.oh + pos * seg.ol + d;
        if (seg.rotate) {
            Elem<T>::store(o, ((((a) * (cs))) - (((bb) * (sn)))));
            Elem<T>::store(o + half, ((((a) * (sn))) + (((bb) * (cs)))));
        } else {
            o[0] = p[0];
            o[half] = p[half];
        }
    }
}

// cos/sin table in float64, stored as float32.
__global__ __launch_bounds__(256) void rope_table_kernel(float* __restrict__ cos_out, float* __restrict__ sin_out,
                                                         int seq_len, int dim, int cols, double theta,
                                                         double scaling) {
    const int half = dim >> 1;
    const int64_t total = (int64_t)seq_len * half;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int d = (int)(i % half);
        const int pos = (int)(i / half);
        const double inv_freq = 1.0 / pow(theta, (double)(2 * d) / (double)dim);
        float t = (float)pos;
        if (scaling != 1.0) t = t / (float)scaling;
        const double ang = (double)t * inv_freq;
        const float cv = (float)cos(ang), sv = (float)sin(ang);
        cos_out[(int64_t)pos * cols + d] = cv;
        sin_out[(int64_t)pos * cols + d] = sv;
        if (cols == dim) {
            cos_out[(int64_t)pos * cols + d + half] = cv;
            sin_out[(int64_t)pos * cols + d + half] = sv;
        }
    }
}

template <typename T>
static void launch_rope(RopeSeg q, RopeSeg k, RopeSeg v3, const float* cos_tab, const float* sin_tab, int table_stride, int B,
                        int L, int D, int pos_offset, bool vec_ok, float sin_sign, hipStream_t s) {
    constexpr int V = Elem<T>::kVec;
    if (vec_ok) {
        const int lanes_per_row = (D / 2) / V;
        const int pos_per_wave = kWave / lanes_per_row;
        const int n_pos_groups = (L + pos_per_wave - 1) / pos_per_wave;
        const bool tab_vec = table_stride % 4 == 0 && aligned16(cos_tab) && aligned16(sin_tab);
        const int total_chunks = q.chunks + k.chunks + v3.chunks;
        const int bpg = (total_chunks + 7) / 8;                       // blocks per (batch, position group)
        const int wpb = (total_chunks + bpg - 1) / bpg;               // waves per block: at most 8, evenly filled
        const int64_t nb = (int64_t)bpg * n_pos_groups * B;
        const size_t lds = (size_t)2 * pos_per_wave * (D / 2) * sizeof(float);
        if (L >= kRopeLongMinPositions)
            hipLaunchKernelGGL((rope_vec_block_kernel<T, kRopeHeadsLong>), dim3((unsigned)nb), dim3(wpb * 64), lds, s, q, k,
                               v3, cos_tab, sin_tab, table_stride, L, D, pos_offset, lanes_per_row, pos_per_wave,
                               n_pos_groups, bpg, tab_vec, sin_sign);
        else
            hipLaunchKernelGGL((rope_vec_block_kernel<T, kRopeHeadsShort>), dim3((unsigned)nb), dim3(wpb * 64), lds, s, q, k,
                               v3, cos_tab, sin_tab, table_stride, L, D, pos_offset, lanes_per_row, pos_per_wave,
                               n_pos_groups, bpg, tab_vec, sin_sign);
    } else {
        const int64_t total = (int64_t)B * (q.heads + k.heads + v3.heads) * L * (D / 2);
        int64_t blocks = (total + 255) / 256;
        if (blocks > 65536) blocks = 65536;
        hipLaunchKernelGGL((rope_scalar_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s, q, k, v3, cos_tab, sin_tab,
                           table_stride, B, L, D, pos_offset, sin_sign);
    }
}

}  // namespace ats

extern "C" int ats_rope_table(float* cos_out, float* sin_out, int seq_len, int dim, int cols, double theta,
                              double scaling_factor, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(cos_out && sin_out, ATS_ERR_INVALID_ARG, "ats_rope_table: null pointer");
    ATS_REQUIRE(seq_len >= 0 && dim > 0 && dim % 2 == 0 && (cols == dim || cols == dim / 2) && theta > 0 &&
                    scaling_factor > 0,
                ATS_ERR_INVALID_ARG, "ats_rope_table: seq_len=%d dim=%d cols=%d theta=%g scaling=%g", seq_len, dim,
                cols, theta, scaling_factor);
    if (seq_len == 0) return ATS_OK;
    const int64_t total = (int64_t)seq_len * (dim / 2);
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), cos_out, sin_out,
                       seq_len, dim, cols, theta, scaling_factor);
    ATS_CHECK_LAUNCH("ats_rope_table");
    return ATS_OK;
}

// Where the rotated keys and the untouched values go when they are appended to a key / value cache
// [B, Hkv, capacity, D] (element strides cb, ch, cl) behind its first `pos` positions.
struct RopeCacheTarget {
    void* k_cache;
    void* v_cache;
    const void* v_in;
    int64_t v_sb, v_sh, v_sl;
    int64_t cb, ch, cl;
    int64_t pos;
};

static int rope_apply(const char* name, float sin_sign, const void* q_in, const void* k_in, void* q_out, void* k_out,
                      const float* cos_tab, const float* sin_tab, int table_stride, int table_len, int B, int Hq,
                      int Hkv, int L, int D, int pos_offset, int64_t q_sb, int64_t q_sh, int64_t q_sl, int64_t k_sb,
                      int64_t k_sh, int64_t k_sl, int dtype, ats_stream_t stream,
                      const RopeCacheTarget* cache = nullptr) {
    using namespace ats;
    ATS_REQUIRE(B >= 0 && Hq >= 0 && Hkv >= 0 && L >= 0 && D > 0 && D % 2 == 0, ATS_ERR_INVALID_ARG,
                "%s: B=%d Hq=%d Hkv=%d L=%d D=%d", name, B, Hq, Hkv, L, D);
    ATS_REQUIRE(dtype == ATS_F32 || dtype == ATS_BF16, ATS_ERR_UNSUPPORTED, "%s: dtype tag %d", name, dtype);
    if (B == 0 || L == 0 || Hq + Hkv == 0) return ATS_OK;
    ATS_REQUIRE(cos_tab && sin_tab && table_stride >= D / 2, ATS_ERR_INVALID_ARG,
                "%s: table pointers/stride (stride=%d, need >= %d)", name, table_stride, D / 2);
    ATS_REQUIRE(pos_offset >= 0 && (int64_t)pos_offset + L <= table_len, ATS_ERR_INVALID_ARG,
                "%s: positions %d..%d exceed table length %d", name, pos_offset, pos_offset + L - 1, table_len);
    ATS_REQUIRE((Hq == 0 || (q_in && q_out)) && (Hkv == 0 || (k_in && (cache ? cache->k_cache : k_out))),
                ATS_ERR_INVALID_ARG, "%s: null tensor pointer", name);
    RopeSeg q = rope_seg(q_in, q_out, q_sb, q_sh, q_sl, Hq, L, D);
    RopeSeg k = rope_seg(k_in, k_out, k_sb, k_sh, k_sl, Hkv, L, D);
    RopeSeg v3 = rope_seg(nullptr, nullptr, 0, 0, 0, 0, L, D);
    if (cache) {
        // keys and values go behind the cache's first cache->pos positions instead of into a tensor of their own
        k.out = static_cast<char*>(cache->k_cache) + cache->pos * cache->cl * (dtype == ATS_F32 ? 4 : 2);
        k.ob = cache->cb, k.oh = cache->ch, k.ol = cache->cl;
        v3 = rope_seg(cache->v_in, static_cast<char*>(cache->v_cache) + cache->pos * cache->cl * (dtype == ATS_F32 ? 4 : 2),
                      cache->v_sb, cache->v_sh, cache->v_sl, Hkv, L, D);
        v3.ob = cache->cb, v3.oh = cache->ch, v3.ol = cache->cl;
        v3.rotate = 0;
    }
    const int V = dtype == ATS_F32 ? 4 : 8;
    auto seg_ok = [&](const RopeSeg& sgm) {
        return sgm.heads == 0 || (aligned16(sgm.in) && aligned16(sgm.out) && sgm.sb % V == 0 && sgm.sh % V == 0 &&
                                  sgm.sl % V == 0 && sgm.ob % V == 0 && sgm.oh % V == 0 && sgm.ol % V == 0);
    };
    const int half = D / 2;
    const bool vec_ok = half % V == 0 && half / V <= kWave && seg_ok(q) && seg_ok(k) && seg_ok(v3);
    if (dtype == ATS_F32)
        launch_rope<float>(q, k, v3, cos_tab, sin_tab, table_stride, B, L, D, pos_offset, vec_ok, sin_sign, as_stream(stream));
    else
        launch_rope<bf16_t>(q, k, v3, cos_tab, sin_tab, table_stride, B, L, D, pos_offset, vec_ok, sin_sign, as_stream(stream));
    ATS_CHECK_LAUNCH(name);
    return ATS_OK;
}

extern "C" int ats_rope_fwd(const void* q_in, const void* k_in, void* q_out, void* k_out, const float* cos_tab,
                            const float* sin_tab, int table_stride, int table_len, int B, int Hq, int Hkv, int L,
                            int D, int pos_offset, int64_t q_sb, int64_t q_sh, int64_t q_sl, int64_t k_sb,
                            int64_t k_sh, int64_t k_sl, int dtype, ats_stream_t stream) {
    return rope_apply("ats_rope_fwd", 1.0f, q_in, k_in, q_out, k_out, cos_tab, sin_tab, table_stride, table_len, B, Hq,
                      Hkv, L, D, pos_offset, q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, dtype, stream);
}

extern "C" int ats_rope_bwd(const void* dq_out, const void* dk_out, void* dq, void* dk, const float* cos_tab,
                            const float* sin_tab, int table_stride, int table_len, int B, int Hq, int Hkv, int L,
                            int D, int pos_offset, int64_t q_sb, int64_t q_sh, int64_t q_sl, int64_t k_sb,
                            int64_t k_sh, int64_t k_sl, int dtype, ats_stream_t stream) {
    return rope_apply("ats_rope_bwd", -1.0f, dq_out, dk_out, dq, dk, cos_tab, sin_tab, table_stride, table_len, B, Hq,
                      Hkv, L, D, pos_offset, q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, dtype, stream);
}

extern "C" int ats_rope_fwd_append(const void* q_in, const void* k_in, const void* v_in, void* q_out, void* k_cache,
                                   void* v_cache, const float* cos_tab, const float* sin_tab, int table_stride,
                                   int table_len, int B, int Hq, int Hkv, int L, int D, int pos_offset, int64_t q_sb,
                                   int64_t q_sh, int64_t q_sl, int64_t k_sb, int64_t k_sh, int64_t k_sl, int64_t v_sb,
                                   int64_t v_sh, int64_t v_sl, int64_t cache_sb, int64_t cache_sh, int64_t cache_sl,
                                   int64_t cache_pos, int64_t cache_capacity, int dtype, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(Hkv > 0 && k_in && v_in && k_cache && v_cache, ATS_ERR_INVALID_ARG,
                "ats_rope_fwd_append: keys, values and both caches are required");
    ATS_REQUIRE(cache_pos >= 0 && L >= 0 && cache_pos + L <= cache_capacity && cache_sl >= D, ATS_ERR_INVALID_ARG,
                "ats_rope_fwd_append: positions %lld..%lld do not fit a cache of %lld (position stride %lld, D=%d)",
                (long long)cache_pos, (long long)(cache_pos + L - 1), (long long)cache_capacity, (long long)cache_sl, D);
    RopeCacheTarget tgt{k_cache, v_cache, v_in, v_sb, v_sh, v_sl, cache_sb, cache_sh, cache_sl, cache_pos};
    return rope_apply("ats_rope_fwd_append", 1.0f, q_in, k_in, q_out, nullptr, cos_tab, sin_tab, table_stride,
                      table_len, B, Hq, Hkv, L, D, pos_offset, q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, dtype, stream, &tgt);
}

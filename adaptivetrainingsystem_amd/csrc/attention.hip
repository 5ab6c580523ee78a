// Causal grouped-query attention forward for gfx950 (bf16, head_dim 64 or 128).
//
// Replaces GroupedQueryAttention._standard_attention / _flash_attention of the reference
// (Src/Main_Scripts/core/model.py:757-839): scores = q.k^T * scale, causal mask, float32 softmax,
// probabilities rounded to bf16, times v; output laid out [B, L, Hq*D].  The [L, L] score matrix is
// never materialised: a block owns 128 query rows of one head (4 waves x 32 rows) and walks the keys in
// tiles of 64 with an online softmax (running maximum and sum per query row).
//
// MFMA layout trick: both products are computed transposed,
//     S^T = K . Q^T      (A operand = K rows from LDS, B operand = Q rows held in registers)
//     O^T = V^T . P^T    (A operand = rows of V^T from LDS, B operand = P^T)
// so a lane of the 32x32 accumulator always owns ONE query row (column lane % 32): the softmax row
// reductions are in-lane loops plus a single cross-lane exchange (lane ^ 32), and the accumulator of
// S^T is already in B-operand order for the second product -- the keys a lane holds for k-step s are
// {4g..4g+3, 8+4g..8+4g+3} + 16s (g = lane / 32); the V^T fragment is read with the same key order,
// which is legal because the contraction over keys is a sum.  V^T ([B, Hkv, D, Lp], keys contiguous) is
// produced once per call by a small transpose kernel, so every operand is read along its contiguous
// dimension.
#include <math.h>

#include "ats_common.hpp"

namespace ats {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 abf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float af32x16_t;
typedef unsigned int au32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int au32x2_t __attribute__((ext_vector_type(2)));

constexpr int kAttBM = 128;   // query rows per block
constexpr int kAttBN = 64;    // keys per tile

__device__ __forceinline__ af32x16_t att_mma(const au32x4_t& a, const au32x4_t& b, af32x16_t c) {
    union {
        au32x4_t u;
        abf16x8_t v;
    } x, y;
    x.u = a;
    y.u = b;
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(x.v, y.v, c, 0, 0, 0);
}

// v: [B, L, *] rows with element strides (batch, position, head; D contiguous) -> vt [B, Hkv, D, Lp],
// zero padded for positions >= L.  One block per (64 positions, head, batch).
template <int D>
__global__ __launch_bounds__(256) void attention_vt_kernel(const bf16_t* __restrict__ v, int64_t sb, int64_t sl,
                                                           int64_t sh, bf16_t* __restrict__ vt, int Hkv, int L,
                                                           int Lp) {
    __shared__ bf16_t tile[D][64 + 8];
    const int l0 = blockIdx.x * 64, h = blockIdx.y, b = blockIdx.z;
    const bf16_t* src = v + b * sb + h * sh;
    for (int i = threadIdx.x; i < 64 * (D / 8); i += 256) {
        const int r = i / (D / 8), c0 = (i % (D / 8)) * 8;
        uint4 raw = make_uint4(0u, 0u, 0u, 0u);
        if (l0 + r < L) raw = *reinterpret_cast<const uint4*>(src + (int64_t)(l0 + r) * sl + c0);
        const bf16_t* e = reinterpret_cast<const bf16_t*>(&raw);
#pragma unroll
        for (int j = 0; j < 8; ++j) tile[c0 + j][r] = e[j];
    }
    __syncthreads();
    bf16_t* dst = vt + ((int64_t)(b * Hkv + h) * D) * Lp + l0;
    for (int i = threadIdx.x; i < D * 8; i += 256) {
        const int d = i / 8, r0 = (i % 8) * 8;
        *reinterpret_cast<uint4*>(dst + (int64_t)d * Lp + r0) = *reinterpret_cast<const uint4*>(&tile[d][r0]);
    }
}

template <int D>
__global__ __launch_bounds__(256) void attention_fwd_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                                                            const bf16_t* __restrict__ vt, bf16_t* __restrict__ out,
                                                            float* __restrict__ lse, int Hq, int Hkv, int L, int Lp,
                                                            float scale_log2) {
    constexpr int KS = D / 16;              // k-steps of the score product
    constexpr int DB = D / 32;              // 32-row blocks of the output (transposed)
    constexpr int KPITCH = D * 2 + 16;      // bytes per K row in LDS
    constexpr int VPITCH = kAttBN * 2 + 8;  // bytes per V^T row in LDS
    constexpr int KTILE = kAttBN * KPITCH;
    constexpr int VTILE = D * VPITCH;
    constexpr int KVEC = kAttBN * (D / 8) / 256;   // 16-byte vectors per thread for a K tile
    constexpr int VVEC = D * (kAttBN / 8) / 256;   // and for a V^T tile
    extern __shared__ __align__(16) unsigned char smem[];   // [2 stages][K tile | V^T tile]
#define ATT_SK(stage_) (smem + (stage_) * (KTILE + VTILE))
#define ATT_SV(stage_) (smem + (stage_) * (KTILE + VTILE) + KTILE)

    const int n_qt = (L + kAttBM - 1) / kAttBM;
    const int qt = n_qt - 1 - blockIdx.x;    // longest rows first
    const int hq = blockIdx.y, b = blockIdx.z;
    const int hkv = hq / (Hq / Hkv);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, g = lane >> 5;
    const int q_row = qt * kAttBM + wave * 32 + col;          // this lane's query
    const int q_clamped = q_row < L ? q_row : L - 1;

    const bf16_t* qp = q + ((int64_t)(b * Hq + hq) * L + q_clamped) * D;
    const bf16_t* kbase = k + (int64_t)(b * Hkv + hkv) * L * D;
    const bf16_t* vbase = vt + (int64_t)(b * Hkv + hkv) * D * Lp;

    au32x4_t qf[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const au32x4_t*>(qp + s * 16 + g * 8);

    af32x16_t acc_o[DB];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc_o[d][v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    const int q_block_last = min(qt * kAttBM + kAttBM - 1, L - 1);
    const int n_tiles = q_block_last / kAttBN + 1;
    const int q_wave_first = qt * kAttBM + wave * 32;
    const int q_wave_last = q_wave_first + 31;

    au32x4_t rk[KVEC], rv[VVEC];
    auto load_tile = [&](int t) {
        const int n0 = t * kAttBN;
#pragma unroll
        for (int i = 0; i < KVEC; ++i) {
            const int idx = tid + i * 256;
            const int r = idx / (D / 8), c = idx % (D / 8);
            int key = n0 + r;
            key = key < L ? key : L - 1;
            rk[i] = *reinterpret_cast<const au32x4_t*>(kbase + (int64_t)key * D + c * 8);
        }
#pragma unroll
        for (int i = 0; i < VVEC; ++i) {
            const int idx = tid + i * 256;
            const int d = idx / (kAttBN / 8), c = idx % (kAttBN / 8);
            rv[i] = *reinterpret_cast<const au32x4_t*>(vbase + (int64_t)d * Lp + n0 + c * 8);
        }
    };
    auto store_tile = [&](int stage) {
#pragma unroll
        for (int i = 0; i < KVEC; ++i) {
            const int idx = tid + i * 256;
            const int r = idx / (D / 8), c = idx % (D / 8);
            *reinterpret_cast<au32x4_t*>(ATT_SK(stage) + r * KPITCH + c * 16) = rk[i];
        }
#pragma unroll
        for (int i = 0; i < VVEC; ++i) {
            const int idx = tid + i * 256;
            const int d = idx / (kAttBN / 8), c = idx % (kAttBN / 8);
            // 8-byte halves: the row pitch keeps 8-byte alignment only
            au32x2_t lo = {rv[i].x, rv[i].y}, hi = {rv[i].z, rv[i].w};
            *reinterpret_cast<au32x2_t*>(ATT_SV(stage) + d * VPITCH + c * 16) = lo;
            *reinterpret_cast<au32x2_t*>(ATT_SV(stage) + d * VPITCH + c * 16 + 8) = hi;
        }
    };

    load_tile(0);
    store_tile(0);
    __syncthreads();
    for (int t = 0; t < n_tiles; ++t) {
        const int st = t & 1;
        const int n0 = t * kAttBN;
        if (t + 1 < n_tiles) load_tile(t + 1);
        if (n0 <= q_wave_last) {   // otherwise every key of the tile is in this wave's future
            // ---- S^T = K . Q^T for 2 blocks of 32 keys
            af32x16_t acc_s[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                for (int v = 0; v < 16; ++v) acc_s[kb][v] = 0.f;
#pragma unroll
                for (int s = 0; s < KS; ++s) {
                    const au32x4_t kf = *reinterpret_cast<const au32x4_t*>(ATT_SK(st) + (kb * 32 + col) * KPITCH + s * 32 + g * 16);
                    acc_s[kb] = att_mma(kf, qf[s], acc_s[kb]);
                }
            }
            // ---- scale, causal mask, online softmax (log2 domain)
            const bool need_mask = n0 + kAttBN - 1 > q_wave_first;
            float mx = m_run;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    float s2 = acc_s[kb][v] * scale_log2;
                    if (need_mask) {
                        const int key = n0 + kb * 32 + (v >> 2) * 8 + g * 4 + (v & 3);
                        if (key > q_row) s2 = -INFINITY;
                    }
                    acc_s[kb][v] = s2;
                    mx = fmaxf(mx, s2);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float alpha = __builtin_amdgcn_exp2f(m_run - mx);   // 0 on the first tile (m_run = -inf)
            float psum = 0.f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float p = __builtin_amdgcn_exp2f(acc_s[kb][v] - mx);
                    acc_s[kb][v] = p;
                    psum += p;
                }
            l_run = l_run * alpha + psum;
            m_run = mx;
#pragma unroll
            for (int d = 0; d < DB; ++d)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc_o[d][v] *= alpha;
            // ---- P^T as B operand: k-step s holds accumulator values 8*(s&1) .. +7 of key block s>>1
            au32x4_t pf[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int kb = s >> 1, v0 = (s & 1) * 8;
                pf[s].x = pack_bf16x2(acc_s[kb][v0 + 0], acc_s[kb][v0 + 1]);
                pf[s].y = pack_bf16x2(acc_s[kb][v0 + 2], acc_s[kb][v0 + 3]);
                pf[s].z = pack_bf16x2(acc_s[kb][v0 + 4], acc_s[kb][v0 + 5]);
                pf[s].w = pack_bf16x2(acc_s[kb][v0 + 6], acc_s[kb][v0 + 7]);
            }
            // ---- O^T += V^T . P^T
#pragma unroll
            for (int d = 0; d < DB; ++d) {
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const unsigned char* vr = ATT_SV(st) + (d * 32 + col) * VPITCH + (s * 16 + g * 4) * 2;
                    const au32x2_t lo = *reinterpret_cast<const au32x2_t*>(vr);
                    const au32x2_t hi = *reinterpret_cast<const au32x2_t*>(vr + 16);
                    const au32x4_t vf = {lo.x, lo.y, hi.x, hi.y};
                    acc_o[d] = att_mma(vf, pf[s], acc_o[d]);
                }
            }
        }
        if (t + 1 < n_tiles) {
            store_tile(st ^ 1);      // the other stage was last read in iteration t-1, before its barrier
        }
        __syncthreads();
    }

    // ---- normalise and write [B, L, Hq*D]
    l_run += __shfl_xor(l_run, 32, 64);
    const float inv = 1.0f / l_run;
    if (q_row < L) {
        bf16_t* orow = out + ((int64_t)b * L + q_row) * (int64_t)(Hq * D) + hq * D;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                au32x2_t w;
                w.x = pack_bf16x2(acc_o[d][r * 4 + 0] * inv, acc_o[d][r * 4 + 1] * inv);
                w.y = pack_bf16x2(acc_o[d][r * 4 + 2] * inv, acc_o[d][r * 4 + 3] * inv);
                *reinterpret_cast<au32x2_t*>(orow + d * 32 + r * 8 + g * 4) = w;
            }
        if (lse && g == 0) lse[(int64_t)(b * Hq + hq) * L + q_row] = (m_run + log2f(l_run)) * 0.6931471805599453f;
    }
#undef ATT_SK
#undef ATT_SV
}

}  // namespace ats

extern "C" int64_t ats_attention_padded_len(int L) { return ((int64_t)L + ats::kAttBN - 1) / ats::kAttBN * ats::kAttBN; }

extern "C" int ats_attention_transpose_v(const void* v, int64_t sb, int64_t sl, int64_t sh, void* vt, int B, int Hkv,
                                         int L, int D, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(B >= 0 && Hkv > 0 && L >= 0 && (D == 64 || D == 128), ATS_ERR_UNSUPPORTED,
                "ats_attention_transpose_v: B=%d Hkv=%d L=%d D=%d (head_dim 64 or 128)", B, Hkv, L, D);
    if (B == 0 || L == 0) return ATS_OK;
    ATS_REQUIRE(v && vt && aligned16(v) && aligned16(vt) && sb % 8 == 0 && sl % 8 == 0 && sh % 8 == 0,
                ATS_ERR_INVALID_ARG, "ats_attention_transpose_v: pointers and strides must be 16-byte aligned");
    const int Lp = (int)ats_attention_padded_len(L);
    const dim3 grid((unsigned)(Lp / 64), (unsigned)Hkv, (unsigned)B);
    if (D == 128)
        hipLaunchKernelGGL((attention_vt_kernel<128>), grid, dim3(256), 0, as_stream(stream),
                           static_cast<const bf16_t*>(v), sb, sl, sh, static_cast<bf16_t*>(vt), Hkv, L, Lp);
    else
        hipLaunchKernelGGL((attention_vt_kernel<64>), grid, dim3(256), 0, as_stream(stream),
                           static_cast<const bf16_t*>(v), sb, sl, sh, static_cast<bf16_t*>(vt), Hkv, L, Lp);
    ATS_CHECK_LAUNCH("ats_attention_transpose_v");
    return ATS_OK;
}

extern "C" int ats_attention_fwd(const void* q, const void* k, const void* vt, void* out, float* lse, int B, int Hq,
                                 int Hkv, int L, int D, float scale, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(B >= 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0 && L >= 0 && scale > 0.f, ATS_ERR_INVALID_ARG,
                "ats_attention_fwd: B=%d Hq=%d Hkv=%d L=%d scale=%g", B, Hq, Hkv, L, scale);
    ATS_REQUIRE(D == 64 || D == 128, ATS_ERR_UNSUPPORTED, "ats_attention_fwd: head_dim %d (64 or 128)", D);
    if (B == 0 || L == 0) return ATS_OK;
    ATS_REQUIRE(q && k && vt && out && aligned16(q) && aligned16(k) && aligned16(vt) && aligned16(out),
                ATS_ERR_INVALID_ARG, "ats_attention_fwd: null or misaligned pointer");
    ATS_REQUIRE(Hq <= 65535 && B <= 65535, ATS_ERR_UNSUPPORTED, "ats_attention_fwd: grid");
    const int Lp = (int)ats_attention_padded_len(L);
    const dim3 grid((unsigned)((L + kAttBM - 1) / kAttBM), (unsigned)Hq, (unsigned)B);
    const float scale_log2 = scale * 1.4426950408889634f;
    if (D == 128) {
        constexpr int smem = 2 * (kAttBN * (128 * 2 + 16) + 128 * (kAttBN * 2 + 8));
        static bool attr = false;
        if (!attr) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_fwd_kernel<128>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, smem);
            ATS_REQUIRE(e == hipSuccess, ATS_ERR_LAUNCH, "ats_attention_fwd: cannot reserve %d bytes of LDS", smem);
            attr = true;
        }
        hipLaunchKernelGGL((attention_fwd_kernel<128>), grid, dim3(256), smem, as_stream(stream),
                           static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k), static_cast<const bf16_t*>(vt),
                           static_cast<bf16_t*>(out), lse, Hq, Hkv, L, Lp, scale_log2);
    } else {
        constexpr int smem = 2 * (kAttBN * (64 * 2 + 16) + 64 * (kAttBN * 2 + 8));
        hipLaunchKernelGGL((attention_fwd_kernel<64>), grid, dim3(256), smem, as_stream(stream),
                           static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k), static_cast<const bf16_t*>(vt),
                           static_cast<bf16_t*>(out), lse, Hq, Hkv, L, Lp, scale_log2);
    }
    ATS_CHECK_LAUNCH("ats_attention_fwd");
    return ATS_OK;
}

// Backward of the causal grouped-query attention for gfx950 (bf16, head_dim 64 or 128).
//
// Gradient of GroupedQueryAttention._standard_attention / _flash_attention of the reference
// (Src/Main_Scripts/core/model.py:757-839), which the reference leaves to autograd.  With
// P = softmax(q.k^T * scale + causal mask) (float32) and delta_i = sum_d dO[i,d] * O[i,d]:
//     dV = P^T . dO        dP = dO . V^T        dS = P * (dP - delta) * scale
//     dQ = dS . K          dK = dS^T . Q
// P is recomputed from the saved log-sum-exp, the [L, Lk] matrices are never materialised, and nothing is
// accumulated with atomics: one kernel owns query rows and walks the keys (dQ), the other owns keys and
// walks the queries of every query head of its kv head (dK, dV), so every output element is summed by
// one lane in a fixed order.
//
// Same MFMA layout trick as the forward: products are formed transposed so that a lane of the 32x32
// accumulator owns one row of the side the block owns (a query in the dQ kernel, a key in the dK/dV
// kernel).  The operand that changes from step to step is the A operand and comes from LDS, where a
// tile is kept as it is in memory (rows of D elements): fragments along D are plain 16-byte reads,
// fragments across rows (K^T for dQ, Q^T and dO^T for dK/dV) come out through the transposing read
// ds_read_b64_tr_b16, so no transposed copy of any operand is made.  A tile is stored once, unpadded, with
// its 16-byte chunks swizzled so that both access patterns stay free of bank conflicts (SwzTile below).
#include <math.h>

#include <type_traits>

#include "ats_common.hpp"
#include "attention_extra.hpp"

namespace ats {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bbf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float bf32x16_t;
typedef unsigned int bu32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int bu32x2_t __attribute__((ext_vector_type(2)));
typedef short btr_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) btr_t* blds_tr_ptr_t;

constexpr int kSgMfma = 0x008, kSgDsRead = 0x100;   // instruction classes of sched_group_barrier
constexpr int kBwdRows = 128;   // rows a block owns: 4 waves x 32
constexpr int kDqBN = 64;       // keys per step of the dQ kernel
constexpr int kDkvBQ = 32;      // queries per step of the dK/dV kernel
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ bf32x16_t bwd_mma(const bu32x4_t& a, const bu32x4_t& b, bf32x16_t c) {
    union {
        bu32x4_t u;
        bbf16x8_t v;
    } x, y;
    x.u = a;
    y.u = b;
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(x.v, y.v, c, 0, 0, 0);
}

// delta[b, h, i] = sum_d dO[b, i, h, d] * O[b, i, h, d]; out and dout are [B, L, Hq*D].
template <int D>
__global__ __launch_bounds__(256) void attention_delta_kernel(const bf16_t* __restrict__ out,
                                                              const bf16_t* __restrict__ dout,
                                                              float* __restrict__ delta, int Hq, int L, int64_t rows) {
    constexpr int TPR = D / 8;   // threads per (token, head) row
    const int64_t row = (int64_t)blockIdx.x * (256 / TPR) + threadIdx.x / TPR;   // index over [B, L, Hq]
    float s = 0.f;
    if (row < rows) {
        const int64_t off = row * D + (threadIdx.x % TPR) * 8;
        const uint4 a = *reinterpret_cast<const uint4*>(out + off);
        const uint4 b = *reinterpret_cast<const uint4*>(dout + off);
        float fa[8], fb[8];
        Elem<bf16_t>::unpack(a, fa);
        Elem<bf16_t>::unpack(b, fb);
#pragma unroll
        for (int j = 0; j < 8; ++j) s += fa[j] * fb[j];
    }
#pragma unroll
    for (int o = TPR / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
    if (row < rows && threadIdx.x % TPR == 0) {
        const int64_t h = row % Hq, bl = row / Hq;
        const int64_t b = bl / L, i = bl % L;
        delta[(b * Hq + h) * L + i] = s;
    }
}

// ------------------------------------------------------------------------------------------ tiles in LDS
// Tiles of rows of D bf16 elements go from memory straight into LDS (buffer_load_dwordx4 ... lds: lane l of an
// instruction deposits its 16 bytes at M0 + 16 l), so rows are unpadded and a tile is stored once, although it is
// read both ways: along D (16-byte reads, 16 consecutive rows per quarter wave) and across rows (transposing
// 8-byte reads, 4 consecutive rows x 64 bytes per half wave).  An XOR swizzle of the 16-byte chunks, applied on the
// global side (which chunk a lane fetches), keeps both patterns free of bank conflicts: slot s of row r holds
// chunk s ^ g(r) with
//     256-byte rows: g(r) = (r % 16) ^ ((r % 4) << 2)       128-byte rows: u = (r / 2) % 8, g = u ^ ((u % 2) << 2)
// g is a bijection of the 16 rows (or 8 row pairs) a quarter wave reads along D, and it moves the 64-byte group
// of each of 4 consecutive rows to a different quarter of the banks.
template <int D>
struct SwzTile {
    static constexpr int ROWB = D * 2;      // bytes per row
    static constexpr int CPR = D / 8;       // 16-byte chunks per row
    static __device__ __forceinline__ int g(int r) {
        if constexpr (D == 128) return (r & 15) ^ ((r & 3) << 2);
        const int u = (r >> 1) & 7;
        return u ^ ((u & 1) << 2);
    }
    // lane offset (bytes from the tile's first row in memory, row stride `row_bytes`) of LDS position p (16-byte units)
    static __device__ __forceinline__ int src_offset(int p, int row_bytes) {
        const int r = p / CPR, sl = p % CPR;
        return r * row_bytes + ((sl ^ g(r)) * 16);
    }
    // LDS byte offset of the A-operand fragment along D for k-step ks: lane (row = lane % 32 of a 32-row block, half g2)
    static __device__ __forceinline__ int row_frag(int lane, int ks) {
        const int col = lane & 31, g2 = lane >> 5;
        return col * ROWB + (((2 * ks + g2) ^ g(col)) * 16);
    }
    // LDS byte offsets of the two 8-byte transposing reads of a fragment across rows (rows r0 + 0..15 of the tile,
    // r0 a multiple of 16, 32 d starting at 32 * G): lane l receives d = 32 G + l % 32 and rows
    // r0 + {4h..4h+3} (lo) and r0 + 8 + {4h..4h+3} (hi), h = l / 32, the order in which a 32x32 accumulator hands
    // its rows to the next product
    static __device__ __forceinline__ int tr_frag(int lane, int G, bool hi) {
        const int rr = 4 * (lane >> 5) + ((lane & 15) >> 2) + (hi ? 8 : 0);
        const int within = 32 * ((lane >> 4) & 1) + 8 * (lane & 3);      // byte inside the 64-byte group
        const int chunk = 4 * G + (within >> 4);
        return rr * ROWB + ((chunk ^ g(rr)) * 16) + (within & 15);
    }
};

typedef __attribute__((address_space(3))) unsigned char* blds_u8_t;
typedef __attribute__((address_space(3))) bu32x4_t* blds_v4_t;
typedef __attribute__((address_space(3))) float* blds_f32_t;
typedef __attribute__((address_space(3))) void* blds_void_t;

__device__ __forceinline__ bu32x4_t tr_fragment_swz(blds_u8_t tile, int lo_off, int hi_off, int const_off) {
    union {
        btr_t t[2];
        bu32x4_t u;
    } cv;
    cv.t[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((blds_tr_ptr_t)(tile + lo_off + const_off));
    cv.t[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((blds_tr_ptr_t)(tile + hi_off + const_off));
    return cv.u;
}

// Wave priority inside the tile loops of both kernels: the three stretches of a step (products, exponentials and
// dS, products) alternate between priority 1 and 0.  The two waves of a SIMD are usually in different stretches,
// and the one in a product stretch then wins the issue slots it needs to keep the matrix pipe fed: backward
// 1.21 -> 1.16 ms at batch 8 x 2048 positions (raising the vector stretch instead measures the same; raising the
// products alone, without lowering in between: 1.19).
// ------------------------------------------------------------------------------------------ dQ
// One 128-row query tile of one (batch, query head): lanes own queries, keys come in tiles of 64.  K and V tiles
// are double buffered: the loads of tile t+1 are issued before the arithmetic of tile t and have the whole
// iteration to land (one barrier per tile).
// EXTRA: pair bias and / or dropout (attention_extra.hpp), the same decisions as the forward made.
// The tile functions of both kernels are inlined functions with __restrict__ pointer parameters, and that is load
// bearing: it gives the transposing LDS reads alias metadata, without which the compiler waits for every
// direct-to-LDS load in flight (s_waitcnt vmcnt(0)) before each ds_read_b64_tr_b16 (see grouped_gemm.hip, where the
// same builtin first came without it).
template <int D, bool BIAS, bool EXTRA = false>
__device__ __forceinline__ void attention_bwd_dq_tile(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                                                      const bf16_t* __restrict__ v, const bf16_t* __restrict__ dout,
                                                      const float* __restrict__ lse, const float* __restrict__ delta,
                                                      const float* __restrict__ key_bias, bf16_t* __restrict__ dq, int Hq,
                                                      int Hkv, int L, int Lk, float scale, int qt, int hq, int b,
                                                      unsigned char* smem, const AttnExtra* ex = nullptr,
                                                      const bf16_t* __restrict__ out_rows = nullptr,
                                                      float* __restrict__ delta_w = nullptr) {
    static_assert(!(EXTRA && BIAS), "a per-key bias is folded into the pair bias");
    using SW = SwzTile<D>;
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int ROWB = SW::ROWB;
    constexpr int TILE = kDqBN * ROWB;              // one K or V tile
    constexpr int STAGE = 2 * TILE;                 // [K | V]
    constexpr int NI = TILE / 1024 / 4;             // load instructions per wave and tile, K (and V)
    static_assert(NI >= 1 && NI * 4 * 1024 == TILE, "loader tiling");
    const blds_u8_t sm = (blds_u8_t)smem;
    const blds_f32_t sBias = (blds_f32_t)(sm + 2 * STAGE);      // [2][64], log2 units
    const float* bias_row = BIAS ? key_bias + (int64_t)b * Lk : nullptr;

    const int hkv = hq / (Hq / Hkv);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, g = lane >> 5;
    const int q_row = qt * kBwdRows + wave * 32 + col;
    const int q_clamped = q_row < L ? q_row : L - 1;
    const int off = Lk - L;
    const int q_pos = q_row + off;
    const float scale_log2 = scale * kLog2e;

    const bf16_t* qp = q + ((int64_t)(b * Hq + hq) * L + q_clamped) * D;
    const bf16_t* dop = dout + ((int64_t)b * L + q_clamped) * (int64_t)(Hq * D) + hq * D;
    bu32x4_t qf[KS], dof[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        qf[s] = *reinterpret_cast<const bu32x4_t*>(qp + s * 16 + g * 8);
        dof[s] = *reinterpret_cast<const bu32x4_t*>(dop + s * 16 + g * 8);
    }
    const float lse2 = lse[(int64_t)(b * Hq + hq) * L + q_clamped] * kLog2e;
    // delta of this lane's query: given, or formed here from the forward's output row and the dO row that the
    // lane holds anyway (lanes l and l + 32 hold the two halves of a row) and left behind for the dK/dV kernel
    float dl;
    if (out_rows != nullptr) {
        const bf16_t* orow = out_rows + ((int64_t)b * L + q_clamped) * (int64_t)(Hq * D) + hq * D;
        float part = 0.f;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const uint4 ov = *reinterpret_cast<const uint4*>(orow + s * 16 + g * 8);
            const uint4 dv4 = make_uint4(dof[s].x, dof[s].y, dof[s].z, dof[s].w);
            float fo[8], fd[8];
            Elem<bf16_t>::unpack(ov, fo);
            Elem<bf16_t>::unpack(dv4, fd);
#pragma unroll
            for (int j = 0; j < 8; ++j) part += fo[j] * fd[j];
        }
        dl = part + __shfl_xor(part, 32, 64);
        if (g == 0 && q_row < L) delta_w[(int64_t)(b * Hq + hq) * L + q_row] = dl;
    } else {
        dl = delta[(int64_t)(b * Hq + hq) * L + q_clamped];
    }
    __amdgpu_buffer_rsrc_t pb_rsrc;
    int pb_row = 0;
    bool ex_bias = false, ex_drop = false;
    uint32_t head_key = 0, drop_counter0 = 0;
    if constexpr (EXTRA) {
        ex_bias = ex->bias_qk != nullptr;
        ex_drop = ex->keep_scale > 0.f;
        pb_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(ex_bias ? ex->bias_qk + (int64_t)b * ex->bias_sb + (int64_t)hq * ex->bias_sh : nullptr),
                                                    0, ex_bias ? (int)((int64_t)L * Lk * 4) : 0, 0x00020000);
        pb_row = q_clamped * Lk * 4;
        head_key = attn_head_key(ex->seed_lo, ex->seed_hi, (uint32_t)(b * Hq + hq));
        drop_counter0 = (uint32_t)q_clamped * (uint32_t)Lk;
    }

    const bf16_t* kbase = k + (int64_t)(b * Hkv + hkv) * Lk * D;
    const bf16_t* vbase = v + (int64_t)(b * Hkv + hkv) * Lk * D;
    // buffer loads: keys past Lk read as zeros
    const __amdgpu_buffer_rsrc_t k_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(kbase), 0, (int)((int64_t)Lk * D * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t v_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(vbase), 0, (int)((int64_t)Lk * D * 2), 0x00020000);
    int ld_off[NI];
#pragma unroll
    for (int j = 0; j < NI; ++j) ld_off[j] = SW::src_offset((j * 4 + wave) * 64 + lane, ROWB);
#define DQ_LOAD(tile_, stage_)                                                                         \
    _Pragma("unroll") for (int j_ = 0; j_ < NI; ++j_) {                                                \
        __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, (blds_void_t)(sm + (stage_) * STAGE + (j_ * 4 + wave) * 1024), 16, \
                                                 ld_off[j_], (tile_) * (kDqBN * D * 2), 0, 0);         \
        __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rsrc, (blds_void_t)(sm + (stage_) * STAGE + TILE + (j_ * 4 + wave) * 1024), \
                                                 16, ld_off[j_], (tile_) * (kDqBN * D * 2), 0, 0);     \
    }
    // Keys past Lk: the rows of K and V that the loads address there must be zeros in LDS (they meet exact
    // zeros of dS and P, but 0 x NaN is not 0); each lane clears the positions of its own loads once they landed.
#define DQ_CLEAR_TAIL(tile_, stage_)                                                                   \
    if (((tile_) + 1) * kDqBN > Lk) {                                                                  \
        _Pragma("unroll") for (int j_ = 0; j_ < NI; ++j_) {                                            \
            const int p_ = (j_ * 4 + wave) * 64 + lane;                                                \
            if ((tile_) * kDqBN + p_ / SW::CPR >= Lk) {                                                \
                *(blds_v4_t)(sm + (stage_) * STAGE + p_ * 16) = bu32x4_t{0u, 0u, 0u, 0u};              \
                *(blds_v4_t)(sm + (stage_) * STAGE + TILE + p_ * 16) = bu32x4_t{0u, 0u, 0u, 0u};       \
            }                                                                                          \
        }                                                                                              \
    }
    int row_addr[KS], tr_lo[DB], tr_hi[DB];
#pragma unroll
    for (int s = 0; s < KS; ++s) row_addr[s] = SW::row_frag(lane, s);
#pragma unroll
    for (int d = 0; d < DB; ++d) {
        tr_lo[d] = SW::tr_frag(lane, d, false);
        tr_hi[d] = SW::tr_frag(lane, d, true);
    }

    bf32x16_t acc_dq[DB];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int x = 0; x < 16; ++x) acc_dq[d][x] = 0.f;

    const int q_block_last = min(qt * kBwdRows + kBwdRows - 1, L - 1) + off;
    const int n_tiles = q_block_last / kDqBN + 1;
    const int q_wave_first = qt * kBwdRows + wave * 32 + off;
    const int q_wave_last = q_wave_first + 31;

    DQ_LOAD(0, 0)
    if (BIAS && tid < kDqBN) sBias[tid] = tid < Lk ? bias_row[tid] * kLog2e : 0.f;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    DQ_CLEAR_TAIL(0, 0)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
    for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(qf[s]), "+v"(dof[s]));

    // log2(scale) joins the exponent, so that P * scale comes out of the exponential: dS = (P * scale) * (dP - delta)
    const float lse2s = lse2 - log2f(scale);
    for (int t = 0; t < n_tiles; ++t) {
        const int n0 = t * kDqBN;
        const int st = (t & 1) * STAGE;             // this tile's stage; the other one receives tile t+1
        float r_bias = 0.f;
        if (t + 1 < n_tiles) {
            if (t & 1) { DQ_LOAD(t + 1, 0) } else { DQ_LOAD(t + 1, 1) }
            if (BIAS && tid < kDqBN) r_bias = n0 + kDqBN + tid < Lk ? bias_row[n0 + kDqBN + tid] * kLog2e : 0.f;
        }
        if (n0 <= q_wave_last) {   // some key of the tile is in this wave's past or present
            // ---- S^T = K . Q^T and dP^T = V . dO^T
            __builtin_amdgcn_s_setprio(1);
            bf32x16_t acc_s[2], acc_p[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int x = 0; x < 16; ++x) {
                    acc_s[kb][x] = 0.f;
                    acc_p[kb][x] = 0.f;
                }
#pragma unroll
            for (int s = 0; s < KS; ++s)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    const blds_u8_t pk = sm + st + row_addr[s] + kb * 32 * ROWB;
                    const bu32x4_t kf = *(blds_v4_t)(pk), vf = *(blds_v4_t)(pk + TILE);
                    acc_s[kb] = bwd_mma(kf, qf[s], acc_s[kb]);
                    acc_p[kb] = bwd_mma(vf, dof[s], acc_p[kb]);
                }
            // ---- dS^T = P^T * (dP^T - delta) * scale, with P^T = exp(S^T * scale - lse)
            __builtin_amdgcn_s_setprio(0);
            const bool diagonal = n0 + kDqBN - 1 > q_wave_first;
            const blds_f32_t bias_t = sBias + (t & 1) * kDqBN;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int x = 0; x < 16; ++x) {
                    // the key of accumulator value x is kb*32 + (x/4)*8 + g*4 + x%4 of the tile
                    float kbias = BIAS ? bias_t[kb * 32 + (x >> 2) * 8 + g * 4 + (x & 3)] : 0.f;
                    float dp = acc_p[kb][x];
                    if constexpr (EXTRA) {
                        const int key = n0 + kb * 32 + (x >> 2) * 8 + g * 4 + (x & 3);
                        if (ex_bias)
                            kbias = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(pb_rsrc, pb_row + key * 4, 0, 0)) *
                                    kLog2e;
                        if (ex_drop)   // dP reaches only the weights that were kept
                            dp = attn_drop_hash(head_key, drop_counter0 + (uint32_t)key) >= ex->drop_threshold ? dp * ex->keep_scale
                                                                                                            : 0.f;
                    }
                    float p = __builtin_amdgcn_exp2f(__builtin_fmaf(acc_s[kb][x], scale_log2, kbias - lse2s));
                    if (diagonal) {
                        const int key = n0 + kb * 32 + (x >> 2) * 8 + g * 4 + (x & 3);
                        if (key > q_pos) p = 0.f;
                    }
                    acc_s[kb][x] = p * (dp - dl);
                }
            bu32x4_t dsf[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int kb = s >> 1, x0 = (s & 1) * 8;
                dsf[s].x = pack_bf16x2(acc_s[kb][x0 + 0], acc_s[kb][x0 + 1]);
                dsf[s].y = pack_bf16x2(acc_s[kb][x0 + 2], acc_s[kb][x0 + 3]);
                dsf[s].z = pack_bf16x2(acc_s[kb][x0 + 4], acc_s[kb][x0 + 5]);
                dsf[s].w = pack_bf16x2(acc_s[kb][x0 + 6], acc_s[kb][x0 + 7]);
            }
            // ---- dQ^T += K^T . dS^T  (keys of a k-step in accumulator order, as in the forward's second product)
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int d = 0; d < DB; ++d)
                    acc_dq[d] = bwd_mma(tr_fragment_swz(sm + st, tr_lo[d], tr_hi[d], s * 16 * ROWB), dsf[s], acc_dq[d]);
            // the transposing reads run two fragments ahead of the MFMAs (unconstrained, the compiler issues all
            // 32 reads first and the first MFMAs wait for the tail of that burst)
            __builtin_amdgcn_sched_group_barrier(kSgDsRead, 4, 0);
#pragma unroll
            for (int i = 0; i + 2 < 4 * DB; ++i) {
                __builtin_amdgcn_sched_group_barrier(kSgDsRead, 2, 0);
                __builtin_amdgcn_sched_group_barrier(kSgMfma, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(kSgMfma, 2, 0);
            __builtin_amdgcn_s_setprio(0);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (t + 1 < n_tiles) {
            if (t & 1) { DQ_CLEAR_TAIL(t + 1, 0) } else { DQ_CLEAR_TAIL(t + 1, 1) }
            if (BIAS && tid < kDqBN) sBias[((t + 1) & 1) * kDqBN + tid] = r_bias;
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
#undef DQ_LOAD
#undef DQ_CLEAR_TAIL

    if (q_row < L) {
        bf16_t* drow = dq + ((int64_t)(b * Hq + hq) * L + q_row) * D;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                bu32x2_t w;
                w.x = pack_bf16x2(acc_dq[d][r * 4 + 0], acc_dq[d][r * 4 + 1]);
                w.y = pack_bf16x2(acc_dq[d][r * 4 + 2], acc_dq[d][r * 4 + 3]);
                *reinterpret_cast<bu32x2_t*>(drow + d * 32 + r * 8 + g * 4) = w;
            }
    }
}

// A workgroup takes a long query tile and its mirror-image short one (equal work per workgroup: the
// hardware hands workgroups out strictly in turn), and the workgroups of one (batch, kv head) share an XCD.
template <int D, bool BIAS, bool EXTRA = false>
__global__ __launch_bounds__(256, 2) void attention_bwd_dq_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const bf16_t* __restrict__ dout, const float* __restrict__ lse, const float* __restrict__ delta,
    const float* __restrict__ key_bias, bf16_t* __restrict__ dq, int Hq, int Hkv, int L, int Lk, float scale, int B,
    AttnExtra ex, const bf16_t* __restrict__ out_rows, float* __restrict__ delta_w) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int n_qt = (L + kBwdRows - 1) / kBwdRows;
    const int n_pairs = (n_qt + 1) / 2;
    const int per_group = n_pairs * (Hq / Hkv);
    const int n_groups = B * Hkv;
    int group, within;
    if (n_groups % 8 == 0) {
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        group = (idx / per_group) * 8 + xcd;
        within = idx % per_group;
    } else {
        group = blockIdx.x / per_group;
        within = blockIdx.x % per_group;
    }
    const int b = group / Hkv;
    const int hq = (group % Hkv) * (Hq / Hkv) + within / n_pairs;
    const int pair = within % n_pairs;
    const int qt_long = n_qt - 1 - pair;
#pragma unroll 1
    for (int half = 0; half < 2; ++half) {
        if (half && pair == qt_long) break;
        attention_bwd_dq_tile<D, BIAS, EXTRA>(q, k, v, dout, lse, delta, key_bias, dq, Hq, Hkv, L, Lk, scale,
                                              half ? pair : qt_long, hq, b, smem, &ex, out_rows, delta_w);
    }
}

// ------------------------------------------------------------------------------------------ dK, dV
// One 128-row key tile of one (batch, kv head): lanes own keys; the queries of every query head of the
// group come in steps of 32, starting at the first query that sees the tile.  The steps of all heads form one
// sequence; the Q and dO rows of step i+1 go from memory straight into the LDS stage that step i-1 used
// (swizzled tiles as in the dQ kernel, read along D for the first two products and across rows for the last
// two) while step i is computed: one barrier per step, and the loads have the whole step to land.
typedef float bf32x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) bf32x4_t* blds_f4_t;
template <int D, bool EXTRA = false>
__device__ __forceinline__ void attention_bwd_dkv_tile(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                                                       const bf16_t* __restrict__ v, const bf16_t* __restrict__ dout,
                                                       const float* __restrict__ lse, const float* __restrict__ delta,
                                                       const float* __restrict__ key_bias, bf16_t* __restrict__ dk,
                                                       bf16_t* __restrict__ dv, int Hq, int Hkv, int L, int Lk, float scale,
                                                       int kt_idx, int hkv, int b, unsigned char* smem,
                                                       const AttnExtra* ex = nullptr) {
    using SW = SwzTile<D>;
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int ROWB = SW::ROWB;
    constexpr int TILE = kDkvBQ * ROWB;              // one Q or dO tile
    constexpr int STAGE = 2 * TILE;                  // [Q | dO]
    constexpr int NI = TILE / 1024 / 4;              // load instructions per wave and tile, Q (and dO)
    static_assert(NI >= 1 && NI * 4 * 1024 == TILE, "loader tiling");
    constexpr int RPITCH = D * 2 + 16;               // bytes per V row in LDS
    const blds_u8_t sm = (blds_u8_t)smem;
    const blds_f32_t sL = (blds_f32_t)(sm + 2 * STAGE);   // [2][32] lse * log2(e)
    const blds_f32_t sD = sL + 2 * kDkvBQ;                // [2][32] delta
    // the block's own V rows stay in LDS for the whole tile: with K rows, both accumulators and V rows in
    // registers a wave would need more than half the register file, i.e. one wave per SIMD
    unsigned char* const sVb = smem + 2 * STAGE + 4 * kDkvBQ * 4;    // [128][RPITCH]

    const int rep = Hq / Hkv;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, g = lane >> 5;
    const int key_row = kt_idx * kBwdRows + wave * 32 + col;
    const int key_clamped = key_row < Lk ? key_row : Lk - 1;
    const int off = Lk - L;
    const float scale_log2 = scale * kLog2e;

    const float kbias = key_bias ? key_bias[(int64_t)b * Lk + key_clamped] * kLog2e : 0.f;   // this lane's key
    bool ex_bias = false, ex_drop = false;
    if constexpr (EXTRA) {
        ex_bias = ex->bias_qk != nullptr;
        ex_drop = ex->keep_scale > 0.f;
    }
    const bf16_t* kp = k + ((int64_t)(b * Hkv + hkv) * Lk + key_clamped) * D;
    bu32x4_t kf[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) kf[s] = *reinterpret_cast<const bu32x4_t*>(kp + s * 16 + g * 8);
    __syncthreads();   // the previous tile of this workgroup is done with the V rows and the stages
    {
        const bf16_t* vblock = v + (int64_t)(b * Hkv + hkv) * Lk * D;
        const __amdgpu_buffer_rsrc_t vb_rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(vblock), 0, (int)((int64_t)Lk * D * 2), 0x00020000);
#pragma unroll
        for (int i = 0; i < kBwdRows * (D / 8) / 256; ++i) {
            const int idx = tid + i * 256;
            const int r = idx / (D / 8), c = idx % (D / 8);
            const bu32x4_t x = __builtin_amdgcn_raw_buffer_load_b128(vb_rsrc, (r * D + c * 8) * 2,
                                                                     kt_idx * kBwdRows * D * 2, 0);
            *reinterpret_cast<bu32x4_t*>(sVb + r * RPITCH + c * 16) = x;
        }
    }
    const unsigned char* const v_row = sVb + (wave * 32 + col) * RPITCH + g * 16;
#pragma unroll
    for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(kf[s]));

    // lane offsets of the loads (Q rows are D elements apart, dO rows Hq * D) and of the fragment reads
    int ld_q[NI], ld_o[NI];
#pragma unroll
    for (int j = 0; j < NI; ++j) {
        ld_q[j] = SW::src_offset((j * 4 + wave) * 64 + lane, ROWB);
        ld_o[j] = SW::src_offset((j * 4 + wave) * 64 + lane, Hq * ROWB);
    }
    // fragment offsets of k-step s / d block G differ from those of k-step 0 / block 0 in the chunk bits only:
    // off(s) = off(0) ^ (s << 5), off(G) = off(0) ^ (G << 6); they are formed per step from three registers
    // (sixteen kept across the loop would not fit beside the accumulators)
    const int row_base = SW::row_frag(lane, 0), tr_lo_base = SW::tr_frag(lane, 0, false),
              tr_hi_base = SW::tr_frag(lane, 0, true);
    // buffer loads: query rows past L are outside the descriptors
#define DKV_LOAD(hh_, q0_, stage_)                                                                     \
    {                                                                                                  \
        const int hq_ = hkv * rep + (hh_);                                                             \
        const __amdgpu_buffer_rsrc_t q_rsrc_ = __builtin_amdgcn_make_buffer_rsrc(                      \
            const_cast<bf16_t*>(q + (int64_t)(b * Hq + hq_) * L * D), 0, (int)((int64_t)L * D * 2), 0x00020000); \
        const __amdgpu_buffer_rsrc_t o_rsrc_ = __builtin_amdgcn_make_buffer_rsrc(                      \
            const_cast<bf16_t*>(dout + (int64_t)b * L * (int64_t)(Hq * D) + hq_ * D), 0,              \
            (int)((((int64_t)L - 1) * Hq * D + D) * 2), 0x00020000);                                   \
        _Pragma("unroll") for (int j_ = 0; j_ < NI; ++j_) {                                            \
            __builtin_amdgcn_raw_ptr_buffer_load_lds(q_rsrc_, (blds_void_t)(sm + (stage_) * STAGE + (j_ * 4 + wave) * 1024), \
                                                     16, ld_q[j_], (q0_) * (D * 2), 0, 0);             \
            __builtin_amdgcn_raw_ptr_buffer_load_lds(o_rsrc_, (blds_void_t)(sm + (stage_) * STAGE + TILE + (j_ * 4 + wave) * 1024), \
                                                     16, ld_o[j_], (q0_) * (Hq * D * 2), 0, 0);        \
        }                                                                                              \
    }
    // Queries past L: their rows of Q and dO must be zeros in LDS (they meet exact zeros of P and dS, but
    // 0 x NaN is not 0); each lane clears the positions of its own loads once they landed.
#define DKV_CLEAR_TAIL(q0_, stage_)                                                                    \
    if ((q0_) + kDkvBQ > L) {                                                                          \
        _Pragma("unroll") for (int j_ = 0; j_ < NI; ++j_) {                                            \
            const int p_ = (j_ * 4 + wave) * 64 + lane;                                                \
            if ((q0_) + p_ / SW::CPR >= L) {                                                           \
                *(blds_v4_t)(sm + (stage_) * STAGE + p_ * 16) = bu32x4_t{0u, 0u, 0u, 0u};              \
                *(blds_v4_t)(sm + (stage_) * STAGE + TILE + p_ * 16) = bu32x4_t{0u, 0u, 0u, 0u};       \
            }                                                                                          \
        }                                                                                              \
    }
    // lse and delta of the step's queries: thread t < 32 fetches those of query q0 + t (raw values: nothing may
    // wait for them before the step's arithmetic is done) and finishes them when it stores them
#define DKV_ROW_SCALARS(hh_, q0_, l_, d_)                                                              \
    if (tid < kDkvBQ) {                                                                                \
        const int qc_ = min((q0_) + tid, L - 1);                                                       \
        const int64_t base_ = (int64_t)(b * Hq + hkv * rep + (hh_)) * L;                               \
        l_ = lse[base_ + qc_];                                                                         \
        d_ = delta[base_ + qc_];                                                                       \
    }
#define DKV_STORE_SCALARS(q0_, par_, l_, d_)                                                           \
    asm volatile("" : "+v"(l_), "+v"(d_));   /* the wait for the two values stays down here */          \
    if (tid < kDkvBQ) {                                                                                \
        const bool in_ = (q0_) + tid < L;                                                              \
        sL[(par_) * kDkvBQ + tid] = in_ ? l_ * kLog2e : INFINITY;   /* exp2(-inf) = 0 for rows past L */ \
        sD[(par_) * kDkvBQ + tid] = in_ ? d_ : 0.f;                                                    \
    }

    bf32x16_t acc_dk[DB], acc_dv[DB];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int x = 0; x < 16; ++x) {
            acc_dk[d][x] = 0.f;
            acc_dv[d][x] = 0.f;
        }

    const int key_block_first = kt_idx * kBwdRows;
    const int key_wave_first = key_block_first + wave * 32;
    const int key_wave_last = key_wave_first + 31;
    // first query that sees any key of the block: q + off >= key_block_first
    const int q_first = max(key_block_first - off, 0) / kDkvBQ * kDkvBQ;
    const int n_steps = rep * ((L - q_first + kDkvBQ - 1) / kDkvBQ);

    DKV_LOAD(0, q_first, 0)
    {
        float l0 = 0.f, d0 = 0.f;
        DKV_ROW_SCALARS(0, q_first, l0, d0)
        DKV_STORE_SCALARS(q_first, 0, l0, d0)
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    DKV_CLEAR_TAIL(q_first, 0)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    int hh = 0, q0 = q_first;
    for (int i = 0; i < n_steps; ++i) {
        const int par = i & 1;
        const blds_u8_t st = sm + par * STAGE;     // this step's stage; the other one receives step i+1
        int hh_n = hh, q0_n = q0 + kDkvBQ;
        if (q0_n >= L) {
            hh_n = hh + 1;
            q0_n = q_first;
        }
        const bool more = i + 1 < n_steps;
        const bool active = q0 + kDkvBQ - 1 + off >= key_wave_first;   // some query of the step sees this wave's keys
        float r_l = 0.f, r_d = 0.f;
        int rb = row_base, tlb = tr_lo_base, thb = tr_hi_base;
        asm volatile("" : "+v"(rb), "+v"(tlb), "+v"(thb));   // keeps the offsets below inside the step
#define DKV_PREFETCH()                                                                                 \
        if (more) {                                                                                    \
            if (par) { DKV_LOAD(hh_n, q0_n, 0) } else { DKV_LOAD(hh_n, q0_n, 1) }                      \
            DKV_ROW_SCALARS(hh_n, q0_n, r_l, r_d)                                                      \
        }
        DKV_PREFETCH()
        if (active) {
            const int hq = hkv * rep + hh;
            const uint32_t head_key = EXTRA ? attn_head_key(ex->seed_lo, ex->seed_hi, (uint32_t)(b * Hq + hq)) : 0u;
            // this head's [L, Lk] matrix of the pair bias; queries past L read as zeros (their probabilities are
            // zeros anyway: lse = +inf)
            __amdgpu_buffer_rsrc_t pb_rsrc;
            if constexpr (EXTRA)
                pb_rsrc = __builtin_amdgcn_make_buffer_rsrc(
                    const_cast<float*>(ex_bias ? ex->bias_qk + (int64_t)b * ex->bias_sb + (int64_t)hq * ex->bias_sh : nullptr), 0,
                    ex_bias ? (int)((int64_t)L * Lk * 4) : 0, 0x00020000);
            // ---- S = Q . K^T and dP = dO . V^T  (rows = queries of the step, column = this lane's key)
            __builtin_amdgcn_s_setprio(1);
            bf32x16_t acc_s, acc_p;
#pragma unroll
            for (int x = 0; x < 16; ++x) {
                acc_s[x] = 0.f;
                acc_p[x] = 0.f;
            }
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const int ra = rb ^ (s << 5);
                const bu32x4_t qa = *(blds_v4_t)(st + ra), oa = *(blds_v4_t)(st + TILE + ra);
                acc_s = bwd_mma(qa, kf[s], acc_s);
                acc_p = bwd_mma(oa, *reinterpret_cast<const bu32x4_t*>(v_row + s * 32), acc_p);
            }
            // the three reads of k-step s+1 go out before the MFMAs of k-step s
            __builtin_amdgcn_sched_group_barrier(kSgDsRead, 3, 0);
#pragma unroll
            for (int s = 0; s + 1 < KS; ++s) {
                __builtin_amdgcn_sched_group_barrier(kSgDsRead, 3, 0);
                __builtin_amdgcn_sched_group_barrier(kSgMfma, 2, 0);
            }
            __builtin_amdgcn_sched_group_barrier(kSgMfma, 2, 0);
            // ---- P = exp(S * scale - lse[q]); dS = P * (dP - delta[q]) * scale; accumulator row x is
            //      query (x / 4) * 8 + g * 4 + x % 4 of the step
            __builtin_amdgcn_s_setprio(0);
            const bool diagonal = q0 + off < key_wave_last;
            bu32x4_t pf[2], dsf[2];
            // rows r of the accumulators (queries r*8 + g*4 + 0..3 of the step) -> words r%2*2, r%2*2+1 of pf / dsf [r/2]
            auto exp_rows = [&](int r) {
                const bf32x4_t l4 = *(blds_f4_t)(sL + par * kDkvBQ + r * 8 + g * 4);
                const bf32x4_t d4 = *(blds_f4_t)(sD + par * kDkvBQ + r * 8 + g * 4);
                const float lv[4] = {l4.x, l4.y, l4.z, l4.w};
                const float dvv[4] = {d4.x, d4.y, d4.z, d4.w};
                float p[4], ds[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int x = r * 4 + j;
                    float kb_x = kbias, dp = acc_p[x], keep_mul = 1.0f;
                    if constexpr (EXTRA) {
                        const int qi = q0 + r * 8 + g * 4 + j;
                        if (ex_bias)
                            kb_x = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                                 pb_rsrc, (qi * Lk + key_clamped) * 4, 0, 0)) *
                                   kLog2e;
                        if (ex_drop) {
                            keep_mul = attn_drop_hash(head_key, (uint32_t)qi * (uint32_t)Lk + (uint32_t)key_clamped) >=
                                               ex->drop_threshold
                                           ? ex->keep_scale
                                           : 0.f;
                            dp *= keep_mul;
                        }
                    }
                    float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(acc_s[x], scale_log2, kb_x - lv[j]));
                    if (diagonal) {
                        const int qi = q0 + r * 8 + g * 4 + j;
                        if (key_row > qi + off) pv = 0.f;
                    }
                    p[j] = pv * keep_mul;          // the weights that met V in the forward
                    ds[j] = pv * (dp - dvv[j]) * scale;
                }
                // k-step s of the second products holds accumulator values 8s .. 8s+7
                const unsigned p01 = pack_bf16x2(p[0], p[1]), p23 = pack_bf16x2(p[2], p[3]);
                const unsigned s01 = pack_bf16x2(ds[0], ds[1]), s23 = pack_bf16x2(ds[2], ds[3]);
                if (r == 0) { pf[0].x = p01; pf[0].y = p23; dsf[0].x = s01; dsf[0].y = s23; }
                if (r == 1) { pf[0].z = p01; pf[0].w = p23; dsf[0].z = s01; dsf[0].w = s23; }
                if (r == 2) { pf[1].x = p01; pf[1].y = p23; dsf[1].x = s01; dsf[1].y = s23; }
                if (r == 3) { pf[1].z = p01; pf[1].w = p23; dsf[1].z = s01; dsf[1].w = s23; }
            };
            exp_rows(0);
            exp_rows(1);
            // ---- dV^T += dO^T . P and dK^T += Q^T . dS  (queries of a k-step in accumulator order).  The
            //      transposing reads of pair i+1 (a fragment of dO^T and one of Q^T) are issued before the MFMAs
            //      of pair i: left to itself the compiler reuses one set of registers for every fragment and
            //      each MFMA waits a full LDS latency.  The exponentials of the second half of the step's queries
            //      run between the MFMAs of the first half.
            __builtin_amdgcn_s_setprio(1);
            {
                constexpr int NP = 2 * DB;   // pairs: (k-step s, d block) = (i / DB, i % DB)
                bu32x4_t fo[2], fq[2];
                fo[0] = tr_fragment_swz(st + TILE, tlb, thb, 0);
                fq[0] = tr_fragment_swz(st, tlb, thb, 0);
#pragma unroll
                for (int i = 0; i < NP; ++i) {
                    if (i == 0) exp_rows(2);
                    if (i == DB / 2) exp_rows(3);
                    if (i + 1 < NP) {
                        const int s1 = (i + 1) / DB, d1 = (i + 1) % DB;
                        const int tl = tlb ^ (d1 << 6), th = thb ^ (d1 << 6);
                        fo[(i + 1) & 1] = tr_fragment_swz(st + TILE, tl, th, s1 * 16 * ROWB);
                        fq[(i + 1) & 1] = tr_fragment_swz(st, tl, th, s1 * 16 * ROWB);
                    }
                    acc_dv[i % DB] = bwd_mma(fo[i & 1], pf[i / DB], acc_dv[i % DB]);
                    acc_dk[i % DB] = bwd_mma(fq[i & 1], dsf[i / DB], acc_dk[i % DB]);
                }
                __builtin_amdgcn_sched_group_barrier(kSgDsRead, 8, 0);
#pragma unroll
                for (int i = 0; i + 2 < NP; ++i) {
                    __builtin_amdgcn_sched_group_barrier(kSgMfma, 2, 0);
                    __builtin_amdgcn_sched_group_barrier(kSgDsRead, 4, 0);
                }
                __builtin_amdgcn_sched_group_barrier(kSgMfma, 4, 0);
            }
            __builtin_amdgcn_s_setprio(0);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (more) {
            if (par) { DKV_CLEAR_TAIL(q0_n, 0) } else { DKV_CLEAR_TAIL(q0_n, 1) }
            DKV_STORE_SCALARS(q0_n, par ^ 1, r_l, r_d)
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        hh = hh_n;
        q0 = q0_n;
    }
#undef DKV_LOAD
#undef DKV_CLEAR_TAIL
#undef DKV_ROW_SCALARS
#undef DKV_STORE_SCALARS
#undef DKV_PREFETCH

    if (key_row < Lk) {
        bf16_t* krow = dk + ((int64_t)(b * Hkv + hkv) * Lk + key_row) * D;
        bf16_t* vrow = dv + ((int64_t)(b * Hkv + hkv) * Lk + key_row) * D;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                bu32x2_t w;
                w.x = pack_bf16x2(acc_dk[d][r * 4 + 0], acc_dk[d][r * 4 + 1]);
                w.y = pack_bf16x2(acc_dk[d][r * 4 + 2], acc_dk[d][r * 4 + 3]);
                *reinterpret_cast<bu32x2_t*>(krow + d * 32 + r * 8 + g * 4) = w;
                w.x = pack_bf16x2(acc_dv[d][r * 4 + 0], acc_dv[d][r * 4 + 1]);
                w.y = pack_bf16x2(acc_dv[d][r * 4 + 2], acc_dv[d][r * 4 + 3]);
                *reinterpret_cast<bu32x2_t*>(vrow + d * 32 + r * 8 + g * 4) = w;
            }
    }
}

// Early key tiles are seen by more queries than late ones: a workgroup takes tile j and tile n-1-j.
template <int D, bool EXTRA = false>
__global__ __launch_bounds__(256, 2) void attention_bwd_dkv_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
    const bf16_t* __restrict__ dout, const float* __restrict__ lse, const float* __restrict__ delta,
    const float* __restrict__ key_bias, bf16_t* __restrict__ dk, bf16_t* __restrict__ dv, int Hq, int Hkv, int L, int Lk,
    float scale, AttnExtra ex) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int n_kt = (Lk + kBwdRows - 1) / kBwdRows;
    const int n_pairs = (n_kt + 1) / 2;
    // consecutive ids go to different XCDs: keep the workgroups of one (batch, kv head), which read the
    // same queries, on one XCD
    const int n_groups = (int)gridDim.x / n_pairs;
    int group, pair;
    if (n_groups % 8 == 0) {
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        group = (idx / n_pairs) * 8 + xcd;
        pair = idx % n_pairs;
    } else {
        group = blockIdx.x / n_pairs;
        pair = blockIdx.x % n_pairs;
    }
    const int hkv = group % Hkv;
    const int b = group / Hkv;
    const int kt_far = n_kt - 1 - pair;
#pragma unroll 1
    for (int half = 0; half < 2; ++half) {
        if (half && pair == kt_far) break;
        attention_bwd_dkv_tile<D, EXTRA>(q, k, v, dout, lse, delta, key_bias, dk, dv, Hq, Hkv, L, Lk, scale,
                                         half ? kt_far : pair, hkv, b, smem, &ex);
    }
}

}  // namespace ats

extern "C" int ats_attention_delta(const void* out, const void* dout, float* delta, int B, int Hq, int L, int D,
                                   ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(B >= 0 && Hq > 0 && L >= 0 && (D == 64 || D == 128), ATS_ERR_UNSUPPORTED,
                "ats_attention_delta: B=%d Hq=%d L=%d D=%d (head_dim 64 or 128)", B, Hq, L, D);
    if (B == 0 || L == 0) return ATS_OK;
    ATS_REQUIRE(out && dout && delta && aligned16(out) && aligned16(dout), ATS_ERR_INVALID_ARG,
                "ats_attention_delta: null or misaligned pointer");
    const int64_t rows = (int64_t)B * L * Hq;
    const int rpb = 256 / (D / 8);
    const int64_t blocks = (rows + rpb - 1) / rpb;
    ATS_REQUIRE(blocks <= 0x7fffffff, ATS_ERR_UNSUPPORTED, "ats_attention_delta: %lld workgroups", (long long)blocks);
    if (D == 128)
        hipLaunchKernelGGL((attention_delta_kernel<128>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const bf16_t*>(out), static_cast<const bf16_t*>(dout), delta, Hq, L, rows);
    else
        hipLaunchKernelGGL((attention_delta_kernel<64>), dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const bf16_t*>(out), static_cast<const bf16_t*>(dout), delta, Hq, L, rows);
    ATS_CHECK_LAUNCH("ats_attention_delta");
    return ATS_OK;
}

extern "C" int ats_attention_bwd(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                                 const float* delta, const float* key_bias, void* dq, void* dk, void* dv, int B, int Hq,
                                 int Hkv, int L, int Lk, int D, float scale, ats_stream_t stream) {
    return ats_attention_bwd_ex(q, k, v, dout, lse, delta, key_bias, nullptr, 0, 0, 0.f, 0, dq, dk, dv, B, Hq, Hkv, L, Lk, D,
                                scale, stream);
}

// out == nullptr: delta is given.  Otherwise the dQ kernel forms delta from out and dout and writes it to
// delta_ws, where the dK/dV kernel (launched behind it on the same stream) reads it.
static int attention_bwd_launch(const void* q, const void* k, const void* v, const void* out, const void* dout,
                                const float* lse, const float* delta, float* delta_ws, const float* key_bias,
                                const float* bias_qk, int64_t bias_sb, int64_t bias_sh, float dropout_p,
                                uint64_t dropout_seed, void* dq, void* dk, void* dv, int B, int Hq, int Hkv, int L, int Lk,
                                int D, float scale, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(B >= 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0 && L >= 0 && Lk >= L && scale > 0.f, ATS_ERR_INVALID_ARG,
                "ats_attention_bwd: B=%d Hq=%d Hkv=%d L=%d Lk=%d scale=%g", B, Hq, Hkv, L, Lk, scale);
    ATS_REQUIRE(D == 64 || D == 128, ATS_ERR_UNSUPPORTED, "ats_attention_bwd: head_dim %d (64 or 128)", D);
    if (B == 0 || L == 0) return ATS_OK;
    ATS_REQUIRE(q && k && v && dout && lse && (out ? delta_ws != nullptr : delta != nullptr) && dq && dk && dv,
                ATS_ERR_INVALID_ARG, "ats_attention_bwd: null pointer");
    ATS_REQUIRE(!out || aligned16(out), ATS_ERR_INVALID_ARG, "ats_attention_bwd: misaligned pointer");
    const bf16_t* out_ = static_cast<const bf16_t*>(out);
    const float* delta_kv = out ? delta_ws : delta;   // what the dK/dV kernel reads
    ATS_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(dout) && aligned16(dq) && aligned16(dk) &&
                    aligned16(dv),
                ATS_ERR_INVALID_ARG, "ats_attention_bwd: misaligned pointer");
    ATS_REQUIRE((int64_t)Lk * D * 2 < 0x7fffffffLL && (int64_t)L * Hq * D * 2 < 0x7fffffffLL, ATS_ERR_UNSUPPORTED,
                "ats_attention_bwd: L=%d Lk=%d (one head's K or V, and one batch entry's dO, must stay under 2 GiB)", L, Lk);
    const int n_qt = (L + kBwdRows - 1) / kBwdRows, n_kt = (Lk + kBwdRows - 1) / kBwdRows;
    const int64_t dq_blocks = (int64_t)((n_qt + 1) / 2) * Hq * B;
    const int64_t dkv_blocks = (int64_t)((n_kt + 1) / 2) * Hkv * B;
    ATS_REQUIRE(dq_blocks <= 0x7fffffff && dkv_blocks <= 0x7fffffff, ATS_ERR_UNSUPPORTED, "ats_attention_bwd: grid");
    const bf16_t* q_ = static_cast<const bf16_t*>(q);
    const bf16_t* k_ = static_cast<const bf16_t*>(k);
    const bf16_t* v_ = static_cast<const bf16_t*>(v);
    const bf16_t* do_ = static_cast<const bf16_t*>(dout);
    hipStream_t s = as_stream(stream);
    AttnExtra ex;
    bool extras = false;
    if (!make_attention_extra("ats_attention_bwd_ex", bias_qk, bias_sb, bias_sh, dropout_p, dropout_seed, L, Lk, &ex, &extras))
        return ATS_ERR_INVALID_ARG;
    ATS_REQUIRE(!extras || key_bias == nullptr, ATS_ERR_INVALID_ARG,
                "ats_attention_bwd_ex: with a pair bias or dropout the per-key bias must be folded into the pair bias");
    if (D == 128) {
        constexpr int smem_dq = 4 * kDqBN * 128 * 2 + 2 * kDqBN * 4;
        constexpr int smem_dkv = 4 * kDkvBQ * 128 * 2 + 4 * kDkvBQ * 4 + kBwdRows * (128 * 2 + 16);
        static LdsReservation reserved, reserved_dq;
        hipError_t e = reserve_lds(reserved, {reinterpret_cast<const void*>(attention_bwd_dkv_kernel<128>)}, smem_dkv);
        ATS_REQUIRE(e == hipSuccess, ATS_ERR_LAUNCH, "ats_attention_bwd: cannot reserve %d bytes of LDS: %s", smem_dkv,
                    hipGetErrorString(e));
        e = reserve_lds(reserved_dq,
                        {reinterpret_cast<const void*>(attention_bwd_dq_kernel<128, true>),
                         reinterpret_cast<const void*>(attention_bwd_dq_kernel<128, false>),
                         reinterpret_cast<const void*>(attention_bwd_dq_kernel<128, false, true>)},
                        smem_dq);
        ATS_REQUIRE(e == hipSuccess, ATS_ERR_LAUNCH, "ats_attention_bwd: cannot reserve %d bytes of LDS: %s", smem_dq,
                    hipGetErrorString(e));
        if (extras) {
            static LdsReservation reserved_x;
            e = reserve_lds(reserved_x, {reinterpret_cast<const void*>(attention_bwd_dkv_kernel<128, true>)}, smem_dkv);
            ATS_REQUIRE(e == hipSuccess, ATS_ERR_LAUNCH, "ats_attention_bwd_ex: cannot reserve %d bytes of LDS: %s", smem_dkv,
                        hipGetErrorString(e));
            hipLaunchKernelGGL((attention_bwd_dq_kernel<128, false, true>), dim3((unsigned)dq_blocks), dim3(256), smem_dq, s,
                               q_, k_, v_, do_, lse, delta, key_bias, static_cast<bf16_t*>(dq), Hq, Hkv, L, Lk, scale, B, ex, out_, delta_ws);
            hipLaunchKernelGGL((attention_bwd_dkv_kernel<128, true>), dim3((unsigned)dkv_blocks), dim3(256), smem_dkv, s, q_,
                               k_, v_, do_, lse, delta_kv, key_bias, static_cast<bf16_t*>(dk), static_cast<bf16_t*>(dv), Hq, Hkv,
                               L, Lk, scale, ex);
        } else {
            if (key_bias)
                hipLaunchKernelGGL((attention_bwd_dq_kernel<128, true>), dim3((unsigned)dq_blocks), dim3(256), smem_dq, s,
                                   q_, k_, v_, do_, lse, delta, key_bias, static_cast<bf16_t*>(dq), Hq, Hkv, L, Lk, scale, B,
                                   ex, out_, delta_ws);
            else
                hipLaunchKernelGGL((attention_bwd_dq_kernel<128, false>), dim3((unsigned)dq_blocks), dim3(256), smem_dq, s,
                                   q_, k_, v_, do_, lse, delta, key_bias, static_cast<bf16_t*>(dq), Hq, Hkv, L, Lk, scale, B,
                                   ex, out_, delta_ws);
            hipLaunchKernelGGL((attention_bwd_dkv_kernel<128>), dim3((unsigned)dkv_blocks), dim3(256), smem_dkv, s, q_, k_,
                               v_, do_, lse, delta_kv, key_bias, static_cast<bf16_t*>(dk), static_cast<bf16_t*>(dv), Hq, Hkv, L,
                               Lk, scale, ex);
        }
    } else {
        constexpr int smem_dq = 4 * kDqBN * 64 * 2 + 2 * kDqBN * 4;
        constexpr int smem_dkv = 4 * kDkvBQ * 64 * 2 + 4 * kDkvBQ * 4 + kBwdRows * (64 * 2 + 16);
        if (extras) {
            hipLaunchKernelGGL((attention_bwd_dq_kernel<64, false, true>), dim3((unsigned)dq_blocks), dim3(256), smem_dq, s,
                               q_, k_, v_, do_, lse, delta, key_bias, static_cast<bf16_t*>(dq), Hq, Hkv, L, Lk, scale, B, ex, out_, delta_ws);
            hipLaunchKernelGGL((attention_bwd_dkv_kernel<64, true>), dim3((unsigned)dkv_blocks), dim3(256), smem_dkv, s, q_,
                               k_, v_, do_, lse, delta_kv, key_bias, static_cast<bf16_t*>(dk), static_cast<bf16_t*>(dv), Hq, Hkv,
                               L, Lk, scale, ex);
        } else {
            if (key_bias)
                hipLaunchKernelGGL((attention_bwd_dq_kernel<64, true>), dim3((unsigned)dq_blocks), dim3(256), smem_dq, s, q_,
                                   k_, v_, do_, lse, delta, key_bias, static_cast<bf16_t*>(dq), Hq, Hkv, L, Lk, scale, B, ex, out_, delta_ws);
            else
                hipLaunchKernelGGL((attention_bwd_dq_kernel<64, false>), dim3((unsigned)dq_blocks), dim3(256), smem_dq, s, q_,
                                   k_, v_, do_, lse, delta, key_bias, static_cast<bf16_t*>(dq), Hq, Hkv, L, Lk, scale, B, ex, out_, delta_ws);
            hipLaunchKernelGGL((attention_bwd_dkv_kernel<64>), dim3((unsigned)dkv_blocks), dim3(256), smem_dkv, s, q_, k_, v_,
                               do_, lse, delta_kv, key_bias, static_cast<bf16_t*>(dk), static_cast<bf16_t*>(dv), Hq, Hkv, L, Lk,
                               scale, ex);
        }
    }
    ATS_CHECK_LAUNCH("ats_attention_bwd");
    return ATS_OK;
}

extern "C" int ats_attention_bwd_ex(const void* q, const void* k, const void* v, const void* dout, const float* lse,
                                    const float* delta, const float* key_bias, const float* bias_qk, int64_t bias_sb,
                                    int64_t bias_sh, float dropout_p, uint64_t dropout_seed, void* dq, void* dk, void* dv, int B, int Hq,
                                    int Hkv, int L, int Lk, int D, float scale, ats_stream_t stream) {
    return attention_bwd_launch(q, k, v, nullptr, dout, lse, delta, nullptr, key_bias, bias_qk, bias_sb, bias_sh, dropout_p,
                                dropout_seed, dq, dk, dv, B, Hq, Hkv, L, Lk, D, scale, stream);
}

extern "C" int ats_attention_bwd_out(const void* q, const void* k, const void* v, const void* out, const void* dout,
                                     const float* lse, float* delta_ws, const float* key_bias, const float* bias_qk,
                                     int64_t bias_sb, int64_t bias_sh, float dropout_p, uint64_t dropout_seed, void* dq,
                                     void* dk, void* dv, int B, int Hq, int Hkv, int L, int Lk, int D, float scale,
                                     ats_stream_t stream) {
    ATS_REQUIRE(out != nullptr || B == 0 || L == 0, ATS_ERR_INVALID_ARG, "ats_attention_bwd_out: null pointer");
    return attention_bwd_launch(q, k, v, out, dout, lse, nullptr, delta_ws, key_bias, bias_qk, bias_sb, bias_sh, dropout_p,
                                dropout_seed, dq, dk, dv, B, Hq, Hkv, L, Lk, D, scale, stream);
}

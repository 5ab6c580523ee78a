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
// which is legal because the contraction over keys is a sum.  V stays as it is in memory ([key][d], any
// batch / position / head strides) all the way into LDS; the V^T fragments come out of LDS through the
// transposing read ds_read_b64_tr_b16, so no transposed copy of V is ever made.
//
// Two bodies share this layout: attention_q_tile_pipe (whole key range; the prefill / training path) loads
// K and V straight into LDS and overlaps the score MFMAs of the next key tile with the softmax of the
// current one inside every wave; attention_q_tile (a key range of a split, for decoding against a long
// cache) keeps the simpler schedule with loads through registers.
#include <math.h>

#include <type_traits>

#include "ats_common.hpp"
#include "attention_extra.hpp"

namespace ats {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 abf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float af32x16_t;
typedef unsigned int au32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int au32x2_t __attribute__((ext_vector_type(2)));
typedef short att_tr_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) att_tr_t* att_lds_tr_ptr_t;

// A block is NT threads = 4 or 8 waves of 32 query rows each.  Four waves (two blocks per CU) for ordinary
// lengths; eight waves share a K/V tile between twice the rows, which pays on long sequences (measured at
// 8192 positions: 1095 vs 1170 us; at 2048: 341 vs 346 us).
constexpr int kAttBN = 64;    // keys per tile
constexpr int att_rows_per_block(int nt) { return nt / 64 * 32; }

// Exchange with the lane 32 positions away by one VALU swap of the wave's halves (v_permlane32_swap) instead of a
// shuffle through the LDS crossbar, whose result a wave can only wait for together with every fragment read it
// has in flight.  All 64 lanes must be active.  Same bits as the shuffle forms (max and sum are symmetric).
__device__ __forceinline__ float xor32_max(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xor32_sum(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ af32x16_t att_mma(const au32x4_t& a, const au32x4_t& b, af32x16_t c) {
    union {
        au32x4_t u;
        abf16x8_t v;
    } x, y;
    x.u = a;
    y.u = b;
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(x.v, y.v, c, 0, 0, 0);
}

// One tile of query rows (32 per wave) against its visible keys.  The rows are the queries of one
// (batch, query head), or -- `pack` -- the queries of all query heads of one (batch, kv head), position
// major: row r is position r / rep of head hkv * rep + r % rep.  Packing fills the tile when there are few
// positions (decoding against a cache: one position, rep rows instead of one).
// SPLIT: the tile sees the keys [key_first, key_first + key_count) only (key_first a multiple of the key tile,
// at or before every query's position, so each row keeps a visible key) and leaves its unnormalised output,
// running maximum and sum in part_out for attention_merge_kernel: rows of D + 4 floats at
// ((b * Hq + hq) * L + position) * n_parts + part.
constexpr int kPartPad = 4;
// EXTRA: a bias per (query, key) pair and / or dropout on the weights (attention_extra.hpp); the bias is read
// from memory in accumulator order (no LDS staging: this is the seldom-used path).
template <int D, bool BIAS, int NT, bool SPLIT = false, bool EXTRA = false>
__device__ __forceinline__ void attention_q_tile(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                                                 int64_t k_sb, int64_t k_sh,
                                                 const bf16_t* __restrict__ v, int64_t v_sb, int v_sl, int64_t v_sh,
                                                 const float* __restrict__ key_bias, bf16_t* __restrict__ out,
                                                 float* __restrict__ lse, int Hq, int Hkv, int L, int Lk,
                                                 float scale_log2, int qt, int head, int b, bool pack,
                                                 unsigned char* smem, float* __restrict__ part_out = nullptr,
                                                 int part = 0, int n_parts = 1, int key_first = 0, int key_count = 0,
                                                 const AttnExtra* ex = nullptr) {
    static_assert(!(EXTRA && (SPLIT || BIAS)), "the extras come alone: a per-key bias is folded into the pair bias");
    constexpr int kAttThreads = NT;
    constexpr int kAttBM = att_rows_per_block(NT);
    constexpr int KS = D / 16;              // k-steps of the score product
    constexpr int DB = D / 32;              // 32-row blocks of the output (transposed)
    constexpr int KPITCH = D * 2 + 16;      // bytes per K row in LDS
    constexpr int VPITCH = D * 2 + 64;      // bytes per V row in LDS (see the transposing read below)
    constexpr int KTILE = kAttBN * KPITCH;
    constexpr int VTILE = kAttBN * VPITCH;
    constexpr int KVEC = kAttBN * (D / 8) / kAttThreads;   // 16-byte vectors per thread for a K tile
    constexpr int VVEC = KVEC;                             // and for a V tile
    // smem: [2 stages][K tile | V tile]
#define ATT_SK(stage_) (smem + (stage_) * (KTILE + VTILE))
#define ATT_SV(stage_) (smem + (stage_) * (KTILE + VTILE) + KTILE)
    // optional additive bias per key (a padding mask), in log2 units: [2 stages][64] floats behind the tiles
    float* const s_bias = reinterpret_cast<float*>(smem + 2 * (KTILE + VTILE));
    const float* bias_row = BIAS ? key_bias + (int64_t)b * Lk + (SPLIT ? key_first : 0) : nullptr;
    // Query i sits at position i + (Lk - L): with cached keys in front the causal diagonal moves right.
    const int off = Lk - L - (SPLIT ? key_first : 0);
    if constexpr (SPLIT) Lk = key_count;      // from here on: the keys of this part, counted from its first
    constexpr bool has_bias = BIAS;
    // with a bias the scores are brought to log2 units before the maximum is taken (sc = 1 afterwards)
    const float sc = (has_bias || EXTRA) ? 1.0f : scale_log2;
    float r_bias = 0.f;

    const int rep = Hq / Hkv;
    const int rp = pack ? rep : 1;                  // rows per position
    const int n_rows = L * rp;
    const int hkv = pack ? head : head / rep;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, g = lane >> 5;
    const int row = qt * kAttBM + wave * 32 + col;            // this lane's row
    const int row_clamped = row < n_rows ? row : n_rows - 1;
    const int q_clamped = row_clamped / rp;                   // its position among the queries
    const int hq = pack ? hkv * rep + row_clamped % rp : head;
    const bool row_valid = row < n_rows;

    const bf16_t* qp = q + ((int64_t)(b * Hq + hq) * L + q_clamped) * D;
    const bf16_t* kbase = k + b * k_sb + hkv * k_sh + (SPLIT ? (int64_t)key_first * D : 0);     // rows of D elements
    const bf16_t* vbase = v + b * v_sb + hkv * v_sh + (SPLIT ? (int64_t)key_first * v_sl : 0);  // key j at + j * v_sl

    au32x4_t qf[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const au32x4_t*>(qp + s * 16 + g * 8);

    // extras: this lane's row of the pair bias (a buffer descriptor over the batch entry's [L, Lk] matrix, so
    // keys past Lk read as zeros) and the dropout key of this (batch, head)
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

    // K and V^T tiles come through buffer loads: a scalar base and tile offset plus one 32-bit lane offset
    // that never changes, so a tile costs no address arithmetic, and keys past Lk read as zeros.
    const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(kbase), 0, (int)((int64_t)Lk * D * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(vbase), 0, (int)((((int64_t)Lk - 1) * v_sl + D) * 2), 0x00020000);
    int k_lane[KVEC], v_lane[VVEC];
#pragma unroll
    for (int i = 0; i < KVEC; ++i) {
        const int idx = tid + i * kAttThreads;
        k_lane[i] = ((idx / (D / 8)) * D + (idx % (D / 8)) * 8) * 2;
    }
#pragma unroll
    for (int i = 0; i < VVEC; ++i) {
        const int idx = tid + i * kAttThreads;
        v_lane[i] = ((idx / (D / 8)) * v_sl + (idx % (D / 8)) * 8) * 2;
    }

    af32x16_t acc_o[DB];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc_o[d][v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    const int q_pos = row / rp + off;                           // last key this lane's query sees
    const int q_block_last = min(qt * kAttBM + kAttBM - 1, n_rows - 1) / rp + off;
    const int n_tiles = SPLIT ? min(q_block_last / kAttBN + 1, (Lk + kAttBN - 1) / kAttBN) : q_block_last / kAttBN + 1;
    const int q_wave_first = (qt * kAttBM + wave * 32) / rp + off;
    // a wave without rows (packed tiles of a short batch) only helps to load
    const int q_wave_last = qt * kAttBM + wave * 32 < n_rows ? (qt * kAttBM + wave * 32 + 31) / rp + off : -1;

    // One barrier per key tile: tile t+1 travels global -> registers while tile t is computed and lands in
    // the other LDS stage at the end of the iteration.  LDS operand fragments are read kRing MFMAs ahead
    // of their use through a small register ring; without it every MFMA would wait a full LDS round trip.
    constexpr int kRing = 6;
    au32x4_t rk[KVEC], rv[VVEC];
    au32x4_t ring[kRing];
    af32x16_t acc_s[2];

    {   // tile 0 -> stage 0
#pragma unroll
        for (int i = 0; i < KVEC; ++i) rk[i] = __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, k_lane[i], 0, 0);
#pragma unroll
        for (int i = 0; i < VVEC; ++i) rv[i] = __builtin_amdgcn_raw_buffer_load_b128(v_rsrc, v_lane[i], 0, 0);
#pragma unroll
        for (int i = 0; i < KVEC; ++i) {
            const int idx = tid + i * kAttThreads;
            const int r = idx / (D / 8), c = idx % (D / 8);
            *reinterpret_cast<au32x4_t*>(ATT_SK(0) + r * KPITCH + c * 16) = rk[i];
        }
#pragma unroll
        for (int i = 0; i < VVEC; ++i) {
            const int idx = tid + i * kAttThreads;
            const int r = idx / (D / 8), c = idx % (D / 8);
            *reinterpret_cast<au32x4_t*>(ATT_SV(0) + r * VPITCH + c * 16) = rv[i];
        }
        if (has_bias && tid < kAttBN) s_bias[tid] = tid < Lk ? bias_row[tid] * 1.4426950408889634f : 0.f;
        __syncthreads();
    }

    // Pin the query fragments here: loads left pending into the loop make the compiler's wait-count
    // bookkeeping hold every score MFMA of every iteration behind that iteration's global loads.
#pragma unroll
    for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(qf[s]));

    for (int t = 0; t < n_tiles; ++t) {
        const int n0 = t * kAttBN;
        const unsigned char* sk = ATT_SK(t & 1);
        const unsigned char* sv = ATT_SV(t & 1);
        const bool has_next = t + 1 < n_tiles;
        // The loads of the next tile are issued one at a time between the MFMAs of the score product: all
        // waves of a CU leave the barrier together, and 8 loads per wave issued back to back queue up behind
        // the CU's one address unit while no wave can reach its MFMAs.
        const int n1 = n0 + kAttBN;
        if (has_bias && has_next && tid < kAttBN) r_bias = n1 + tid < Lk ? bias_row[n1 + tid] * 1.4426950408889634f : 0.f;
#define ATT_LOAD_ONE(i_)                                                                               \
    {                                                                                                  \
        if ((i_) < KVEC)                                                                               \
            rk[(i_) < KVEC ? (i_) : 0] =                                                               \
                __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, k_lane[(i_) < KVEC ? (i_) : 0], n1 * D * 2, 0); \
        else                                                                                           \
            rv[(i_) < KVEC ? 0 : (i_) - KVEC] = __builtin_amdgcn_raw_buffer_load_b128(                 \
                v_rsrc, v_lane[(i_) < KVEC ? 0 : (i_) - KVEC], n1 * v_sl * 2, 0);                      \
    }
        constexpr int NLOAD = KVEC + VVEC;
        constexpr int LOAD_EVERY = 2 * KS / NLOAD;
        static_assert(LOAD_EVERY >= 1 && LOAD_EVERY * NLOAD == 2 * KS, "one load per LOAD_EVERY score MFMAs");
        if (has_next && n0 > q_wave_last) {   // this wave skips the tile's arithmetic but still loads its share
#pragma unroll
            for (int i = 0; i < NLOAD; ++i) ATT_LOAD_ONE(i);
        }

        if (n0 <= q_wave_last) {   // some key of the tile is visible to this wave
            // ---- S^T = K . Q^T: fragment f = (k-step f/2, key block f%2)
            const unsigned char* kr = sk + col * KPITCH + g * 16;
#define ATT_KFRAG(f_) (*reinterpret_cast<const au32x4_t*>(kr + ((f_) & 1) * 32 * KPITCH + ((f_) >> 1) * 32))
#pragma unroll
            for (int f = 0; f < kRing; ++f) ring[f] = ATT_KFRAG(f);
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc_s[kb][v] = 0.f;
#pragma unroll
            for (int f = 0; f < 2 * KS; ++f) {
                acc_s[f & 1] = att_mma(ring[f % kRing], qf[f >> 1], acc_s[f & 1]);
                if (f + kRing < 2 * KS) ring[f % kRing] = ATT_KFRAG(f + kRing);
                if (has_next && f % LOAD_EVERY == LOAD_EVERY - 1) ATT_LOAD_ONE(f / LOAD_EVERY);
                __builtin_amdgcn_sched_barrier(0);   // keep the reads kRing fragments ahead of their use
            }
#undef ATT_KFRAG
#undef ATT_LOAD_ONE
            // First fragments of V^T travel during the softmax: fragment f = (k-step f/DB, output block f%DB).
            // V sits in LDS as it does in memory ([key][d]); the A operand wants, per lane, one d and eight
            // keys.  ds_read_b64_tr_b16 does 4x4 transposes inside groups of 16 lanes: the four lanes
            // r = a + 4j (j = 0..3) each point at 4 consecutive d of key j, and lane 4a + c receives element
            // c of all four, i.e. d = 4a + c for 4 consecutive keys.  With the addresses below lane l ends up
            // with d = l % 32 and keys 4g .. 4g+3 (first read) and 8+4g .. 8+4g+3 (second read) of the
            // k-step, which is the key order P^T has as the B operand.  The row pitch of D*2+64 bytes puts
            // the 4 keys of a read 16 banks apart.
            const unsigned char* vr =
                sv + (4 * (lane >> 5) + ((lane & 15) >> 2)) * VPITCH + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
#define ATT_VFRAG(f_, dst_)                                                                            \
    {                                                                                                  \
        const unsigned char* p_ = vr + (((f_) / DB) * 16) * VPITCH + ((f_) % DB) * 64;                 \
        const att_tr_t lo_ = __builtin_amdgcn_ds_read_tr16_b64_v4i16((att_lds_tr_ptr_t)(p_));           \
        const att_tr_t hi_ = __builtin_amdgcn_ds_read_tr16_b64_v4i16((att_lds_tr_ptr_t)(p_ + 8 * VPITCH)); \
        union { att_tr_t t[2]; au32x4_t u; } cv_;                                                     \
        cv_.t[0] = lo_; cv_.t[1] = hi_;                                                                \
        dst_ = cv_.u;                                                                                  \
    }
#pragma unroll
            for (int f = 0; f < kRing; ++f) ATT_VFRAG(f, ring[f]);
            __builtin_amdgcn_sched_barrier(0);

            if (has_bias) {   // scores to log2 units plus the key's bias; accumulator value x of block kb is key
                              // kb*32 + (x/4)*8 + g*4 + x%4 of the tile
                const float* bt = s_bias + (t & 1) * kAttBN + g * 4;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float4 b4 = *reinterpret_cast<const float4*>(bt + kb * 32 + r * 8);
                        acc_s[kb][r * 4 + 0] = __builtin_fmaf(acc_s[kb][r * 4 + 0], scale_log2, b4.x);
                        acc_s[kb][r * 4 + 1] = __builtin_fmaf(acc_s[kb][r * 4 + 1], scale_log2, b4.y);
                        acc_s[kb][r * 4 + 2] = __builtin_fmaf(acc_s[kb][r * 4 + 2], scale_log2, b4.z);
                        acc_s[kb][r * 4 + 3] = __builtin_fmaf(acc_s[kb][r * 4 + 3], scale_log2, b4.w);
                    }
            }
            if constexpr (EXTRA) {   // scores to log2 units plus the pair bias of (this lane's query, key)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    float bq[16];
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int key = n0 + kb * 32 + (v >> 2) * 8 + g * 4 + (v & 3);
                        bq[v] = ex_bias ? __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                              pb_rsrc, pb_row + key * 4, 0, 0))
                                        : 0.f;
                    }
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        acc_s[kb][v] = __builtin_fmaf(acc_s[kb][v], scale_log2, bq[v] * 1.4426950408889634f);
                }
            }
            if (n0 + kAttBN - 1 > q_wave_first) {   // diagonal tile: causal mask
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int key = n0 + kb * 32 + (v >> 2) * 8 + g * 4 + (v & 3);
                        if (key > q_pos) acc_s[kb][v] = -INFINITY;
                    }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) mx = fmaxf(mx, acc_s[kb][v]);
            mx = xor32_max(mx);
            // The reference point of the exponentials follows the running maximum lazily: it moves only when
            // the maximum has grown by more than kLazy (log2 units), so p <= 2^kLazy, which float32 sums and
            // bf16 operands hold without loss of relative precision, and the rescaling of the output
            // accumulator (64 multiplies per lane) becomes rare; the result l and o / l is the same quantity.
            constexpr float kLazy = 8.0f;
            const float m_cand = fmaxf(m_run, mx * sc);   // a positive factor keeps the order
            const float m_new = m_cand - m_run > kLazy ? m_cand : m_run;   // -inf on the first tile: moves
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);   // 0 on the first tile
            float psum = 0.f;
            // p = exp2(s * c - m * c): one fused multiply-add per element, c = scale * log2(e)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(acc_s[kb][v], sc, -m_new));
                    acc_s[kb][v] = p;
                    psum += p;
                }
            l_run = l_run * alpha + psum;
            m_run = m_new;
            if (!__all(alpha == 1.0f)) {   // the running maximum moved for some row of this wave
#pragma unroll
                for (int d = 0; d < DB; ++d)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc_o[d][v] *= alpha;
            }
            if constexpr (EXTRA) {   // dropout acts on the weights that meet V; the row sum keeps all of them
                if (ex_drop) {
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int key = n0 + kb * 32 + (v >> 2) * 8 + g * 4 + (v & 3);
                            const bool keep = attn_drop_hash(head_key, drop_counter0 + (uint32_t)key) >= ex->drop_threshold;
                            acc_s[kb][v] = keep ? acc_s[kb][v] * ex->keep_scale : 0.f;
                        }
                }
            }
            // P^T as B operand: k-step s holds accumulator values 8*(s&1) .. +7 of key block s>>1
            au32x4_t pf[4];
#pragma unroll
            for (int s_ = 0; s_ < 4; ++s_) {
                const int kb = s_ >> 1, v0 = (s_ & 1) * 8;
                pf[s_].x = pack_bf16x2(acc_s[kb][v0 + 0], acc_s[kb][v0 + 1]);
                pf[s_].y = pack_bf16x2(acc_s[kb][v0 + 2], acc_s[kb][v0 + 3]);
                pf[s_].z = pack_bf16x2(acc_s[kb][v0 + 4], acc_s[kb][v0 + 5]);
                pf[s_].w = pack_bf16x2(acc_s[kb][v0 + 6], acc_s[kb][v0 + 7]);
            }
            // ---- O^T += V^T . P^T
#pragma unroll
            for (int f = 0; f < 4 * DB; ++f) {
                acc_o[f % DB] = att_mma(ring[f % kRing], pf[f / DB], acc_o[f % DB]);
                if (f + kRing < 4 * DB) ATT_VFRAG(f + kRing, ring[f % kRing]);
                __builtin_amdgcn_sched_barrier(0);
            }
#undef ATT_VFRAG
        }

        if (has_next) {   // stage (t+1)&1 was last read in iteration t-1, before its closing barrier
            if (has_bias && tid < kAttBN) s_bias[((t + 1) & 1) * kAttBN + tid] = r_bias;
            unsigned char* dk = ATT_SK((t + 1) & 1);
            unsigned char* dv = ATT_SV((t + 1) & 1);
#pragma unroll
            for (int i = 0; i < KVEC; ++i) {
                const int idx = tid + i * kAttThreads;
                const int r = idx / (D / 8), c = idx % (D / 8);
                *reinterpret_cast<au32x4_t*>(dk + r * KPITCH + c * 16) = rk[i];
            }
#pragma unroll
            for (int i = 0; i < VVEC; ++i) {
                const int idx = tid + i * kAttThreads;
                const int r = idx / (D / 8), c = idx % (D / 8);
                *reinterpret_cast<au32x4_t*>(dv + r * VPITCH + c * 16) = rv[i];
            }
        }
        __syncthreads();
    }

    l_run = xor32_sum(l_run);
    if constexpr (SPLIT) {
        if (row_valid) {
            float* prow = part_out + ((((int64_t)b * Hq + hq) * L + q_clamped) * n_parts + part) * (D + kPartPad);
#pragma unroll
            for (int d = 0; d < DB; ++d)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    *reinterpret_cast<float4*>(prow + d * 32 + r * 8 + g * 4) =
                        make_float4(acc_o[d][r * 4 + 0], acc_o[d][r * 4 + 1], acc_o[d][r * 4 + 2], acc_o[d][r * 4 + 3]);
            if (g == 0) {
                prow[D] = m_run;
                prow[D + 1] = l_run;
            }
        }
        return;
    }
    // ---- normalise and write [B, L, Hq*D]
    const float inv = 1.0f / l_run;
    if (row_valid) {
        bf16_t* orow = out + ((int64_t)b * L + q_clamped) * (int64_t)(Hq * D) + hq * D;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                au32x2_t w;
                w.x = pack_bf16x2(acc_o[d][r * 4 + 0] * inv, acc_o[d][r * 4 + 1] * inv);
                w.y = pack_bf16x2(acc_o[d][r * 4 + 2] * inv, acc_o[d][r * 4 + 3] * inv);
                *reinterpret_cast<au32x2_t*>(orow + d * 32 + r * 8 + g * 4) = w;
            }
        if (lse && g == 0) lse[(int64_t)(b * Hq + hq) * L + q_clamped] = (m_run + log2f(l_run)) * 0.6931471805599453f;
    }
#undef ATT_SK
#undef ATT_SV
}

// Order of the MFMAs of one iteration of attention_q_tile_pipe.  NS score MFMAs (tile t+1) and 4 * DB output
// MFMAs (tile t; DB per group of 16 keys) are dealt into four groups and a tail:
//     group 0: NS/4 score MFMAs;   group g = 1..3: NS/4 score MFMAs, then the DB output MFMAs of key group g-1;
//     tail: the DB output MFMAs of key group 3.
// The exponentials of key group g are computed during group g, so the output MFMAs of a key group always find
// their probabilities ready.
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

template <int NS, int DB>
struct PipeSeq {
    static constexpr int SPG = NS / 4;
    static constexpr int GS = SPG + DB;     // slots of groups 1..3
    static_assert(SPG * 4 == NS && 8 % SPG == 0 && 8 % GS == 0, "slots per group must divide the 8 elements of a key group");
    static constexpr int group(int u) { return u < SPG ? 0 : 1 + (u - SPG) / GS; }      // 4 = tail
    static constexpr int slot_in_group(int u) { return u < SPG ? u : (u - SPG) % GS; }
    static constexpr int group_slots(int g) { return g == 0 ? SPG : GS; }
    static constexpr bool is_s(int u) { return group(u) < 4 && slot_in_group(u) < SPG; }
    static constexpr int idx(int u) {
        return is_s(u) ? group(u) * SPG + slot_in_group(u)
                       : (group(u) < 4 ? (group(u) - 1) * DB + slot_in_group(u) - SPG : 3 * DB + (u - SPG - 3 * GS));
    }
};

// Software-pipelined variant of attention_q_tile (same arguments and results, without the key-range split).
//
// A wave's two units have about the same amount of work per key tile at head_dim 128: ~1000 cycles of MFMA
// (score and output products) and ~900 cycles of vector ALU (32 exponentials per lane at a quarter rate, the
// maximum, the sum, the conversion).  In attention_q_tile the two alternate inside a wave and overlap only
// by the luck of the other wave on the SIMD being in the other phase.  Here the score product of tile t+1
// is issued between the softmax instructions of tile t, so every wave keeps both units busy by itself:
//     iteration t:   S(t+1) = K(t+1) . Q^T  interleaved with  P(t) = softmax step of S(t)
//                    O^T   += V(t)^T . P(t)^T
// which takes a second score accumulator (32 registers).  The registers come from the loads: K and V tiles
// go from memory straight into LDS (buffer_load_dwordx4 ... lds, lane l of an instruction deposits its 16
// bytes at M0 + 16 l), so no tile passes through registers and no ds_write is issued.  Such a load writes
// 1 KiB of consecutive LDS, so rows cannot be padded; bank conflicts are avoided by an XOR swizzle applied on
// the global side instead (which 16-byte chunk of a row a lane fetches):
//     K: slot s of row r holds chunk s ^ fK(r); the 16 rows that a quarter wave reads with ds_read_b128 hit
//        16 different slots (fK(r) = r % 16 for 256-byte rows; (r / 2) % 8 for 128-byte rows, where two rows
//        share a 256-byte line),
//     V: the transposing read takes 64 consecutive bytes from each of 4 consecutive rows per half wave; the
//        64-byte group index is XORed with fV(r) (r % 4, or (r / 2) % 2 for 128-byte rows), so the four rows
//        land on four different groups of 16 banks.
// K runs one tile ahead of V: at the start of iteration t the loads of K(t+2) and V(t+1) are issued into the
// stages that K(t) and V(t-1) occupied (everybody was done with them at the barrier that ended iteration
// t-1) and have the whole iteration to land; two stages each, 4 x 16 KiB at head_dim 128.
template <int D, bool BIAS, int NT>
__device__ __forceinline__ void attention_q_tile_pipe(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                                                      int64_t k_sb, int64_t k_sh, const bf16_t* __restrict__ v,
                                                      int64_t v_sb, int v_sl, int64_t v_sh,
                                                      const float* __restrict__ key_bias, bf16_t* __restrict__ out,
                                                      float* __restrict__ lse, int Hq, int Hkv, int L, int Lk,
                                                      float scale_log2, int qt, int head, int b, bool pack,
                                                      unsigned char* smem) {
    typedef __attribute__((address_space(3))) void* lds_ptr_t;
    typedef __attribute__((address_space(3))) unsigned char* lds_u8_t;
    typedef __attribute__((address_space(3))) au32x4_t* lds_v4_t;
    typedef __attribute__((address_space(3))) float* lds_f32_t;
    typedef float att_f32x4_t __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) att_f32x4_t* lds_f32x4_t;
    const lds_u8_t sm = (lds_u8_t)smem;     // every LDS access below goes through this typed base
    constexpr int NW = NT / 64;
    constexpr int kAttBM = att_rows_per_block(NT);
    constexpr int KS = D / 16;              // k-steps of the score product
    constexpr int DB = D / 32;              // 32-row blocks of the output (transposed)
    constexpr int ROWB = D * 2;             // bytes per K or V row in LDS
    constexpr int CPR = D / 8;              // 16-byte chunks per row
    constexpr int TILE = kAttBN * ROWB;
    constexpr int NI = TILE / 1024 / NW;    // load instructions per wave for a K tile (and for a V tile)
    static_assert(NI >= 1 && NI * NW * 1024 == TILE, "loader tiling");
    constexpr int NS = 2 * KS;              // score MFMAs per tile
    constexpr int NO = 4 * DB;              // output MFMAs per tile
    constexpr int kRing = (BIAS && D == 128) ? 4 : 6;   // the bias variant needs the registers
    static_assert(kRing <= NO, "the fragment ring runs through both products");
    using SEQ = PipeSeq<NS, DB>;
    // LDS map: [K stage 0][K stage 1][V stage 0][V stage 1][bias: 2 x 64 floats]
    constexpr int V_BASE = 2 * TILE;
    const lds_f32_t s_bias = (lds_f32_t)(sm + 4 * TILE);
    const float* bias_row = BIAS ? key_bias + (int64_t)b * Lk : nullptr;
    const int off = Lk - L;                 // query i sits at position i + (Lk - L)
    constexpr bool has_bias = BIAS;
    const float sc = has_bias ? 1.0f : scale_log2;
    float r_bias = 0.f;

    const int rep = Hq / Hkv;
    const int rp = pack ? rep : 1;
    const int n_rows = L * rp;
    const int hkv = pack ? head : head / rep;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, g = lane >> 5;
    const int row = qt * kAttBM + wave * 32 + col;
    const int row_clamped = row < n_rows ? row : n_rows - 1;
    const int q_clamped = row_clamped / rp;
    const int hq = pack ? hkv * rep + row_clamped % rp : head;
    const bool row_valid = row < n_rows;

    const bf16_t* qp = q + ((int64_t)(b * Hq + hq) * L + q_clamped) * D;
    const bf16_t* kbase = k + b * k_sb + hkv * k_sh;
    const bf16_t* vbase = v + b * v_sb + hkv * v_sh;

    au32x4_t qf[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const au32x4_t*>(qp + s * 16 + g * 8);

    const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(kbase), 0, (int)((int64_t)Lk * D * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(vbase), 0, (int)((((int64_t)Lk - 1) * v_sl + D) * 2), 0x00020000);
    // load instruction j of this wave fills LDS positions (j * NW + wave) * 64 + lane (16-byte units) of a stage
    int k_off[NI], v_off[NI];
#pragma unroll
    for (int j = 0; j < NI; ++j) {
        const int p = (j * NW + wave) * 64 + lane;
        const int r = p / CPR, s = p % CPR;
        const int fk = D == 128 ? (r & 15) : ((r >> 1) & 7);
        const int fv = D == 128 ? (r & 3) : ((r >> 1) & 1);
        k_off[j] = (r * D + (s ^ fk) * 8) * 2;
        v_off[j] = (r * v_sl + (s ^ (fv << 2)) * 8) * 2;
    }
#define PIPE_LOAD_K(tile_, stage_)                                                                     \
    _Pragma("unroll") for (int j_ = 0; j_ < NI; ++j_) __builtin_amdgcn_raw_ptr_buffer_load_lds(        \
        k_rsrc, (lds_ptr_t)(sm + (stage_) * TILE + (j_ * NW + wave) * 1024), 16, k_off[j_],            \
        (tile_) * (kAttBN * D * 2), 0, 0)
#define PIPE_LOAD_V(tile_, stage_)                                                                     \
    _Pragma("unroll") for (int j_ = 0; j_ < NI; ++j_) __builtin_amdgcn_raw_ptr_buffer_load_lds(        \
        v_rsrc, (lds_ptr_t)(sm + V_BASE + (stage_) * TILE + (j_ * NW + wave) * 1024), 16, v_off[j_],   \
        (tile_) * kAttBN * v_sl * 2, 0, 0)
    // Keys past Lk: their V rows must be zeros in LDS (their probabilities are exact zeros, but 0 x NaN is
    // not); each lane clears the positions its own loads address, after those loads have landed.
#define PIPE_CLEAR_V_TAIL(tile_, stage_)                                                               \
    if (((tile_) + 1) * kAttBN > Lk) {                                                                 \
        _Pragma("unroll") for (int j_ = 0; j_ < NI; ++j_) {                                            \
            const int p_ = (j_ * NW + wave) * 64 + lane;                                               \
            if ((tile_) * kAttBN + p_ / CPR >= Lk)                                                     \
                *(lds_v4_t)(sm + V_BASE + (stage_) * TILE + p_ * 16) = au32x4_t{0u, 0u, 0u, 0u};       \
        }                                                                                              \
    }

    // fragment addresses (byte offsets into smem, stage and fragment row blocks added as constants)
    int k_addr[KS], v_addr[DB];
    {
        const int fk = D == 128 ? (col & 15) : ((col >> 1) & 7);
#pragma unroll
        for (int s = 0; s < KS; ++s) k_addr[s] = col * ROWB + (((2 * s + g) ^ fk) * 16);
        const int rr = 4 * g + ((lane & 15) >> 2);
        const int fv = D == 128 ? (rr & 3) : ((rr >> 1) & 1);
        const int within = 32 * ((lane >> 4) & 1) + 8 * (lane & 3);
#pragma unroll
        for (int d = 0; d < DB; ++d) v_addr[d] = V_BASE + rr * ROWB + ((d ^ fv) * 64) + within;
    }
    // fragment f of the score product = (k-step f/2, key block f%2); fragment f of the output product =
    // (k-step f/DB, output block f%DB), read transposed (see attention_q_tile for the lane arithmetic)
#define PIPE_KFRAG(stage_, f_, dst_)                                                                   \
    dst_ = *(lds_v4_t)(sm + k_addr[(f_) >> 1] + (stage_) * TILE + ((f_) & 1) * 32 * ROWB)
#define PIPE_VFRAG(stage_, f_, dst_)                                                                   \
    {                                                                                                  \
        const lds_u8_t p_ = sm + v_addr[(f_) % DB] + (stage_) * TILE + ((f_) / DB) * 16 * ROWB;        \
        const att_tr_t lo_ = __builtin_amdgcn_ds_read_tr16_b64_v4i16((att_lds_tr_ptr_t)(p_));           \
        const att_tr_t hi_ = __builtin_amdgcn_ds_read_tr16_b64_v4i16((att_lds_tr_ptr_t)(p_ + 8 * ROWB)); \
        union { att_tr_t t[2]; au32x4_t u; } cv_;                                                     \
        cv_.t[0] = lo_; cv_.t[1] = hi_;                                                                \
        dst_ = cv_.u;                                                                                  \
    }
    af32x16_t acc_o[DB];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int x = 0; x < 16; ++x) acc_o[d][x] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    const int q_pos = row / rp + off;
    const int q_block_last = min(qt * kAttBM + kAttBM - 1, n_rows - 1) / rp + off;
    const int n_tiles = q_block_last / kAttBN + 1;
    const int q_wave_first = (qt * kAttBM + wave * 32) / rp + off;
    const int q_wave_last = qt * kAttBM + wave * 32 < n_rows ? (qt * kAttBM + wave * 32 + 31) / rp + off : -1;
    const int my_tiles = q_wave_last >= 0 ? min(q_wave_last / kAttBN + 1, n_tiles) : 0;   // tiles this wave computes

    au32x4_t ring[kRing];
    af32x16_t acc_sa[2], acc_sb[2];
    au32x4_t pf[4];

    // ---- prologue: K(0), V(0), K(1) land; S(0)
    PIPE_LOAD_K(0, 0);
    PIPE_LOAD_V(0, 0);
    if (n_tiles > 1) PIPE_LOAD_K(1, 1);
    if (has_bias && tid < kAttBN) s_bias[tid] = tid < Lk ? bias_row[tid] * 1.4426950408889634f : 0.f;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    PIPE_CLEAR_V_TAIL(0, 0)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
    for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(qf[s]));
    if (my_tiles > 0) {
#pragma unroll
        for (int f = 0; f < kRing; ++f) PIPE_KFRAG(0, f, ring[f]);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int x = 0; x < 16; ++x) acc_sa[kb][x] = 0.f;
#pragma unroll
        for (int f = 0; f < NS; ++f) {
            acc_sa[f & 1] = att_mma(ring[f % kRing], qf[f >> 1], acc_sa[f & 1]);
            if (f + kRing < NS) PIPE_KFRAG(0, f + kRing, ring[f % kRing]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // every wave is done with K stage 0 before K(2) may land there
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    // Iteration t with PAR = t % 2: S(t) is in CUR, S(t+1) goes to NXT; K(t+1) sits in K stage PAR^1, V(t) in V
    // stage PAR; K(t+2) is loaded into K stage PAR, V(t+1) into V stage PAR^1.
    // The 64 keys of a tile form four groups of 16 (one k-step of the output product each).  After the row
    // maximum is known, the iteration runs through NS + NO MFMA slots in the order given by PipeSeq: group g
    // holds a quarter of the score MFMAs of tile t+1 and the output MFMAs of key group g-1 of tile t, and behind
    // every MFMA comes a share of the exponentials of key group g; so MFMAs and vector instructions alternate
    // through the whole iteration, and a wave that has to wait for the matrix pipe (the other wave of the SIMD
    // is using it) is never more than one MFMA behind with its vector work.  The stretch runs at raised wave
    // priority (s_setprio 1; back to 0 behind it): the other wave of the SIMD, which belongs to another workgroup
    // and is usually somewhere else in its iteration, then yields while it is in its vector-only parts (mask, row
    // maximum, rescaling): 315 -> 309 us at batch 8 x 2048 positions (priority 3: 311; raising the vector-only
    // parts instead: no gain).
#define PIPE_SLOT_FRAG(kstage_, vstage_, u_, dst_)                                                     \
    {                                                                                                  \
        if constexpr (SEQ::is_s(u_)) { PIPE_KFRAG(kstage_, SEQ::idx(u_), dst_); }                      \
        else PIPE_VFRAG(vstage_, SEQ::idx(u_), dst_)                                                   \
    }
#define PIPE_BODY(t_, PAR, CUR, NXT)                                                                   \
    {                                                                                                  \
        const int n0 = (t_) * kAttBN;                                                                  \
        if ((t_) + 2 < n_tiles) PIPE_LOAD_K((t_) + 2, PAR);                           \
        if ((t_) + 1 < n_tiles) PIPE_LOAD_V((t_) + 1, (PAR) ^ 1);                     \
        if (has_bias && (t_) + 1 < n_tiles && tid < kAttBN)                                            \
            r_bias = n0 + kAttBN + tid < Lk ? bias_row[n0 + kAttBN + tid] * 1.4426950408889634f : 0.f; \
        if ((t_) < my_tiles) {                                                                         \
            static_for<0, kRing>([&](auto uc) __attribute__((always_inline)) {                         \
                constexpr int u = decltype(uc)::value;                                                 \
                PIPE_SLOT_FRAG((PAR) ^ 1, PAR, u, ring[u]);                                            \
            });                                                                                        \
            if (has_bias) {                                                                            \
                const lds_f32_t bt = s_bias + (PAR) * kAttBN + g * 4;                                  \
                _Pragma("unroll") for (int kb = 0; kb < 2; ++kb)                                       \
                _Pragma("unroll") for (int r = 0; r < 4; ++r) {                                        \
                    const att_f32x4_t b4 = *(lds_f32x4_t)(bt + kb * 32 + r * 8);                       \
                    CUR[kb][r * 4 + 0] = __builtin_fmaf(CUR[kb][r * 4 + 0], scale_log2, b4.x);         \
                    CUR[kb][r * 4 + 1] = __builtin_fmaf(CUR[kb][r * 4 + 1], scale_log2, b4.y);         \
                    CUR[kb][r * 4 + 2] = __builtin_fmaf(CUR[kb][r * 4 + 2], scale_log2, b4.z);         \
                    CUR[kb][r * 4 + 3] = __builtin_fmaf(CUR[kb][r * 4 + 3], scale_log2, b4.w);         \
                }                                                                                      \
            }                                                                                          \
            if (n0 + kAttBN - 1 > q_wave_first) {                                                      \
                _Pragma("unroll") for (int kb = 0; kb < 2; ++kb)                                       \
                _Pragma("unroll") for (int x = 0; x < 16; ++x) {                                       \
                    const int key = n0 + kb * 32 + (x >> 2) * 8 + g * 4 + (x & 3);                     \
                    if (key > q_pos) CUR[kb][x] = -INFINITY;                                           \
                }                                                                                      \
            }                                                                                          \
            float mx = -INFINITY;                                                                      \
            _Pragma("unroll") for (int kb = 0; kb < 2; ++kb)                                           \
            _Pragma("unroll") for (int x = 0; x < 16; ++x) mx = fmaxf(mx, CUR[kb][x]);                 \
            mx = xor32_max(mx);                                                    \
            const float m_cand = fmaxf(m_run, mx * sc);                                                \
            const float m_new = m_cand - m_run > kLazyMax ? m_cand : m_run;                            \
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);                                 \
            float psum = 0.f;                                                                          \
            if (!__all(alpha == 1.0f)) {                                                               \
                _Pragma("unroll") for (int d = 0; d < DB; ++d)                                         \
                _Pragma("unroll") for (int x = 0; x < 16; ++x) acc_o[d][x] *= alpha;                   \
            }                                                                                          \
            __builtin_amdgcn_sched_barrier(0);                                                         \
            __builtin_amdgcn_s_setprio(1);   /* the MFMA / exponential stretch outranks the other wave's vector-only parts */ \
            static_for<0, NS + NO>([&](auto uc) __attribute__((always_inline)) {                       \
                constexpr int u = decltype(uc)::value;                                                 \
                constexpr int f = SEQ::idx(u);                                                         \
                if constexpr (SEQ::is_s(u)) {                                                          \
                    if constexpr (f < 2) {                                                             \
                        _Pragma("unroll") for (int x = 0; x < 16; ++x) NXT[f & 1][x] = 0.f;            \
                    }                                                                                  \
                    NXT[f & 1] = att_mma(ring[u % kRing], qf[f >> 1], NXT[f & 1]);                     \
                } else {                                                                               \
                    acc_o[f % DB] = att_mma(ring[u % kRing], pf[f / DB], acc_o[f % DB]);               \
                }                                                                                      \
                if constexpr (u + kRing < NS + NO) PIPE_SLOT_FRAG((PAR) ^ 1, PAR, u + kRing, ring[u % kRing]); \
                if constexpr (SEQ::group(u) < 4) {                                                     \
                    constexpr int gq = SEQ::group(u), w = SEQ::slot_in_group(u), n = SEQ::group_slots(gq); \
                    static_for<w * 8 / n, (w + 1) * 8 / n>([&](auto jc) __attribute__((always_inline)) { \
                        constexpr int j = decltype(jc)::value;                                         \
                        constexpr int kb = gq >> 1, x = (gq & 1) * 8 + j;                              \
                        float p = __builtin_amdgcn_exp2f(__builtin_fmaf(CUR[kb][x], sc, -m_new));      \
                        asm volatile("" : "+v"(p));   /* keeps the exponential here, between the MFMAs */ \
                        CUR[kb][x] = p;                                                                \
                        psum += p;                                                                     \
                        if constexpr (j & 1) pf[gq][j >> 1] = pack_bf16x2(CUR[kb][x - 1], p);          \
                    });                                                                                \
                }                                                                                      \
                __builtin_amdgcn_sched_barrier(0);                                                     \
            });                                                                                        \
            __builtin_amdgcn_s_setprio(0);                                                             \
            l_run = l_run * alpha + psum;                                                              \
            m_run = m_new;                                                                             \
        }                                                                                              \
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                               \
        if ((t_) + 1 < n_tiles) {                                                                      \
            PIPE_CLEAR_V_TAIL((t_) + 1, (PAR) ^ 1)                                                     \
            if (has_bias && tid < kAttBN) s_bias[((PAR) ^ 1) * kAttBN + tid] = r_bias;                 \
        }                                                                                              \
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");                                \
    }

    constexpr float kLazyMax = 8.0f;   // see attention_q_tile: the reference point of the exponentials moves lazily
    for (int t = 0; t < n_tiles; t += 2) {
        PIPE_BODY(t, 0, acc_sa, acc_sb)
        if (t + 1 >= n_tiles) break;
        PIPE_BODY(t + 1, 1, acc_sb, acc_sa)
    }
#undef PIPE_BODY
#undef PIPE_SLOT_FRAG
#undef PIPE_VFRAG
#undef PIPE_KFRAG
#undef PIPE_CLEAR_V_TAIL
#undef PIPE_LOAD_V
#undef PIPE_LOAD_K

    l_run = xor32_sum(l_run);
    const float inv = 1.0f / l_run;
    if (row_valid) {
        bf16_t* orow = out + ((int64_t)b * L + q_clamped) * (int64_t)(Hq * D) + hq * D;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                au32x2_t w;
                w.x = pack_bf16x2(acc_o[d][r * 4 + 0] * inv, acc_o[d][r * 4 + 1] * inv);
                w.y = pack_bf16x2(acc_o[d][r * 4 + 2] * inv, acc_o[d][r * 4 + 3] * inv);
                *reinterpret_cast<au32x2_t*>(orow + d * 32 + r * 8 + g * 4) = w;
            }
        if (lse && g == 0) lse[(int64_t)(b * Hq + hq) * L + q_clamped] = (m_run + log2f(l_run)) * 0.6931471805599453f;
    }
}

// Each workgroup takes a long query tile and its mirror-image short one, so every workgroup of a launch
// does the same work: the hardware hands workgroups to XCDs and shader engines strictly in turn and waits
// for the next target to have room, so workgroups of uneven length leave whole shader engines idle.
// Consecutive ids go to different XCDs; the blocks of one (batch, kv head) are kept on one XCD so that
// its K and V stay in that XCD's L2.  Two waves per SIMD (register budget 256): one wave's softmax runs
// in the shadow of the other's MFMAs.
template <int D, bool BIAS, int NT>
__global__ __launch_bounds__(NT, 512 / NT) void attention_fwd_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k,
                                                            int64_t k_sb, int64_t k_sh,
                                                            const bf16_t* __restrict__ v, int64_t v_sb, int v_sl, int64_t v_sh,
                                                            const float* __restrict__ key_bias, bf16_t* __restrict__ out,
                                                            float* __restrict__ lse, int Hq, int Hkv, int L, int Lk,
                                                            float scale_log2, int B, int pack) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int kAttBM = att_rows_per_block(NT);
    const int heads_per_group = pack ? 1 : Hq / Hkv;     // packed: the group's heads share the rows of a tile
    const int n_qt = (L * (pack ? Hq / Hkv : 1) + kAttBM - 1) / kAttBM;
    const int n_pairs = (n_qt + 1) / 2;
    const int per_group = n_pairs * heads_per_group;     // workgroups sharing one K/V
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
    const int head = pack ? group % Hkv : (group % Hkv) * heads_per_group + within / n_pairs;
    const int pair = within % n_pairs;
    const int qt_long = n_qt - 1 - pair;
#pragma unroll 1
    for (int half = 0; half < 2; ++half) {
        if (half && pair == qt_long) break;   // an odd tile count leaves the middle tile on its own
        attention_q_tile_pipe<D, BIAS, NT>(q, k, k_sb, k_sh, v, v_sb, v_sl, v_sh, key_bias, out, lse, Hq, Hkv, L, Lk,
                                           scale_log2, half ? pair : qt_long, head, b, pack != 0, smem);
    }
}

// The same launch shape for calls with a bias per (query, key) pair or dropout: the non-pipelined body with
// the extras switched on (four waves; rows are never packed).
template <int D>
__global__ __launch_bounds__(256, 2) void attention_fwd_extra_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, int64_t k_sb, int64_t k_sh, const bf16_t* __restrict__ v,
    int64_t v_sb, int v_sl, int64_t v_sh, bf16_t* __restrict__ out, float* __restrict__ lse, int Hq, int Hkv, int L, int Lk,
    float scale_log2, int B, AttnExtra ex) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int kAttBM = att_rows_per_block(256);
    const int heads_per_group = Hq / Hkv;
    const int n_qt = (L + kAttBM - 1) / kAttBM;
    const int n_pairs = (n_qt + 1) / 2;
    const int per_group = n_pairs * heads_per_group;
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
    const int head = (group % Hkv) * heads_per_group + within / n_pairs;
    const int pair = within % n_pairs;
    const int qt_long = n_qt - 1 - pair;
#pragma unroll 1
    for (int half = 0; half < 2; ++half) {
        if (half && pair == qt_long) break;
        attention_q_tile<D, false, 256, false, true>(q, k, k_sb, k_sh, v, v_sb, v_sl, v_sh, nullptr, out, lse, Hq, Hkv, L, Lk,
                                                     scale_log2, half ? pair : qt_long, head, b, false, smem, nullptr, 0, 1,
                                                     0, 0, &ex);
    }
}

// Few query rows against many keys (decoding): the keys are cut into n_parts ranges and every (batch, head
// group, range) gets a workgroup, so that a handful of sequences still fills the chip; the ranges are merged
// by attention_merge_kernel.  One query tile per group (rows <= 128), part p covers part_len keys from
// p * part_len, the last one the rest.
template <int D, bool BIAS>
__global__ __launch_bounds__(256, 2) void attention_splitkv_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k, int64_t k_sb, int64_t k_sh, const bf16_t* __restrict__ v,
    int64_t v_sb, int v_sl, int64_t v_sh, const float* __restrict__ key_bias, float* __restrict__ part_out, int Hq, int Hkv,
    int L, int Lk, float scale_log2, int B, int pack, int n_parts, int part_len) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int heads_per_group = pack ? 1 : Hq / Hkv;
    const int n_base = B * Hkv * heads_per_group;
    const int part = blockIdx.x / n_base;
    const int base = blockIdx.x - part * n_base;
    const int group = base / heads_per_group;
    const int b = group / Hkv;
    const int head = pack ? group % Hkv : (group % Hkv) * heads_per_group + base % heads_per_group;
    const int key_first = part * part_len;
    const int key_count = part == n_parts - 1 ? Lk - key_first : part_len;
    attention_q_tile<D, BIAS, 256, true>(q, k, k_sb, k_sh, v, v_sb, v_sl, v_sh, key_bias, nullptr, nullptr, Hq, Hkv, L, Lk,
                                         scale_log2, 0, head, b, pack != 0, smem, part_out, part, n_parts, key_first,
                                         key_count);
}

// One wave per query row: out = sum_p 2^(m_p - M) O_p / sum_p 2^(m_p - M) l_p with M = max_p m_p.  Lane p
// holds the maximum and sum of part p (at most 64 parts), so the weights are ready before the rows of
// partial outputs are streamed; the sums run over the parts in order.
template <int D>
__global__ __launch_bounds__(256) void attention_merge_kernel(const float* __restrict__ part_out, bf16_t* __restrict__ out,
                                                              float* __restrict__ lse, int64_t n_rows, int Hq, int L,
                                                              int n_parts) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);      // (b * Hq + hq) * L + position
    if (row >= n_rows) return;
    const float* p0 = part_out + row * n_parts * (D + kPartPad);
    const float2 ml = lane < n_parts ? *reinterpret_cast<const float2*>(p0 + lane * (D + kPartPad) + D)
                                     : make_float2(-INFINITY, 0.f);
    float M = ml.x;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o, 64));
    const float w_lane = lane < n_parts ? __builtin_amdgcn_exp2f(ml.x - M) : 0.f;
    float denom = 0.f, acc[D / 64];
#pragma unroll
    for (int j = 0; j < D / 64; ++j) acc[j] = 0.f;
#pragma unroll 4
    for (int p = 0; p < n_parts; ++p) {
        const float w = __shfl(w_lane, p, 64);
        denom += w * __shfl(ml.y, p, 64);
        const float* pr = p0 + p * (D + kPartPad);
#pragma unroll
        for (int j = 0; j < D / 64; ++j) acc[j] += w * pr[j * 64 + lane];
    }
    const int64_t bh = row / L, pos = row - bh * L;
    const int64_t b = bh / Hq, hq = bh - b * Hq;
    bf16_t* orow = out + (b * L + pos) * (int64_t)(Hq * D) + hq * D;
    const float inv = 1.0f / denom;
#pragma unroll
    for (int j = 0; j < D / 64; ++j) orow[j * 64 + lane].bits = static_cast<uint16_t>(float_to_bf16_bits(acc[j] * inv));
    if (lse && lane == 0) lse[row] = (M + log2f(denom)) * 0.6931471805599453f;
}

// Key ranges for the split: aim at ~1024 workgroups, ranges of whole key tiles and at least two tiles, every
// range starting at or before the first query's position (so that each row sees a key of each range).
// Measured (32 query / 8 kv heads, D 128, one new token): 1 sequence x 16384 keys 291 -> 33 us, 8 x 8192
// 150 -> 50 us, 16 x 2048 41 -> 30 us; from 64 sequences on the single pass is as fast or faster.
static int attention_split_plan(int B, int Hq, int Hkv, int L, int Lk, int* part_len_out) {
    const int rep = Hq / Hkv;
    const bool pack = L < att_rows_per_block(256) && Hq > Hkv;
    const int64_t rows = pack ? (int64_t)L * rep : L;
    if (rows > att_rows_per_block(256) || Lk - L < 4 * kAttBN) return 1;
    const int64_t n_base = (int64_t)B * (pack ? Hkv : Hq);
    if (n_base > 256) return 1;      // one workgroup per (batch, head group) already fills the chip twice over
    int64_t want = 1024 / n_base;
    if (want > 64) want = 64;
    int part_len = (int)(((Lk + want - 1) / want + kAttBN - 1) / kAttBN) * kAttBN;
    if (part_len < 2 * kAttBN) part_len = 2 * kAttBN;
    int n_parts = (Lk + part_len - 1) / part_len;
    while (n_parts > 1 && (int64_t)(n_parts - 1) * part_len > Lk - L) --n_parts;
    *part_len_out = part_len;
    return n_parts;
}

}  // namespace ats

extern "C" size_t ats_attention_fwd_workspace(int B, int Hq, int Hkv, int L, int Lk, int D) {
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || L <= 0 || Lk < L || (D != 64 && D != 128)) return 0;
    int part_len = 0;
    const int n_parts = ats::attention_split_plan(B, Hq, Hkv, L, Lk, &part_len);
    return n_parts > 1 ? (size_t)B * Hq * L * n_parts * (D + ats::kPartPad) * sizeof(float) : 0;
}

// Fills the kernels' view of the optional extras; returns false (with the error text set) on bad arguments.
namespace ats {
bool make_attention_extra(const char* who, const float* bias_qk, int64_t bias_sb, int64_t bias_sh, float dropout_p,
                          uint64_t seed, int L,
                          int Lk, AttnExtra* ex, bool* any) {
    *any = bias_qk != nullptr || dropout_p > 0.f;
    ex->bias_qk = bias_qk;
    ex->bias_sb = bias_sb;
    ex->bias_sh = bias_sh;
    ex->keep_scale = 0.f;
    ex->drop_threshold = 0;
    ex->seed_lo = (uint32_t)seed;
    ex->seed_hi = (uint32_t)(seed >> 32);
    if (!(dropout_p >= 0.f && dropout_p < 1.f)) {
        set_error("%s: dropout probability %g (must be in [0, 1))", who, dropout_p);
        return false;
    }
    if (bias_qk && (bias_sb < 0 || bias_sh < 0 || (reinterpret_cast<uintptr_t>(bias_qk) & 3) ||
                    (int64_t)L * Lk * 4 >= 0x7fffffffLL)) {
        set_error("%s: pair bias (batch stride %lld, head stride %lld; one [L, Lk] matrix must stay under 2 GiB)", who,
                  (long long)bias_sb, (long long)bias_sh);
        return false;
    }
    if (dropout_p > 0.f) {
        if ((int64_t)L * Lk > 0xffffffffLL) {
            set_error("%s: dropout needs L * Lk < 2^32", who);
            return false;
        }
        ex->keep_scale = 1.0f / (1.0f - dropout_p);
        double t = (double)dropout_p * 4294967296.0;
        ex->drop_threshold = t >= 4294967295.0 ? 0xffffffffu : (uint32_t)t;
    }
    return true;
}
}  // namespace ats

extern "C" int ats_attention_fwd(const void* q, const void* k, int64_t k_sb, int64_t k_sh, const void* v, int64_t v_sb,
                                 int64_t v_sl, int64_t v_sh, const float* key_bias, void* out, float* lse, int B, int Hq,
                                 int Hkv, int L, int Lk, int D, float scale, void* workspace, size_t workspace_bytes,
                                 ats_stream_t stream) {
    return ats_attention_fwd_ex(q, k, k_sb, k_sh, v, v_sb, v_sl, v_sh, key_bias, nullptr, 0, 0, 0.f, 0, out, lse, B, Hq, Hkv, L,
                                Lk, D, scale, workspace, workspace_bytes, stream);
}

extern "C" int ats_attention_fwd_ex(const void* q, const void* k, int64_t k_sb, int64_t k_sh, const void* v, int64_t v_sb,
                                    int64_t v_sl, int64_t v_sh, const float* key_bias, const float* bias_qk,
                                    int64_t bias_sb, int64_t bias_sh, float dropout_p, uint64_t dropout_seed, void* out,
                                    float* lse, int B,
                                    int Hq, int Hkv, int L, int Lk, int D, float scale, void* workspace,
                                    size_t workspace_bytes, ats_stream_t stream) {
    using namespace ats;
    ATS_REQUIRE(B >= 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0 && L >= 0 && Lk >= L && scale > 0.f, ATS_ERR_INVALID_ARG,
                "ats_attention_fwd: B=%d Hq=%d Hkv=%d L=%d Lk=%d scale=%g", B, Hq, Hkv, L, Lk, scale);
    ATS_REQUIRE(D == 64 || D == 128, ATS_ERR_UNSUPPORTED, "ats_attention_fwd: head_dim %d (64 or 128)", D);
    if (B == 0 || L == 0) return ATS_OK;
    ATS_REQUIRE(q && k && v && out && aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out),
                ATS_ERR_INVALID_ARG, "ats_attention_fwd: null or misaligned pointer");
    ATS_REQUIRE(k_sb % 8 == 0 && k_sh % 8 == 0 && k_sb >= 0 && k_sh >= 0, ATS_ERR_INVALID_ARG,
                "ats_attention_fwd: batch and head strides of k (%lld, %lld) must be multiples of 8 elements",
                (long long)k_sb, (long long)k_sh);
    ATS_REQUIRE(v_sl >= D && v_sl % 8 == 0 && v_sb % 8 == 0 && v_sh % 8 == 0 && v_sb >= 0 && v_sh >= 0, ATS_ERR_INVALID_ARG,
                "ats_attention_fwd: strides of v (%lld, %lld, %lld) must be multiples of 8 elements, rows apart",
                (long long)v_sb, (long long)v_sl, (long long)v_sh);
    ATS_REQUIRE((int64_t)Lk * D * 2 < 0x7fffffffLL && ((int64_t)Lk * v_sl + D) * 2 < 0x7fffffffLL, ATS_ERR_UNSUPPORTED,
                "ats_attention_fwd: %d keys (one head's K or V must stay under 2 GiB)", Lk);
    // few query positions (decoding, short chunks): the query heads of a kv group share a tile's rows
    const float scale_log2 = scale * 1.4426950408889634f;
    AttnExtra ex;
    bool extras = false;
    if (!make_attention_extra("ats_attention_fwd_ex", bias_qk, bias_sb, bias_sh, dropout_p, dropout_seed, L, Lk, &ex, &extras))
        return ATS_ERR_INVALID_ARG;
    if (extras) {
        ATS_REQUIRE(key_bias == nullptr, ATS_ERR_INVALID_ARG,
                    "ats_attention_fwd_ex: with a pair bias or dropout the per-key bias must be folded into the pair bias");
        const int64_t blocks = (int64_t)(((L + 127) / 128 + 1) / 2) * Hq * B;
        ATS_REQUIRE(blocks <= 0x7fffffff, ATS_ERR_UNSUPPORTED, "ats_attention_fwd_ex: %lld workgroups", (long long)blocks);
        const int smem_x = 2 * kAttBN * ((D * 2 + 16) + (D * 2 + 64));
        static LdsReservation reserved_x[2];
        auto launch_x = [&](auto kernel, LdsReservation& reserved) -> int {
            if (smem_x > 64 * 1024) {
                hipError_t e = reserve_lds(reserved, {reinterpret_cast<const void*>(kernel)}, smem_x);
                ATS_REQUIRE(e == hipSuccess, ATS_ERR_LAUNCH, "ats_attention_fwd_ex: cannot reserve %d bytes of LDS: %s",
                            smem_x, hipGetErrorString(e));
            }
            hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), smem_x, as_stream(stream),
                               static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k), k_sb, k_sh,
                               static_cast<const bf16_t*>(v), v_sb, (int)v_sl, v_sh, static_cast<bf16_t*>(out), lse, Hq, Hkv,
                               L, Lk, scale_log2, B, ex);
            return ATS_OK;
        };
        const int rc = D == 128 ? launch_x(attention_fwd_extra_kernel<128>, reserved_x[0])
                                : launch_x(attention_fwd_extra_kernel<64>, reserved_x[1]);
        if (rc != ATS_OK) return rc;
        ATS_CHECK_LAUNCH("ats_attention_fwd_ex");
        return ATS_OK;
    }
    // decoding sizes with a workspace: key ranges in parallel, then a merge
    int part_len = 0;
    const int n_parts = workspace ? attention_split_plan(B, Hq, Hkv, L, Lk, &part_len) : 1;
    if (n_parts > 1 && workspace_bytes >= (size_t)B * Hq * L * n_parts * (D + kPartPad) * sizeof(float) &&
        aligned16(workspace)) {
        const int pack = (L < att_rows_per_block(256) && Hq > Hkv) ? 1 : 0;
        const int64_t n_base = (int64_t)B * (pack ? Hkv : Hq);
        const int smem = 2 * kAttBN * ((D * 2 + 16) + (D * 2 + 64)) + (key_bias ? 2 * kAttBN * 4 : 0);
        float* parts = static_cast<float*>(workspace);
        static LdsReservation reserved_split[4];
        auto launch_split = [&](auto kernel, LdsReservation& reserved) -> int {
            if (smem > 64 * 1024) {
                hipError_t e = reserve_lds(reserved, {reinterpret_cast<const void*>(kernel)}, smem);
                ATS_REQUIRE(e == hipSuccess, ATS_ERR_LAUNCH, "ats_attention_fwd: cannot reserve %d bytes of LDS: %s", smem,
                            hipGetErrorString(e));
            }
            hipLaunchKernelGGL(kernel, dim3((unsigned)(n_base * n_parts)), dim3(256), smem, as_stream(stream),
                               static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k), k_sb, k_sh,
                               static_cast<const bf16_t*>(v), v_sb, (int)v_sl, v_sh, key_bias, parts, Hq, Hkv, L, Lk,
                               scale_log2, B, pack, n_parts, part_len);
            return ATS_OK;
        };
        int rc;
        if (D == 128)
            rc = key_bias ? launch_split(attention_splitkv_kernel<128, true>, reserved_split[0])
                          : launch_split(attention_splitkv_kernel<128, false>, reserved_split[1]);
        else
            rc = key_bias ? launch_split(attention_splitkv_kernel<64, true>, reserved_split[2])
                          : launch_split(attention_splitkv_kernel<64, false>, reserved_split[3]);
        if (rc != ATS_OK) return rc;
        ATS_CHECK_LAUNCH("ats_attention_fwd(key ranges)");
        const int64_t n_rows = (int64_t)B * Hq * L;
        const dim3 mgrid((unsigned)((n_rows + 3) / 4));
        if (D == 128)
            hipLaunchKernelGGL((attention_merge_kernel<128>), mgrid, dim3(256), 0, as_stream(stream), parts,
                               static_cast<bf16_t*>(out), lse, n_rows, Hq, L, n_parts);
        else
            hipLaunchKernelGGL((attention_merge_kernel<64>), mgrid, dim3(256), 0, as_stream(stream), parts,
                               static_cast<bf16_t*>(out), lse, n_rows, Hq, L, n_parts);
        ATS_CHECK_LAUNCH("ats_attention_fwd(merge)");
        return ATS_OK;
    }
    const int nt = L >= 4096 ? 512 : 256;
    const int kAttBM = att_rows_per_block(nt);
    const int pack = (L < kAttBM && Hq > Hkv) ? 1 : 0;
    const int64_t n_blocks = pack ? (int64_t)((((int64_t)L * (Hq / Hkv) + kAttBM - 1) / kAttBM + 1) / 2) * Hkv * B
                                  : (int64_t)(((L + kAttBM - 1) / kAttBM + 1) / 2) * Hq * B;
    ATS_REQUIRE(n_blocks <= 0x7fffffff, ATS_ERR_UNSUPPORTED, "ats_attention_fwd: %lld workgroups", (long long)n_blocks);
    const dim3 grid((unsigned)n_blocks);
    static LdsReservation reserved_lds[8];      // one per kernel instance
    auto launch = [&](auto kernel, int smem, LdsReservation& reserved) -> int {
        if (smem > 64 * 1024) {
            hipError_t e = reserve_lds(reserved, {reinterpret_cast<const void*>(kernel)}, smem);
            ATS_REQUIRE(e == hipSuccess, ATS_ERR_LAUNCH, "ats_attention_fwd: cannot reserve %d bytes of LDS: %s", smem,
                        hipGetErrorString(e));
        }
        hipLaunchKernelGGL(kernel, grid, dim3(nt), smem, as_stream(stream), static_cast<const bf16_t*>(q),
                           static_cast<const bf16_t*>(k), k_sb, k_sh, static_cast<const bf16_t*>(v), v_sb, (int)v_sl, v_sh,
                           key_bias,
                           static_cast<bf16_t*>(out), lse, Hq, Hkv, L, Lk, scale_log2, B, pack);
        return ATS_OK;
    };
    // K tile, V tile (two stages each, rows unpadded) and, with a bias, two stages of one float per key
    const int smem = 4 * kAttBN * D * 2 + (key_bias ? 2 * kAttBN * 4 : 0);
    int rc;
    if (D == 128 && nt == 256)
        rc = key_bias ? launch(attention_fwd_kernel<128, true, 256>, smem, reserved_lds[0])
                      : launch(attention_fwd_kernel<128, false, 256>, smem, reserved_lds[1]);
    else if (D == 128)
        rc = key_bias ? launch(attention_fwd_kernel<128, true, 512>, smem, reserved_lds[2])
                      : launch(attention_fwd_kernel<128, false, 512>, smem, reserved_lds[3]);
    else if (nt == 256)
        rc = key_bias ? launch(attention_fwd_kernel<64, true, 256>, smem, reserved_lds[4])
                      : launch(attention_fwd_kernel<64, false, 256>, smem, reserved_lds[5]);
    else
        rc = key_bias ? launch(attention_fwd_kernel<64, true, 512>, smem, reserved_lds[6])
                      : launch(attention_fwd_kernel<64, false, 512>, smem, reserved_lds[7]);
    if (rc != ATS_OK) return rc;
    ATS_CHECK_LAUNCH("ats_attention_fwd");
    return ATS_OK;
}

// Optional extras of the attention kernels: an additive bias per (query, key) pair and dropout on the
// attention weights (GroupedQueryAttention._standard_attention, Src/Main_Scripts/core/model.py:819-833:
// a [B, 1, L, Lk] mask is added as (1 - mask) * -1e4, nn.Dropout acts on the weights while training).
//
// Dropout needs the same keep / drop decision for element (batch, head, query, key) in the forward and in
// both backward kernels, whatever tile or lane the element falls into, so the decision is a pure function of
// the coordinates and a 64-bit seed: a 32-bit counter (query * Lk + key) is mixed with a per-(batch, head)
// key by the finaliser of MurmurHash3 (two multiply / xor-shift rounds), and the element is kept when the
// result is at or above p * 2^32.  torch's generator stream cannot be reproduced by a kernel that visits
// the elements in tile order; the host-side restatement of this function is what the tests compare with.
#pragma once
#include <stdint.h>

#ifndef ATS_HD
#ifdef __HIPCC__
#define ATS_HD __host__ __device__
#else
#define ATS_HD
#endif
#endif

namespace ats {

struct AttnExtra {
    const float* bias_qk;     // [B, L, Lk] float32 added to the scaled scores, or null
    int64_t bias_sb;          // floats between the matrices of two batch entries (0: one matrix for all)
    int64_t bias_sh;          // floats between the matrices of two query heads (0: one matrix for all heads)
    float keep_scale;         // 1 / (1 - p) with dropout, 0 without
    uint32_t drop_threshold;  // keep an element iff its hash >= threshold
    uint32_t seed_lo, seed_hi;
};

ATS_HD inline uint32_t attn_head_key(uint32_t seed_lo, uint32_t seed_hi, uint32_t batch_head) {
    uint32_t x = seed_lo ^ (batch_head * 0x9E3779B1u);
    x ^= x >> 15;
    x *= 0x2C1B3C6Du;
    x ^= seed_hi;
    x ^= x >> 12;
    return x;
}

// counter = query * Lk + key (the caller guarantees L * Lk < 2^32)
ATS_HD inline uint32_t attn_drop_hash(uint32_t head_key, uint32_t counter) {
    uint32_t x = counter ^ head_key;
    x ^= x >> 16;
    x *= 0x85EBCA6Bu;
    x ^= x >> 13;
    x *= 0xC2B2AE35u;
    x ^= x >> 16;
    return x;
}

// Fills `ex` from the arguments of the extended entry points; false (error text set) on bad arguments.
// `any` tells whether a pair bias or dropout was asked for at all.
bool make_attention_extra(const char* who, const float* bias_qk, int64_t bias_sb, int64_t bias_sh, float dropout_p, uint64_t seed, int L,
                          int Lk, AttnExtra* ex, bool* any);

}  // namespace ats

// Block id -> (expert, m-tile, n-tile) for the grouped expert GEMMs.
//
// MI355X has 8 XCDs with a private L2 each, and the hardware deals consecutive
// workgroup ids round-robin over the XCDs.  The schedule therefore takes
// xcd = id % 8 and gives every XCD whole "supertiles" of SM x SN neighbouring
// tiles (32 blocks, one per CU of the XCD): the blocks of a supertile advance
// through K together and share operand-A panels and weight panels in that
// XCD's L2.
//
// The m-tiles of all groups form one list (group 0's tiles, then group 1's, ...;
// a group is an expert, or a K slice of an expert); a supertile covers SM
// consecutive entries of that list ("band") and SN consecutive n-tiles.
// Groups with few rows therefore leave no holes: a band simply continues into
// the next group ("packed" list).  Launches whose groups are large (thousands of
// rows) use the "aligned" list instead, in which every group's tile count is
// rounded up to a multiple of SM, so that no band mixes the weight panels of two
// experts; the few list entries past a group's last tile are empty.  A band belongs to the group in which it starts; supertiles are
// ordered group -> n-group -> band of that group, so the XCDs working side by
// side stream the same weight panels of one expert (shared through the
// memory-side cache) and a weight panel is needed only once per expert.  Blocks
// past the end of the list or of N return at once.
//
// Finding the group of a list entry is a search in the prefix sums of the
// per-group tile counts.  On the device a wave does it in parallel: lane l loads
// the row count of group l, a shuffle scan forms the prefix sums, a ballot finds
// the group (64 groups per step) - one memory round trip instead of one per
// group, which matters for blocks that only find out that they have no tile.
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

constexpr int kNumXcd = 8;
constexpr int kSuperBlocks = 32;  // blocks per supertile = CUs per XCD

struct TileCoord {
    int e, mt, nt;
};

struct TileSlot {
    int64_t S;   // supertile index
    int dm, dn;  // position inside the supertile
};

ATS_HD inline TileSlot tile_slot(int64_t block, int SN) {
    const int xcd = (int)(block % kNumXcd);
    const int64_t li = block / kNumXcd;
    TileSlot s;
    s.S = (li / kSuperBlocks) * kNumXcd + xcd;
    const int w = (int)(li % kSuperBlocks);
    s.dn = w % SN;
    s.dm = w / SN;
    return s;
}

// Bands that start before list position `pos` (band b starts at b * SM).
ATS_HD inline int64_t bands_before(int64_t pos, int SM) { return (pos + SM - 1) / SM; }

// Host reference of the schedule (sequential prefix walk).  k_slices > 1: the list is repeated per K slice,
// slice-major; *slice receives the slice.  SM * SN must equal kSuperBlocks.
inline int list_tiles(int count, int BM, int SM, bool aligned) {
    const int t = count > 0 ? (count + BM - 1) / BM : 0;
    return aligned ? (t + SM - 1) / SM * SM : t;
}

inline bool decode_tile(int64_t block, const int32_t* row_count, int E, int BM, int n_tiles, int SM, int SN,
                        bool aligned, TileCoord* out, int k_slices = 1, int* slice = nullptr) {
    const int n_groups = (n_tiles + SN - 1) / SN;
    const TileSlot s = tile_slot(block, SN);
    const int G = E * k_slices;
    // owner group of supertile S: first g with bands_before(prefix_incl[g]) * n_groups > S
    int64_t excl = 0;
    int64_t gm = -1;
    int nt = 0;
    for (int g = 0; g < G; ++g) {
        const int t = list_tiles(row_count[g % E], BM, SM, aligned);
        const int64_t first_band = bands_before(excl, SM), end_band = bands_before(excl + t, SM);
        if (end_band * n_groups > s.S) {
            const int64_t r = s.S - first_band * n_groups;
            const int64_t nb = end_band - first_band;
            gm = (first_band + r % nb) * SM + s.dm;
            nt = (int)(r / nb) * SN + s.dn;
            break;
        }
        excl += t;
    }
    if (gm < 0 || nt >= n_tiles) return false;
    // group of list position gm
    excl = 0;
    for (int g = 0; g < G; ++g) {
        const int t = list_tiles(row_count[g % E], BM, SM, aligned);
        if (gm < excl + t) {
            if ((gm - excl) * BM >= row_count[g % E]) return false;    // padding entry of an aligned list
            out->e = g % E;
            out->mt = (int)(gm - excl);
            out->nt = nt;
            if (slice) *slice = g / E;
            return true;
        }
        excl += t;
    }
    return false;
}

#ifdef __HIPCC__
// Device version: every lane of the calling wave takes part (call it with all 64 lanes active and wave-uniform
// arguments); the result is the same in all lanes.  Groups are taken 64 at a time.
__device__ __forceinline__ void tile_scan64(const int32_t* __restrict__ row_count, int E, int G, int g0, int BM,
                                            int SM, bool aligned, int lane, int* t_out, int* p_out) {
    const int g = g0 + lane;
    const int cnt = g < G ? row_count[g % E] : 0;
    int t = cnt > 0 ? (cnt + BM - 1) / BM : 0;
    if (aligned) t = (t + SM - 1) / SM * SM;
    const int p = wave_inclusive_scan(t);     // ats_common.hpp
    *t_out = t;
    *p_out = p;   // inclusive prefix inside this chunk
}

__device__ __forceinline__ bool decode_tile_wave(int64_t block, const int32_t* __restrict__ row_count, int E, int BM,
                                                 int n_tiles, int SM, int SN, bool aligned, TileCoord* out,
                                                 int k_slices = 1, int* slice = nullptr) {
    const int lane = threadIdx.x & 63;
    const int n_groups = (n_tiles + SN - 1) / SN;
    const TileSlot s = tile_slot(block, SN);
    const int G = E * k_slices;
    // owner group of the supertile
    int64_t base = 0, gm = -1;
    int nt = 0;
    int t0 = 0, p0 = 0;
    for (int g0 = 0; g0 < G; g0 += 64) {
        int t, p;
        tile_scan64(row_count, E, G, g0, BM, SM, aligned, lane, &t, &p);
        if (g0 == 0) {
            t0 = t;
            p0 = p;
        }
        const int64_t incl = base + p;
        const unsigned long long hit = __ballot(bands_before(incl, SM) * n_groups > s.S);
        if (hit) {
            // lane values through v_readlane: scalars, so that everything derived from them (the tile, the
            // loads' descriptors, the branches below) is uniform for the compiler too
            const int first = __ffsll((long long)hit) - 1;
            const int64_t incl_g = base + __builtin_amdgcn_readlane(p, first);
            const int64_t excl_g = incl_g - __builtin_amdgcn_readlane(t, first);
            const int64_t first_band = bands_before(excl_g, SM), nb = bands_before(incl_g, SM) - first_band;
            const int64_t r = s.S - first_band * n_groups;
            gm = (first_band + r % nb) * SM + s.dm;
            nt = (int)(r / nb) * SN + s.dn;
            break;
        }
        base += __builtin_amdgcn_readlane(p, 63);
    }
    if (gm < 0 || nt >= n_tiles) return false;
    // group of list position gm (it is the owner or a later group)
    base = 0;
    for (int g0 = 0; g0 < G; g0 += 64) {
        int t = t0, p = p0;
        if (g0 > 0) tile_scan64(row_count, E, G, g0, BM, SM, aligned, lane, &t, &p);
        const unsigned long long hit = __ballot(base + p > gm);
        if (hit) {
            const int first = __ffsll((long long)hit) - 1;
            const int pe = __builtin_amdgcn_readlane(p, first), te = __builtin_amdgcn_readlane(t, first);
            const int g = g0 + first;
            const int mt = (int)(gm - (base + pe - te));
            if (aligned && (int64_t)mt * BM >= __builtin_amdgcn_readfirstlane(row_count[g % E])) return false;  // padding
            out->e = g % E;
            out->mt = mt;
            out->nt = nt;
            if (slice) *slice = g / E;
            return true;
        }
        base += __builtin_amdgcn_readlane(p, 63);
    }
    return false;
}
#endif

// Groups of at least this many rows on average use the aligned list.
#ifndef ATS_ALIGNED_MIN
#define ATS_ALIGNED_MIN 1536
#endif
constexpr int64_t kAlignedBandsMinAvgRows = ATS_ALIGNED_MIN;

// Supertile shape for a launch: SN from {8, 4, 2} with the fewest unused n-slots (the larger SN wins ties),
// SM = kSuperBlocks / SN.  Tile configurations that stream weights (one m-tile per group) pass their own shape.
inline void pick_supertile(int n_tiles, int* SM, int* SN) {
    int best = 8, best_pad = 1 << 30;
    for (int sn : {8, 4, 2}) {
        const int pad = (n_tiles + sn - 1) / sn * sn - n_tiles;
        if (pad < best_pad) {
            best_pad = pad;
            best = sn;
        }
    }
    *SN = best;
    *SM = kSuperBlocks / best;
}

// Number of blocks to launch so that every existing tile is covered, given only an upper bound on the total
// row count (max_rows and E already multiplied by the number of K slices, if any).
inline int64_t grid_blocks(int64_t max_rows, int E, int BM, int n_tiles, int SM, int SN, bool aligned) {
    const int n_groups = (n_tiles + SN - 1) / SN;
    // sum of ceil(count / BM) <= max_rows / BM + E; rounding every group up to a multiple of SM adds < SM each
    const int64_t mtiles_bound = max_rows / BM + (int64_t)E * (aligned ? SM : 1);
    const int64_t supertiles = (mtiles_bound + SM - 1) / SM * n_groups;
    const int64_t blocks = supertiles * kSuperBlocks;
    const int64_t round = (int64_t)kNumXcd * kSuperBlocks;
    return (blocks + round - 1) / round * round;
}

}  // namespace ats

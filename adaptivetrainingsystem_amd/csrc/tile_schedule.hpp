// Block id -> (expert, m-tile, n-tile) for the grouped expert GEMMs.
//
// MI355X has 8 XCDs with a private L2 each, and the hardware deals consecutive
// workgroup ids round-robin over the XCDs.  The schedule therefore takes
// xcd = id % 8 and gives every XCD whole "supertiles" of SM x SN neighbouring
// tiles (32 blocks, one per CU of the XCD): the blocks of a supertile advance
// through K together and share SM operand-A panels and SN weight panels in that
// XCD's L2.  Supertiles are ordered expert -> n-group -> m-group, so the XCDs
// working side by side stream the same weight panels (shared through the
// memory-side cache) and a weight panel is needed only once per expert.
// Ragged experts: tiles past an expert's last row do not exist; their blocks
// return at once.
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

// SM * SN must equal kSuperBlocks.
ATS_HD inline bool decode_tile(int64_t block, const int32_t* row_count, int E, int BM, int n_tiles, int SM, int SN,
                               TileCoord* out) {
    const int xcd = (int)(block % kNumXcd);
    const int64_t li = block / kNumXcd;
    int64_t S = (li / kSuperBlocks) * kNumXcd + xcd;
    const int w = (int)(li % kSuperBlocks);
    const int dn = w % SN, dm = w / SN;
    const int n_groups = (n_tiles + SN - 1) / SN;
    for (int e = 0; e < E; ++e) {
        const int cnt = row_count[e];
        if (cnt <= 0) continue;
        const int mtiles = (cnt + BM - 1) / BM;
        const int mgroups = (mtiles + SM - 1) / SM;
        const int64_t st = (int64_t)mgroups * n_groups;
        if (S < st) {
            const int mg = (int)(S % mgroups);
            const int ng = (int)(S / mgroups);
            const int mt = mg * SM + dm;
            const int nt = ng * SN + dn;
            if (mt >= mtiles || nt >= n_tiles) return false;
            out->e = e;
            out->mt = mt;
            out->nt = nt;
            return true;
        }
        S -= st;
    }
    return false;
}

// Split K: E * k_slices groups, slice-major (group g is slice g / E of expert g % E); the slice is found
// by counting, so the walk divides by nothing new and stays on the scalar unit.
ATS_HD inline bool decode_tile_sliced(int64_t block, const int32_t* row_count, int E, int BM, int n_tiles, int SM,
                                      int SN, int k_slices, TileCoord* out, int* slice) {
    const int xcd = (int)(block % kNumXcd);
    const int64_t li = block / kNumXcd;
    int64_t S = (li / kSuperBlocks) * kNumXcd + xcd;
    const int w = (int)(li % kSuperBlocks);
    const int dn = w % SN, dm = w / SN;
    const int n_groups = (n_tiles + SN - 1) / SN;
    for (int ks = 0; ks < k_slices; ++ks) {
        for (int e = 0; e < E; ++e) {
            const int cnt = row_count[e];
            if (cnt <= 0) continue;
            const int mtiles = (cnt + BM - 1) / BM;
            const int mgroups = (mtiles + SM - 1) / SM;
            const int64_t st = (int64_t)mgroups * n_groups;
            if (S < st) {
                const int mg = (int)(S % mgroups);
                const int ng = (int)(S / mgroups);
                const int mt = mg * SM + dm;
                const int nt = ng * SN + dn;
                if (mt >= mtiles || nt >= n_tiles) return false;
                out->e = e;
                out->mt = mt;
                out->nt = nt;
                *slice = ks;
                return true;
            }
            S -= st;
        }
    }
    return false;
}

// Number of blocks to launch so that every existing tile is covered, given only
// an upper bound on the total row count.
inline int64_t grid_blocks(int64_t max_rows, int E, int BM, int n_tiles, int SM, int SN) {
    const int n_groups = (n_tiles + SN - 1) / SN;
    const int64_t supertiles = (max_rows / ((int64_t)BM * SM) + E) * n_groups;
    const int64_t blocks = supertiles * kSuperBlocks;
    const int64_t round = (int64_t)kNumXcd * kSuperBlocks;
    return (blocks + round - 1) / round * round;
}

}  // namespace ats

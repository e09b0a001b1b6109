// Tile scheduling of the grouped GEMM for gfx950: which (expert, row tile, column tile, piece of the contraction) a
// workgroup works on, derived on the device from expert_offsets by one wavefront.  Takes the place of the reference's
// fixed grid of row blocks that may straddle experts (scattermoe/triton_implementation/kernels.py:40-75).
// Kept apart from the kernels so that the same source also compiles for the host, with the wave primitives replaced
// by an emulation (tests/host/tile_schedule_host.cpp), where every shape of expert_offsets can be walked exhaustively:
// each tile dealt exactly once, pieces of a split tile covering the contraction exactly, no position past the grid.
#pragma once

namespace ck {

// Expert tile lookup: row tile `mt` (counted over all experts, each expert's rows cut into BM-row tiles)
// -> expert, first row, valid rows.  Executed by the first wave; result broadcast through LDS.
template <int BM>
__device__ __forceinline__ void find_tile(const int64_t* __restrict__ offsets, int E, int mt, int* sh_info) {
    if (threadIdx.x < CK_WAVE) {
        const int lane = lane_id();
        int base_tiles = 0;
        int found_e = -1, found_start = 0, found_rows = 0;
        for (int e0 = 0; e0 < E && found_e < 0; e0 += CK_WAVE) {
            const int e = e0 + lane;
            int begin = 0, end = 0;
            if (e < E) {
                end = (int)offsets[e];
                begin = e == 0 ? 0 : (int)offsets[e - 1];
            }
            const int tiles = (end - begin + BM - 1) / BM;
            const int incl = wave_inclusive_scan_i(tiles) + base_tiles;
            const uint64_t hit = __ballot(e < E && incl > mt);
            if (hit != 0) {
                const int src = __ffsll((unsigned long long)hit) - 1;
                const int excl = __shfl(incl - tiles, src, CK_WAVE);
                const int b = __shfl(begin, src, CK_WAVE);
                const int en = __shfl(end, src, CK_WAVE);
                found_e = e0 + src;
                found_start = b + (mt - excl) * BM;
                found_rows = min(BM, en - found_start);
            }
            base_tiles = __shfl(incl, CK_WAVE - 1, CK_WAVE);
        }
        if (lane == 0) {
            sh_info[0] = found_e;
            sh_info[1] = found_start;
            sh_info[2] = found_rows;
        }
    }
    __syncthreads();
}

// XCD-aware tile order: consecutive workgroup ids land on different XCDs (8 of them, one L2 each), so
// give every XCD a contiguous range of logical tile ids; inside the range, walk GROUP_M row tiles for
// one column tile before moving to the next column tile, so concurrent tiles share operands in L2.
__device__ __forceinline__ bool logical_tile(int m_tiles, int n_tiles, int& mt, int& nt) {
    constexpr int XCDS = 8, GROUP_M = 8;
    const int total = m_tiles * n_tiles;
    const int per_xcd = (total + XCDS - 1) / XCDS;
    const int bid = blockIdx.x;
    const int L = (bid % XCDS) * per_xcd + bid / XCDS;
    if (L >= total) return false;
    const int group_span = GROUP_M * n_tiles;
    const int group = L / group_span;
    const int first_m = group * GROUP_M;
    const int gm = min(GROUP_M, m_tiles - first_m);
    const int in_group = L - group * group_span;
    mt = first_m + in_group % gm;
    nt = in_group / gm;
    return true;
}

// Row tiles of all experts, and the expert that owns row tile mt.  Both are run by one wavefront.  With at most 64
// experts lane e keeps the bounds and the running tile count of expert e from the first function, and the second
// needs no further pass over the offsets (one round trip to memory per tile search instead of two).
struct ExpertTiles {
    int begin, end, tiles, incl;
};

template <int BM>
__device__ __forceinline__ int count_row_tiles(const int64_t* __restrict__ offsets, int E, int lane, ExpertTiles& mine) {
    if (E <= CK_WAVE) {
        mine.begin = 0;
        mine.end = 0;
        if (lane < E) {
            mine.end = (int)offsets[lane];
            mine.begin = lane == 0 ? 0 : (int)offsets[lane - 1];
        }
        mine.tiles = (mine.end - mine.begin + BM - 1) / BM;
        mine.incl = wave_inclusive_scan_i(mine.tiles);
        return __shfl(mine.incl, CK_WAVE - 1, CK_WAVE);
    }
    int m_tiles = 0;
    for (int e0 = 0; e0 < E; e0 += CK_WAVE) {
        const int e = e0 + lane;
        int tiles = 0;
        if (e < E) tiles = ((int)offsets[e] - (e == 0 ? 0 : (int)offsets[e - 1]) + BM - 1) / BM;
        m_tiles += wave_sum_i(tiles);
    }
    return m_tiles;
}

template <int BM>
__device__ __forceinline__ void expert_of_row_tile(const int64_t* __restrict__ offsets, int E, int lane, int mt,
                                                   const ExpertTiles& mine, int& found_e, int& found_start,
                                                   int& found_rows) {
    if (E <= CK_WAVE) {
        const uint64_t hit = __ballot(lane < E && mine.incl > mt);
        if (hit != 0) {
            const int src = __ffsll((unsigned long long)hit) - 1;
            const int excl = __shfl(mine.incl - mine.tiles, src, CK_WAVE);
            const int b = __shfl(mine.begin, src, CK_WAVE);
            const int en = __shfl(mine.end, src, CK_WAVE);
            found_e = src;
            found_start = b + (mt - excl) * BM;
            found_rows = min(BM, en - found_start);
        }
        return;
    }
    int base_tiles = 0;
    for (int e0 = 0; e0 < E && found_e < 0; e0 += CK_WAVE) {
        const int e = e0 + lane;
        int begin = 0, end = 0;
        if (e < E) {
            end = (int)offsets[e];
            begin = e == 0 ? 0 : (int)offsets[e - 1];
        }
        const int tiles = (end - begin + BM - 1) / BM;
        const int incl = wave_inclusive_scan_i(tiles) + base_tiles;
        const uint64_t hit = __ballot(e < E && incl > mt);
        if (hit != 0) {
            const int src = __ffsll((unsigned long long)hit) - 1;
            const int excl = __shfl(incl - tiles, src, CK_WAVE);
            const int b = __shfl(begin, src, CK_WAVE);
            const int en = __shfl(end, src, CK_WAVE);
            found_e = e0 + src;
            found_start = b + (mt - excl) * BM;
            found_rows = min(BM, en - found_start);
        }
        base_tiles = __shfl(incl, CK_WAVE - 1, CK_WAVE);
    }
}

// Tile of workgroup blockIdx.x for the products whose rows are cut per expert (forward and input gradient): the
// XCD-aware order above, applied to the number of row tiles the experts really have.  The host can only bound
// that number (rows / BM + E); dealing out the bound would leave the XCD that owns the end of the range with
// mostly empty tiles while the others carry all the work.  Executed by the first wave; the result (expert, first
// row, valid rows, column tile; expert < 0: nothing to do) is broadcast through LDS.
template <int BM>
__device__ __forceinline__ void find_tile_balanced(const int64_t* __restrict__ offsets, int E, int n_tiles, int* sh_info) {
    if (threadIdx.x < CK_WAVE) {
        constexpr int XCDS = 8, GROUP_M = 8;
        const int lane = lane_id();
        ExpertTiles mine;
        const int m_tiles = count_row_tiles<BM>(offsets, E, lane, mine);
        int found_e = -1, found_start = 0, found_rows = 0, nt = 0;
        const int total = m_tiles * n_tiles;
        // an even share of the tiles where rows of the tile grid are long; whole rows of it where they are short
        // (measured at 16 column tiles: 1-2 % better than shares that end in the middle of a row, while at 56 and
        // 112 column tiles the even share is 2-4 % better)
        const int per_xcd = n_tiles >= 32 ? (total + XCDS - 1) / XCDS : (m_tiles + XCDS - 1) / XCDS * n_tiles;
        const int xcd = blockIdx.x % XCDS, pos = blockIdx.x / XCDS;
        const int L = xcd * per_xcd + pos;
        if (pos < per_xcd && L < total) {
            const int group_span = GROUP_M * n_tiles;
            const int group = L / group_span;
            const int first_m = group * GROUP_M;
            const int gm = min(GROUP_M, m_tiles - first_m);
            const int in_group = L - group * group_span;
            const int mt = first_m + in_group % gm;
            nt = in_group / gm;
            expert_of_row_tile<BM>(offsets, E, lane, mt, mine, found_e, found_start, found_rows);
        }
        if (lane == 0) {
            sh_info[0] = found_e;
            sh_info[1] = found_start;
            sh_info[2] = found_rows;
            sh_info[3] = nt;
        }
    }
    __syncthreads();
}

// The same search with the last, partly filled round of every XCD split along the contraction.  A product with few
// column tiles has only a few rounds of tiles per CU (1088 tiles of a Mixtral c_proj over 256 CUs: 4.25), and the
// CUs without a tile in the last round idle for a whole tile time.  Every XCD (32 CUs) takes an even share of the
// tiles; if the share leaves a last round of rem <= 16 tiles, each of them is cut into s = 32 / rem pieces of the
// contraction range, worked on by s workgroups that write fp32 partial tiles to a workspace; a second launch
// (MODE 2) adds the pieces up and runs the epilogue.  Pieces are at least 32 contraction tiles long (the partial
// tiles cost two passes over 256 KB per piece and the second launch a few microseconds).
//   sh_info: 0 expert (< 0: nothing to do), 1 first row, 2 valid rows, 3 column tile, 4 / 5 first and end
//   contraction tile of this workgroup, 6 partial slot (< 0: a whole tile), 7 pieces per tile in this XCD's tail
// fixup = true (MODE 2): workgroup (x, i) = (blockIdx.x % 8, blockIdx.x / 8) owns tail tile i of XCD x, if there is one.
constexpr int kSplitSlots = 256, kSplitMinTiles = 32, kSplitMax = 8;

template <int BM, int BK>
__device__ __forceinline__ void find_tile_split(const int64_t* __restrict__ offsets, int E, int n_tiles, int K, bool fixup,
                                                int* sh_info) {
    if (threadIdx.x < CK_WAVE) {
        constexpr int XCDS = 8, GROUP_M = 8, CUS = 32;
        const int lane = lane_id();
        ExpertTiles et;
        const int m_tiles = count_row_tiles<BM>(offsets, E, lane, et);
        const int total = m_tiles * n_tiles;
        const int per_xcd = (total + XCDS - 1) / XCDS;
        const int xcd = blockIdx.x % XCDS, pos = blockIdx.x / XCDS;
        const int base = xcd * per_xcd;
        const int mine = max(0, min(per_xcd, total - base));  // tiles of this XCD
        const int full = mine / CUS * CUS, rem = mine - full;
        const int k_tiles = (K + BK - 1) / BK;
        int pieces = 1;
        if (rem > 0 && rem <= CUS / 2) pieces = max(1, min(min(CUS / rem, kSplitMax), k_tiles / kSplitMinTiles));
        int L = -1, kt_b = 0, kt_e = k_tiles, slot = -1;
        if (fixup) {
            if (pieces > 1 && pos < rem) {
                L = base + full + pos;
                slot = xcd * CUS + pos * pieces;  // the first of the tile's pieces
            }
        } else if (pos < full) {
            L = base + pos;
        } else {
            const int i = pos - full;
            if (i < rem * pieces) {
                L = base + full + i / pieces;
                if (pieces > 1) {
                    const int c = i % pieces;
                    kt_b = (int)((int64_t)c * k_tiles / pieces);
                    kt_e = (int)((int64_t)(c + 1) * k_tiles / pieces);
                    slot = xcd * CUS + i;
                }
            }
        }
        int found_e = -1, found_start = 0, found_rows = 0, nt = 0;
        if (L >= 0) {
            const int group_span = GROUP_M * n_tiles;
            const int group = L / group_span;
            const int first_m = group * GROUP_M;
            const int gm = min(GROUP_M, m_tiles - first_m);
            const int in_group = L - group * group_span;
            const int mt = first_m + in_group % gm;
            nt = in_group / gm;
            expert_of_row_tile<BM>(offsets, E, lane, mt, et, found_e, found_start, found_rows);
        }
        if (lane == 0) {
            sh_info[0] = found_e;
            sh_info[1] = found_start;
            sh_info[2] = found_rows;
            sh_info[3] = nt;
            sh_info[4] = kt_b;
            sh_info[5] = kt_e;
            sh_info[6] = slot;
            sh_info[7] = pieces;
        }
    }
    __syncthreads();
}

// Tile order of the per-expert weight-gradient products.  A tile's cost grows with its expert's row count, which
// routing can skew by orders of magnitude, and workgroup w always runs on XCD w % 8.  So every XCD gets an
// eighth of the tiles of EVERY expert (a contiguous piece of the expert's tile grid in the grouped order used
// above: 8 row tiles per column tile), and takes the experts in the order of falling row count - the long tiles
// start first, the short ones fill the gaps at the end.
//   workgroup w -> XCD x = w % 8, position s = w / 8 in that XCD's list; list = for rank r: piece x of expert(r)
// Returns false for the workgroups past the end of a list.
__device__ __forceinline__ bool weight_grad_tile(int E, int i_tiles, int n_tiles, int& rank, int& it, int& nt) {
    constexpr int XCDS = 8, GROUP_M = 8;
    const int per_expert = i_tiles * n_tiles;
    const int x = blockIdx.x % XCDS, s = blockIdx.x / XCDS;
    const int lo = per_expert / XCDS, rem = per_expert % XCDS;
    const int mine = lo + (x < rem ? 1 : 0);
    if (mine == 0 || s >= E * mine) return false;
    rank = s / mine;
    const int q = x * lo + min(x, rem) + s % mine;  // position in the expert's grid, grouped order
    const int group_span = GROUP_M * n_tiles;
    const int group = q / group_span;
    const int first = group * GROUP_M;
    const int gm = min(GROUP_M, i_tiles - first);
    const int in_group = q - group * group_span;
    it = first + in_group % gm;
    nt = in_group / gm;
    return true;
}

// Expert with the `rank`-th largest row count (ties: lower index first).  Every wave works it out for itself from
// the offsets: lane e holds the count of expert e and counts the experts ahead of it.  More than 64 experts keep
// their index order (the split over the XCDs above is what matters most).
__device__ __forceinline__ int expert_of_rank(const int64_t* __restrict__ offsets, int E, int rank) {
    if (E > CK_WAVE) return rank;
    const int lane = lane_id();
    int count = -1;
    if (lane < E) count = (int)offsets[lane] - (lane == 0 ? 0 : (int)offsets[lane - 1]);
    int ahead = 0;
    for (int e = 0; e < E; ++e) {
        const int other = __shfl(count, e, CK_WAVE);
        ahead += (other > count || (other == count && e < lane)) ? 1 : 0;
    }
    const uint64_t hit = __ballot(lane < E && ahead == rank);
    return __builtin_amdgcn_readfirstlane(__ffsll((unsigned long long)hit) - 1);
}

// ---- host side: how many workgroups each way of dealing needs ------------------------------------------------------
// m_tiles is the host's bound of the row tile count of the per-expert products (rows / BM + E; the device counts the
// tiles the experts really have), i_tiles the row tiles of one expert's weight gradient.
namespace tile_grid {

// find_tile_balanced: 8 XCD lists, each long enough for either way it deals (an eighth of the tiles, or whole rows of
// the tile grid)
inline int64_t balanced(int64_t m_tiles, int64_t n_tiles) {
    const int64_t even = (m_tiles * n_tiles + 7) / 8;
    const int64_t rows = ((m_tiles + 7) / 8) * n_tiles;
    return 8 * (even > rows ? even : rows);
}
// find_tile_split, first launch: an eighth of the tiles per XCD, and the pieces of a tail take up to 32 places
inline int64_t split(int64_t m_tiles, int64_t n_tiles) { return 8 * ((m_tiles * n_tiles + 7) / 8 + 32); }
// find_tile_split, second launch (fixup): at most 16 split tiles per XCD
inline int64_t split_fixup() { return 8 * 16; }
// weight_grad_tile: 8 lists, each with ceil(tiles per expert / 8) entries per expert
inline int64_t weight_grad(int64_t E, int64_t i_tiles, int64_t n_tiles) { return 8 * E * ((i_tiles * n_tiles + 7) / 8); }

}  // namespace tile_grid

}  // namespace ck

// Host build of the grouped GEMM's tile scheduling (csrc/ck_tile_schedule.h): the device source itself, compiled with
// g++, with a wavefront emulated lane by lane in lockstep at the wave primitives (ballot, shuffle, scan, sum).
// For expert_offsets of many shapes it walks every workgroup of every launch form and checks what the kernels rely on:
//   find_tile_balanced   every (expert, row tile, column tile) exactly once, nothing else, rows inside the expert
//   find_tile_split      the same, with the pieces of a split tile covering the contraction range exactly once, partial
//                        slots unique and below kSplitSlots; the fix-up launch finds every split tile once, with the
//                        first slot and the piece count of the first launch
//   weight_grad_tile     every (expert, row tile, column tile) of every expert's weight gradient exactly once, the
//   + expert_of_rank     experts taken in the order of falling row count
//   find_tile + logical_tile (the 64-bit-address kernel's order)   every tile of the bound grid at most once, every real
//                        tile exactly once
// Exit status 0 and "ok" on success; the first violation is printed and the status is 1.
#include <setjmp.h>

#include <algorithm>
#include <array>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <set>
#include <string>
#include <tuple>
#include <vector>

// ---- the wavefront ---------------------------------------------------------------------------------------------------
#define CK_WAVE 64
#define __device__
#define __forceinline__ inline
#define __restrict__

namespace emu {
// Lockstep by replay: the lanes run one after the other; a lane that reaches a wave primitive whose result is not known
// yet leaves its value there and stops, and once all 64 have stopped at it the results are computed and the lanes start
// over, taking the known results from the log.  The scheduling code has the same control flow in every lane, so all
// lanes stop at the same primitive in every round and finish in the same round (checked).
constexpr int kLanes = CK_WAVE;
enum Kind { kNone, kBallot, kShuffle, kFirst, kScan, kSum, kSync };
int current = 0;     // the lane being run
int known = 0;       // primitives whose results are in the log
int position = 0;    // next primitive of the current lane's run
std::vector<std::array<long long, kLanes>> results;
long long given[kLanes];
int argument[kLanes];
Kind kind_of[kLanes];
jmp_buf leave;

long long primitive(Kind kind, long long mine, int arg = 0) {
    if (position < known) return results[position++][current];
    given[current] = mine;
    argument[current] = arg;
    kind_of[current] = kind;
    longjmp(leave, 1);
}

void run_wave(void (*f)()) {
    results.clear();
    known = 0;
    for (;;) {
        int finished = 0;
        for (int l = 0; l < kLanes; ++l) {
            current = l;
            position = 0;
            kind_of[l] = kNone;
            if (setjmp(leave) == 0) {
                f();
                ++finished;
            }
        }
        if (finished == kLanes) return;
        if (finished != 0) {
            std::printf("FAILED: the lanes of a wave took different paths\n");
            std::exit(1);
        }
        std::array<long long, kLanes> r{};
        for (int l = 1; l < kLanes; ++l)
            if (kind_of[l] != kind_of[0]) {
                std::printf("FAILED: the lanes of a wave stopped at different primitives\n");
                std::exit(1);
            }
        long long running = 0, mask = 0;
        for (int l = 0; l < kLanes; ++l) {
            running += given[l];
            mask |= (long long)((unsigned long long)(given[l] & 1) << l);
            if (kind_of[0] == kScan) r[l] = running;
        }
        for (int l = 0; l < kLanes; ++l) {
            if (kind_of[0] == kBallot) r[l] = mask;
            else if (kind_of[0] == kShuffle) r[l] = given[argument[l] & (kLanes - 1)];
            else if (kind_of[0] == kFirst) r[l] = given[0];
            else if (kind_of[0] == kSum) r[l] = running;
        }
        results.push_back(r);
        ++known;
    }
}
}  // namespace emu

struct Dim3 {
    unsigned x;
};
Dim3 blockIdx{0};
struct ThreadIdx {
    // only the first wavefront of a workgroup runs the searches; the emulated lanes are its threads
    operator unsigned() const { return (unsigned)emu::current; }
};
struct {
    ThreadIdx x;
} threadIdx;

inline int __ffsll(unsigned long long v) { return __builtin_ffsll((long long)v); }
inline uint64_t __ballot(bool p) { return (uint64_t)emu::primitive(emu::kBallot, p ? 1 : 0); }
inline int __shfl(int v, int src, int) { return (int)emu::primitive(emu::kShuffle, v, src); }
inline int __builtin_amdgcn_readfirstlane(int v) { return (int)emu::primitive(emu::kFirst, v); }
inline void __syncthreads() { emu::primitive(emu::kSync, 0); }

namespace ck {
using std::max;
using std::min;
inline int lane_id() { return emu::current; }
inline int wave_inclusive_scan_i(int v) { return (int)emu::primitive(emu::kScan, v); }
inline int wave_sum_i(int v) { return (int)emu::primitive(emu::kSum, v); }
}  // namespace ck

#include "../../kernel-hyperdrive_amd/csrc/ck_tile_schedule.h"

// ---- the checks --------------------------------------------------------------------------------------------------------
namespace {
constexpr int BM = 256, BK = 64;

[[noreturn]] void fail(const char* what, const std::vector<int64_t>& offsets, int n_tiles, int K, long long a = 0, long long b = 0,
                       long long c = 0) {
    std::printf("FAILED: %s (%lld, %lld, %lld)  E=%zu n_tiles=%d K=%d offsets:", what, a, b, c, offsets.size(), n_tiles, K);
    for (size_t i = 0; i < offsets.size() && i < 70; ++i) std::printf(" %lld", (long long)offsets[i]);
    std::printf("\n");
    std::exit(1);
}

struct Problem {
    std::vector<int64_t> offsets;  // inclusive ends
    int E, n_tiles, K;
    int rows() const { return (int)offsets.back(); }
    int begin(int e) const { return e == 0 ? 0 : (int)offsets[e - 1]; }
    int end(int e) const { return (int)offsets[e]; }
    int m_tiles_bound() const { return rows() / BM + E; }
};
const Problem* g_problem;
int g_info[8];
bool g_fixup;
bool g_short_grid = false;  // --short-grid: launch too few workgroups on purpose, to show that the checks notice

// every (expert, first row, column tile) the experts really have
std::set<std::tuple<int, int, int>> real_tiles(const Problem& p) {
    std::set<std::tuple<int, int, int>> s;
    for (int e = 0; e < p.E; ++e)
        for (int r = p.begin(e); r < p.end(e); r += BM)
            for (int nt = 0; nt < p.n_tiles; ++nt) s.insert({e, r, nt});
    return s;
}

void check_rows(const Problem& p, const int* info, const char* what) {
    const int e = info[0], start = info[1], valid = info[2], nt = info[3];
    if (e >= p.E || nt < 0 || nt >= p.n_tiles) fail(what, p.offsets, p.n_tiles, p.K, e, start, nt);
    if (start < p.begin(e) || (start - p.begin(e)) % BM != 0 || valid != std::min(BM, p.end(e) - start) || valid <= 0)
        fail(what, p.offsets, p.n_tiles, p.K, e, start, valid);
}

void balanced(const Problem& p) {
    g_problem = &p;
    auto expected = real_tiles(p);
    std::set<std::tuple<int, int, int>> seen;
    const int64_t grid = ck::tile_grid::balanced(p.m_tiles_bound(), p.n_tiles) - (g_short_grid ? 8 : 0);
    for (int64_t b = 0; b < grid; ++b) {
        blockIdx.x = (unsigned)b;
        emu::run_wave([] { ck::find_tile_balanced<BM>(g_problem->offsets.data(), g_problem->E, g_problem->n_tiles, g_info); });
        if (g_info[0] < 0) continue;
        check_rows(p, g_info, "find_tile_balanced: tile outside its expert");
        if (!seen.insert({g_info[0], g_info[1], g_info[3]}).second)
            fail("find_tile_balanced: tile dealt twice", p.offsets, p.n_tiles, p.K, g_info[0], g_info[1], g_info[3]);
    }
    if (seen != expected) fail("find_tile_balanced: tiles missing", p.offsets, p.n_tiles, p.K, (long long)seen.size(), (long long)expected.size());
}

void split(const Problem& p) {
    g_problem = &p;
    auto expected = real_tiles(p);
    const int k_tiles = (p.K + BK - 1) / BK;
    // tile -> pieces [kt_b, kt_e), slot
    std::map<std::tuple<int, int, int>, std::vector<std::tuple<int, int, int, int>>> pieces;
    std::set<int> slots;
    const int64_t grid = ck::tile_grid::split(p.m_tiles_bound(), p.n_tiles);
    for (int64_t b = 0; b < grid; ++b) {
        blockIdx.x = (unsigned)b;
        g_fixup = false;
        emu::run_wave([] {
            ck::find_tile_split<BM, BK>(g_problem->offsets.data(), g_problem->E, g_problem->n_tiles, g_problem->K, g_fixup, g_info);
        });
        if (g_info[0] < 0) continue;
        check_rows(p, g_info, "find_tile_split: tile outside its expert");
        const int kt_b = g_info[4], kt_e = g_info[5], slot = g_info[6], n = g_info[7];
        if (slot >= 0) {
            if (slot >= ck::kSplitSlots || !slots.insert(slot).second || n < 2 || n > ck::kSplitMax)
                fail("find_tile_split: partial slot", p.offsets, p.n_tiles, p.K, slot, n);
            if (kt_e - kt_b < 1) fail("find_tile_split: empty piece", p.offsets, p.n_tiles, p.K, kt_b, kt_e);
        } else if (kt_b != 0 || kt_e != k_tiles) {
            fail("find_tile_split: a whole tile with a piece's range", p.offsets, p.n_tiles, p.K, kt_b, kt_e);
        }
        pieces[{g_info[0], g_info[1], g_info[3]}].push_back({kt_b, kt_e, slot, n});
    }
    std::map<std::tuple<int, int, int>, std::pair<int, int>> split_tiles;  // tile -> (first slot, pieces)
    for (auto& [tile, list] : pieces) {
        std::sort(list.begin(), list.end());
        int at = 0;
        for (auto& [kb, ke, slot, n] : list) {
            if (kb != at) fail("find_tile_split: pieces do not tile the contraction", p.offsets, p.n_tiles, p.K, kb, at);
            at = ke;
        }
        if (at != k_tiles) fail("find_tile_split: contraction not covered", p.offsets, p.n_tiles, p.K, at, k_tiles);
        if (list.size() > 1) {
            for (size_t i = 0; i < list.size(); ++i)
                if (std::get<2>(list[i]) != std::get<2>(list[0]) + (int)i || std::get<3>(list[i]) != (int)list.size())
                    fail("find_tile_split: slots of a tile not consecutive in piece order", p.offsets, p.n_tiles, p.K, (long long)i);
            split_tiles[tile] = {std::get<2>(list[0]), (int)list.size()};
        } else if (std::get<2>(list[0]) >= 0) {
            fail("find_tile_split: a single piece with a slot", p.offsets, p.n_tiles, p.K);
        }
    }
    std::set<std::tuple<int, int, int>> seen;
    for (auto& kv : pieces) seen.insert(kv.first);
    if (seen != expected) fail("find_tile_split: tiles missing", p.offsets, p.n_tiles, p.K, (long long)seen.size(), (long long)expected.size());
    // the launch that adds the pieces up
    std::set<std::tuple<int, int, int>> fixed;
    for (int64_t b = 0; b < ck::tile_grid::split_fixup(); ++b) {
        blockIdx.x = (unsigned)b;
        g_fixup = true;
        emu::run_wave([] {
            ck::find_tile_split<BM, BK>(g_problem->offsets.data(), g_problem->E, g_problem->n_tiles, g_problem->K, g_fixup, g_info);
        });
        if (g_info[0] < 0) continue;
        check_rows(p, g_info, "find_tile_split (fix-up): tile outside its expert");
        const std::tuple<int, int, int> tile{g_info[0], g_info[1], g_info[3]};
        auto it = split_tiles.find(tile);
        if (it == split_tiles.end() || it->second.first != g_info[6] || it->second.second != g_info[7] || !fixed.insert(tile).second)
            fail("find_tile_split (fix-up): not the first launch's split tile", p.offsets, p.n_tiles, p.K, g_info[0], g_info[1], g_info[6]);
    }
    if (fixed.size() != split_tiles.size()) fail("find_tile_split (fix-up): split tiles left without their sum", p.offsets, p.n_tiles, p.K, (long long)fixed.size(), (long long)split_tiles.size());
}

int g_rank, g_expert;
void weight_grad(const Problem& p, int i_tiles) {
    g_problem = &p;
    std::vector<int> order(p.E);
    for (int e = 0; e < p.E; ++e) order[e] = e;
    if (p.E <= CK_WAVE)
        std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return p.end(a) - p.begin(a) > p.end(b) - p.begin(b); });
    std::set<std::tuple<int, int, int>> seen;
    const int64_t grid = ck::tile_grid::weight_grad(p.E, i_tiles, p.n_tiles);
    int last_rank_of_xcd[8] = {-1, -1, -1, -1, -1, -1, -1, -1};
    for (int64_t b = 0; b < grid; ++b) {
        blockIdx.x = (unsigned)b;
        int rank, it, nt;
        if (!ck::weight_grad_tile(p.E, i_tiles, p.n_tiles, rank, it, nt)) continue;
        if (rank < 0 || rank >= p.E || it < 0 || it >= i_tiles || nt < 0 || nt >= p.n_tiles)
            fail("weight_grad_tile: outside the grid", p.offsets, p.n_tiles, p.K, rank, it, nt);
        if (rank < last_rank_of_xcd[b % 8]) fail("weight_grad_tile: an XCD's list goes back to a larger expert", p.offsets, p.n_tiles, p.K, rank);
        last_rank_of_xcd[b % 8] = rank;
        g_rank = rank;
        emu::run_wave([] {
            const int e = ck::expert_of_rank(g_problem->offsets.data(), g_problem->E, g_rank);
            if (emu::current == 0) g_expert = e;
        });
        if (g_expert != order[rank]) fail("expert_of_rank: not the expert with the rank-th largest row count", p.offsets, p.n_tiles, p.K, rank, g_expert, order[rank]);
        if (!seen.insert({g_expert, it, nt}).second) fail("weight_grad_tile: tile dealt twice", p.offsets, p.n_tiles, p.K, g_expert, it, nt);
    }
    if ((int64_t)seen.size() != (int64_t)p.E * i_tiles * p.n_tiles) fail("weight_grad_tile: tiles missing", p.offsets, p.n_tiles, p.K, (long long)seen.size());
}

int g_mt;
void bound_grid(const Problem& p) {
    // the 64-bit-address kernel: every workgroup of the bound grid maps to a distinct (row tile, column tile); row tiles
    // beyond the experts' own find no expert
    g_problem = &p;
    const int m_tiles = p.m_tiles_bound();
    auto expected = real_tiles(p);
    std::set<std::tuple<int, int, int>> seen;
    std::set<std::pair<int, int>> logical;
    const int grid = (m_tiles * p.n_tiles + 7) / 8 * 8;
    for (int b = 0; b < grid; ++b) {
        blockIdx.x = (unsigned)b;
        int mt, nt;
        if (!ck::logical_tile(m_tiles, p.n_tiles, mt, nt)) continue;
        if (mt < 0 || mt >= m_tiles || nt < 0 || nt >= p.n_tiles || !logical.insert({mt, nt}).second)
            fail("logical_tile: outside the grid or dealt twice", p.offsets, p.n_tiles, p.K, mt, nt);
        g_mt = mt;
        emu::run_wave([] { ck::find_tile<BM>(g_problem->offsets.data(), g_problem->E, g_mt, g_info); });
        if (g_info[0] < 0) continue;
        g_info[3] = nt;
        check_rows(p, g_info, "find_tile: tile outside its expert");
        seen.insert({g_info[0], g_info[1], nt});
    }
    if ((int)logical.size() != m_tiles * p.n_tiles || seen != expected)
        fail("find_tile / logical_tile: tiles missing", p.offsets, p.n_tiles, p.K, (long long)seen.size(), (long long)expected.size());
}

Problem make(std::mt19937& rng, int E, int rows, double skew, int empty, int n_tiles, int K) {
    std::vector<double> w(E);
    for (int e = 0; e < E; ++e) w[e] = 1.0 / std::pow(e + 1.0, skew);
    std::shuffle(w.begin(), w.end(), rng);
    for (int i = 0; i < empty && i < E; ++i) w[rng() % E] = 0.0;
    double total = 0;
    for (double v : w) total += v;
    Problem p;
    p.E = E;
    p.n_tiles = n_tiles;
    p.K = K;
    int64_t at = 0;
    for (int e = 0; e < E; ++e) {
        const int64_t n = total > 0 ? (int64_t)(rows * w[e] / total) : 0;
        at += n;
        p.offsets.push_back(at);
    }
    if (at == 0) p.offsets.back() = std::min(rows, 1);  // at least one row somewhere, unless asked for none
    return p;
}
}  // namespace

int main(int argc, char** argv) {
    g_short_grid = argc > 1 && std::string(argv[1]) == "--short-grid";
    std::mt19937 rng(12345);
    int problems = 0;
    // experts, rows, skew of the row counts, experts emptied, column tiles, contraction length
    const int shapes[][6] = {
        {8, 16384, 0, 0, 16, 14336},  {8, 16384, 0, 0, 16, 28672},  {8, 16384, 0, 0, 112, 4096}, {8, 16384, 0, 0, 56, 4096},
        {64, 98304, 1, 5, 6, 2048},   {64, 98304, 1, 5, 11, 2048},  {64, 98304, 1, 5, 8, 1408},  {3, 600, 0, 0, 1, 4096},
        {4, 200, 0, 1, 2, 8192},      {2, 260, 0, 0, 2, 4160},      {1, 5000, 0, 0, 3, 4096},    {100, 30000, 1, 20, 2, 6400},
        {7, 900, 2, 2, 1, 200},       {33, 70000, 0, 0, 5, 12288},  {8, 1, 0, 0, 1, 64},         {70, 2000, 2, 30, 3, 5000},
    };
    for (auto& s : shapes)
        for (int rep = 0; rep < 2; ++rep) {
            const Problem p = make(rng, s[0], s[1] - rep * (int)(rng() % 97), s[2] * 1.2, s[3], s[4], s[5]);
            balanced(p);
            split(p);
            bound_grid(p);
            weight_grad(p, 1 + (int)(rng() % 12));
            ++problems;
        }
    std::printf("ok: %d problems\n", problems);
    return 0;
}

// Embedding gather (forward) and scatter-add (backward) for gfx950.
//   forward : out[i, :] = W[ids[i], :]                    bit-exact row copy
//             (cute_kernels/kernels/embedding/triton_implementation/kernels_forward.py:13-39)
//   backward: dW = one_hot(ids)^T @ dy  with fp32 accumulation and ONE rounding per element
//             (math: cute_kernels/kernels/embedding/README.md:7-15).  The reference adds rows with
//             floating-point atomics into a zeroed table (kernels_backward.py:13-45); here the token
//             ids are sorted first so that every table row has exactly one writer:
//               1. stable radix sort of (id, position) spread over the GPU (histogram / scan / scatter
//                  per 9-bit digit), then one workgroup marks which table rows are selected at all
//                  and records, for every sorted slot, the first slot of its run of equal ids.
//               2. rows kernel, one launch for two jobs: rows no id selects are written as zeros (the
//                  bulk of the traffic; a part of them rides, as extra workgroups, on the small launches
//                  of step 1 - whole ranges of rows on the two launches before the marks exist, the unmarked
//                  rows of a range on the later ones); a run of equal ids is cut into chunks of
//                  kChunk slots.  A chunk of one row is copied by one wave; the others are summed by the four
//                  waves of a workgroup, a quarter of the columns each, in fp32 registers and in ascending
//                  token position.  A run that fits one chunk is rounded and stored straight into dW; longer
//                  runs leave one fp32 partial row per chunk in the workspace.
//               3. combine kernel: sums the partial rows of each long run and stores the dW row.
//             No floating-point atomics, deterministic.  Of the rows that receive a sum, only those inside the two
//             ranges cleared before the marks exist are written twice.
#include <cstdlib>

#include "ck_block_sort.h"
#include "ck_grid_sort.h"

namespace ck {

// slots of one run summed in one go (measured at 32768 Zipf(1.1) ids, table [128256, 4096]: 16 / 32 / 64 slots 353 /
// 362 / 325 us - fewer partial rows to write and to add up again; ids spread evenly do not care)
constexpr int kChunk = 64;
constexpr int kRowPacks = 8;    // packets per lane per column tile (tile = 64 lanes * 8 packets)

// accumulator of the backward sums
template <typename T>
struct AccOf {
    typedef float type;
};
template <>
struct AccOf<F32> {
    typedef double type;
};

template <bool I32>
__device__ __forceinline__ int64_t load_tok(const void* p, int64_t i) {
    return I32 ? (int64_t) reinterpret_cast<const int32_t*>(p)[i] : reinterpret_cast<const int64_t*>(p)[i];
}

// ---- forward ---------------------------------------------------------------------------------
// One wave per output row, 4 rows per workgroup.  VEC = T::kVec (16-byte packets) or 1.
template <typename T, int VEC, bool I32>
__global__ void __launch_bounds__(256)
    embedding_fwd_kernel(const void* __restrict__ ids, const typename T::storage_t* __restrict__ w,
                         typename T::storage_t* __restrict__ out, int64_t n, int64_t V, int64_t H) {
    typedef VPack<T, VEC> P;
    const int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / CK_WAVE;
    if (row >= n) return;
    const int lane = lane_id();
    const int64_t id = load_tok<I32>(ids, row);
    const int64_t packs = H / VEC;
    P* dst = reinterpret_cast<P*>(out + row * H);
    if (id < 0 || id >= V) {
        P z;
#pragma unroll
        for (int j = 0; j < VEC; ++j) z.v[j] = T::down(0.f);
        for (int64_t p = lane; p < packs; p += CK_WAVE) dst[p] = z;
        return;
    }
    const P* src = reinterpret_cast<const P*>(w + id * H);
    int64_t p = lane;
    // four packets in flight per lane
    for (; p + 3 * CK_WAVE < packs; p += 4 * CK_WAVE) {
        const P a = src[p], b = src[p + CK_WAVE], c = src[p + 2 * CK_WAVE], d = src[p + 3 * CK_WAVE];
        nt_store(a, dst + p);
        nt_store(b, dst + p + CK_WAVE);
        nt_store(c, dst + p + 2 * CK_WAVE);
        nt_store(d, dst + p + 3 * CK_WAVE);
    }
    for (; p < packs; p += CK_WAVE) nt_store(src[p], dst + p);
}

// ---- backward 1: sort -------------------------------------------------------------------------
struct EmbWorkspace {
    uint32_t* keys[2];
    uint32_t* vals[2];
    uint32_t* hist;      // [bins][waves] of the grid sort
    uint32_t* run_head;  // [n] first sorted slot of the run of equal ids that slot i belongs to
    uint8_t* touched;    // [V] 1 when some id selects the row
    float* partial;      // [2 * ceil(n / kChunk)][H]
};

static inline int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

static inline int64_t emb_carve(void* base, int64_t n, int64_t V, int64_t H, EmbWorkspace* ws) {
    int64_t off = 0;
    char* b = (char*)base;
    const int64_t arr = align_up(n * 4, 256);
    for (int i = 0; i < 2; ++i) {
        if (ws) ws->keys[i] = (uint32_t*)(b + off);
        off += arr;
        if (ws) ws->vals[i] = (uint32_t*)(b + off);
        off += arr;
    }
    if (ws) ws->hist = (uint32_t*)(b + off);
    off += align_up((int64_t)(1 << kGridSortMaxBits) * grid_sort_waves(n) * 4, 256);
    if (ws) ws->run_head = (uint32_t*)(b + off);
    off += arr;
    if (ws) ws->touched = (uint8_t*)(b + off);
    off += align_up(V, 256);
    if (ws) ws->partial = (float*)(b + off);
    off += align_up(2 * ((n + kChunk - 1) / kChunk) * H * 4, 256);
    return off;
}

// Sort of the token ids, spread over the GPU (ck_grid_sort.h).  Ids outside [0, V) get the key V: they sort
// last and are skipped by the later kernels.
template <bool I32>
struct IdLoader {
    const void* ids;
    int64_t V;
    __device__ __forceinline__ void operator()(int i, uint32_t& k, uint32_t& v) const {
        const int64_t id = load_tok<I32>(ids, i);
        k = (id < 0 || id >= V) ? (uint32_t)V : (uint32_t)id;
        v = (uint32_t)i;
    }
};
struct PairLoader {
    const uint32_t* keys;
    const uint32_t* vals;
    __device__ __forceinline__ void operator()(int i, uint32_t& k, uint32_t& v) const {
        k = keys[i];
        v = vals[i];
    }
};
struct PairStorer {
    uint32_t* keys;
    uint32_t* vals;
    __device__ __forceinline__ void operator()(int pos, uint32_t k, uint32_t v) const {
        keys[pos] = k;
        vals[pos] = v;
    }
};

// Zero fill of the table rows no id selects, as a side job of the launches that come after the row marks are known.
// Those launches (the sort's scatter / histogram / scan kernels, the run heads) are a handful of workgroups each and
// bound by latency, about 8 us apiece and one behind the other; the fill is the bulk of the operator's bytes and needs
// nothing from them but the marks.  Each of them gets a share of the table's rows as extra workgroups behind its own
// (`first_block` on), so the sort no longer costs time of its own.  One wave takes four consecutive rows: the four
// marks first, then 16-byte packets of zeros (zero bits are zero in every storage type).
struct FillJob {
    const uint8_t* touched;       // null: the marks are not known yet, every row of the share is cleared (the row sums,
                                  // which run later, overwrite the selected ones among them)
    char* dw;
    int64_t row_bytes;            // a multiple of 16
    int64_t row_begin, row_end;   // this launch's share of the rows
    int first_block;              // workgroups [first_block, gridDim.x) belong to the job
};
constexpr int kFillRowsPerWave = 4;

__device__ __forceinline__ bool run_fill_job(const FillJob& f) {
    if ((int)blockIdx.x < f.first_block) return false;
    typedef uint32_t zero_t __attribute__((ext_vector_type(4)));
    const int lane = lane_id();
    const int waves = blockDim.x / CK_WAVE;
    const int64_t row0 =
        f.row_begin + (((int64_t)blockIdx.x - f.first_block) * waves + threadIdx.x / CK_WAVE) * kFillRowsPerWave;
    uint8_t mark[kFillRowsPerWave];
#pragma unroll
    for (int r = 0; r < kFillRowsPerWave; ++r)
        mark[r] = row0 + r < f.row_end ? (f.touched != nullptr ? f.touched[row0 + r] : 0) : 1;
    const zero_t z = {0u, 0u, 0u, 0u};
    const int64_t packs = f.row_bytes / 16;
#pragma unroll
    for (int r = 0; r < kFillRowsPerWave; ++r) {
        if (mark[r]) continue;
        zero_t* dst = reinterpret_cast<zero_t*>(f.dw + (row0 + r) * f.row_bytes);
        for (int64_t p = lane; p < packs; p += CK_WAVE) dst[p] = z;
    }
    return true;
}
// workgroups a launch with `threads` lanes per workgroup needs for the job's rows
static inline int64_t fill_job_blocks(int64_t rows, int threads) {
    const int64_t per_block = (int64_t)(threads / CK_WAVE) * kFillRowsPerWave;
    return (rows + per_block - 1) / per_block;
}

template <typename Loader>
__global__ void __launch_bounds__(256)
    embedding_sort_hist_kernel(Loader load, int n, int shift, int bits, uint32_t* __restrict__ hist, int num_waves,
                               uint32_t* __restrict__ clear, int64_t clear_words, FillJob fill) {
    __shared__ GridSortShared sh;
    if (run_fill_job(fill)) return;
    // side job of the first pass: clear the row marks
    const int64_t own = min((int64_t)gridDim.x, (int64_t)fill.first_block);  // the workgroups that are not the fill's
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < clear_words; i += own * blockDim.x) clear[i] = 0u;
    grid_sort_histogram(sh, n, shift, bits, hist, num_waves, load);
}

// Workgroup 0 scans the histogram.  In the first pass the workgroups behind it mark the table rows some id selects
// (the marks were cleared by the launch before; Loader gives the key V to ids outside the table); in later passes
// they carry a share of the zero fill.
template <typename Loader, bool MARK>
__global__ void __launch_bounds__(1024)
    embedding_sort_scan_kernel(uint32_t* __restrict__ hist, int total, Loader load, int n, int64_t V,
                               uint8_t* __restrict__ touched, FillJob fill) {
    if (blockIdx.x == 0) {
        grid_sort_scan(hist, total);
        return;
    }
    if (run_fill_job(fill)) return;
    if (MARK) {
        // workgroups 1 .. fill.first_block - 1 (all the others, where the launch carries no fill)
        const int64_t markers = min((int64_t)gridDim.x, (int64_t)fill.first_block) - 1;
        const int64_t stride = markers * blockDim.x;
        for (int64_t i = (int64_t)(blockIdx.x - 1) * blockDim.x + threadIdx.x; i < n; i += stride) {
            uint32_t key, val;
            load((int)i, key, val);
            if ((int64_t)key < V) touched[key] = 1;
        }
    }
}

template <typename Loader>
__global__ void __launch_bounds__(256)
    embedding_sort_scatter_kernel(Loader load, PairStorer store, int n, int shift, int bits,
                                  const uint32_t* __restrict__ offsets, int num_waves, FillJob fill) {
    __shared__ GridSortShared sh;
    if (run_fill_job(fill)) return;
    grid_sort_scatter(sh, n, shift, bits, offsets, num_waves, load, store);
}

// Runs of equal ids in the sorted order: records, for every sorted slot, the first slot of its run.  Every wave owns
// kRunsWaveSlots consecutive slots: it first finds the head of the run it starts in (among the 64 slots before its
// first one, else by a 64-way search), then walks its slots 64 at a time carrying the latest head forward with a wave
// max-scan.
constexpr int kRunsWaveSlots = 4 * CK_WAVE;
// the slots [begin, end) of one wave
__device__ __forceinline__ void run_heads_of_range(const uint32_t* __restrict__ skeys, uint32_t* __restrict__ run_head,
                                                   int begin, int end) {
    const int lane = lane_id();
    // head of the run that contains slot `begin`: the last slot j <= begin with skeys[j - 1] != skeys[j]
    int carry = -1;
    const uint32_t first_key = skeys[begin];
    {
        const int j = begin - lane;  // lane 0 looks at begin, lane 63 at begin - 63
        const bool is_head = j >= 0 && (j == 0 || skeys[j - 1] != first_key);
        const uint64_t found = __ballot(is_head);
        if (found != 0) carry = begin - (__ffsll((unsigned long long)found) - 1);
    }
    if (carry < 0) {
        // A run longer than that (a popular id): the keys are sorted, so its head is the first slot that holds the
        // key.  The wave probes 64 evenly spaced slots of the range still in question per round trip, which narrows
        // the range 64 times - three rounds for any number of ids, where a walk back costs one per 64 slots of the run.
        int lo = 0, hi = begin - CK_WAVE;  // the head is in [lo, hi]: slots hi + 1 .. begin were just seen to hold the key
        while (lo < hi) {
            const int step = (hi - lo + CK_WAVE - 1) / CK_WAVE;
            const int pos = min(lo + lane * step, hi);
            const uint64_t eq = __ballot(skeys[pos] == first_key);  // false ... false true ... true along the lanes
            if (eq == 0) {
                lo = min(lo + (CK_WAVE - 1) * step, hi) + 1;
            } else {
                const int f = __ffsll((unsigned long long)eq) - 1;
                hi = min(lo + f * step, hi);
                if (f > 0) lo = min(lo + (f - 1) * step, hi) + 1;
            }
        }
        carry = lo;
    }
    for (int i0 = begin; i0 < end; i0 += CK_WAVE) {
        const int i = i0 + lane;
        int head = -1;
        if (i < end) {
            const uint32_t k = skeys[i];
            if (i == 0 || skeys[i - 1] != k) head = i;
        }
        const int incl = max(wave_inclusive_max_i(head), carry);
        if (i < end) run_head[i] = (uint32_t)incl;
        carry = __shfl(incl, CK_WAVE - 1, CK_WAVE);
    }
}

__global__ void __launch_bounds__(256)
    embedding_runs_kernel(const uint32_t* __restrict__ skeys, uint32_t* __restrict__ run_head, int n, FillJob fill) {
    if (run_fill_job(fill)) return;
    const int gw = (blockIdx.x * blockDim.x + threadIdx.x) / CK_WAVE;
    const int begin = gw * kRunsWaveSlots;
    if (begin >= n) return;
    run_heads_of_range(skeys, run_head, begin, min(begin + kRunsWaveSlots, n));
}

// ---- backward 1, the short form: three launches instead of seven ----------------------------------------------------
// For the id counts this operator sees (tens of thousands) one workgroup sorts the pairs in tens of microseconds
// (ck_block_sort.h: three passes of 6 bits for a 17-bit vocabulary, all in one launch, then the run heads), which is
// less than the zero fill needs anyway: the launch's other workgroups carry all of the fill that is left, in one
// piece and at the rate of a plain fill, where the seven launches of the grid-wide sort each pay a ramp up and down.
// Before it, two small launches clear and set the row marks (and carry an unconditional share of the fill each).
__global__ void __launch_bounds__(256)
    embedding_clear_marks_kernel(uint32_t* __restrict__ clear, int64_t clear_words, FillJob fill) {
    if (run_fill_job(fill)) return;
    const int64_t own = min((int64_t)gridDim.x, (int64_t)fill.first_block);
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < clear_words; i += own * blockDim.x) clear[i] = 0u;
}

template <bool I32>
__global__ void __launch_bounds__(256)
    embedding_mark_kernel(IdLoader<I32> load, int n, int64_t V, uint8_t* __restrict__ touched, FillJob fill) {
    if (run_fill_job(fill)) return;
    const int64_t own = min((int64_t)gridDim.x, (int64_t)fill.first_block);
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += own * blockDim.x) {
        uint32_t key, val;
        load((int)i, key, val);
        if ((int64_t)key < V) touched[key] = 1;
    }
}

// Workgroup 0 sorts (id, position) by id - the sorted pairs end in keys[(passes - 1) & 1] / vals[(passes - 1) & 1], as
// the grid-wide sort leaves them - and records the run heads; the others fill.
template <bool I32>
__global__ void __launch_bounds__(kSortThreads)
    embedding_block_sort_kernel(IdLoader<I32> first_load, uint32_t* keys0, uint32_t* vals0, uint32_t* keys1, uint32_t* vals1,
                                uint32_t* __restrict__ run_head, int n, int key_bits, FillJob fill) {
    __shared__ SortShared sh;
    if (run_fill_job(fill)) return;
    const int passes = ck_sort_passes(key_bits);
    const int bits_per_pass = (key_bits + passes - 1) / passes;
    uint32_t* kbuf[2] = {keys0, keys1};
    uint32_t* vbuf[2] = {vals0, vals1};
    for (int p = 0; p < passes; ++p) {
        const int shift = p * bits_per_pass;
        const int bits = min(bits_per_pass, key_bits - shift);
        const bool first = p == 0;
        const uint32_t* kin = kbuf[(p + 1) & 1];
        const uint32_t* vin = vbuf[(p + 1) & 1];
        uint32_t* kout = kbuf[p & 1];
        uint32_t* vout = vbuf[p & 1];
        auto load = [&](int i, uint32_t& k, uint32_t& v) {
            if (first) {
                first_load(i, k, v);
            } else {
                k = kin[i];
                v = vin[i];
            }
        };
        auto store = [&](int pos, uint32_t k, uint32_t v) {
            kout[pos] = k;
            vout[pos] = v;
        };
        block_radix_pass(sh, n, shift, bits, load, store);
    }
    const uint32_t* skeys = kbuf[(passes - 1) & 1];
    const int wave = threadIdx.x / CK_WAVE;
    for (int begin = wave * kRunsWaveSlots; begin < n; begin += kSortWaves * kRunsWaveSlots)
        run_heads_of_range(skeys, run_head, begin, min(begin + kRunsWaveSlots, n));
}

// ---- backward 2: one launch for the two row-wise jobs ---------------------------------------------
// Workgroups [0, chunk_groups) sum chunks of runs (two dependent memory round trips per wave: latency-bound);
// the remaining workgroups write zeros into the rows nobody selects (pure streaming writes, the bulk of the
// bytes).  Running both in one grid lets the streaming part hide the latency of the other.
//   chunk job: a run of equal ids is cut into chunks of kChunk slots; the dy rows of a chunk are summed in fp32
//   (fp64 for fp32 tables) in ascending token position.  A run that fits one chunk is rounded and stored
//   straight into dW; longer runs leave one fp32 partial row per chunk in the workspace.
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
    embedding_bwd_rows_kernel(const uint32_t* __restrict__ skeys, const uint32_t* __restrict__ spos,
                              const uint32_t* __restrict__ run_head, const uint8_t* __restrict__ touched,
                              const typename T::storage_t* __restrict__ dy, typename T::storage_t* __restrict__ dw,
                              float* __restrict__ partial, int n, int chunk_groups, int64_t V, int64_t H,
                              int64_t fill_begin) {
    typedef VPack<T, VEC> P;
    const int lane = lane_id();
    const int64_t packs = H / VEC;

    if ((int)blockIdx.x >= chunk_groups) {
        // ---- zero fill of the rows [fill_begin, V): what the launches before this one did not carry ----
        const int64_t row = fill_begin + (int64_t)(blockIdx.x - chunk_groups) * 4 + threadIdx.x / CK_WAVE;
        if (row >= V) return;
        if (touched[row]) return;
        P z;
#pragma unroll
        for (int j = 0; j < VEC; ++j) z.v[j] = T::down(0.f);
        P* dst = reinterpret_cast<P*>(dw + row * H);
        for (int64_t p = lane; p < packs; p += CK_WAVE) nt_store(z, dst + p);
        return;
    }

    // ---- chunk sums ----
    // Wave w of the workgroup looks at sorted slot 4 * blockIdx.x + w.  A slot that starts a chunk with a single
    // row is copied by its wave alone.  The other chunk starts are summed by the four waves together, one after the
    // other: each wave takes a quarter of the columns and keeps four rows of the chunk in flight, so a chunk of 32
    // rows is 8 dependent round trips instead of 32 - under the load of the fill a round trip takes several
    // microseconds, and with skewed ids the longest chain set the time of the launch.  The rows are still added in
    // ascending token position, one accumulator per element.
    static_assert(kChunk <= CK_WAVE, "a wave looks at the slots of a chunk with one lane each");
    __shared__ uint32_t sh_pos[4][kChunk];
    __shared__ int sh_cnt[4];     // rows of the chunk that starts at the wave's slot; 0: nothing left to sum
    __shared__ int sh_multi[4];   // 0: the run is this chunk, rounded and stored; else 1 + (slot is the run's head)
    __shared__ uint32_t sh_id[4];
    const int wave = threadIdx.x / CK_WAVE;
    const int i = blockIdx.x * 4 + wave;
    {
        int cnt = 0;
        bool multi = false;
        uint32_t id = 0, pos_l = 0;
        int head = 0;
        if (i < n) {
            // every index load is issued before any of them is used: one round trip
            id = skeys[i];
            head = (int)run_head[i];
            const bool in_range = lane < kChunk && i + lane < n;
            const uint32_t key_l = in_range ? skeys[i + lane] : 0xffffffffu;
            const uint32_t key_next = i + kChunk < n ? skeys[i + kChunk] : 0xffffffffu;  // first slot past the chunk
            pos_l = in_range ? spos[i + lane] : 0u;
            if ((int64_t)id < V && (i - head) % kChunk == 0) {
                // slots of this chunk: leading slots i, i+1, ... with the same id, at most kChunk
                const uint64_t bal = __ballot(key_l == id);
                cnt = bal == ~0ull ? CK_WAVE : __ffsll((unsigned long long)~bal) - 1;  // lane 0 always matches, so cnt >= 1
                const bool continues = cnt == kChunk && key_next == id;
                multi = (i != head) || continues;
            }
        }
        if (cnt == 1 && !multi) {
            // the only row of its id (nearly every slot when ids are spread over a large table): widened and rounded
            // back, the row comes out as it went in, so it is copied - eight packets per lane in flight, no accumulators
            const uint32_t pos = __shfl(pos_l, 0, CK_WAVE);
            const P* src = reinterpret_cast<const P*>(dy + (int64_t)pos * H);
            P* dst = reinterpret_cast<P*>(dw + (int64_t)id * H);
            for (int64_t p0 = 0; p0 < packs; p0 += (int64_t)CK_WAVE * kRowPacks) {
                P v[kRowPacks];
#pragma unroll
                for (int q = 0; q < kRowPacks; ++q) {
                    const int64_t p = p0 + lane + (int64_t)q * CK_WAVE;
                    if (p < packs) v[q] = nt_load(src + p);
                }
#pragma unroll
                for (int q = 0; q < kRowPacks; ++q) {
                    const int64_t p = p0 + lane + (int64_t)q * CK_WAVE;
                    if (p < packs) nt_store(v[q], dst + p);
                }
            }
            cnt = 0;
        }
        if (lane < kChunk) sh_pos[wave][lane] = pos_l;
        if (lane == 0) {
            sh_cnt[wave] = cnt;
            sh_multi[wave] = multi ? 1 + (i == head ? 1 : 0) : 0;
            sh_id[wave] = id;
        }
    }
    __syncthreads();

    // fp32 tables sum in fp64 so that the result is the correctly rounded sum whatever the order
    typedef typename AccOf<T>::type acc_t;
    constexpr int kWavePacks = kRowPacks / 4;  // packets per lane and column tile that one of the four waves takes
    constexpr int kRowsInFlight = 4;
    const int64_t tile = (int64_t)CK_WAVE * kRowPacks;
    for (int owner = 0; owner < 4; ++owner) {
        const int cnt = sh_cnt[owner];
        if (cnt == 0) continue;  // the same for all four waves
        const int multi = sh_multi[owner];
        const int64_t id = sh_id[owner];
        const int slot_i = blockIdx.x * 4 + owner;
        for (int64_t p0 = 0; p0 < packs; p0 += tile) {
            acc_t acc[kWavePacks][VEC];
#pragma unroll
            for (int q = 0; q < kWavePacks; ++q)
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[q][j] = 0;
            for (int r0 = 0; r0 < cnt; r0 += kRowsInFlight) {
                P v[kRowsInFlight][kWavePacks];
#pragma unroll
                for (int u = 0; u < kRowsInFlight; ++u) {
                    if (r0 + u < cnt) {
                        const P* src = reinterpret_cast<const P*>(dy + (int64_t)sh_pos[owner][r0 + u] * H);
#pragma unroll
                        for (int q = 0; q < kWavePacks; ++q) {
                            const int64_t p = p0 + lane + (int64_t)(wave * kWavePacks + q) * CK_WAVE;
                            if (p < packs) v[u][q] = nt_load(src + p);
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < kRowsInFlight; ++u) {
                    if (r0 + u < cnt) {
#pragma unroll
                        for (int q = 0; q < kWavePacks; ++q) {
                            const int64_t p = p0 + lane + (int64_t)(wave * kWavePacks + q) * CK_WAVE;
                            if (p < packs) {
#pragma unroll
                                for (int j = 0; j < VEC; ++j) acc[q][j] += (acc_t)T::up(v[u][q].v[j]);
                            }
                        }
                    }
                }
            }
            if (multi == 0) {
                P* dst = reinterpret_cast<P*>(dw + id * H);
#pragma unroll
                for (int q = 0; q < kWavePacks; ++q) {
                    const int64_t p = p0 + lane + (int64_t)(wave * kWavePacks + q) * CK_WAVE;
                    if (p < packs) {
                        P o;
#pragma unroll
                        for (int j = 0; j < VEC; ++j) o.v[j] = T::down((float)acc[q][j]);
                        nt_store(o, dst + p);
                    }
                }
            } else {
                // at most two chunk starts of long runs fall into one window of kChunk slots: the last chunk
                // of one run and the head of the next, told apart by the low bit
                const int64_t slot = 2 * (int64_t)(slot_i / kChunk) + (multi == 2 ? 1 : 0);
                float* dst = partial + slot * H;
#pragma unroll
                for (int q = 0; q < kWavePacks; ++q) {
                    const int64_t p = p0 + lane + (int64_t)(wave * kWavePacks + q) * CK_WAVE;
                    if (p < packs) {
                        if (VEC % 4 == 0) {
#pragma unroll
                            for (int j = 0; j + 3 < VEC; j += 4)
                                *reinterpret_cast<float4*>(dst + p * VEC + j) = make_float4(
                                    (float)acc[q][j], (float)acc[q][j + 1], (float)acc[q][j + 2], (float)acc[q][j + 3]);
                        } else {
#pragma unroll
                            for (int j = 0; j < VEC; ++j) dst[p * VEC + j] = (float)acc[q][j];
                        }
                    }
                }
            }
        }
    }
}

// ---- backward 3: add up the partial rows of long runs ------------------------------------------------
// Workgroup (g, part) looks at the 64 sorted slots [64 g, 64 g + 64): the slots that head a run longer than kChunk
// are found with one coalesced look, then the whole workgroup sums, for each of them in turn, the partial rows
// of the run over its share (`part`) of the columns, eight partial rows in flight per lane.
constexpr int kCombineParts = 16;

template <typename T>
__global__ void __launch_bounds__(256)
    embedding_bwd_combine_kernel(const uint32_t* __restrict__ skeys, const uint32_t* __restrict__ run_head,
                                 const float* __restrict__ partial, typename T::storage_t* __restrict__ dw, int n,
                                 int64_t V, int64_t H) {
    __shared__ unsigned long long sh_hits;
    if (threadIdx.x < CK_WAVE) {
        const int i = blockIdx.x * CK_WAVE + threadIdx.x;
        bool hit = false;
        if (i < n) {
            const uint32_t id = skeys[i];
            hit = (int64_t)id < V && (int)run_head[i] == i && i + kChunk < n && skeys[i + kChunk] == id;
        }
        const uint64_t hits = __ballot(hit);
        if (threadIdx.x == 0) sh_hits = hits;
    }
    __syncthreads();
    uint64_t hits = sh_hits;
    typedef typename AccOf<T>::type acc_t;
    const int64_t cols = (H + kCombineParts - 1) / kCombineParts;
    const int64_t c0 = (int64_t)blockIdx.y * cols;
    const int64_t c1 = c0 + cols < H ? c0 + cols : H;
    while (hits != 0) {
        const int i = blockIdx.x * CK_WAVE + (__ffsll((unsigned long long)hits) - 1);
        hits &= hits - 1;
        const uint32_t id = skeys[i];
        // number of chunks of the run: chunk starts i, i + kChunk, ... that still hold this id
        int chunks = 0;
        for (int base = 0;; base += 256) {
            const int64_t s = (int64_t)i + (int64_t)(base + threadIdx.x) * kChunk;
            const int c = __syncthreads_count(s < n && skeys[s] == id);
            chunks += c;
            if (c < 256) break;
        }
        const int64_t first_slot = 2 * (int64_t)(i / kChunk) + 1;
        for (int64_t c = c0 + threadIdx.x; c < c1; c += 256) {
            acc_t acc = (acc_t)partial[first_slot * H + c];
            int k = 1;
            for (; k + 7 < chunks; k += 8) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = partial[2 * (int64_t)((i + (k + u) * kChunk) / kChunk) * H + c];
#pragma unroll
                for (int u = 0; u < 8; ++u) acc += (acc_t)v[u];
            }
            for (; k < chunks; ++k) acc += (acc_t)partial[2 * (int64_t)((i + k * kChunk) / kChunk) * H + c];
            dw[(int64_t)id * H + c] = T::down((float)acc);
        }
    }
}

}  // namespace ck

template <typename T, int VEC, bool I32>
static void launch_fwd(unsigned grid, hipStream_t s, const void* ids, const void* weight, void* output, int64_t n,
                       int64_t V, int64_t H) {
    typedef typename T::storage_t S;
    hipLaunchKernelGGL((ck::embedding_fwd_kernel<T, VEC, I32>), dim3(grid), dim3(256), 0, s, ids, (const S*)weight,
                       (S*)output, n, V, H);
}

extern "C" int ck_embedding_forward(const void* ids, int ids_are_i32, const void* weight, void* output,
                                    int64_t num_ids, int64_t V, int64_t H, int dtype, void* stream) {
    if (num_ids < 0 || V < 0 || H < 0) return CK_ERR_SHAPE;
    if (num_ids == 0 || H == 0) return CK_OK;
    if (!ids || !output || (V > 0 && !weight)) return CK_ERR_NULL;
    if (!ck_aligned_elem(output, dtype) || (weight && !ck_aligned_elem(weight, dtype))) return CK_ERR_ALIGN;
    const int64_t grid = ck_ceil_div(num_ids, 4);
    if (grid > 0x7fffffff) return CK_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    CK_DISPATCH_DTYPE(dtype, {
        const bool vec = ck_aligned16(weight) && ck_aligned16(output) && (H % T::kVec == 0);
        if (vec) {
            if (ids_are_i32) launch_fwd<T, T::kVec, true>((unsigned)grid, s, ids, weight, output, num_ids, V, H);
            else launch_fwd<T, T::kVec, false>((unsigned)grid, s, ids, weight, output, num_ids, V, H);
        } else {
            if (ids_are_i32) launch_fwd<T, 1, true>((unsigned)grid, s, ids, weight, output, num_ids, V, H);
            else launch_fwd<T, 1, false>((unsigned)grid, s, ids, weight, output, num_ids, V, H);
        }
    });
    return ck_launch_status();
}

extern "C" int64_t ck_embedding_backward_workspace_size(int64_t num_ids, int64_t V, int64_t H) {
    if (num_ids < 0 || V < 0 || H < 0) return 0;
    return ck::emb_carve(nullptr, num_ids, V, H, nullptr);
}

// (measured at a table of [128256, 4096] and 32768 ids, seven carrying launches: 290 / 285 / 285 / 288 / 292 us with
// 60 / 80 / 100 / 120 / 150 MB each; Zipf(1.1) ids 352 / 343 / 339 / 338 / 339 us)
constexpr int64_t kCarrierFillBytes = (int64_t)100 << 20;

// ids the one-workgroup sort of the short prelude takes (beyond that the grid-wide sort is the faster one by far)
constexpr int kBlockSortMaxIds = 1 << 17;
// CK_EMBEDDING_BWD_PRELUDE=short selects the three-launch prelude where it applies (default: the grid-wide sort)
static int embedding_backward_prelude() {
    const char* v = getenv("CK_EMBEDDING_BWD_PRELUDE");
    return v && v[0] == 's' ? 1 : 0;
}

template <typename T, int VEC>
static void launch_bwd(hipStream_t s, const ck::EmbWorkspace& ws, int passes, const void* dy, void* dw, int n,
                       int64_t V, int64_t H, int64_t fill_begin) {
    typedef typename T::storage_t S;
    const uint32_t* skeys = ws.keys[(passes - 1) & 1];
    const uint32_t* spos = ws.vals[(passes - 1) & 1];
    const int chunk_groups = (int)ck_ceil_div(n, 4);
    const int64_t fill_groups = ck_ceil_div(V - fill_begin, 4);
    if (chunk_groups + fill_groups > 0)
        hipLaunchKernelGGL((ck::embedding_bwd_rows_kernel<T, VEC>), dim3((unsigned)(chunk_groups + fill_groups)), dim3(256),
                           0, s, skeys, spos, ws.run_head, ws.touched, (const S*)dy, (S*)dw, ws.partial, n, chunk_groups, V, H,
                           fill_begin);
    if (n > 0)
        hipLaunchKernelGGL((ck::embedding_bwd_combine_kernel<T>), dim3((unsigned)ck_ceil_div(n, CK_WAVE), ck::kCombineParts),
                           dim3(256), 0, s, skeys, ws.run_head, ws.partial, (S*)dw, n, V, H);
}

extern "C" int ck_embedding_backward(const void* ids, int ids_are_i32, const void* output_grad, void* weight_grad,
                                     void* workspace, int64_t workspace_bytes, int64_t num_ids, int64_t V, int64_t H,
                                     int dtype, void* stream) {
    if (num_ids < 0 || V < 0 || H < 0 || num_ids > 0x7fffffff || V >= 0xffffffffll) return CK_ERR_SHAPE;
    if (dtype != CK_F32 && dtype != CK_F16 && dtype != CK_BF16) return CK_ERR_DTYPE;
    if (V == 0 || H == 0) return CK_OK;
    if (!weight_grad || (num_ids > 0 && (!ids || !output_grad))) return CK_ERR_NULL;
    if (!ck_aligned_elem(weight_grad, dtype) || (output_grad && !ck_aligned_elem(output_grad, dtype)))
        return CK_ERR_ALIGN;
    if (ck_ceil_div(V, 4) + ck_ceil_div(num_ids, 4) > 0x7fffffff) return CK_ERR_SHAPE;
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return CK_ERR_WORKSPACE;
    if (workspace_bytes < ck_embedding_backward_workspace_size(num_ids, V, H)) return CK_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    ck::EmbWorkspace ws;
    ck::emb_carve(workspace, num_ids, V, H, &ws);
    const int key_bits = ck::ck_key_bits(V + 1);  // one extra key value marks ids outside [0, V)
    const int passes = (key_bits + ck::kGridSortMaxBits - 1) / ck::kGridSortMaxBits;
    const int bits_per_pass = (key_bits + passes - 1) / passes;
    const int n = (int)num_ids;
    const int num_waves = ck::grid_sort_waves(n);
    const unsigned sort_grid = (unsigned)(num_waves > 0 ? ck_ceil_div(num_waves, ck::kGridSortBlockWaves) : 1);
    const int64_t clear_words = (V + 3) / 4;
    // The zero fill of the rows nobody selects rides on the launches before the row sums: the three launches of every
    // pass and the run heads.  The first two launches run before the marks exist (the second one sets them): their
    // shares are cleared whole, and the row sums overwrite the selected rows among them later.  Needs rows of whole
    // 16-byte packets; otherwise (and without ids) the rows kernel fills, as it sums.
    const int64_t row_bytes = H * ck_elem_size(dtype);
    const bool spread_fill = n > 0 && row_bytes % 16 == 0 && ck_aligned16(weight_grad);
    const int carriers = 3 * passes + 1;
    // a carrier's own work leaves most of the GPU idle for about 8 us: that much fill is free, more only moves time
    // from the row-sum launch, where the fill hides the latency of the sums, to here
    int64_t spread_rows = spread_fill ? carriers * (kCarrierFillBytes / row_bytes) : 0;
    if (spread_rows > V) spread_rows = V;
    const bool short_prelude = spread_fill && n <= kBlockSortMaxIds && embedding_backward_prelude() == 1;
    if (short_prelude) {
        // clear marks | set marks | sort + run heads, with the fill on all three: an unconditional share on each of the
        // first two (the marks do not exist yet), everything else - by the marks - on the third
        const int64_t share = kCarrierFillBytes / row_bytes < V / 2 ? kCarrierFillBytes / row_bytes : V / 2;
        ck::FillJob f = {nullptr, (char*)weight_grad, row_bytes, 0, share, 4};
        hipLaunchKernelGGL(ck::embedding_clear_marks_kernel, dim3((unsigned)(4 + ck::fill_job_blocks(share, 256))), dim3(256),
                           0, s, (uint32_t*)ws.touched, clear_words, f);
        const int mark_own = (int)ck_ceil_div(n, 4 * 256);
        const unsigned mark_grid = (unsigned)(mark_own + ck::fill_job_blocks(share, 256));
        const unsigned sort_grid_1 = (unsigned)(1 + ck::fill_job_blocks(V - 2 * share, ck::kSortThreads));
        const ck::FillJob mark_fill = {nullptr, (char*)weight_grad, row_bytes, share, 2 * share, mark_own};
        const ck::FillJob sort_fill = {ws.touched, (char*)weight_grad, row_bytes, 2 * share, V, 1};
        if (ids_are_i32) {
            const ck::IdLoader<true> load = {ids, V};
            hipLaunchKernelGGL(ck::embedding_mark_kernel<true>, dim3(mark_grid), dim3(256), 0, s, load, n, V, ws.touched,
                               mark_fill);
            hipLaunchKernelGGL(ck::embedding_block_sort_kernel<true>, dim3(sort_grid_1), dim3(ck::kSortThreads), 0, s, load,
                               ws.keys[0], ws.vals[0], ws.keys[1], ws.vals[1], ws.run_head, n, key_bits, sort_fill);
        } else {
            const ck::IdLoader<false> load = {ids, V};
            hipLaunchKernelGGL(ck::embedding_mark_kernel<false>, dim3(mark_grid), dim3(256), 0, s, load, n, V, ws.touched,
                               mark_fill);
            hipLaunchKernelGGL(ck::embedding_block_sort_kernel<false>, dim3(sort_grid_1), dim3(ck::kSortThreads), 0, s, load,
                               ws.keys[0], ws.vals[0], ws.keys[1], ws.vals[1], ws.run_head, n, key_bits, sort_fill);
        }
        const int sort_passes = ck::ck_sort_passes(key_bits);
        CK_DISPATCH_DTYPE(dtype, {
            const bool vec = ck_aligned16(weight_grad) && (!output_grad || ck_aligned16(output_grad)) && (H % T::kVec == 0);
            if (vec) launch_bwd<T, T::kVec>(s, ws, sort_passes, output_grad, weight_grad, (int)num_ids, V, H, V);
            else launch_bwd<T, 1>(s, ws, sort_passes, output_grad, weight_grad, (int)num_ids, V, H, V);
        });
        return ck_launch_status();
    }
    int carrier = 0;
    auto fill_share = [&](int own_blocks, int threads, unsigned& grid, bool marks_known = true) {
        ck::FillJob f = {marks_known ? ws.touched : nullptr, (char*)weight_grad, row_bytes, 0, 0, 0x7fffffff};
        grid = (unsigned)own_blocks;
        if (spread_fill) {
            f.row_begin = spread_rows * carrier / carriers;
            f.row_end = spread_rows * (carrier + 1) / carriers;
            f.first_block = own_blocks;
            grid = (unsigned)(own_blocks + ck::fill_job_blocks(f.row_end - f.row_begin, threads));
            ++carrier;
        }
        return f;
    };
    // workgroups of the second launch that mark the selected rows (behind the one that scans)
    const unsigned mark_blocks = (unsigned)(n > 0 ? ck_ceil_div(n, 4 * 1024) : 0);
    for (int p = 0; p < passes; ++p) {
        const int shift = p * bits_per_pass;
        const int bits = key_bits - shift < bits_per_pass ? key_bits - shift : bits_per_pass;
        const int total = (1 << bits) * num_waves;
        ck::PairStorer store = {ws.keys[p & 1], ws.vals[p & 1]};
        unsigned grid = 0;
        if (p == 0) {
            // the clear of the row marks rides on the first histogram launch (needs at least one workgroup)
            if (ids_are_i32) {
                ck::IdLoader<true> load = {ids, V};
                ck::FillJob f = fill_share((int)sort_grid, 256, grid, false);
                hipLaunchKernelGGL((ck::embedding_sort_hist_kernel<ck::IdLoader<true>>), dim3(grid), dim3(256), 0, s,
                                   load, n, shift, bits, ws.hist, num_waves, (uint32_t*)ws.touched, clear_words, f);
                f = fill_share(1 + (int)mark_blocks, 1024, grid, false);
                hipLaunchKernelGGL((ck::embedding_sort_scan_kernel<ck::IdLoader<true>, true>), dim3(grid), dim3(1024), 0, s,
                                   ws.hist, total, load, n, V, ws.touched, f);
                f = fill_share((int)sort_grid, 256, grid);
                hipLaunchKernelGGL((ck::embedding_sort_scatter_kernel<ck::IdLoader<true>>), dim3(grid), dim3(256), 0, s,
                                   load, store, n, shift, bits, ws.hist, num_waves, f);
            } else {
                ck::IdLoader<false> load = {ids, V};
                ck::FillJob f = fill_share((int)sort_grid, 256, grid, false);
                hipLaunchKernelGGL((ck::embedding_sort_hist_kernel<ck::IdLoader<false>>), dim3(grid), dim3(256), 0, s,
                                   load, n, shift, bits, ws.hist, num_waves, (uint32_t*)ws.touched, clear_words, f);
                f = fill_share(1 + (int)mark_blocks, 1024, grid, false);
                hipLaunchKernelGGL((ck::embedding_sort_scan_kernel<ck::IdLoader<false>, true>), dim3(grid), dim3(1024), 0, s,
                                   ws.hist, total, load, n, V, ws.touched, f);
                f = fill_share((int)sort_grid, 256, grid);
                hipLaunchKernelGGL((ck::embedding_sort_scatter_kernel<ck::IdLoader<false>>), dim3(grid), dim3(256), 0, s,
                                   load, store, n, shift, bits, ws.hist, num_waves, f);
            }
        } else {
            ck::PairLoader load = {ws.keys[(p + 1) & 1], ws.vals[(p + 1) & 1]};
            ck::FillJob f = fill_share((int)sort_grid, 256, grid);
            hipLaunchKernelGGL((ck::embedding_sort_hist_kernel<ck::PairLoader>), dim3(grid), dim3(256), 0, s, load, n, shift,
                               bits, ws.hist, num_waves, (uint32_t*)nullptr, (int64_t)0, f);
            f = fill_share(1, 1024, grid);
            hipLaunchKernelGGL((ck::embedding_sort_scan_kernel<ck::PairLoader, false>), dim3(grid), dim3(1024), 0, s, ws.hist,
                               total, load, n, V, ws.touched, f);
            f = fill_share((int)sort_grid, 256, grid);
            hipLaunchKernelGGL((ck::embedding_sort_scatter_kernel<ck::PairLoader>), dim3(grid), dim3(256), 0, s, load, store,
                               n, shift, bits, ws.hist, num_waves, f);
        }
    }
    if (n > 0) {
        unsigned grid = 0;
        const ck::FillJob f = fill_share((int)ck_ceil_div(n, 4 * ck::kRunsWaveSlots), 256, grid);
        hipLaunchKernelGGL(ck::embedding_runs_kernel, dim3(grid), dim3(256), 0, s, ws.keys[(passes - 1) & 1], ws.run_head, n,
                           f);
    }
    CK_DISPATCH_DTYPE(dtype, {
        const bool vec = ck_aligned16(weight_grad) && (!output_grad || ck_aligned16(output_grad)) && (H % T::kVec == 0);
        if (vec) launch_bwd<T, T::kVec>(s, ws, passes, output_grad, weight_grad, (int)num_ids, V, H, spread_rows);
        else launch_bwd<T, 1>(s, ws, passes, output_grad, weight_grad, (int)num_ids, V, H, spread_rows);
    });
    return ck_launch_status();
}

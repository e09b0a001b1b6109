// Grouped GEMMs of the scattermoe layer for gfx950:
//   ck_scatter2scatter : out[out_row(i)] = X[in_row(i)] @ W[e(i)]        (forward and dX)
//       cute_kernels/kernels/scattermoe/triton_implementation/kernels.py:8-149
//   ck_group_bwd_W     : DW[e] = X_e^T @ DY_e                            (dW)
//       cute_kernels/kernels/scattermoe/triton_implementation/kernels.py:152-240
//   ck_group           : out[i] = A[idx[i] / fan_out] * coeff[idx[i]]    (row gather)
//       cute_kernels/kernels/scattermoe/triton_implementation/kernels.py:243-298
//
// 16-bit types run on the matrix cores: v_mfma_f32_16x16x32_{bf16,f16} (which sustains a higher rate on real data
// under the power limit than the 32x32x16 shape), fp32 accumulators, operand tiles copied straight into
// double-buffered LDS.  Tiles are scheduled per expert from expert_offsets, so a tile
// never mixes rows of two experts (the reference lets a 128-row block straddle experts and repeats the
// product once per expert present in it).  fp32, and shapes whose contiguous dimensions are not
// multiples of 8 elements, go through a plain kernel with exact (fp64) accumulation.
#include <cstdlib>
#include <type_traits>

#include "ck_device.h"
#include "ck_gemm_prims.h"

namespace ck {

// ---- MFMA wrappers ---------------------------------------------------------------------------
template <typename T>
struct Mma;
template <>
struct Mma<BF16> {
    typedef bf16x8_t frag_t;
    static __device__ __forceinline__ f32x16_t mma(frag_t a, frag_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <>
struct Mma<F16> {
    typedef f16x8_t frag_t;
    static __device__ __forceinline__ f32x16_t mma(frag_t a, frag_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

template <typename T>
struct Mma16;
template <>
struct Mma16<BF16> {
    typedef bf16x8_t frag_t;
    static __device__ __forceinline__ f32x4_t mma(frag_t a, frag_t b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    // the same with the accumulator pinned to the accumulation half of the register file
    static __device__ __forceinline__ void mma_acc(frag_t a, frag_t b, f32x4_t& c) { mfma16_acc(a, b, c); }
};
template <>
struct Mma16<F16> {
    typedef f16x8_t frag_t;
    static __device__ __forceinline__ f32x4_t mma(frag_t a, frag_t b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void mma_acc(frag_t a, frag_t b, f32x4_t& c) { mfma16_acc(a, b, c); }
};

struct GemmParams {
    const void* A;  // S2S: X [*, K]            XTY: P [rows, I]  (C = P^T Q)
    const void* B;  // S2S: W view              XTY: Q [rows, J]
    void* C;        // S2S: out [slots, N]      XTY: C [E, I, J], J contiguous
    int64_t lda, ldb, ldc;
    int64_t b_stride_e, c_stride_e;
    const int64_t* row_idx;  // S2S: sorted_scattered_idxs
    const int64_t* offsets;  // inclusive expert ends, [E]
    int M, N, K, E;          // S2S: slots, N, K.  XTY: rows, J (= N), I (= K)
    int fan_out, x_grouped, y_grouped;
    int m_tiles, n_tiles;    // S2S: upper bound of row tiles; XTY: tiles along I
    int wide;                // operands too large for 32-bit byte offsets inside a tile's source
    // SwiGLU fused into the epilogue (kernel template argument GLU):
    //   1: C = h [slots, 2 * glu_half] (up | gate halves), aux = act [slots, glu_half] written as well
    //   2: the product is d_act (N = glu_half columns), aux = h read, C = d_h [slots, 2 * glu_half] written
    void* aux;
    int64_t ld_aux;
    int glu_half;
    // Tail splitting of the per-expert products (kernel template argument MODE, see find_tile_split): fp32 partial
    // tiles, kSplitSlots of them, BM * BN floats each
    float* partials;
    // S2S without activation: bias [E, N] of the operands' type, or null.  Added to the fp32 sums before they are
    // rounded, as F.linear(rows, W[e], bias[e]) rounds once (cute_kernels/kernels/scattermoe/torch_implementation.py:35-43).
    const void* bias;
    int waves;  // host side only: which loop the launch takes (0: the library's choice, 4, 8)
};

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

}  // namespace ck

#include "ck_tile_schedule.h"

namespace ck {

// Tile shape of the MFMA kernel.  BM x BN outputs per workgroup, BK of the contraction per step,
// WM x WN wavefronts each owning a (BM/WM) x (BN/WN) block of 32x32 MFMA tiles.
template <int BM_, int BN_, int BK_, int WM_, int WN_>
struct Tile {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
    static constexpr int THREADS = WM * WN * CK_WAVE;
    static constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
};

typedef short v4i16_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4i16_t* lds_v4i16_ptr;

// Operand tile in LDS.
//   KC = true : [ROWS][BK + 8]  (contraction contiguous); an MFMA fragment is one 16-byte read per lane; the
//               8-element pad makes consecutive rows fall 36 dwords apart, which spreads 16 lanes over all banks
//   KC = false: [BK][ROWS + 32] (output dimension contiguous); fragments come from two transposing reads
//               (ds_read_b64_tr_b16): inside each group of 16 lanes, 4 lanes fetch one contraction row of 16
//               elements and lane i receives element i of each of the 4 rows
template <typename S, int ROWS, int BK, bool KC>
struct OperandTile {
    static constexpr int LD = KC ? BK + 8 : ROWS + 32;
    static constexpr int LINES = KC ? ROWS : BK;
    static constexpr int ELEMS = LINES * LD;
    static constexpr int CHUNKS_PER_LINE = (KC ? BK : ROWS) / 8;

    // fragment for the 32 rows starting at `r0`, contraction offset `kk` (multiple of 16)
    template <typename frag_t>
    static __device__ __forceinline__ frag_t fragment(const S* tile, int r0, int kk, int lane) {
        if (KC) {
            return *reinterpret_cast<const frag_t*>(tile + (r0 + lane % 32) * LD + kk + (lane / 32) * 8);
        } else {
            const int g = lane / 16, i = lane % 16;
            const S* p = tile + (kk + (g / 2) * 8 + i / 4) * LD + r0 + (g % 2) * 16 + (i % 4) * 4;
            union {
                v4i16_t h[2];
                frag_t f;
            } u;
            u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(p));
            u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(p + 4 * LD));
            return u.f;
        }
    }
};

// GROUP_K = false ("S2S"): C[row map] = A[row map] (k contiguous) x B, B k-contiguous (B_KC) or n-contiguous.
// GROUP_K = true  ("XTY"): C[e] = P_e^T Q_e, both operands contiguous along the output dimension; the
//                          contraction runs over the expert's rows.
template <typename T, typename TL, bool B_KC, bool GROUP_K>
__global__ void __launch_bounds__(TL::THREADS) grouped_gemm_kernel(GemmParams p) {
    typedef typename T::storage_t S;
    typedef typename Mma<T>::frag_t frag_t;
    constexpr int BM = TL::BM, BN = TL::BN, BK = TL::BK, WM = TL::WM, WN = TL::WN;
    constexpr int THREADS = TL::THREADS, TM = TL::TM, TN = TL::TN;
    constexpr bool A_KC = !GROUP_K;
    constexpr bool B_KCC = GROUP_K ? false : B_KC;
    typedef OperandTile<S, BM, BK, A_KC> ATile;
    typedef OperandTile<S, BN, BK, B_KCC> BTile;
    constexpr int C_LD = BN + 8;  // staged output tile [BM][BN + 8]
    constexpr int STAGE_ELEMS = ATile::ELEMS + BTile::ELEMS;
    constexpr int LDS_ELEMS = (2 * STAGE_ELEMS > BM * C_LD) ? 2 * STAGE_ELEMS : BM * C_LD;
    __shared__ __attribute__((aligned(16))) S lds[LDS_ELEMS];
    __shared__ int sh_info[4];

    int mt, nt;
    if (!logical_tile(p.m_tiles, p.n_tiles, mt, nt)) return;

    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int wave = tid / CK_WAVE;
    const int wm = wave / WN, wn = wave % WN;

    // ---- which rows / which contraction range ------------------------------------------------
    int expert, row_start, rows_valid;  // S2S: rows of this tile.  XTY: output rows of this tile
    int k_begin, k_end;                 // contraction range
    int i_base;                         // XTY: first output row of this tile
    if (!GROUP_K) {
        find_tile<BM>(p.offsets, p.E, mt, sh_info);
        expert = sh_info[0];
        row_start = sh_info[1];
        rows_valid = sh_info[2];
        if (expert < 0) return;
        k_begin = 0;
        k_end = p.K;
        i_base = 0;
    } else {
        const int i_tiles = p.m_tiles / p.E;
        expert = mt / i_tiles;
        i_base = (mt % i_tiles) * BM;
        k_begin = expert == 0 ? 0 : (int)p.offsets[expert - 1];
        k_end = (int)p.offsets[expert];
        row_start = 0;
        rows_valid = min(BM, p.K - i_base);
    }
    const int n_base = nt * BN;

    // ---- global -> register staging ------------------------------------------------------------
    constexpr int A_CH = ATile::LINES * ATile::CHUNKS_PER_LINE / THREADS;
    constexpr int B_CH = BTile::LINES * BTile::CHUNKS_PER_LINE / THREADS;
    static_assert(ATile::LINES * ATile::CHUNKS_PER_LINE % THREADS == 0, "A tile / threads");
    static_assert(BTile::LINES * BTile::CHUNKS_PER_LINE % THREADS == 0, "B tile / threads");

    const S* a_src[A_CH];  // S2S: row base pointers (nullptr = row outside the tile)
    if (A_KC) {
#pragma unroll
        for (int i = 0; i < A_CH; ++i) {
            const int r = (tid + i * THREADS) / ATile::CHUNKS_PER_LINE;
            a_src[i] = nullptr;
            if (r < rows_valid) {
                const int64_t slot = row_start + r;
                const int64_t src_row = p.x_grouped ? slot : p.row_idx[slot] / p.fan_out;
                a_src[i] = reinterpret_cast<const S*>(p.A) + src_row * p.lda;
            }
        }
    }
    const S* Abase = reinterpret_cast<const S*>(p.A);
    const S* Bbase = reinterpret_cast<const S*>(p.B) + (GROUP_K ? 0 : (int64_t)expert * p.b_stride_e);

    u32x4_t a_reg[A_CH], b_reg[B_CH];
    auto load_tiles = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_CH; ++i) {
            const int c = tid + i * THREADS;
            const int r = c / ATile::CHUNKS_PER_LINE;
            const int cc = (c % ATile::CHUNKS_PER_LINE) * 8;
            u32x4_t v = {0u, 0u, 0u, 0u};
            if (A_KC) {
                // row r of the tile, k = k0 + cc .. +7
                if (a_src[i] != nullptr && k0 + cc < k_end) v = *reinterpret_cast<const u32x4_t*>(a_src[i] + k0 + cc);
            } else {
                // contraction row k0 + r, output rows i_base + cc .. +7
                if (k0 + r < k_end && i_base + cc < p.K)
                    v = *reinterpret_cast<const u32x4_t*>(Abase + (int64_t)(k0 + r) * p.lda + i_base + cc);
            }
            a_reg[i] = v;
        }
#pragma unroll
        for (int i = 0; i < B_CH; ++i) {
            const int c = tid + i * THREADS;
            const int r = c / BTile::CHUNKS_PER_LINE;
            const int cc = (c % BTile::CHUNKS_PER_LINE) * 8;
            u32x4_t v = {0u, 0u, 0u, 0u};
            if (B_KCC) {
                // column n_base + r, k = k0 + cc .. +7
                if (n_base + r < p.N && k0 + cc < k_end)
                    v = *reinterpret_cast<const u32x4_t*>(Bbase + (int64_t)(n_base + r) * p.ldb + k0 + cc);
            } else {
                // contraction row k0 + r, columns n_base + cc .. +7
                if (k0 + r < k_end && n_base + cc < p.N)
                    v = *reinterpret_cast<const u32x4_t*>(Bbase + (int64_t)(k0 + r) * p.ldb + n_base + cc);
            }
            b_reg[i] = v;
        }
    };
    auto store_tiles = [&](int buf) {
        S* At = lds + buf * STAGE_ELEMS;
        S* Bt = At + ATile::ELEMS;
#pragma unroll
        for (int i = 0; i < A_CH; ++i) {
            const int c = tid + i * THREADS;
            *reinterpret_cast<u32x4_t*>(At + (c / ATile::CHUNKS_PER_LINE) * ATile::LD + (c % ATile::CHUNKS_PER_LINE) * 8) =
                a_reg[i];
        }
#pragma unroll
        for (int i = 0; i < B_CH; ++i) {
            const int c = tid + i * THREADS;
            *reinterpret_cast<u32x4_t*>(Bt + (c / BTile::CHUNKS_PER_LINE) * BTile::LD + (c % BTile::CHUNKS_PER_LINE) * 8) =
                b_reg[i];
        }
    };

    f32x16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int k_tiles = (k_end - k_begin + BK - 1) / BK;
    if (k_tiles > 0) {
        load_tiles(k_begin);
        store_tiles(0);
    }
    __syncthreads();
    for (int kt = 0; kt < k_tiles; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < k_tiles) load_tiles(k_begin + (kt + 1) * BK);
        const S* At = lds + buf * STAGE_ELEMS;
        const S* Bt = At + ATile::ELEMS;
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            frag_t af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                af[i] = ATile::template fragment<frag_t>(At, wm * (BM / WM) + i * 32, kk, lane);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                bf[j] = BTile::template fragment<frag_t>(Bt, wn * (BN / WN) + j * 32, kk, lane);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = Mma<T>::mma(af[i], bf[j], acc[i][j]);
        }
        if (kt + 1 < k_tiles) store_tiles(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue -------------------------------------------------------------------------------
    // Accumulators (lane: column lane % 32, rows 8 * (r / 4) + 4 * (lane / 32) + r % 4 of each 32x32 tile) are
    // rounded and staged in LDS, then written out as 16-byte packets along rows, rows going to their mapped
    // position.  The loop above ended with a barrier, so the operand buffers can be reused.
    S* Ct = lds;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = wm * (BM / WM) + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
                const int col = wn * (BN / WN) + j * 32 + lane % 32;
                float v = acc[i][j][r];
                if (!GROUP_K && p.bias != nullptr)
                    v += T::up(reinterpret_cast<const S*>(p.bias)[(int64_t)expert * p.N + min(n_base + col, p.N - 1)]);
                Ct[row * C_LD + col] = T::down(v);
            }
    __syncthreads();
    S* Cbase = reinterpret_cast<S*>(p.C) + (GROUP_K ? (int64_t)expert * p.c_stride_e : 0);
    constexpr int C_CHUNKS_PER_ROW = BN / 8;
    constexpr int C_CH = BM * C_CHUNKS_PER_ROW / THREADS;
#pragma unroll
    for (int i = 0; i < C_CH; ++i) {
        const int c = tid + i * THREADS;
        const int row = c / C_CHUNKS_PER_ROW;
        const int col = (c % C_CHUNKS_PER_ROW) * 8;
        if (row < rows_valid && n_base + col < p.N) {
            int64_t out_row;
            if (GROUP_K) {
                out_row = i_base + row;
            } else {
                const int64_t slot = row_start + row;
                out_row = p.y_grouped ? slot : p.row_idx[slot];
            }
            *reinterpret_cast<u32x4_t*>(Cbase + out_row * p.ldc + n_base + col) =
                *reinterpret_cast<const u32x4_t*>(Ct + row * C_LD + col);
        }
    }
}

// =====================================================================================================
// Direct-to-LDS version of the MFMA kernel (BK = 64, two LDS stages)
// =====================================================================================================
// Operand tiles go from global memory straight into LDS with global_load_lds_dwordx4: no staging
// registers, no ds_write burst at the end of a step, and the copy overlaps the MFMAs of the current step.
// One wave instruction fills 64 consecutive 16-byte slots, so rows cannot be padded; bank conflicts are
// avoided by an XOR swizzle applied on the global side (which 16-byte chunk a lane fetches) and undone
// when fragments are read:
//   k-contiguous operand, row = 128 B = 8 slots:   slot = chunk ^ ((row >> 1) & 7)
//   other layout, contraction row = ROWS * 2 B:    slot = chunk ^ (((k & 3) << 2) | (((k >> 3) & 1) << 1))
// (a transposing read takes contraction rows 8 g + r, g = lane / 16, r = 0 .. 3, 32 bytes of each per 16 lanes, and
// the LDS serves 32 lanes at a time: the first term spreads the four r over the 256 bytes of the banks in steps of
// 64, the second puts the odd g into the 32-byte gaps between them.  Without it the two g of a half-wave met in
// the same banks: half of the LDS cycles of the weight-gradient product were conflict cycles.)
// LDS positions whose contraction index lies beyond the end of the contraction range are cleared with a
// plain store in the (single) partial step; positions of rows / columns outside the problem keep whatever
// they held, which only reaches outputs that are never stored.
template <typename S, int ROWS, bool KC, int NWAVES>
struct DtlOperand {
    static constexpr int BK = 64;
    static constexpr int STAGE_BYTES = ROWS * BK * 2;
    static constexpr int SLOTS = STAGE_BYTES / 16;
    static constexpr int IPW = SLOTS / (CK_WAVE * NWAVES);  // load instructions per wave per stage
    static constexpr int SLOTS_PER_LINE = KC ? 8 : ROWS / 8;
    static_assert(SLOTS % (CK_WAVE * NWAVES) == 0, "operand tile / waves");

    // slot p of the stage -> (line, chunk) it has to hold; line = row (KC) or contraction index (other)
    static __device__ __forceinline__ void slot_source(int p, int& line, int& chunk) {
        line = p / SLOTS_PER_LINE;
        const int slot = p % SLOTS_PER_LINE;
        chunk = KC ? (slot ^ ((line >> 1) & 7)) : (slot ^ (((line & 3) << 2) | (((line >> 3) & 1) << 1)));
    }
};

// two fp32 values rounded to the storage type (round to nearest even) and packed into one dword, first value low
template <typename T>
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    typedef typename T::storage_t S2 __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t f = {a, b};
    const S2 h = __builtin_convertvector(f, S2);
    uint32_t w;
    __builtin_memcpy(&w, &h, 4);
    return w;
}

// the reverse: the two storage values of a dword as fp32
template <typename T>
__device__ __forceinline__ void unpack2(uint32_t w, float& a, float& b) {
    typename T::storage_t h[2];
    __builtin_memcpy(h, &w, 4);
    a = T::up(h[0]);
    b = T::up(h[1]);
}

// MODE 0: one workgroup per tile.  MODE 1: tiles dealt by find_tile_split; a workgroup with a piece of a tile writes its
// fp32 accumulators to p.partials instead of running the epilogue.  MODE 2: the launch that follows MODE 1 - one
// workgroup per split tile adds the pieces up and runs the epilogue.
template <typename T, typename TL, bool B_KC, bool GROUP_K, int GLU = 0, int MODE = 0>
// Two waves per SIMD is all the LDS footprint allows; telling the compiler keeps it from spilling to reach a
// higher occupancy that cannot happen.
__global__ void __launch_bounds__(TL::THREADS) CK_WAVES_PER_SIMD(TL::WM * TL::WN / 4)
    grouped_gemm_m16_kernel(GemmParams p) {
    static_assert(MODE == 0 || (GLU == 0 && !GROUP_K), "tail splitting is for the plain per-expert products");
    typedef typename T::storage_t S;
    typedef typename Mma16<T>::frag_t frag_t;
    constexpr int BM = TL::BM, BN = TL::BN, BK = 64, WM = TL::WM, WN = TL::WN;
    constexpr int THREADS = TL::THREADS, NWAVES = WM * WN;
    constexpr int TM = BM / WM / 16, TN = BN / WN / 16, TH = TM / 2;  // 16 x 16 tiles per wave; TH: half of the rows
    static_assert(TM % 2 == 0, "the loop works on one half of a wave's rows at a time");
    static_assert(TL::BK == 64, "the direct-to-LDS kernel is written for BK = 64");
    static_assert(WM == 2, "the epilogue stages one half of the rows per stage buffer");
    constexpr bool A_KC = !GROUP_K;
    constexpr bool B_KCC = GROUP_K ? false : B_KC;
    // Each operand tile lies in LDS as two halves of 128 lines, [A lower | A upper | B lower | B upper], 16 KB each.
    // The halves are the tile's rows [0, BM / 2) and [BM / 2, BM), columns [0, BN / 2) and [BN / 2, BN): where rows or
    // columns are the contiguous dimension in memory, a half's lines are then whole 256-byte runs (interleaved
    // 32-column groups split every 128-byte line between the halves and measured 47 % more requests to L2).  Wave
    // (wm, wn) owns rows wm * RW .. + RW of either A half and columns wn * CW .. + CW of either B half.
    typedef DtlOperand<S, BM / 2, A_KC, NWAVES> AOp;
    typedef DtlOperand<S, BN / 2, B_KCC, NWAVES> BOp;
    static_assert(AOp::IPW == BOp::IPW && AOp::IPW * NWAVES == 16, "square tile; the wait counts of the loops assume 16 copies per half operand");
    static_assert(NWAVES == 8 || NWAVES == 4, "two loops: two wave groups in antiphase (8 waves), one software-pipelined wave per SIMD (4)");
    constexpr int IPW = AOp::IPW;  // copy instructions per wave and half operand
    constexpr int A_HALF = AOp::STAGE_BYTES, B_HALF = BOp::STAGE_BYTES, B_AT = 2 * A_HALF;
    constexpr int STAGE_BYTES = 2 * A_HALF + 2 * B_HALF;
    constexpr int RW = BM / WM / 2, CW = BN / WN / 2;  // lines of one half that belong to one wave
    constexpr int TNH = TN / 2;
    constexpr int C_LD = BN + 8;
    constexpr int HALF_C_BYTES = (BM / 2) * C_LD * 2;  // staged output rows of one wave row-group
    constexpr int BUF_BYTES = STAGE_BYTES > HALF_C_BYTES ? STAGE_BYTES : HALF_C_BYTES;
    __shared__ __attribute__((aligned(1024))) char lds0[BUF_BYTES];
    __shared__ __attribute__((aligned(1024))) char lds1[BUF_BYTES];
    __shared__ int sh_info[8];

    int nt = 0;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / CK_WAVE);
    const int wm = wave / WN, wn = wave % WN;

    int expert, row_start, rows_valid, k_begin, k_end, i_base;
    int part_slot = -1, part_pieces = 1;
    if (!GROUP_K) {
        if (MODE == 0)
            find_tile_balanced<BM>(p.offsets, p.E, p.n_tiles, sh_info);
        else
            find_tile_split<BM, BK>(p.offsets, p.E, p.n_tiles, p.K, MODE == 2, sh_info);
        expert = __builtin_amdgcn_readfirstlane(sh_info[0]);
        row_start = __builtin_amdgcn_readfirstlane(sh_info[1]);
        rows_valid = __builtin_amdgcn_readfirstlane(sh_info[2]);
        nt = __builtin_amdgcn_readfirstlane(sh_info[3]);
        if (expert < 0) return;
        k_begin = 0;
        k_end = p.K;
        if (MODE != 0) {
            part_slot = __builtin_amdgcn_readfirstlane(sh_info[6]);
            part_pieces = __builtin_amdgcn_readfirstlane(sh_info[7]);
            if (MODE == 1 && part_slot >= 0) {
                k_begin = __builtin_amdgcn_readfirstlane(sh_info[4]) * BK;
                k_end = min(p.K, __builtin_amdgcn_readfirstlane(sh_info[5]) * BK);
            }
        }
        i_base = 0;
    } else {
        int rank, it;
        if (!weight_grad_tile(p.E, p.m_tiles / p.E, p.n_tiles, rank, it, nt)) return;
        expert = expert_of_rank(p.offsets, p.E, rank);
        i_base = it * BM;
        k_begin = expert == 0 ? 0 : (int)p.offsets[expert - 1];
        k_end = (int)p.offsets[expert];
        row_start = 0;
        rows_valid = min(BM, p.K - i_base);
    }
    const bool upper_rows_live = rows_valid > BM / 2;  // the same for every wave of the workgroup
    static_assert(GLU == 0 || !GROUP_K, "the fused activation belongs to the per-expert products");
    static_assert(GLU != 1 || B_KC, "the forward fusion reads the weight with the contraction contiguous");
    // GLU == 1: a tile holds BN / 2 "up" columns n_base .. and the BN / 2 "gate" columns glu_half + n_base ..
    // that pair with them (glu_half is a multiple of BN / 2, checked by the host)
    const int n_base = GLU == 1 ? nt * (BN / 2) : nt * BN;
    const int cols_valid = GLU == 1 ? BN : min(BN, p.N - n_base);  // > 0 and a multiple of 8
    const bool upper_cols_live = cols_valid > BN / 2;  // likewise for the last column tile of an odd half-tile count

    // ---- global sources of the LDS slots this lane fills ---------------------------------------------
    typedef __attribute__((address_space(1))) const char* gchar_t;
    const gchar_t a_base = (gchar_t)p.A + (A_KC ? (int64_t)k_begin : (int64_t)k_begin * p.lda + i_base) * 2;
    const gchar_t b_base = (gchar_t)p.B + ((GROUP_K ? 0 : (int64_t)expert * p.b_stride_e) +
                                          (B_KCC ? (int64_t)k_begin : (int64_t)k_begin * p.ldb + n_base)) * 2;
    const int64_t a_step = (A_KC ? (int64_t)BK : (int64_t)BK * p.lda) * 2;
    const int64_t b_step = (B_KCC ? (int64_t)BK : (int64_t)BK * p.ldb) * 2;
    uint32_t a_voff[2][IPW], b_voff[2][IPW];
    {
        const int lane = lane_id();
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < IPW; ++j) {
                int line, chunk;
                AOp::slot_source((wave * IPW + j) * CK_WAVE + lane, line, chunk);
                if (A_KC) {
                    const int trow = h * (BM / 2) + line;
                    const int64_t slot = row_start + min(trow, rows_valid - 1);
                    const int64_t src_row = p.x_grouped ? slot : (int64_t)((uint32_t)p.row_idx[slot] / (uint32_t)p.fan_out);
                    a_voff[h][j] = (uint32_t)((src_row * p.lda + chunk * 8) * 2);
                } else {
                    const int tcol = h * (BM / 2) + chunk * 8;
                    const int cc = tcol < rows_valid ? tcol : 0;
                    a_voff[h][j] = (uint32_t)(((int64_t)line * p.lda + cc) * 2);
                }
            }
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < IPW; ++j) {
                int line, chunk;
                BOp::slot_source((wave * IPW + j) * CK_WAVE + lane, line, chunk);
                if (B_KCC) {
                    const int tcol = h * (BN / 2) + line;
                    const int r = min(tcol, cols_valid - 1);
                    const int w_row = (GLU == 1 && r >= BN / 2) ? p.glu_half + n_base + r - BN / 2 : n_base + r;
                    b_voff[h][j] = (uint32_t)(((int64_t)w_row * p.ldb + chunk * 8) * 2);
                } else {
                    const int tcol = h * (BN / 2) + chunk * 8;
                    const int cc = tcol < cols_valid ? tcol : 0;
                    b_voff[h][j] = (uint32_t)(((int64_t)line * p.ldb + cc) * 2);
                }
            }
    }

    // One copy instruction: 64 lanes x 16 bytes from (wave-uniform base + 32-bit lane offset) to 1 KB of LDS at dst
    // (lds_copy16: the compiler's wait-count bookkeeping does not see it; the waits are placed by hand below)
    auto dma = [&](gchar_t base, uint32_t voff, const char* dst) __attribute__((always_inline)) {
        lds_copy16(lds_address(dst), voff, (uint64_t)base);
    };
    // one half operand (0: A lower, 1: A upper, 2: B lower, 3: B upper) of tile t, which lies inside the contraction range
    auto issue_part = [&](char* st, int part, int t) __attribute__((always_inline)) {
        if (part < 2) {
            const gchar_t at = a_base + (int64_t)t * a_step;
#pragma unroll
            for (int j = 0; j < IPW; ++j) dma(at, a_voff[part][j], st + part * A_HALF + (wave * IPW + j) * 1024);
        } else {
            const gchar_t bt = b_base + (int64_t)t * b_step;
#pragma unroll
            for (int j = 0; j < IPW; ++j)
                dma(bt, b_voff[part - 2][j], st + B_AT + (part - 2) * B_HALF + (wave * IPW + j) * 1024);
        }
    };
    // copy instruction j (of IPW) of one half operand
    auto issue_one = [&](char* st, int part, int t, int j) __attribute__((always_inline)) {
        if (part < 2)
            dma(a_base + (int64_t)t * a_step, a_voff[part][j], st + part * A_HALF + (wave * IPW + j) * 1024);
        else
            dma(b_base + (int64_t)t * b_step, b_voff[part - 2][j], st + B_AT + (part - 2) * B_HALF + (wave * IPW + j) * 1024);
    };
    // tile t whatever its position: slots past the end of the contraction range are cleared instead of copied
    auto issue = [&](int t, char* st) __attribute__((always_inline)) {
        const int k0 = k_begin + t * BK;
        if (k0 + BK <= k_end) {
#pragma unroll
            for (int part = 0; part < 4; ++part) issue_part(st, part, t);
            return;
        }
        const gchar_t at = a_base + (int64_t)t * a_step;
        const gchar_t bt = b_base + (int64_t)t * b_step;
        const int lane = opaque(lane_id());
        const u32x4_t zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < IPW; ++j) {
                int line, chunk;
                AOp::slot_source((wave * IPW + j) * CK_WAVE + lane, line, chunk);
                char* dst = st + h * A_HALF + (wave * IPW + j) * 1024;
                if (k0 + (A_KC ? chunk * 8 : line) < k_end)
                    dma(at, a_voff[h][j], dst);
                else
                    *reinterpret_cast<u32x4_t*>(dst + lane * 16) = zero;
            }
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < IPW; ++j) {
                int line, chunk;
                BOp::slot_source((wave * IPW + j) * CK_WAVE + lane, line, chunk);
                char* dst = st + B_AT + h * B_HALF + (wave * IPW + j) * 1024;
                if (k0 + (B_KCC ? chunk * 8 : line) < k_end)
                    dma(bt, b_voff[h][j], dst);
                else
                    *reinterpret_cast<u32x4_t*>(dst + lane * 16) = zero;
            }
    };

    // ---- fragment addresses (bytes inside a stage) -----------------------------------------------------
    int frag_row, frag_swz;
    int a_off[TM], b_off[TN];
    // transposed layouts: the odd 16-row block of a pair lies 32 bytes after the even one, before the swizzle; the
    // swizzle flips that bit for odd lane / 16, so there it lies 32 bytes before
    const int odd_step = (lane_id() / 16) & 1 ? -32 : 32;
    {
        const int lane = lane_id();
        frag_row = (lane % 16) * 128;
        frag_swz = ((lane / 16) ^ ((lane % 16) >> 1)) << 4;
        const int g = lane / 16, q = lane % 16;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int l0 = wm * RW + (i % TH) * 16;
            if (A_KC) {
                a_off[i] = (i / TH) * A_HALF + l0 * 128;
            } else {
                const int col = l0 + (q % 4) * 4;
                a_off[i] = (i / TH) * A_HALF + (g * 8 + q / 4) * BM + (((col / 8) ^ ((q / 4) << 2) ^ ((g & 1) << 1)) << 4) + (col % 8) * 2;
            }
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int l0 = wn * CW + (j % TNH) * 16;
            if (B_KCC) {
                b_off[j] = B_AT + (j / TNH) * B_HALF + l0 * 128;
            } else {
                const int col = l0 + (q % 4) * 4;
                b_off[j] = B_AT + (j / TNH) * B_HALF + (g * 8 + q / 4) * BN + (((col / 8) ^ ((q / 4) << 2) ^ ((g & 1) << 1)) << 4) + (col % 8) * 2;
            }
        }
    }
    // fragments of one half of the wave's rows, both contraction groups of 32: af[kk / 32][i]
    auto read_a = [&](const char* st, int h, frag_t (*af)[TH]) __attribute__((always_inline)) {
#pragma unroll
        for (int kki = 0; kki < 2; ++kki) {
            const int kk = kki * 32;
            const int kc = frag_row + (opaque(frag_swz) ^ ((kk / 8) << 4));
#pragma unroll
            for (int i = 0; i < TH; ++i) {
                const int ii = h * TH + i;
                if (A_KC) {
                    af[kki][i] = *reinterpret_cast<const frag_t*>(st + kc + a_off[ii]);
                } else {
                    // a contraction row of a half operand is BM / 2 elements = BM bytes
                    const char* q = st + a_off[ii & ~1] + (ii & 1) * odd_step + kk * BM;
                    union {
                        v4i16_t h2[2];
                        frag_t f;
                    } u;
                    u.h2[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(q));
                    u.h2[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(q + 4 * BM));
                    af[kki][i] = u.f;
                }
            }
        }
    };
    auto read_b = [&](const char* st, int h, frag_t (*bf)[TNH]) __attribute__((always_inline)) {
#pragma unroll
        for (int kki = 0; kki < 2; ++kki) {
            const int kk = kki * 32;
            const int kc = frag_row + (opaque(frag_swz) ^ ((kk / 8) << 4));
#pragma unroll
            for (int j = 0; j < TNH; ++j) {
                const int jj = h * TNH + j;
                if (B_KCC) {
                    bf[kki][j] = *reinterpret_cast<const frag_t*>(st + kc + b_off[jj]);
                } else {
                    const char* q = st + b_off[jj & ~1] + (jj & 1) * odd_step + kk * BN;
                    union {
                        v4i16_t h2[2];
                        frag_t f;
                    } u;
                    u.h2[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(q));
                    u.h2[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(q + 4 * BN));
                    bf[kki][j] = u.f;
                }
            }
        }
    };

    f32x4_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
    // The per-expert bias is what the sums start from (not in a piece of a split tile: there the launch that adds
    // the pieces up starts from it): it joins the fp32 sums at no cost and is rounded with them, once.
    // (eight waves only: with four, 256 initial values that depend on a branch wait in ordinary registers until the
    // loop takes them over, and spill; the host sends products with a bias to the eight-wave loop)
    if (NWAVES == 8 && GLU == 0 && !GROUP_K && p.bias != nullptr && !(MODE == 1 && part_slot >= 0)) {
        // a lane's four columns of every 16-column block, the same for all of its rows (see the epilogue)
        const S* brow = reinterpret_cast<const S*>(p.bias) + (int64_t)expert * p.N;
        const int lane = lane_id();
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = n_base + (j / TNH) * (BN / 2) + wn * CW + (j % TNH) * 16 + 4 * (lane / 16);
            const u32x2_t four = *reinterpret_cast<const u32x2_t*>(brow + (col < p.N ? col : 0));  // N is a multiple of 8
            float b[4];
            unpack2<T>(four.x, b[0], b[1]);
            unpack2<T>(four.y, b[2], b[3]);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[i][j][r] = b[r];
        }
    }

    // one quarter of the wave's block: rows of half ha times columns of half hb, over the whole tile depth.  The
    // MFMA gets the column fragment as its first operand, i.e. it computes the 16 x 16 block transposed: a lane
    // then holds four consecutive columns of one row (row lane % 16, columns 4 * (lane / 16) + r), which the
    // epilogue stages with one 8-byte LDS store instead of four 2-byte ones.
    auto mma_quad = [&](int ha, int hb, frag_t (*af)[TH], frag_t (*bf)[TNH]) __attribute__((always_inline)) {
#pragma unroll
        for (int kki = 0; kki < 2; ++kki)
#pragma unroll
            for (int i = 0; i < TH; ++i)
#pragma unroll
                for (int j = 0; j < TNH; ++j)
                    if constexpr (NWAVES == 4)
                        Mma16<T>::mma_acc(bf[kki][j], af[kki][i], acc[ha * TH + i][hb * TNH + j]);
                    else
                        acc[ha * TH + i][hb * TNH + j] = Mma16<T>::mma(bf[kki][j], af[kki][i], acc[ha * TH + i][hb * TNH + j]);
    };
    frag_t fa[2][TH], fb0[2][TNH], fb1[2][TNH];
    // one whole tile, outside the pipelined loop
    auto multiply_tile = [&](const char* st) __attribute__((always_inline)) {
        read_a(st, 0, fa);
        read_b(st, 0, fb0);
        if (upper_cols_live) read_b(st, 1, fb1);
        mma_quad(0, 0, fa, fb0);
        if (upper_cols_live) mma_quad(0, 1, fa, fb1);
        __builtin_amdgcn_sched_barrier(0);
        if (upper_rows_live) {
            read_a(st, 1, fa);
            if (upper_cols_live) mma_quad(1, 1, fa, fb1);
            mma_quad(1, 0, fa, fb0);
        }
    };

    // ---- the pipelined loop ----------------------------------------------------------------------------
    // The waves of the lower row group (0 .. 3, one per SIMD) and of the upper row group (4 .. 7) run the same
    // sequence of phases, the upper group one phase behind: while one wave of a SIMD issues a quarter of its
    // matrix instructions (C phase), the other reads the next fragments and requests copies (M phase).  A wave
    // that waits for the copy path to take its request then never holds up matrix instructions.  Every phase ends
    // at a workgroup barrier.  Tile kt is read from X while tile kt + 2 is copied over the halves of X as they
    // fall free:
    //   M0 reads A lower of X           copies B lower (last read in M3 of the step before)
    //   M1 reads B upper                copies A lower
    //   M2 reads A upper                copies B upper
    //   M3 reads B lower of Y           copies A upper
    // so every copy has seven M phases until its half is read again, and a wait that leaves the twelve most recent
    // copies of the wave outstanding (two per M phase) at the end of each M phase covers it: what the next M phase
    // of either group reads was requested at least six M phases before this one, and the barrier that ends the
    // phase passes that on to the other waves.  The count only works because nothing but these copies is
    // outstanding on the vector-memory counter inside the loop: the copies complete in the order they were
    // issued, but an ordinary load issued among them can complete ahead of older copies (tried: wrong results).
#define CK_PHASE_END()                           \
    do {                                         \
        __builtin_amdgcn_sched_barrier(0);       \
        __builtin_amdgcn_s_barrier();            \
        __builtin_amdgcn_sched_barrier(0);       \
    } while (0)
    // An M phase ends with a wait that leaves the twelve most recent copies of the wave outstanding.
#define CK_M_END(PART)                                        \
    do {                                                      \
        issue_part(X, PART, tf);                              \
        wait_copies<12>();     \
        __builtin_amdgcn_s_waitcnt(0xC07F); /* lgkmcnt(0) */  \
        CK_PHASE_END();                                       \
    } while (0)
    const int k_tiles = (k_end - k_begin + BK - 1) / BK;
    const int n_full = (k_end - k_begin) / BK;  // leading tiles that lie completely inside the range
    // `upper` says, as a type, whether the upper half of the tile's rows holds any row of the segment: where it holds
    // none (the last row tile of an expert with at most BM / 2 rows left) its fragments are not read and its matrix
    // instructions not issued, while barriers and copies stay as they are, so the counts of the waits still hold.
    // `upper_cols` says the same of the upper half of the tile's columns (an output width of an odd number of half
    // tiles, 1408 = 5.5 x 256 for instance).
    auto pp_step = [&](auto upper, auto upper_cols, int kt, char* X, char* Y, frag_t (*bl)[TNH], frag_t (*bu)[TNH]) __attribute__((always_inline)) {
        constexpr bool UPPER = decltype(upper)::value;
        constexpr bool UCOLS = decltype(upper_cols)::value;
        // The last two steps of a range have no tile left to request; they request the last tile once more, into
        // halves that nobody reads again, which keeps the count of outstanding copies the same in every step (a
        // branch around the copies, with its own wait, measured slower than the 2 / 64 of copy work it saves).
        const int tf = min(kt + 2, n_full - 1);
        read_a(X, 0, fa);
        CK_M_END(2);
        __builtin_amdgcn_s_setprio(1);
        mma_quad(0, 0, fa, bl);
        __builtin_amdgcn_s_setprio(0);
        CK_PHASE_END();
        if (UCOLS) read_b(X, 1, bu);
        CK_M_END(0);
        __builtin_amdgcn_s_setprio(1);
        if (UCOLS) mma_quad(0, 1, fa, bu);
        __builtin_amdgcn_s_setprio(0);
        CK_PHASE_END();
        if (UPPER) read_a(X, 1, fa);
        CK_M_END(3);
        __builtin_amdgcn_s_setprio(1);
        if (UPPER && UCOLS) mma_quad(1, 1, fa, bu);
        __builtin_amdgcn_s_setprio(0);
        CK_PHASE_END();
        // lower columns of the next tile, over the registers of this tile's upper columns (after the last tile of a
        // range this reads a stage that nobody uses any more)
        read_b(Y, 0, bu);
        CK_M_END(1);
        __builtin_amdgcn_s_setprio(1);
        if (UPPER) mma_quad(1, 0, fa, bl);
        __builtin_amdgcn_s_setprio(0);
        CK_PHASE_END();
    };

    int kt = 0;
    if (MODE == 2) kt = k_tiles;  // nothing to multiply: the accumulators come from the partial tiles below
    if constexpr (NWAVES == 4) {
        // ---- one wave per SIMD: the same pipeline inside a single instruction stream ----------------------------
        // Every wave owns a 128 x 128 block (64 rows of either A half x 64 columns of either B half; 256 accumulator
        // registers, which the compiler keeps in the accumulation half of the register file), so a step reads
        // 128 KB of fragments from LDS per CU where eight waves of 128 x 64 read 192 KB.  A step is four quarters of
        // 32 matrix instructions (row half x column half over the tile depth).  While a quarter multiplies, the wave
        // reads the one half operand the next quarter lacks into registers that are free, and requests four copies:
        //   Q0  A lower x B lower      reads B upper of X            copies B lower of X <- tile kt + 2
        //   Q1  A lower x B upper      reads A upper of X            copies B upper of X <- tile kt + 2
        //   Q2  A upper x B upper      reads A lower of Y            copies A upper of X <- tile kt + 2
        //   Q3  A upper x B lower      reads B lower of Y            copies A lower of Y <- tile kt + 3
        // (X holds tile kt, Y tile kt + 1.)  A half is overwritten in the quarter after the one that read it, and read
        // seven quarters after its copy was requested.  A quarter ends with a wait that leaves the 24 most recent
        // copies of the wave outstanding (four per quarter, so everything older than six quarters has landed), a
        // wait for the wave's own LDS reads (the half they came from is overwritten next), and a workgroup barrier.
        // The loads and copies are spread between the matrix instructions, two of those per slot, and the slots are
        // fenced for the instruction scheduler so that the spacing survives.
        static_assert(NWAVES != 4 || (TH == 4 && TNH == 4), "a quarter is 4 x 4 blocks");
        auto ld_a = [&](const char* st, int h, int kki, int i) __attribute__((always_inline)) -> frag_t {
            const int kk = kki * 32;
            const int kc = frag_row + (opaque(frag_swz) ^ ((kk / 8) << 4));
            const int ii = h * TH + i;
            if (A_KC) {
                return *reinterpret_cast<const frag_t*>(st + kc + a_off[ii]);
            } else {
                const char* q = st + a_off[ii & ~1] + (ii & 1) * odd_step + kk * BM;
                union {
                    v4i16_t h2[2];
                    frag_t f;
                } u;
                u.h2[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(q));
                u.h2[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(q + 4 * BM));
                return u.f;
            }
        };
        auto ld_b = [&](const char* st, int h, int kki, int j) __attribute__((always_inline)) -> frag_t {
            const int kk = kki * 32;
            const int kc = frag_row + (opaque(frag_swz) ^ ((kk / 8) << 4));
            const int jj = h * TNH + j;
            if (B_KCC) {
                return *reinterpret_cast<const frag_t*>(st + kc + b_off[jj]);
            } else {
                const char* q = st + b_off[jj & ~1] + (jj & 1) * odd_step + kk * BN;
                union {
                    v4i16_t h2[2];
                    frag_t f;
                } u;
                u.h2[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(q));
                u.h2[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16_ptr)(q + 4 * BN));
                return u.f;
            }
        };
#define CK_Q_END()                                                \
    do {                                                          \
        __builtin_amdgcn_sched_barrier(0);                        \
        wait_copies<24>();         \
        __builtin_amdgcn_s_waitcnt(0xC07F); /* lgkmcnt(0) */      \
        __builtin_amdgcn_s_barrier();                             \
        __builtin_amdgcn_sched_barrier(0);                        \
    } while (0)
        // One quarter: the matrix instructions of rows half ha x columns half hb (if `mma`), fragment n of the next
        // half operand through load_one(n) in every other slot (if `load`), copy instruction c of half `cpart` of
        // tile ct into stage cst in slots 1, 5, 9, 13.
        auto quarter = [&](auto mma, auto load, int ha, int hb, frag_t (*af)[TH], frag_t (*bf)[TNH], auto load_one,
                           char* cst, int cpart, int ct) __attribute__((always_inline)) {
            constexpr bool MMA = decltype(mma)::value;
            constexpr bool LOAD = decltype(load)::value;
#pragma unroll
            for (int sl = 0; sl < 16; ++sl) {
                if (LOAD && sl % 2 == 0) load_one(sl / 2);
                if (sl % 4 == 1) issue_one(cst, cpart, ct, sl / 4);
                if (MMA) {
#pragma unroll
                    for (int m = 2 * sl; m < 2 * sl + 2; ++m) {
                        const int kki = m / 16, i = (m / 4) % 4, j = m % 4;
                        Mma16<T>::mma_acc(bf[kki][j], af[kki][i], acc[ha * TH + i][hb * TNH + j]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            CK_Q_END();
        };
        frag_t fa0[2][TH], fa1[2][TH], fbx[2][TNH], fby[2][TNH];
        // one step: bl holds B lower of tile kt on entry and is free on exit, bu receives B upper of tile kt, then
        // B lower of tile kt + 1
        auto w4_step = [&](auto upper, auto upper_cols, int kt_, char* X, char* Y, frag_t (*bl)[TNH], frag_t (*bu)[TNH]) __attribute__((always_inline)) {
            constexpr bool UPPER = decltype(upper)::value;
            constexpr bool UCOLS = decltype(upper_cols)::value;
            typedef std::integral_constant<bool, UPPER> up_t;
            typedef std::integral_constant<bool, UCOLS> uc_t;
            typedef std::integral_constant<bool, UPPER && UCOLS> both_t;
            // the last steps of a range have no tile left to request: they request the last tile once more, into
            // halves that nobody reads again, which keeps the count of outstanding copies the same in every quarter
            const int t2 = min(kt_ + 2, n_full - 1), t3 = min(kt_ + 3, n_full - 1);
            quarter(std::true_type{}, uc_t{}, 0, 0, fa0, bl, [&](int n) __attribute__((always_inline)) { bu[n / 4][n % 4] = ld_b(X, 1, n / 4, n % 4); }, X, 2, t2);
            quarter(uc_t{}, up_t{}, 0, 1, fa0, bu, [&](int n) __attribute__((always_inline)) { fa1[n / 4][n % 4] = ld_a(X, 1, n / 4, n % 4); }, X, 3, t2);
            quarter(both_t{}, std::true_type{}, 1, 1, fa1, bu, [&](int n) __attribute__((always_inline)) { fa0[n / 4][n % 4] = ld_a(Y, 0, n / 4, n % 4); }, X, 1, t2);
            quarter(up_t{}, std::true_type{}, 1, 0, fa1, bl, [&](int n) __attribute__((always_inline)) { bu[n / 4][n % 4] = ld_b(Y, 0, n / 4, n % 4); }, Y, 0, t3);
        };
        if (MODE != 2 && n_full >= 2) {
            // tiles 0 and 1 in the order of the loop's requests (A lower, B lower, B upper, A upper); A lower and B
            // lower of tile 0 go to the registers, then A lower of tile 2 may follow over A lower of tile 0
            issue_part(lds0, 0, 0);
            issue_part(lds0, 2, 0);
            issue_part(lds0, 3, 0);
            issue_part(lds0, 1, 0);
            issue_part(lds1, 0, 1);
            issue_part(lds1, 2, 1);
            issue_part(lds1, 3, 1);
            issue_part(lds1, 1, 1);
            CK_Q_END();  // the first 8 of 32 have landed: A lower and B lower of tile 0
#pragma unroll
            for (int n = 0; n < 8; ++n) {
                fa0[n / 4][n % 4] = ld_a(lds0, 0, n / 4, n % 4);
                fbx[n / 4][n % 4] = ld_b(lds0, 0, n / 4, n % 4);
            }
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
            issue_part(lds0, 0, min(2, n_full - 1));
            CK_Q_END();  // B upper of tile 0 has landed: 24 younger copies
            auto run = [&](auto upper, auto upper_cols) __attribute__((always_inline)) {
                for (; kt + 1 < n_full; kt += 2) {
                    w4_step(upper, upper_cols, kt, lds0, lds1, fbx, fby);
                    w4_step(upper, upper_cols, kt + 1, lds1, lds0, fby, fbx);
                }
            };
            if (upper_rows_live && upper_cols_live) run(std::true_type{}, std::true_type{});
            else if (upper_cols_live) run(std::false_type{}, std::true_type{});
            else if (upper_rows_live) run(std::true_type{}, std::false_type{});
            else run(std::false_type{}, std::false_type{});
            wait_copies<0>();
            __syncthreads();
            if (kt < n_full) {  // an odd number of full tiles: the last one is complete in lds0
                multiply_tile(lds0);
                ++kt;
                __syncthreads();
            }
        }
#undef CK_Q_END
    } else
    if (MODE != 2 && n_full >= 2) {
#pragma unroll
        for (int part = 0; part < 4; ++part) issue_part(lds0, part, 0);
        // Tile 1 is requested in the order in which the first two steps read it (B lower, A lower, B upper, A
        // upper), so the waits of the loop (twelve copies outstanding, two more per M phase) cover each half in
        // time, and only tile 0 has to be complete before the loop starts: the 128 copy instructions of the two
        // tiles take the request path about 2 us, half of which now runs beside the first step.
        issue_part(lds1, 2, 1);
        issue_part(lds1, 0, 1);
        issue_part(lds1, 3, 1);
        issue_part(lds1, 1, 1);
        wait_copies<8>();
        __syncthreads();
        read_b(lds0, 0, fb0);
        __builtin_amdgcn_s_waitcnt(0xC07F);
        CK_PHASE_END();
        if (wm == 1) CK_PHASE_END();  // the upper group falls one phase behind
        // two steps per turn so that each names its buffers and registers statically
        auto run = [&](auto upper, auto upper_cols) __attribute__((always_inline)) {
            for (; kt + 1 < n_full; kt += 2) {
                pp_step(upper, upper_cols, kt, lds0, lds1, fb0, fb1);
                pp_step(upper, upper_cols, kt + 1, lds1, lds0, fb1, fb0);
            }
        };
        if (upper_rows_live && upper_cols_live) run(std::true_type{}, std::true_type{});
        else if (upper_cols_live) run(std::false_type{}, std::true_type{});
        else if (upper_rows_live) run(std::true_type{}, std::false_type{});
        else run(std::false_type{}, std::false_type{});
        if (wm == 0) CK_PHASE_END();
        wait_copies<0>();
        __syncthreads();
        if (kt < n_full) {  // an odd number of full tiles: the last one is complete in lds0
            multiply_tile(lds0);
            ++kt;
            __syncthreads();
        }
    }
    for (; kt < k_tiles; ++kt) {
        issue(kt, lds0);
        wait_copies<0>();
        __syncthreads();
        multiply_tile(lds0);
        __syncthreads();
    }
#undef CK_M_END
#undef CK_PHASE_END
    if constexpr (NWAVES == 4 && MODE != 2) {  // (the eight-wave loop's matrix instructions are builtins: the compiler counts)
        static_assert(NWAVES != 4 || TN == 8, "one statement per row of eight accumulators");
        settle_matrix_results<true>(acc[0]);
#pragma unroll
        for (int i = 1; i < TM; ++i) settle_matrix_results<false>(acc[i]);
    }

    // ---- pieces of a split tile ------------------------------------------------------------------------
    // A partial tile is stored the way the accumulators lie in the registers: float4 number
    // ((wave * TM + i) * TN + j) * 64 + lane of the slot, so both directions move 1 KB per wave instruction.
    if (MODE == 1 && part_slot >= 0) {
        f32x4_t* dst = reinterpret_cast<f32x4_t*>(p.partials) + (int64_t)part_slot * (BM * BN / 4);
        const int l = lane_id();
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) dst[((wave * TM + i) * TN + j) * CK_WAVE + l] = acc[i][j];
        return;
    }
    if (MODE == 2) {
        const f32x4_t* src = reinterpret_cast<const f32x4_t*>(p.partials) + (int64_t)part_slot * (BM * BN / 4);
        const int l = lane_id();
        for (int c = 0; c < part_pieces; ++c) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const f32x4_t v = src[(int64_t)c * (BM * BN / 4) + ((wave * TM + i) * TN + j) * CK_WAVE + l];
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[i][j][r] += v[r];
                }
        }
    }

    // ---- epilogue -----------------------------------------------------------------------------------
    // Accumulators (lane: row lane % 16, columns 4 * (lane / 16) + r of each 16x16 tile) are
    // rounded and staged in LDS - the tile's upper half of the rows in one stage buffer, the lower half in the other -
    // then written out as 16-byte packets along rows, rows going to their mapped position.
    const int lane = opaque(lane_id());
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        S* Ch = reinterpret_cast<S*>(i / TH == 0 ? lds0 : lds1);  // tile rows [0, BM / 2) are staged in lds0, the rest in lds1
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int row = wm * RW + (i % TH) * 16 + lane % 16;  // inside this half of the tile
            const int col = (j / TNH) * (BN / 2) + wn * CW + (j % TNH) * 16 + 4 * (lane / 16);
            u32x2_t four;
            four.x = pack2<T>(acc[i][j][0], acc[i][j][1]);
            four.y = pack2<T>(acc[i][j][2], acc[i][j][3]);
            *reinterpret_cast<u32x2_t*>(Ch + row * C_LD + col) = four;
        }
    }
    // The tile leaves LDS as 16-byte packets along rows.  Two copies of that code: the eight-wave kernels keep theirs
    // statement for statement, so that they compile to the instructions that were measured (written as passes, the
    // same code was scheduled and register-allocated differently); the four-wave kernels, with twice the packets per
    // lane, take them in two passes over one set of registers.
    if constexpr (NWAVES == 8) {
        S* Cbase = reinterpret_cast<S*>(p.C) + (GROUP_K ? (int64_t)expert * p.c_stride_e : 0);
        typedef VPack<T, 8> P8;
        // GLU == 1: a lane takes an "up" packet together with its "gate" packet, so packets are counted over half a row
        constexpr int C_CHUNKS_PER_ROW = (GLU == 1 ? BN / 2 : BN) / 8;
        constexpr int C_CH = BM * C_CHUNKS_PER_ROW / THREADS;
        // The loads an output packet depends on are all requested before anything is stored, and without branches
        // (positions outside the tile are redirected to a valid one): the destination rows of scattered outputs, the
        // up / gate packets of h for GLU == 2 - both while the workgroup is on its way to the barrier - and, behind the
        // barrier, the staged packets themselves.  Packet by packet, every store would wait for its own loads in turn
        // (and, with one counter for loads and stores, for the store before it).
        constexpr int H_CH = GLU == 2 ? C_CH : 1;
        P8 h_up[H_CH], h_gate[H_CH];
        int64_t out_row[C_CH];
    #pragma unroll
        for (int i = 0; i < C_CH; ++i) {
            const int row = min((tid + i * THREADS) / C_CHUNKS_PER_ROW, rows_valid - 1);
            out_row[i] = GROUP_K ? i_base + row : row_start + row;
        }
        if (!GROUP_K && !p.y_grouped) {
    #pragma unroll
            for (int i = 0; i < C_CH; ++i) out_row[i] = p.row_idx[out_row[i]];
        }
        if (GLU == 2) {
    #pragma unroll
            for (int i = 0; i < C_CH; ++i) {
                const int col = min(((tid + i * THREADS) % C_CHUNKS_PER_ROW) * 8, cols_valid - 8);
                const S* hrow = reinterpret_cast<const S*>(p.aux) + out_row[i] * p.ld_aux + n_base + col;
                h_up[i] = nt_load(reinterpret_cast<const P8*>(hrow));
                h_gate[i] = nt_load(reinterpret_cast<const P8*>(hrow + p.glu_half));
            }
        }
        __syncthreads();
        constexpr int G_CH = GLU == 1 ? C_CH : 1;
        P8 staged[C_CH], staged_gate[G_CH];
    #pragma unroll
        for (int i = 0; i < C_CH; ++i) {
            const int c = tid + i * THREADS;
            const int row = c / C_CHUNKS_PER_ROW;
            const int col = (c % C_CHUNKS_PER_ROW) * 8;
            const S* src = reinterpret_cast<const S*>(row < BM / 2 ? lds0 : lds1) + (row % (BM / 2)) * C_LD + col;
            staged[i] = *reinterpret_cast<const P8*>(src);
            // GLU == 1: columns [0, BN / 2) of the tile are "up", [BN / 2, BN) the matching "gate"
            if (GLU == 1) staged_gate[i] = *reinterpret_cast<const P8*>(src + BN / 2);
        }
    #pragma unroll
        for (int i = 0; i < C_CH; ++i) {
            const int c = tid + i * THREADS;
            const int row = c / C_CHUNKS_PER_ROW;
            const int col = (c % C_CHUNKS_PER_ROW) * 8;
            if (row < rows_valid && col < cols_valid) {
                if (GLU == 0) {
                    *reinterpret_cast<P8*>(Cbase + out_row[i] * p.ldc + n_base + col) = staged[i];
                } else if (GLU == 1) {
                    // both halves go to h, and the activation is computed from the rounded values exactly as the
                    // separate kernel would from h
                    const P8 u = staged[i];
                    const P8 g = staged_gate[GLU == 1 ? i : 0];
                    P8 y;
    #pragma unroll
                    for (int e = 0; e < 8; ++e) y.v[e] = T::down(swiglu_fwd_1<T>(T::up(g.v[e]), T::up(u.v[e])));
                    S* hrow = Cbase + out_row[i] * p.ldc + n_base + col;
                    *reinterpret_cast<P8*>(hrow) = u;
                    *reinterpret_cast<P8*>(hrow + p.glu_half) = g;
                    *reinterpret_cast<P8*>(reinterpret_cast<S*>(p.aux) + out_row[i] * p.ld_aux + n_base + col) = y;
                } else {
                    // the staged tile is d_act (rounded, as the separate kernels would hand it over); h supplies up
                    // and gate of the same positions, and d_h receives both derivatives
                    const P8 u = h_up[GLU == 2 ? i : 0];
                    const P8 g = h_gate[GLU == 2 ? i : 0];
                    const P8 d = staged[i];
                    P8 du, dg;
    #pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        float fg, fu;
                        swiglu_bwd_1<T>(T::up(g.v[e]), T::up(u.v[e]), T::up(d.v[e]), fg, fu);
                        dg.v[e] = T::down(fg);
                        du.v[e] = T::down(fu);
                    }
                    S* drow = Cbase + out_row[i] * p.ldc + n_base + col;
                    *reinterpret_cast<P8*>(drow) = du;
                    *reinterpret_cast<P8*>(drow + p.glu_half) = dg;
                }
            }
        }
    } else {
        S* Cbase = reinterpret_cast<S*>(p.C) + (GROUP_K ? (int64_t)expert * p.c_stride_e : 0);
        typedef VPack<T, 8> P8;
        // GLU == 1: a lane takes an "up" packet together with its "gate" packet, so packets are counted over half a row
        constexpr int C_CHUNKS_PER_ROW = (GLU == 1 ? BN / 2 : BN) / 8;
        // packets per lane: with four waves twice as many as with eight, taken in two passes over the same registers
        constexpr int PASSES = NWAVES == 4 ? 2 : 1;
        constexpr int C_CH = BM * C_CHUNKS_PER_ROW / THREADS / PASSES;
        // The loads an output packet depends on are all requested before anything is stored, and without branches
        // (positions outside the tile are redirected to a valid one): the destination rows of scattered outputs, the
        // up / gate packets of h for GLU == 2 - in the first pass while the workgroup is on its way to the barrier - and,
        // behind the barrier, the staged packets themselves.  Packet by packet, every store would wait for its own loads
        // in turn (and, with one counter for loads and stores, for the store before it).
        constexpr int H_CH = GLU == 2 ? C_CH : 1;
        P8 h_up[H_CH], h_gate[H_CH];
        int64_t out_row[C_CH];
        auto request = [&](int pass) __attribute__((always_inline)) {
    #pragma unroll
            for (int i = 0; i < C_CH; ++i) {
                const int row = min((tid + (pass * C_CH + i) * THREADS) / C_CHUNKS_PER_ROW, rows_valid - 1);
                out_row[i] = GROUP_K ? i_base + row : row_start + row;
            }
            if (!GROUP_K && !p.y_grouped) {
    #pragma unroll
                for (int i = 0; i < C_CH; ++i) out_row[i] = p.row_idx[out_row[i]];
            }
            if (GLU == 2) {
    #pragma unroll
                for (int i = 0; i < C_CH; ++i) {
                    const int col = min(((tid + (pass * C_CH + i) * THREADS) % C_CHUNKS_PER_ROW) * 8, cols_valid - 8);
                    const S* hrow = reinterpret_cast<const S*>(p.aux) + out_row[i] * p.ld_aux + n_base + col;
                    h_up[i] = nt_load(reinterpret_cast<const P8*>(hrow));
                    h_gate[i] = nt_load(reinterpret_cast<const P8*>(hrow + p.glu_half));
                }
            }
        };
        constexpr int G_CH = GLU == 1 ? C_CH : 1;
        auto write_out = [&](int pass) __attribute__((always_inline)) {
            P8 staged[C_CH], staged_gate[G_CH];
    #pragma unroll
            for (int i = 0; i < C_CH; ++i) {
                const int c = tid + (pass * C_CH + i) * THREADS;
                const int row = c / C_CHUNKS_PER_ROW;
                const int col = (c % C_CHUNKS_PER_ROW) * 8;
                const S* src = reinterpret_cast<const S*>(row < BM / 2 ? lds0 : lds1) + (row % (BM / 2)) * C_LD + col;
                staged[i] = *reinterpret_cast<const P8*>(src);
                // GLU == 1: columns [0, BN / 2) of the tile are "up", [BN / 2, BN) the matching "gate"
                if (GLU == 1) staged_gate[i] = *reinterpret_cast<const P8*>(src + BN / 2);
            }
    #pragma unroll
            for (int i = 0; i < C_CH; ++i) {
                const int c = tid + (pass * C_CH + i) * THREADS;
                const int row = c / C_CHUNKS_PER_ROW;
                const int col = (c % C_CHUNKS_PER_ROW) * 8;
                if (row < rows_valid && col < cols_valid) {
                    if (GLU == 0) {
                        *reinterpret_cast<P8*>(Cbase + out_row[i] * p.ldc + n_base + col) = staged[i];
                    } else if (GLU == 1) {
                        // both halves go to h, and the activation is computed from the rounded values exactly as the
                        // separate kernel would from h
                        const P8 u = staged[i];
                        const P8 g = staged_gate[GLU == 1 ? i : 0];
                        P8 y;
    #pragma unroll
                        for (int e = 0; e < 8; ++e) y.v[e] = T::down(swiglu_fwd_1<T>(T::up(g.v[e]), T::up(u.v[e])));
                        S* hrow = Cbase + out_row[i] * p.ldc + n_base + col;
                        *reinterpret_cast<P8*>(hrow) = u;
                        *reinterpret_cast<P8*>(hrow + p.glu_half) = g;
                        *reinterpret_cast<P8*>(reinterpret_cast<S*>(p.aux) + out_row[i] * p.ld_aux + n_base + col) = y;
                    } else {
                        // the staged tile is d_act (rounded, as the separate kernels would hand it over); h supplies up
                        // and gate of the same positions, and d_h receives both derivatives
                        const P8 u = h_up[GLU == 2 ? i : 0];
                        const P8 g = h_gate[GLU == 2 ? i : 0];
                        const P8 d = staged[i];
                        P8 du, dg;
    #pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            float fg, fu;
                            swiglu_bwd_1<T>(T::up(g.v[e]), T::up(u.v[e]), T::up(d.v[e]), fg, fu);
                            dg.v[e] = T::down(fg);
                            du.v[e] = T::down(fu);
                        }
                        S* drow = Cbase + out_row[i] * p.ldc + n_base + col;
                        *reinterpret_cast<P8*>(drow) = du;
                        *reinterpret_cast<P8*>(drow + p.glu_half) = dg;
                    }
                }
            }
        };
        request(0);
        __syncthreads();
        write_out(0);
        if (PASSES == 2) {
            request(1);
            write_out(1);
        }
    }
}

// ---- plain kernels (fp32 and irregular shapes) ---------------------------------------------------
// One lane per output element, fp64 accumulation: the fp32 path promises 1e-5, which an fp32 sum of a few
// hundred O(1) terms does not keep in any order, so the sum is made exact and rounded once.
template <typename T>
__global__ void __launch_bounds__(256)
    s2s_plain_kernel(const typename T::storage_t* __restrict__ X, int64_t ldx, const typename T::storage_t* __restrict__ W,
                     int64_t se, int64_t sk, int64_t sn, const int64_t* __restrict__ row_idx,
                     const int64_t* __restrict__ offsets, typename T::storage_t* __restrict__ out, int64_t ldo,
                     int64_t slots, int K, int N, int E, int fan_out, int x_grouped, int y_grouped,
                     const typename T::storage_t* __restrict__ bias) {
    const int n = blockIdx.x * 64 + threadIdx.x % 64;
    const int64_t slot = (int64_t)blockIdx.y * 4 + threadIdx.x / 64;
    if (slot >= slots || n >= N) return;
    // expert of this slot: first e with offsets[e] > slot (binary search)
    int lo = 0, hi = E - 1;
    while (lo < hi) {
        const int mid = (lo + hi) / 2;
        if (offsets[mid] > slot) hi = mid;
        else lo = mid + 1;
    }
    const int64_t src_row = x_grouped ? slot : row_idx[slot] / fan_out;
    const int64_t dst_row = y_grouped ? slot : row_idx[slot];
    const typename T::storage_t* x = X + src_row * ldx;
    const typename T::storage_t* w = W + (int64_t)lo * se + (int64_t)n * sn;
    double acc = 0.0;
    for (int k = 0; k < K; ++k) acc = fma((double)T::up(x[k]), (double)T::up(w[(int64_t)k * sk]), acc);
    if (bias != nullptr) acc += (double)T::up(bias[(int64_t)lo * N + n]);
    out[dst_row * ldo + n] = T::down((float)acc);
}

template <typename T>
__global__ void __launch_bounds__(256)
    xty_plain_kernel(const typename T::storage_t* __restrict__ DY, int64_t lddy, const typename T::storage_t* __restrict__ X,
                     int64_t ldx, const int64_t* __restrict__ offsets, typename T::storage_t* __restrict__ DW, int64_t se,
                     int64_t sk, int64_t sn, int K, int N, int E) {
    // lanes run along the contiguous dimension of DW
    const bool k_fast = sk == 1;
    const int fast = blockIdx.x * 64 + threadIdx.x % 64;
    const int slow = blockIdx.y * 4 + threadIdx.x / 64;
    const int e = blockIdx.z;
    const int k = k_fast ? fast : slow;
    const int n = k_fast ? slow : fast;
    if (k >= K || n >= N) return;
    const int64_t begin = e == 0 ? 0 : offsets[e - 1];
    const int64_t end = offsets[e];
    double acc = 0.0;
    for (int64_t m = begin; m < end; ++m)
        acc = fma((double)T::up(X[m * ldx + k]), (double)T::up(DY[m * lddy + n]), acc);
    DW[(int64_t)e * se + (int64_t)k * sk + (int64_t)n * sn] = T::down((float)acc);
}

// ---- row gather ------------------------------------------------------------------------------
// One wave per output row, 4 rows per workgroup.
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
    group_kernel(const typename T::storage_t* __restrict__ A, int64_t lda, const int64_t* __restrict__ idx,
                 const typename T::storage_t* __restrict__ coeff, typename T::storage_t* __restrict__ out, int64_t ldo,
                 int64_t rows, int64_t K, int64_t fan_out) {
    typedef VPack<T, VEC> P;
    const int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / CK_WAVE;
    if (row >= rows) return;
    const int64_t id = idx[row];
    const float c = coeff != nullptr ? T::up(coeff[id]) : 1.0f;
    const P* src = reinterpret_cast<const P*>(A + (id / fan_out) * lda);
    P* dst = reinterpret_cast<P*>(out + row * ldo);
    const int64_t packs = K / VEC;
    for (int64_t p = lane_id(); p < packs; p += CK_WAVE) {
        P v = src[p];
        if (coeff != nullptr) {
            // the reference multiplies in the storage type (kernels.py:284-286): one rounding of the product
#pragma unroll
            for (int j = 0; j < VEC; ++j) v.v[j] = T::down(T::up(v.v[j]) * c);
        }
        nt_store(v, dst + p);
    }
}

// ---- SwiGLU passes for the shapes the fused epilogues do not take ------------------------------------------
// act[r][c] = swiglu(up = h[r][c], gate = h[r][half + c]); one lane per element.
template <typename T>
__global__ void __launch_bounds__(256)
    glu_rows_fwd_kernel(const typename T::storage_t* __restrict__ h, int64_t ldh, typename T::storage_t* __restrict__ act,
                        int64_t ld_act, int64_t rows, int64_t half) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t r = blockIdx.y;
    if (c >= half) return;
    for (int64_t row = r; row < rows; row += gridDim.y)
        act[row * ld_act + c] = T::down(swiglu_fwd_1<T>(T::up(h[row * ldh + half + c]), T::up(h[row * ldh + c])));
}
// d_h[r][c] holds d_act[r][c] on entry; on exit d_h[r][c] = d_up and d_h[r][half + c] = d_gate.  Every lane
// reads its own element before it writes, so the pass works in place.
template <typename T>
__global__ void __launch_bounds__(256)
    glu_rows_bwd_kernel(const typename T::storage_t* __restrict__ h, int64_t ldh, typename T::storage_t* d_h, int64_t ld_dh,
                        int64_t rows, int64_t half) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t r = blockIdx.y;
    if (c >= half) return;
    for (int64_t row = r; row < rows; row += gridDim.y) {
        float dg, du;
        swiglu_bwd_1<T>(T::up(h[row * ldh + half + c]), T::up(h[row * ldh + c]), T::up(d_h[row * ld_dh + c]), dg, du);
        d_h[row * ld_dh + c] = T::down(du);
        d_h[row * ld_dh + half + c] = T::down(dg);
    }
}

}  // namespace ck

// ---- host side ------------------------------------------------------------------------------
namespace {

#ifndef CK_TILE_CONFIG
#define CK_TILE_CONFIG 256, 256, 64, 2, 4
#endif
typedef ck::Tile<CK_TILE_CONFIG> MainTile;
typedef ck::Tile<256, 256, 64, 2, 2> FourWaveTile;  // the same tile by four waves, one per SIMD
constexpr int kBM = MainTile::BM, kBN = MainTile::BN;
static_assert(FourWaveTile::BM == kBM && FourWaveTile::BN == kBN, "both loops work on one tile grid");

// Workgroups for the products cut per expert, at the bound of the row tile count
int64_t dealt_grid(const ck::GemmParams& p) { return ck::tile_grid::balanced(p.m_tiles, p.n_tiles); }

// Which of the two loops a launch takes (the tile grid is the same): 8 = two wave groups in antiphase, 4 = one
// software-pipelined wave per SIMD.
// `waves` of the entry points: 0 = the library's choice (eight, unless the environment variable CK_GEMM_WAVES says 4 -
// a switch for measurements), 4 or 8 = that loop.  Products with a bias always take eight.
int default_gemm_waves() {
    static const int waves = [] {
        const char* v = getenv("CK_GEMM_WAVES");
        return v && v[0] == '4' ? 4 : 8;
    }();
    return waves;
}
bool valid_waves(int waves) { return waves == 0 || waves == 4 || waves == 8; }

template <typename T, bool B_KC, bool GROUP_K, int GLU = 0, int MODE = 0>
void launch_m16(unsigned grid, const ck::GemmParams& p, hipStream_t s) {
    if ((p.waves == 0 ? default_gemm_waves() : p.waves) == 4 && p.bias == nullptr)
        hipLaunchKernelGGL((ck::grouped_gemm_m16_kernel<T, FourWaveTile, B_KC, GROUP_K, GLU, MODE>), dim3(grid),
                           dim3(FourWaveTile::THREADS), 0, s, p);
    else
        hipLaunchKernelGGL((ck::grouped_gemm_m16_kernel<T, MainTile, B_KC, GROUP_K, GLU, MODE>), dim3(grid),
                           dim3(MainTile::THREADS), 0, s, p);
}

template <typename T, bool B_KC, bool GROUP_K>
void launch_mfma(const ck::GemmParams& p, hipStream_t s) {
    const int total = p.m_tiles * p.n_tiles;
    const int grid = (total + 7) / 8 * 8;
    if (p.wide)
        hipLaunchKernelGGL((ck::grouped_gemm_kernel<T, MainTile, B_KC, GROUP_K>), dim3((unsigned)grid),
                           dim3(MainTile::THREADS), 0, s, p);
    else if (GROUP_K) {
        // 8 lists (one per XCD): see weight_grad_tile; < 2^31: m_tiles * n_tiles is checked by the caller
        launch_m16<T, B_KC, GROUP_K>((unsigned)ck::tile_grid::weight_grad(p.E, p.m_tiles / p.E, p.n_tiles), p, s);
    } else
        launch_m16<T, B_KC, GROUP_K>((unsigned)dealt_grid(p), p, s);
}

// per-expert product whose last round of tiles is split along the contraction (see find_tile_split): the tiles,
// then the sums of the split ones
template <typename T, bool B_KC>
void launch_mfma_split(const ck::GemmParams& p, hipStream_t s) {
    launch_m16<T, B_KC, false, 0, 1>((unsigned)ck::tile_grid::split(p.m_tiles, p.n_tiles), p, s);
    launch_m16<T, B_KC, false, 0, 2>((unsigned)ck::tile_grid::split_fixup(), p, s);
}

constexpr int64_t kSplitWorkspaceBytes = (int64_t)ck::kSplitSlots * kBM * kBN * 4;
// contraction lengths from which a tile can be cut into two pieces of kSplitMinTiles contraction tiles
constexpr int64_t kSplitMinK = 2 * ck::kSplitMinTiles * 64;

// per-expert product with the SwiGLU epilogue GLU (1: forward, 2: backward); never the wide kernel
template <typename T, bool B_KC, int GLU>
void launch_mfma_glu(const ck::GemmParams& p, hipStream_t s) {
    launch_m16<T, B_KC, false, GLU>((unsigned)dealt_grid(p), p, s);
}

bool mult8(int64_t v) { return (v & 7) == 0; }

}  // namespace

extern "C" int64_t ck_scatter2scatter_workspace_size(int64_t num_slots, int64_t K, int64_t N, int64_t E, int dtype) {
    if (num_slots <= 0 || N <= 0 || E <= 0 || dtype == CK_F32 || K < kSplitMinK) return 0;
    return kSplitWorkspaceBytes;
}

extern "C" int ck_scatter2scatter(const void* X, int64_t x_stride, const void* W, int64_t w_stride_e,
                                  int64_t w_stride_k, int64_t w_stride_n, const int64_t* sorted_scattered_idxs,
                                  const int64_t* expert_offsets, void* out, int64_t out_stride, int64_t num_slots,
                                  int64_t K, int64_t N, int64_t E, int64_t fan_out, int x_grouped, int y_grouped,
                                  const void* bias, int dtype, void* stream) {
    return ck_scatter2scatter_ws(X, x_stride, W, w_stride_e, w_stride_k, w_stride_n, sorted_scattered_idxs, expert_offsets,
                                 out, out_stride, num_slots, K, N, E, fan_out, x_grouped, y_grouped, bias, dtype, 0, nullptr,
                                 0, stream);
}

extern "C" int ck_scatter2scatter_ws(const void* X, int64_t x_stride, const void* W, int64_t w_stride_e,
                                     int64_t w_stride_k, int64_t w_stride_n, const int64_t* sorted_scattered_idxs,
                                     const int64_t* expert_offsets, void* out, int64_t out_stride, int64_t num_slots,
                                     int64_t K, int64_t N, int64_t E, int64_t fan_out, int x_grouped, int y_grouped,
                                     const void* bias, int dtype, int waves, void* workspace,
                                     int64_t workspace_bytes, void* stream) {
    if (num_slots < 0 || K < 0 || N < 0 || E <= 0 || fan_out <= 0 || !valid_waves(waves)) return CK_ERR_SHAPE;
    if (num_slots > 0x7fffffff || K > 0x7fffffff || N > 0x7fffffff || E > 0x7fffffff) return CK_ERR_SHAPE;
    if (dtype != CK_F32 && dtype != CK_F16 && dtype != CK_BF16) return CK_ERR_DTYPE;
    if (num_slots == 0 || N == 0) return CK_OK;
    if (!out || !expert_offsets || (K > 0 && (!X || !W))) return CK_ERR_NULL;
    if ((!x_grouped || !y_grouped) && !sorted_scattered_idxs) return CK_ERR_NULL;
    if (!ck_aligned_elem(X, dtype) || !ck_aligned_elem(W, dtype) || !ck_aligned_elem(out, dtype)) return CK_ERR_ALIGN;
    if (bias && !ck_aligned_elem(bias, dtype)) return CK_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;

    const bool b_kc = w_stride_k == 1, b_nc = w_stride_n == 1;
    const bool fast = dtype != CK_F32 && K > 0 && (b_kc || b_nc) && ck_aligned16(X) && ck_aligned16(W) && mult8(K) &&
                      mult8(x_stride) && mult8(w_stride_e) && mult8(b_kc ? w_stride_n : w_stride_k) && mult8(N) &&
                      ck_aligned16(out) && mult8(out_stride) && (!bias || ck_aligned16(bias));
    if (fast) {
        ck::GemmParams p = {};
        p.A = X;
        p.B = W;
        p.C = out;
        p.lda = x_stride;
        p.ldb = b_kc ? w_stride_n : w_stride_k;
        p.ldc = out_stride;
        p.b_stride_e = w_stride_e;
        p.row_idx = sorted_scattered_idxs;
        p.offsets = expert_offsets;
        p.M = (int)num_slots;
        p.N = (int)N;
        p.K = (int)K;
        p.E = (int)E;
        p.fan_out = (int)fan_out;
        p.x_grouped = x_grouped;
        p.y_grouped = y_grouped;
        p.bias = bias;
        p.waves = waves;
        // the direct-to-LDS kernel addresses a tile's sources with 32-bit byte offsets from a per-tile base
        p.wide = num_slots * x_stride * 2 >= (int64_t)1 << 32 || (b_kc ? N : K) * p.ldb * 2 >= (int64_t)1 << 32;
        p.m_tiles = (int)(num_slots / kBM + E);
        p.n_tiles = (int)ck_ceil_div(N, kBN);
        if ((int64_t)(p.m_tiles + 8) * p.n_tiles > 0x7ffffff0 - 256) return CK_ERR_SHAPE;
        // with a workspace, the last round of tiles of every XCD is split along the contraction
        if (workspace != nullptr && !p.wide && K >= kSplitMinK) {
            if (workspace_bytes < kSplitWorkspaceBytes || !ck_aligned16(workspace)) return CK_ERR_WORKSPACE;
            p.partials = static_cast<float*>(workspace);
            if (dtype == CK_BF16) {
                if (b_kc) launch_mfma_split<ck::BF16, true>(p, s);
                else launch_mfma_split<ck::BF16, false>(p, s);
            } else {
                if (b_kc) launch_mfma_split<ck::F16, true>(p, s);
                else launch_mfma_split<ck::F16, false>(p, s);
            }
            return ck_launch_status();
        }
        if (dtype == CK_BF16) {
            if (b_kc) launch_mfma<ck::BF16, true, false>(p, s);
            else launch_mfma<ck::BF16, false, false>(p, s);
        } else {
            if (b_kc) launch_mfma<ck::F16, true, false>(p, s);
            else launch_mfma<ck::F16, false, false>(p, s);
        }
        return ck_launch_status();
    }
    const dim3 grid((unsigned)ck_ceil_div(N, 64), (unsigned)ck_ceil_div(num_slots, 4));
    if (grid.y > 65535u * 1024u) return CK_ERR_SHAPE;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        hipLaunchKernelGGL((ck::s2s_plain_kernel<T>), grid, dim3(256), 0, s, (const S*)X, x_stride, (const S*)W,
                           w_stride_e, w_stride_k, w_stride_n, sorted_scattered_idxs, expert_offsets, (S*)out,
                           out_stride, num_slots, (int)K, (int)N, (int)E, (int)fan_out, x_grouped, y_grouped,
                           (const S*)bias);
    });
    return ck_launch_status();
}

extern "C" int ck_scatter2scatter_glu(const void* X, int64_t x_stride, const void* W, int64_t w_stride_e,
                                      int64_t w_stride_k, int64_t w_stride_n, const int64_t* sorted_scattered_idxs,
                                      const int64_t* expert_offsets, void* h, int64_t h_stride, void* act,
                                      int64_t act_stride, int64_t num_slots, int64_t K, int64_t I, int64_t E,
                                      int64_t fan_out, int x_grouped, int dtype, int waves, void* stream) {
    if (num_slots < 0 || K < 0 || I < 0 || E <= 0 || fan_out <= 0 || !valid_waves(waves)) return CK_ERR_SHAPE;
    if (num_slots > 0x7fffffff || K > 0x7fffffff || I > 0x3fffffff || E > 0x7fffffff) return CK_ERR_SHAPE;
    if (dtype != CK_F32 && dtype != CK_F16 && dtype != CK_BF16) return CK_ERR_DTYPE;
    if (num_slots == 0 || I == 0) return CK_OK;
    if (!h || !act || !expert_offsets || (K > 0 && (!X || !W))) return CK_ERR_NULL;
    if (!x_grouped && !sorted_scattered_idxs) return CK_ERR_NULL;
    if (!ck_aligned_elem(X, dtype) || !ck_aligned_elem(W, dtype) || !ck_aligned_elem(h, dtype) ||
        !ck_aligned_elem(act, dtype))
        return CK_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    const int64_t N = 2 * I;

    const bool fused = dtype != CK_F32 && K > 0 && w_stride_k == 1 && ck_aligned16(X) && ck_aligned16(W) && mult8(K) &&
                       mult8(x_stride) && mult8(w_stride_e) && mult8(w_stride_n) && I % (kBN / 2) == 0 &&
                       ck_aligned16(h) && mult8(h_stride) && ck_aligned16(act) && mult8(act_stride) &&
                       num_slots * x_stride * 2 < (int64_t)1 << 32 && N * w_stride_n * 2 < (int64_t)1 << 32;
    if (fused) {
        ck::GemmParams p = {};
        p.A = X;
        p.B = W;
        p.C = h;
        p.lda = x_stride;
        p.ldb = w_stride_n;
        p.ldc = h_stride;
        p.b_stride_e = w_stride_e;
        p.row_idx = sorted_scattered_idxs;
        p.offsets = expert_offsets;
        p.M = (int)num_slots;
        p.N = (int)N;
        p.K = (int)K;
        p.E = (int)E;
        p.fan_out = (int)fan_out;
        p.x_grouped = x_grouped;
        p.y_grouped = 1;
        p.aux = act;
        p.ld_aux = act_stride;
        p.glu_half = (int)I;
        p.waves = waves;
        p.m_tiles = (int)(num_slots / kBM + E);
        p.n_tiles = (int)(I / (kBN / 2));
        if ((int64_t)(p.m_tiles + 8) * p.n_tiles > 0x7ffffff0) return CK_ERR_SHAPE;
        if (dtype == CK_BF16) launch_mfma_glu<ck::BF16, true, 1>(p, s);
        else launch_mfma_glu<ck::F16, true, 1>(p, s);
        return ck_launch_status();
    }
    const int st = ck_scatter2scatter(X, x_stride, W, w_stride_e, w_stride_k, w_stride_n, sorted_scattered_idxs,
                                      expert_offsets, h, h_stride, num_slots, K, N, E, fan_out, x_grouped, 1, nullptr, dtype,
                                      stream);
    if (st != CK_OK) return st;
    const dim3 grid((unsigned)ck_ceil_div(I, 256), (unsigned)(num_slots < 65535 ? num_slots : 65535));
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        hipLaunchKernelGGL((ck::glu_rows_fwd_kernel<T>), grid, dim3(256), 0, s, (const S*)h, h_stride, (S*)act, act_stride,
                           num_slots, I);
    });
    return ck_launch_status();
}

extern "C" int ck_scatter2scatter_glu_bwd(const void* DY, int64_t dy_stride, const void* W, int64_t w_stride_e,
                                          int64_t w_stride_k, int64_t w_stride_n, const int64_t* expert_offsets,
                                          const void* h, int64_t h_stride, void* d_h, int64_t d_h_stride,
                                          int64_t num_slots, int64_t K, int64_t I, int64_t E, int dtype, int waves,
                                          void* stream) {
    if (num_slots < 0 || K < 0 || I < 0 || E <= 0 || !valid_waves(waves)) return CK_ERR_SHAPE;
    if (num_slots > 0x7fffffff || K > 0x7fffffff || I > 0x3fffffff || E > 0x7fffffff) return CK_ERR_SHAPE;
    if (dtype != CK_F32 && dtype != CK_F16 && dtype != CK_BF16) return CK_ERR_DTYPE;
    if (num_slots == 0 || I == 0) return CK_OK;
    if (!h || !d_h || !expert_offsets || (K > 0 && (!DY || !W))) return CK_ERR_NULL;
    if (!ck_aligned_elem(DY, dtype) || !ck_aligned_elem(W, dtype) || !ck_aligned_elem(h, dtype) ||
        !ck_aligned_elem(d_h, dtype))
        return CK_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;

    const bool fused = dtype != CK_F32 && K > 0 && w_stride_n == 1 && ck_aligned16(DY) && ck_aligned16(W) && mult8(K) &&
                       mult8(dy_stride) && mult8(w_stride_e) && mult8(w_stride_k) && mult8(I) && ck_aligned16(h) &&
                       mult8(h_stride) && ck_aligned16(d_h) && mult8(d_h_stride) &&
                       num_slots * dy_stride * 2 < (int64_t)1 << 32 && K * w_stride_k * 2 < (int64_t)1 << 32;
    if (fused) {
        ck::GemmParams p = {};
        p.A = DY;
        p.B = W;
        p.C = d_h;
        p.lda = dy_stride;
        p.ldb = w_stride_k;
        p.ldc = d_h_stride;
        p.b_stride_e = w_stride_e;
        p.offsets = expert_offsets;
        p.M = (int)num_slots;
        p.N = (int)I;
        p.K = (int)K;
        p.E = (int)E;
        p.fan_out = 1;
        p.x_grouped = 1;
        p.y_grouped = 1;
        p.aux = const_cast<void*>(h);
        p.ld_aux = h_stride;
        p.glu_half = (int)I;
        p.waves = waves;
        p.m_tiles = (int)(num_slots / kBM + E);
        p.n_tiles = (int)ck_ceil_div(I, kBN);
        if ((int64_t)(p.m_tiles + 8) * p.n_tiles > 0x7ffffff0) return CK_ERR_SHAPE;
        if (dtype == CK_BF16) launch_mfma_glu<ck::BF16, false, 2>(p, s);
        else launch_mfma_glu<ck::F16, false, 2>(p, s);
        return ck_launch_status();
    }
    // d_act goes into the first half of every d_h row, then one pass turns the row into (d_up | d_gate) in place
    const int st = ck_scatter2scatter(DY, dy_stride, W, w_stride_e, w_stride_k, w_stride_n, nullptr, expert_offsets, d_h,
                                      d_h_stride, num_slots, K, I, E, 1, 1, 1, nullptr, dtype, stream);
    if (st != CK_OK) return st;
    const dim3 grid((unsigned)ck_ceil_div(I, 256), (unsigned)(num_slots < 65535 ? num_slots : 65535));
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        hipLaunchKernelGGL((ck::glu_rows_bwd_kernel<T>), grid, dim3(256), 0, s, (const S*)h, h_stride, (S*)d_h, d_h_stride,
                           num_slots, I);
    });
    return ck_launch_status();
}

extern "C" int ck_group_bwd_W(const void* DY, int64_t dy_stride, const void* X, int64_t x_stride,
                              const int64_t* expert_offsets, void* DW, int64_t dw_stride_e, int64_t dw_stride_k,
                              int64_t dw_stride_n, int64_t M, int64_t K, int64_t N, int64_t E, int dtype, int waves,
                              void* stream) {
    if (M < 0 || K < 0 || N < 0 || E <= 0 || !valid_waves(waves)) return CK_ERR_SHAPE;
    if (M > 0x7fffffff || K > 0x7fffffff || N > 0x7fffffff || E > 65535) return CK_ERR_SHAPE;
    if (dtype != CK_F32 && dtype != CK_F16 && dtype != CK_BF16) return CK_ERR_DTYPE;
    if (K == 0 || N == 0) return CK_OK;
    if (!DW || !expert_offsets || (M > 0 && (!DY || !X))) return CK_ERR_NULL;
    if (!ck_aligned_elem(DW, dtype) || !ck_aligned_elem(X, dtype) || !ck_aligned_elem(DY, dtype)) return CK_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;

    const bool k_fast = dw_stride_k == 1, n_fast = dw_stride_n == 1;
    const bool fast = dtype != CK_F32 && (k_fast || n_fast) && ck_aligned16(X) && ck_aligned16(DY) && mult8(K) &&
                      mult8(N) && mult8(x_stride) && mult8(dy_stride) && ck_aligned16(DW) && mult8(dw_stride_e) &&
                      mult8(k_fast ? dw_stride_n : dw_stride_k);
    if (fast) {
        // C[e][i][j] = sum_r P[r][i] * Q[r][j] with j the contiguous dimension of DW
        ck::GemmParams p = {};
        const bool swap = k_fast;  // j = k: P = DY (i = n), Q = X
        p.A = swap ? DY : X;
        p.lda = swap ? dy_stride : x_stride;
        p.B = swap ? X : DY;
        p.ldb = swap ? x_stride : dy_stride;
        p.C = DW;
        p.ldc = swap ? dw_stride_n : dw_stride_k;
        p.c_stride_e = dw_stride_e;
        p.offsets = expert_offsets;
        p.M = (int)M;
        p.K = (int)(swap ? N : K);  // I
        p.N = (int)(swap ? K : N);  // J
        p.E = (int)E;
        p.waves = waves;
        p.wide = 64 * p.lda * 2 >= (int64_t)1 << 32 || 64 * p.ldb * 2 >= (int64_t)1 << 32;
        p.m_tiles = (int)(E * ck_ceil_div(p.K, kBM));
        p.n_tiles = (int)ck_ceil_div(p.N, kBN);
        if ((int64_t)(p.m_tiles + 8) * p.n_tiles > 0x7ffffff0) return CK_ERR_SHAPE;
        if (dtype == CK_BF16) launch_mfma<ck::BF16, false, true>(p, s);
        else launch_mfma<ck::F16, false, true>(p, s);
        return ck_launch_status();
    }
    const int64_t fast_dim = k_fast ? K : N, slow_dim = k_fast ? N : K;
    const dim3 grid((unsigned)ck_ceil_div(fast_dim, 64), (unsigned)ck_ceil_div(slow_dim, 4), (unsigned)E);
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        hipLaunchKernelGGL((ck::xty_plain_kernel<T>), grid, dim3(256), 0, s, (const S*)DY, dy_stride, (const S*)X,
                           x_stride, expert_offsets, (S*)DW, dw_stride_e, dw_stride_k, dw_stride_n, (int)K, (int)N,
                           (int)E);
    });
    return ck_launch_status();
}

extern "C" int ck_group(const void* A, int64_t a_stride, const int64_t* idx, const void* coeff, void* out,
                        int64_t out_stride, int64_t num_rows, int64_t K, int64_t fan_out, int dtype, void* stream) {
    if (num_rows < 0 || K < 0 || fan_out <= 0) return CK_ERR_SHAPE;
    if (num_rows == 0 || K == 0) return CK_OK;
    if (!A || !idx || !out) return CK_ERR_NULL;
    if (!ck_aligned_elem(A, dtype) || !ck_aligned_elem(out, dtype) || (coeff && !ck_aligned_elem(coeff, dtype)))
        return CK_ERR_ALIGN;
    const int64_t grid = ck_ceil_div(num_rows, 4);
    if (grid > 0x7fffffff) return CK_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        const bool vec = ck_aligned16(A) && ck_aligned16(out) && K % T::kVec == 0 && a_stride % T::kVec == 0 &&
                         out_stride % T::kVec == 0;
        if (vec)
            hipLaunchKernelGGL((ck::group_kernel<T, T::kVec>), dim3((unsigned)grid), dim3(256), 0, s, (const S*)A,
                               a_stride, idx, (const S*)coeff, (S*)out, out_stride, num_rows, K, fan_out);
        else
            hipLaunchKernelGGL((ck::group_kernel<T, 1>), dim3((unsigned)grid), dim3(256), 0, s, (const S*)A, a_stride,
                               idx, (const S*)coeff, (S*)out, out_stride, num_rows, K, fan_out);
    });
    return ck_launch_status();
}

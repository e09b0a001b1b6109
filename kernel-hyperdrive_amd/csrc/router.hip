// Routing weights of the MoE layer in one pass: the k largest router logits of every token, their positions, and
// the softmax over those k values.  The reference does this with stock torch ops - topk (or max for k = 1), a cast
// to fp32, softmax, a cast back (cute_kernels/kernels/scattermoe/torch_implementation.py:121-132, 193-199) - and
// autograd strings the matching backward ops together; here each direction is one launch, one wavefront per token.
//   forward : selected[t, j]  = position of the j-th largest logit of token t (ties: the lower position first;
//                               NaN counts as larger than every number, as in torch.topk)
//             weights[t, j]   = exp(v_j - v_0) / sum_i exp(v_i - v_0) over the k selected values, fp32 math,
//                               rounded once to the storage type; the fp32 values are kept for the backward
//   backward: d_v[t, j]       = w_j * (g_j - sum_i g_i w_i)     (softmax backward on the fp32 weights)
//             d_logits[t, e]  = d_v[t, j] where e = selected[t, j], else 0  (every element of the row is written)
// The forward also exists with the router's linear in front (logits = x W^T, torch_implementation.py:122): a
// workgroup multiplies 16 tokens by all experts' rows with MFMAs, its waves splitting the hidden dimension, adds
// the partial blocks up through LDS in a fixed order, rounds the logits once to the storage type, writes them, and
// selects from the rounded values - as the stock sequence does, which selects from the stored logits.
#include <math.h>

#include "ck_device.h"

namespace ck {

// is (a, ai) ahead of (b, bi) in the order "larger value first, NaN before everything, lower position first"?
__device__ __forceinline__ bool router_ahead(float a, int ai, float b, int bi) {
    const bool an = a != a, bn = b != b;
    const bool gt = (a > b) || (an && !bn);
    const bool eq = (a == b) || (an && bn);
    return gt || (eq && ai < bi);
}

// Selection and softmax for one token by one wavefront: lane l holds the logits of experts l, l + 64, ... in v.
template <typename T, int VPL>
__device__ __forceinline__ void router_select_token(const float (&v)[VPL], int lane, int E, int k, int64_t t,
                                                    typename T::storage_t* __restrict__ weights,
                                                    float* __restrict__ weights_f32, int64_t* __restrict__ selected) {
    uint32_t taken = 0;  // bit i: v[i] is already among the selected
    float my_val = 0.f;  // lane j < k ends up with the j-th largest value and its position
    int my_idx = 0;
    for (int j = 0; j < k; ++j) {
        float best = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const int e = i * CK_WAVE + lane;
            if (e < E && !((taken >> i) & 1u) && router_ahead(v[i], e, best, bi)) {
                best = v[i];
                bi = e;
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(best, off, CK_WAVE);
            const int oi = __shfl_xor(bi, off, CK_WAVE);
            if (router_ahead(ov, oi, best, bi)) {
                best = ov;
                bi = oi;
            }
        }
        if (lane == j) {
            my_val = best;
            my_idx = bi;
        }
        if ((bi % CK_WAVE) == lane) taken |= 1u << (bi / CK_WAVE);
    }
    const float top = __shfl(my_val, 0, CK_WAVE);
    const float p = lane < k ? expf(my_val - top) : 0.f;
    const float w = p / wave_sum(p);
    if (lane < k) {
        weights[t * k + lane] = T::down(w);
        weights_f32[t * k + lane] = w;
        selected[t * k + lane] = my_idx;
    }
}

template <typename T, int VPL>
__global__ void __launch_bounds__(256)
    router_fwd_kernel(const typename T::storage_t* __restrict__ logits, int64_t ld,
                      typename T::storage_t* __restrict__ weights, float* __restrict__ weights_f32,
                      int64_t* __restrict__ selected, int64_t tokens, int E, int k) {
    const int64_t t = (int64_t)blockIdx.x * 4 + threadIdx.x / CK_WAVE;
    if (t >= tokens) return;
    const int lane = lane_id();
    float v[VPL];
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int e = i * CK_WAVE + lane;
        v[i] = e < E ? T::up(logits[t * ld + e]) : 0.f;
    }
    router_select_token<T, VPL>(v, lane, E, k, t, weights, weights_f32, selected);
}

// ---- the router's linear and the selection in one launch ---------------------------------------------------
template <typename T>
struct RouterMma;
template <>
struct RouterMma<BF16> {
    typedef bf16x8_t frag_t;
    static __device__ __forceinline__ f32x4_t mma(frag_t a, frag_t b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};
template <>
struct RouterMma<F16> {
    typedef f16x8_t frag_t;
    static __device__ __forceinline__ f32x4_t mma(frag_t a, frag_t b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};

constexpr int kRouterTokens = 16;  // tokens per workgroup: one MFMA row tile

// NT column tiles of 16 experts.  Operand fragments come straight from memory: lane l of a 16 x 16 x 32 MFMA supplies
// the 8 consecutive hidden positions 8 * (l / 16) ... of row l % 16 of either operand - one 16-byte load each, and
// the weight rows stay in L2.  Wave w of NW takes the blocks of 32 hidden positions w, w + NW, ...; U of them are in
// flight.  Many waves per workgroup keep both chains short: the blocks a wave walks through, and the tokens it then
// selects for one after the other (16 / NW; a selection is a chain of dependent shuffles).
// The result lane l holds of tile nt is (token 4 * (l / 16) + r, expert 16 nt + l % 16), r = 0 .. 3.
template <typename T, int NT, int NW>
__global__ void __launch_bounds__(NW * CK_WAVE)
    router_linear_fwd_kernel(const typename T::storage_t* __restrict__ x, int64_t ldx,
                             const typename T::storage_t* __restrict__ w, int64_t ldw,
                             typename T::storage_t* __restrict__ logits, int64_t ld_logits,
                             typename T::storage_t* __restrict__ weights, float* __restrict__ weights_f32,
                             int64_t* __restrict__ selected, int64_t tokens, int H, int E, int k) {
    typedef typename T::storage_t S;
    typedef typename RouterMma<T>::frag_t frag_t;
    constexpr int EP = NT * 16, VPL = (EP + CK_WAVE - 1) / CK_WAVE, U = NT <= 1 ? 4 : NT <= 2 ? 2 : 1;
    constexpr int TPW = kRouterTokens / NW;  // tokens a wave selects for
    static_assert(kRouterTokens % NW == 0, "whole tokens per wave");
    __shared__ float part[NW][kRouterTokens][EP + 1];
    const int wave = threadIdx.x / CK_WAVE, lane = lane_id();
    const int row = lane % 16, kc = lane / 16;
    const int64_t t0 = (int64_t)blockIdx.x * kRouterTokens;
    const S* xrow = x + min(t0 + row, tokens - 1) * ldx + kc * 8;
    const S* wrow[NT];
    bool live[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int n = nt * 16 + row;
        live[nt] = n < E;
        wrow[nt] = w + (int64_t)(live[nt] ? n : 0) * ldw + kc * 8;
    }
    f32x4_t acc[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const frag_t zero = {};
    const int k_last = H - 8 - kc * 8;  // (relative to the lane's first packet) the last packet of the row
    for (int kb = wave; kb * 32 < H; kb += NW * U) {
        // All loads of a turn are issued before any is used, and none sits behind a branch: a packet past the end of
        // the row (H is a multiple of 8, so it lies wholly inside or outside) or in a row past the last expert is
        // read from a valid place instead and replaced by zeros afterwards.
        frag_t a[U], b[U][NT];
        bool in[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k0 = (kb + NW * u) * 32;
            in[u] = k0 <= k_last;
            const int kl = in[u] ? k0 : -kc * 8;  // the row's first packet (xrow / wrow point kc packets into the row)
            a[u] = nt_load(reinterpret_cast<const frag_t*>(xrow + kl));
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) b[u][nt] = *reinterpret_cast<const frag_t*>(wrow[nt] + kl);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            a[u] = in[u] ? a[u] : zero;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[nt] = RouterMma<T>::mma(a[u], live[nt] ? b[u][nt] : zero, acc[nt]);
        }
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) part[wave][4 * kc + r][nt * 16 + row] = acc[nt][r];
    __syncthreads();
    // wave w finishes tokens TPW w ...: lane l holds experts l, l + 64
    for (int i = 0; i < TPW; ++i) {
        const int tt = wave * TPW + i;
        const int64_t t = t0 + tt;
        if (t >= tokens) break;
        float v[VPL];
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const int e = j * CK_WAVE + lane;
            v[j] = 0.f;
            if (e < E) {
                float sum = part[0][tt][e];
#pragma unroll
                for (int pw = 1; pw < NW; ++pw) sum += part[pw][tt][e];
                const S rounded = T::down(sum);
                logits[t * ld_logits + e] = rounded;
                v[j] = T::up(rounded);
            }
        }
        router_select_token<T, VPL>(v, lane, E, k, t, weights, weights_f32, selected);
    }
}

template <typename T, int VPL>
__global__ void __launch_bounds__(256)
    router_bwd_kernel(const typename T::storage_t* __restrict__ d_weights, const float* __restrict__ weights_f32,
                      const int64_t* __restrict__ selected, typename T::storage_t* __restrict__ d_logits, int64_t ld,
                      int64_t tokens, int E, int k) {
    const int64_t t = (int64_t)blockIdx.x * 4 + threadIdx.x / CK_WAVE;
    if (t >= tokens) return;
    const int lane = lane_id();
    const bool live = lane < k;
    const float w = live ? weights_f32[t * k + lane] : 0.f;
    const float g = live ? T::up(d_weights[t * k + lane]) : 0.f;
    const int sel = live ? (int)selected[t * k + lane] : -1;
    const float dv = w * (g - wave_sum(g * w));
    float out[VPL];
#pragma unroll
    for (int i = 0; i < VPL; ++i) out[i] = 0.f;
    for (int j = 0; j < k; ++j) {
        const int sj = __shfl(sel, j, CK_WAVE);
        const float dj = __shfl(dv, j, CK_WAVE);
#pragma unroll
        for (int i = 0; i < VPL; ++i)
            if (i * CK_WAVE + lane == sj) out[i] = dj;
    }
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int e = i * CK_WAVE + lane;
        if (e < E) d_logits[t * ld + e] = T::down(out[i]);
    }
}


// ---- gradient of the router's weight -----------------------------------------------------------------------
// d_weight[e, h] = sum_t d_logits[t, e] * x[t, h]: few outputs, a sum over every token.  The tokens are cut into
// pieces; workgroup (column group, piece) multiplies its piece for 256 columns and writes an fp32 partial block, and
// a second launch adds the pieces up in their order and rounds once.  d_logits comes transposed ([E, T], a small
// tensor), so the MFMA's row operand is one 16-byte load per lane; x is contracted along its rows, so each wave
// copies 32 tokens x 64 columns to its own LDS region with 16-byte accesses and picks the column operand from there
// element by element.  Lane l holds (expert 16 nt + 4 (l / 16) + r, column 16 ht + l % 16) of tile (nt, ht).
constexpr int kWgPieceTokens = 32;   // tokens per step
constexpr int kWgWaveCols = 64;      // columns per wave
constexpr int kWgCols = 4 * kWgWaveCols;
constexpr int kWgRowPad = kWgWaveCols + 8;  // LDS row length in elements (16-byte aligned rows)

template <typename T, int NT>
__global__ void __launch_bounds__(256)
    router_weight_grad_kernel(const typename T::storage_t* __restrict__ dlt, const typename T::storage_t* __restrict__ x,
                              int64_t ldx, float* __restrict__ partial, int tokens, int H, int E, int piece_tokens) {
    typedef typename T::storage_t S;
    typedef typename RouterMma<T>::frag_t frag_t;
    __shared__ __attribute__((aligned(16))) S tile[4][kWgPieceTokens][kWgRowPad];
    const int wave = threadIdx.x / CK_WAVE, lane = lane_id();
    const int row = lane % 16, g = lane / 16;
    const int h0 = blockIdx.x * kWgCols + wave * kWgWaveCols;
    const int piece = blockIdx.y;
    const int t_begin = piece * piece_tokens, t_end = min(tokens, t_begin + piece_tokens);
    f32x4_t acc[NT][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int ht = 0; ht < 4; ++ht) acc[nt][ht] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const frag_t zero = {};
    // the lane's part in copying the x tile: token lane / 8 + 8 i of the step, columns 8 (lane % 8) ... of the wave's 64
    const int ct = lane / 8, cc = (lane % 8) * 8;
    const int col = min(h0 + cc, H - 8);  // columns past H are read from a valid place and never stored
    if (h0 < H) {
        for (int t0 = t_begin; t0 < t_end; t0 += kWgPieceTokens) {
            frag_t xin[4], a[NT];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int t = t0 + ct + 8 * i;
                xin[i] = nt_load(reinterpret_cast<const frag_t*>(x + (int64_t)min(t, tokens - 1) * ldx + col));
            }
            const int ta = t0 + 8 * g;  // tokens are a multiple of 8: the packet lies inside the row or outside
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int e = nt * 16 + row;
                a[nt] = *reinterpret_cast<const frag_t*>(dlt + (int64_t)min(e, E - 1) * tokens + min(ta, tokens - 8));
                if (e >= E || ta >= t_end) a[nt] = zero;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int t = t0 + ct + 8 * i;
                *reinterpret_cast<frag_t*>(&tile[wave][ct + 8 * i][cc]) = t < t_end ? xin[i] : zero;
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);  // the wave's own LDS writes (lgkmcnt 0)
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int ht = 0; ht < 4; ++ht) {
                union {
                    S e[8];
                    frag_t f;
                } b;
#pragma unroll
                for (int j = 0; j < 8; ++j) b.e[j] = tile[wave][8 * g + j][ht * 16 + row];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc[nt][ht] = RouterMma<T>::mma(a[nt], b.f, acc[nt][ht]);
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
        }
    }
    float* out = partial + (int64_t)piece * E * H;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int ht = 0; ht < 4; ++ht)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int e = nt * 16 + 4 * g + r, h = h0 + ht * 16 + row;
                if (e < E && h < H) out[(int64_t)e * H + h] = acc[nt][ht][r];
            }
}

// d_weight[e, h] = sum over the pieces of partial[piece][e][h], four columns per lane, in a fixed order (four running
// sums over the pieces p % 4, so that four loads are under way); one rounding
template <typename T>
__global__ void __launch_bounds__(256)
    router_weight_grad_sum_kernel(const float* __restrict__ partial, typename T::storage_t* __restrict__ dw, int64_t ld,
                                  int pieces, int H, int E) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;  // H is a multiple of 8: the four share a row
    const int64_t n = (int64_t)E * H;
    if (i >= n) return;
    f32x4_t sum[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) sum[u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    int p = 0;
    for (; p + 4 <= pieces; p += 4) {
        f32x4_t v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const f32x4_t*>(partial + (int64_t)(p + u) * n + i);
#pragma unroll
        for (int u = 0; u < 4; ++u) sum[u] += v[u];
    }
    for (; p < pieces; ++p) sum[p % 4] += *reinterpret_cast<const f32x4_t*>(partial + (int64_t)p * n + i);
    const f32x4_t total = (sum[0] + sum[1]) + (sum[2] + sum[3]);
    VPack<T, 4> out;
#pragma unroll
    for (int r = 0; r < 4; ++r) out.v[r] = T::down(total[r]);
    typename T::storage_t* dst = dw + (i / H) * ld + i % H;
    if ((reinterpret_cast<uintptr_t>(dst) & 7u) == 0) {
        *reinterpret_cast<VPack<T, 4>*>(dst) = out;
    } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) dst[r] = out.v[r];
    }
}

}  // namespace ck

namespace {
constexpr int64_t kMaxRouterExperts = 1024;  // 16 values per lane
constexpr int64_t kMaxLinearExperts = 128;   // 8 MFMA column tiles
}

#define CK_ROUTER_LAUNCH(KERNEL, ...)                                                                              \
    do {                                                                                                           \
        const int vpl = (int)ck_ceil_div(E, (int64_t)CK_WAVE);                                                     \
        if (vpl <= 1)                                                                                              \
            hipLaunchKernelGGL((ck::KERNEL<T, 1>), dim3((unsigned)grid), dim3(256), 0, s, __VA_ARGS__);            \
        else if (vpl <= 2)                                                                                         \
            hipLaunchKernelGGL((ck::KERNEL<T, 2>), dim3((unsigned)grid), dim3(256), 0, s, __VA_ARGS__);            \
        else if (vpl <= 4)                                                                                         \
            hipLaunchKernelGGL((ck::KERNEL<T, 4>), dim3((unsigned)grid), dim3(256), 0, s, __VA_ARGS__);            \
        else if (vpl <= 8)                                                                                         \
            hipLaunchKernelGGL((ck::KERNEL<T, 8>), dim3((unsigned)grid), dim3(256), 0, s, __VA_ARGS__);            \
        else                                                                                                       \
            hipLaunchKernelGGL((ck::KERNEL<T, 16>), dim3((unsigned)grid), dim3(256), 0, s, __VA_ARGS__);           \
    } while (0)

extern "C" int ck_router_topk_softmax_forward(const void* logits, int64_t logits_stride, void* weights,
                                              float* weights_f32, int64_t* selected, int64_t tokens, int64_t E,
                                              int64_t k, int dtype, void* stream) {
    if (tokens < 0 || E <= 0 || E > kMaxRouterExperts || k <= 0 || k > E || k > CK_WAVE || logits_stride < E)
        return CK_ERR_SHAPE;
    if (tokens == 0) return CK_OK;
    if (!logits || !weights || !weights_f32 || !selected) return CK_ERR_NULL;
    if (!ck_aligned_elem(logits, dtype) || !ck_aligned_elem(weights, dtype)) return CK_ERR_ALIGN;
    const int64_t grid = ck_ceil_div(tokens, 4);
    if (grid > 0x7fffffff) return CK_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        CK_ROUTER_LAUNCH(router_fwd_kernel, (const S*)logits, logits_stride, (S*)weights, weights_f32, selected, tokens,
                         (int)E, (int)k);
    });
    return ck_launch_status();
}

extern "C" int ck_router_forward(const void* x, int64_t x_stride, const void* gate_weight, int64_t gate_weight_stride,
                                 void* logits, int64_t logits_stride, void* weights, float* weights_f32,
                                 int64_t* selected, int64_t tokens, int64_t H, int64_t E, int64_t k, int dtype,
                                 void* stream) {
    if (dtype != CK_BF16 && dtype != CK_F16) return CK_ERR_DTYPE;
    if (tokens < 0 || H <= 0 || H > 0x7fffffff - 1024 || (H & 7) || E <= 0 || E > kMaxLinearExperts || k <= 0 || k > E ||
        k > CK_WAVE || x_stride < H || gate_weight_stride < H || (x_stride & 7) || (gate_weight_stride & 7) ||
        logits_stride < E)
        return CK_ERR_SHAPE;
    if (tokens == 0) return CK_OK;
    if (!x || !gate_weight || !logits || !weights || !weights_f32 || !selected) return CK_ERR_NULL;
    if (!ck_aligned16(x) || !ck_aligned16(gate_weight) || !ck_aligned_elem(logits, dtype) || !ck_aligned_elem(weights, dtype))
        return CK_ERR_ALIGN;
    const int64_t grid = ck_ceil_div(tokens, ck::kRouterTokens);
    if (grid > 0x7fffffff) return CK_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    const int nt = (int)ck_ceil_div(E, 16);
#define CK_ROUTER_LINEAR(TT, NT)                                                                                    \
    hipLaunchKernelGGL((ck::router_linear_fwd_kernel<TT, NT, NT <= 4 ? 16 : 8>), dim3((unsigned)grid),             \
                       dim3((NT <= 4 ? 16 : 8) * CK_WAVE), 0, s,                                                   \
                       (const TT::storage_t*)x, x_stride, (const TT::storage_t*)gate_weight, gate_weight_stride,  \
                       (TT::storage_t*)logits, logits_stride, (TT::storage_t*)weights, weights_f32, selected, tokens, \
                       (int)H, (int)E, (int)k)
#define CK_ROUTER_LINEAR_NT(TT)            \
    do {                                   \
        if (nt <= 1)                       \
            CK_ROUTER_LINEAR(TT, 1);       \
        else if (nt <= 2)                  \
            CK_ROUTER_LINEAR(TT, 2);       \
        else if (nt <= 4)                  \
            CK_ROUTER_LINEAR(TT, 4);       \
        else                               \
            CK_ROUTER_LINEAR(TT, 8);       \
    } while (0)
    if (dtype == CK_BF16)
        CK_ROUTER_LINEAR_NT(ck::BF16);
    else
        CK_ROUTER_LINEAR_NT(ck::F16);
#undef CK_ROUTER_LINEAR_NT
#undef CK_ROUTER_LINEAR
    return ck_launch_status();
}

extern "C" int ck_router_topk_softmax_backward(const void* d_weights, const float* weights_f32, const int64_t* selected,
                                               void* d_logits, int64_t d_logits_stride, int64_t tokens, int64_t E,
                                               int64_t k, int dtype, void* stream) {
    if (tokens < 0 || E <= 0 || E > kMaxRouterExperts || k <= 0 || k > E || k > CK_WAVE || d_logits_stride < E)
        return CK_ERR_SHAPE;
    if (tokens == 0) return CK_OK;
    if (!d_weights || !weights_f32 || !selected || !d_logits) return CK_ERR_NULL;
    if (!ck_aligned_elem(d_weights, dtype) || !ck_aligned_elem(d_logits, dtype)) return CK_ERR_ALIGN;
    const int64_t grid = ck_ceil_div(tokens, 4);
    if (grid > 0x7fffffff) return CK_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    CK_DISPATCH_DTYPE(dtype, {
        typedef typename T::storage_t S;
        CK_ROUTER_LAUNCH(router_bwd_kernel, (const S*)d_weights, weights_f32, selected, (S*)d_logits, d_logits_stride,
                         tokens, (int)E, (int)k);
    });
    return ck_launch_status();
}

namespace {
// pieces of the token range for ck_router_weight_grad: about two workgroups per CU, pieces of whole 32-token steps
void weight_grad_pieces(int64_t tokens, int64_t H, int64_t* pieces, int64_t* piece_tokens) {
    const int64_t groups = ck_ceil_div(H, ck::kWgCols);
    int64_t want = ck_ceil_div(512, groups);
    const int64_t steps = ck_ceil_div(tokens, ck::kWgPieceTokens);
    if (want > steps) want = steps;
    if (want < 1) want = 1;
    *piece_tokens = ck_ceil_div(steps, want) * ck::kWgPieceTokens;
    *pieces = ck_ceil_div(tokens, *piece_tokens);
}
}  // namespace

extern "C" int64_t ck_router_weight_grad_workspace_size(int64_t tokens, int64_t H, int64_t E) {
    if (tokens <= 0 || H <= 0 || E <= 0) return 0;
    int64_t pieces, piece_tokens;
    weight_grad_pieces(tokens, H, &pieces, &piece_tokens);
    return pieces * E * H * (int64_t)sizeof(float);
}

extern "C" int ck_router_weight_grad(const void* d_logits_t, const void* x, int64_t x_stride, void* d_weight,
                                     int64_t d_weight_stride, void* workspace, int64_t workspace_bytes, int64_t tokens,
                                     int64_t H, int64_t E, int dtype, void* stream) {
    if (dtype != CK_BF16 && dtype != CK_F16) return CK_ERR_DTYPE;
    if (tokens <= 0 || tokens > 0x7fffffff - 1024 || (tokens & 7) || H <= 0 || H > 0x7fffffff - 1024 || (H & 7) || E <= 0 ||
        E > kMaxLinearExperts || x_stride < H || (x_stride & 7) || d_weight_stride < H)
        return CK_ERR_SHAPE;
    if (!d_logits_t || !x || !d_weight || !workspace) return CK_ERR_NULL;
    if (!ck_aligned16(d_logits_t) || !ck_aligned16(x) || !ck_aligned_elem(d_weight, dtype)) return CK_ERR_ALIGN;
    if ((reinterpret_cast<uintptr_t>(workspace) & 15u) || workspace_bytes < ck_router_weight_grad_workspace_size(tokens, H, E))
        return CK_ERR_WORKSPACE;
    int64_t pieces, piece_tokens;
    weight_grad_pieces(tokens, H, &pieces, &piece_tokens);
    if (pieces > 65535) return CK_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)ck_ceil_div(H, ck::kWgCols), (unsigned)pieces);
    const int nt = (int)ck_ceil_div(E, 16);
#define CK_WEIGHT_GRAD(TT, NT)                                                                                       \
    hipLaunchKernelGGL((ck::router_weight_grad_kernel<TT, NT>), grid, dim3(256), 0, s, (const TT::storage_t*)d_logits_t, \
                       (const TT::storage_t*)x, x_stride, (float*)workspace, (int)tokens, (int)H, (int)E,           \
                       (int)piece_tokens)
#define CK_WEIGHT_GRAD_NT(TT)                                                                                   \
    do {                                                                                                        \
        if (nt <= 1)                                                                                            \
            CK_WEIGHT_GRAD(TT, 1);                                                                              \
        else if (nt <= 2)                                                                                       \
            CK_WEIGHT_GRAD(TT, 2);                                                                              \
        else if (nt <= 4)                                                                                       \
            CK_WEIGHT_GRAD(TT, 4);                                                                              \
        else                                                                                                    \
            CK_WEIGHT_GRAD(TT, 8);                                                                              \
        hipLaunchKernelGGL((ck::router_weight_grad_sum_kernel<TT>), dim3((unsigned)ck_ceil_div(E * H, 1024)),   \
                           dim3(256), 0, s, (const float*)workspace, (TT::storage_t*)d_weight, d_weight_stride, \
                           (int)pieces, (int)H, (int)E);                                                        \
    } while (0)
    if (dtype == CK_BF16)
        CK_WEIGHT_GRAD_NT(ck::BF16);
    else
        CK_WEIGHT_GRAD_NT(ck::F16);
#undef CK_WEIGHT_GRAD_NT
#undef CK_WEIGHT_GRAD
    return ck_launch_status();
}

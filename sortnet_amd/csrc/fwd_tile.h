// Register/LDS-tiled forward kernel shared by every distance-neuron forward op, and the
// per-op policies plugged into it.
//
// One workgroup = 256 work-items laid out 16 (output channel) x 16 (batch row).  It owns a
// (16*TB) x (16*TM) tile of outputs; each work-item keeps a TB x TM block of accumulators in
// registers (rows tb + 16*i, channels tm + 16*j).  The reduction axis is walked in chunks of
// KT = 32 inputs: the x tile (one or two of them for interval kernels) and the w tile of a
// chunk are staged in LDS with 128-bit global loads, rows padded to 36 floats so that the
// 128-bit LDS reads of the 16 distinct rows of a wavefront fall on distinct banks, and are then
// consumed four inputs at a time.  grid.z carries the group and, for ops whose result can be
// merged with an atomic max, a slice of the reduction range (split-N) so that small batches
// still fill 256 compute units.
#pragma once
#include <float.h>
#include <stdlib.h>
#include "common.h"


namespace sd {

constexpr int KT = 32;        // inputs per LDS chunk
constexpr int LDP = KT + 4;   // padded LDS row length in floats

// -------------------------------------------------------------------------------------------
// tile loaders
// -------------------------------------------------------------------------------------------
__device__ __forceinline__ float mask_value(float v, uint32_t key, uint32_t n, uint32_t t16) {
    return (rng_word(key, n) >> 16) < t16 ? v : __builtin_nanf("");
}

// NX = 1: one input tile.  NX = 2: lower/upper tiles with the inverted-interval repair
// (core/cuda/bound_inf_dist_cuda.cu:63).
template <int NX, int BB>
__device__ __forceinline__ void load_x_tiles(float (*xs0)[LDP], float (*xs1)[LDP], const FwdArgs& a,
                                             int g, int r0, int k0, int n_end) {
    const int tid = threadIdx.x;
    const bool masked = (NX == 1) && a.mask_mode == SD_MASK_FACTORED;
    if (a.fast_x) {
        constexpr int NV = BB * (KT / 4);
        #pragma unroll
        for (int e0 = 0; e0 < NV; e0 += 256) {
            int e = e0 + tid;
            if (NV % 256 != 0 && e >= NV) break;
            int row = e >> 3, c4 = (e & 7) * 4;
            int r = r0 + row, n = k0 + c4;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f), u = v;
            if (r < a.R && n < n_end) {
                size_t off = (size_t)(r * a.G + g) * a.CIg + n;
                v = *reinterpret_cast<const float4*>(a.x0 + off);
                if (NX == 2) {
                    u = *reinterpret_cast<const float4*>(a.x1 + off);
                    if (v.x > u.x) v.x = u.x = (v.x + u.x) * 0.5f;
                    if (v.y > u.y) v.y = u.y = (v.y + u.y) * 0.5f;
                    if (v.z > u.z) v.z = u.z = (v.z + u.z) * 0.5f;
                    if (v.w > u.w) v.w = u.w = (v.w + u.w) * 0.5f;
                }
                if (masked) {
                    uint32_t key = rng_row_key(a.seed, 1u, (uint32_t)(r * a.G + g));
                    v.x = mask_value(v.x, key, n, a.t16);
                    v.y = mask_value(v.y, key, n + 1, a.t16);
                    v.z = mask_value(v.z, key, n + 2, a.t16);
                    v.w = mask_value(v.w, key, n + 3, a.t16);
                }
            }
            *reinterpret_cast<float4*>(&xs0[row][c4]) = v;
            if (NX == 2) *reinterpret_cast<float4*>(&xs1[row][c4]) = u;
        }
    } else {
        for (int e = tid; e < BB * KT; e += 256) {
            int row, c;
            if (a.HW > 1) { c = e / BB; row = e - c * BB; }   // neighbouring rows are contiguous in memory
            else { row = e / KT; c = e - row * KT; }
            int r = r0 + row, n = k0 + c;
            float v = 0.f, u = 0.f;
            if (r < a.R && n < n_end) {
                int b = r / a.HW, hw = r - b * a.HW;
                size_t off = ((size_t)(b * a.G + g) * a.CIg + n) * a.HW + hw;
                v = a.x0[off];
                if (NX == 2) {
                    u = a.x1[off];
                    if (v > u) v = u = (v + u) * 0.5f;
                }
                if (masked) v = mask_value(v, rng_row_key(a.seed, 1u, (uint32_t)((b * a.G + g) * a.HW + hw)), n, a.t16);
            }
            xs0[row][c] = v;
            if (NX == 2) xs1[row][c] = u;
        }
    }
}

template <int BM>
__device__ __forceinline__ void load_w_tile(float (*ws)[LDP], const FwdArgs& a,
                                            int g, int s, int m0, int k0, int n_end) {
    const int tid = threadIdx.x;
    const bool masked = a.mask_mode == SD_MASK_FACTORED;
    if (a.fast_w) {
        constexpr int NV = BM * (KT / 4);
        #pragma unroll
        for (int e0 = 0; e0 < NV; e0 += 256) {
            int e = e0 + tid;
            if (NV % 256 != 0 && e >= NV) break;
            int row = e >> 3, c4 = (e & 7) * 4;
            int m = m0 + row, n = k0 + c4;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (m < a.COg && n < n_end) {
                int wrow = a.co_idx ? a.co_idx[(s * a.G + g) * a.COg + m] : m;
                v = *reinterpret_cast<const float4*>(a.w + (size_t)(g * a.W_COg + wrow) * a.W_CIg + n);
                if (masked) {
                    uint32_t key = rng_row_key(a.seed, 2u, (uint32_t)(g * a.COg + m));
                    v.x = mask_value(v.x, key, n, a.t16);
                    v.y = mask_value(v.y, key, n + 1, a.t16);
                    v.z = mask_value(v.z, key, n + 2, a.t16);
                    v.w = mask_value(v.w, key, n + 3, a.t16);
                }
            }
            *reinterpret_cast<float4*>(&ws[row][c4]) = v;
        }
    } else {
        // a work-item stages one column of the chunk (256 is a multiple of KT): its input index is looked up once
        const int c = tid % KT, n = k0 + c;
        const bool n_ok = n < n_end;
        const int wcol = n_ok ? (a.ci_idx ? a.ci_idx[(s * a.G + g) * a.CIg + n] : n) : 0;
        #pragma unroll
        for (int row = tid / KT; row < BM; row += 256 / KT) {
            int m = m0 + row;
            float v = 0.f;
            if (m < a.COg && n_ok) {
                int wrow = a.co_idx ? a.co_idx[(s * a.G + g) * a.COg + m] : m;
                v = a.w[(size_t)(g * a.W_COg + wrow) * a.W_CIg + wcol];
                if (masked) v = mask_value(v, rng_row_key(a.seed, 2u, (uint32_t)(g * a.COg + m)), n, a.t16);
            }
            ws[row][c] = v;
        }
    }
}

// -------------------------------------------------------------------------------------------
// the kernel
// -------------------------------------------------------------------------------------------
template <class P, int TB, int TM>
__global__ void __launch_bounds__(256, P::MIN_WAVES) fwd_kernel(FwdArgs a) {
    if constexpr (P::GATED) { if (gate_closed(a.gate, a.gate_limit, a.gate_above)) return; }
    constexpr int BB = 16 * TB, BM = 16 * TM, NX = P::NX;
    __shared__ __attribute__((aligned(16))) float xs[NX][BB][LDP];
    __shared__ __attribute__((aligned(16))) float ws[BM][LDP];

    const int tid = threadIdx.x, tm = tid & 15, tb = tid >> 4;
    const int g = blockIdx.z % a.G, split = blockIdx.z / a.G;
    const int r0 = blockIdx.y * BB, m0 = blockIdx.x * BM;
    const int s = (r0 / a.HW) / kSubBatch;

    const int nchunks = (a.CIg + KT - 1) / KT;
    const int n_begin = (int)((long long)split * nchunks / a.nsplit) * KT;
    int n_end = (int)((long long)(split + 1) * nchunks / a.nsplit) * KT;
    if (n_end > a.CIg) n_end = a.CIg;

    typename P::Acc acc[TB][TM];
    #pragma unroll
    for (int i = 0; i < TB; i++) {
        #pragma unroll
        for (int j = 0; j < TM; j++) {
            int r = r0 + tb + 16 * i, m = m0 + tm + 16 * j;
            int b = r / a.HW, hw = r - b * a.HW;
            size_t o = ((size_t)(b * a.G + g) * a.COg + m) * a.HW + hw;
            P::init(acc[i][j], a, o, r < a.R && m < a.COg, split);
        }
    }

    for (int k0 = n_begin; k0 < n_end; k0 += KT) {
        load_x_tiles<NX, BB>(xs[0], xs[NX - 1], a, g, r0, k0, n_end);
        load_w_tile<BM>(ws, a, g, s, m0, k0, n_end);
        __syncthreads();
        #pragma unroll
        for (int pass = 0; pass < P::PASSES; pass++) {
            #pragma unroll P::UNROLL4
            for (int n4 = 0; n4 < KT; n4 += 4) {
                float4 wv[TM];
                const int n4l = n4;
                #pragma unroll
                for (int j = 0; j < TM; j++) wv[j] = *reinterpret_cast<const float4*>(&ws[tm + 16 * j][n4l]);
                #pragma unroll
                for (int i = 0; i < TB; i++) {
                    float4 xl = *reinterpret_cast<const float4*>(&xs[0][tb + 16 * i][n4l]);
                    float4 xu = (NX == 2) ? *reinterpret_cast<const float4*>(&xs[NX - 1][tb + 16 * i][n4l]) : xl;
                    #pragma unroll
                    for (int j = 0; j < TM; j++) P::step4(acc[i][j], a, xl, xu, wv[j], k0 + n4, pass);
                }
            }
            #pragma unroll
            for (int i = 0; i < TB; i++) {
                #pragma unroll
                for (int j = 0; j < TM; j++) P::chunk_end(acc[i][j], a, pass, k0);
            }
        }
        __syncthreads();
    }

    #pragma unroll
    for (int i = 0; i < TB; i++) {
        #pragma unroll
        for (int j = 0; j < TM; j++) {
            int r = r0 + tb + 16 * i, m = m0 + tm + 16 * j;
            if (r < a.R && m < a.COg) {
                int b = r / a.HW, hw = r - b * a.HW;
                size_t o = ((size_t)(b * a.G + g) * a.COg + m) * a.HW + hw;
                P::store(acc[i][j], a, o, split);
            }
        }
    }
}

// -------------------------------------------------------------------------------------------
// Pipelined variant for the vector-load case (HW == 1, reduction length a multiple of 4, no input
// index list).  The global loads of chunk k+1 are issued into registers, branch-free, right after
// chunk k has been published in LDS, and are written to LDS once chunk k has been consumed, so
// HBM/L2 latency hides behind the VALU work of the same workgroup.  One LDS buffer keeps four
// workgroups resident per compute unit: the fp32 vector ALUs only reach their full rate when at
// least two wavefronts per SIMD have VALU work ready.
// In the factored mask mode the keep bits come from bit-mask words built by build_masks_kernel
// (one 32-bit word per row and chunk).
// -------------------------------------------------------------------------------------------
// waves per SIMD the pipelined kernels are compiled for and the unroll factor of their inner loop: a policy may
// name other values for register tiles of at most four channels per work-item (PIPE_WAVES_TM4, UNROLL4_TM4;
// 0 = same)
template <class P, int TB, int TM>
constexpr int pipe_waves() { return (TM <= 4 && P::PIPE_WAVES_TM4) ? P::PIPE_WAVES_TM4 : P::PIPE_WAVES; }
template <class P, int TB, int TM>
constexpr int pipe_unroll() { return (TM <= 4 && P::UNROLL4_TM4) ? P::UNROLL4_TM4 : P::UNROLL4; }

template <class P, int TB, int TM>
__global__ void __launch_bounds__(256, (pipe_waves<P, TB, TM>())) fwd_kernel_pipe(FwdArgs a) {
    if constexpr (P::GATED) { if (gate_closed(a.gate, a.gate_limit, a.gate_above)) return; }
    constexpr int BB = 16 * TB, BM = 16 * TM, NX = P::NX;
    constexpr int NXV = (BB * 8 + 255) / 256, NWV = (BM * 8 + 255) / 256;
    __shared__ __attribute__((aligned(16))) float xs[NX][BB][LDP];
    __shared__ __attribute__((aligned(16))) float ws[BM][LDP];

    const int tid = threadIdx.x, tm = tid & 15, tb = tid >> 4;
    const int g = blockIdx.z % a.G, split = blockIdx.z / a.G;
    const int r0 = blockIdx.y * BB, m0 = blockIdx.x * BM;
    const int s = r0 / kSubBatch;
    const bool masked = (NX == 1) && a.mask_mode == SD_MASK_FACTORED;

    const int nchunks = (a.CIg + KT - 1) / KT;
    const int n_begin = (int)((long long)split * nchunks / a.nsplit) * KT;
    int n_end = (int)((long long)(split + 1) * nchunks / a.nsplit) * KT;
    if (n_end > a.CIg) n_end = a.CIg;

    // staging slot v of a work-item: float4 number v * 256 + tid of a tile = row (tid >> 3) + 32 v,
    // columns (tid & 7) * 4 .. +3.  Rows outside the tensor read row 0 of the tile's first valid
    // row instead (always a legal address) and are zeroed afterwards.
    const int lrow = tid >> 3, lc4 = (tid & 7) * 4;
    // 32-bit element offsets of the rows this work-item stages (pointers would cost twice the registers)
    int xoff[NXV], woff[NWV], xmoff[NXV], wmoff[NWV];
    uint32_t okbits = 0;   // bit v: x row v valid, bit 8 + v: w row v valid
    #pragma unroll
    for (int v = 0; v < NXV; v++) {
        int row = lrow + 32 * v, r = r0 + row;
        bool ok = row < BB && r < a.R;
        int rr = ok ? r : r0;
        okbits |= ok ? 1u << v : 0u;
        xoff[v] = (rr * a.G + g) * a.CIg;
        xmoff[v] = masked ? (rr * a.G + g) * nchunks : 0;
    }
    #pragma unroll
    for (int v = 0; v < NWV; v++) {
        int row = lrow + 32 * v, m = m0 + row;
        bool ok = row < BM && m < a.COg;
        int mm = ok ? m : m0;
        okbits |= ok ? 1u << (8 + v) : 0u;
        int wrow = a.co_idx ? a.co_idx[(s * a.G + g) * a.COg + mm] : mm;
        woff[v] = (g * a.W_COg + wrow) * a.W_CIg;
        wmoff[v] = masked ? (g * a.COg + mm) * nchunks : 0;
    }
    // unmasked: the mask pointers alias x and word 0 is read and ignored
    const uint32_t* xmbase = masked ? a.xmask : reinterpret_cast<const uint32_t*>(a.x0);
    const uint32_t* wmbase = masked ? a.wmask : reinterpret_cast<const uint32_t*>(a.x0);
    const int mstep = masked ? 1 : 0;

    float4 px0[NXV], px1[NXV], pw[NWV];
    uint32_t mx[NXV], mw[NWV];

    auto gload = [&](int k0) {
        int n = k0 + lc4;
        if (n > a.CIg - 4) n = a.CIg - 4;     // keeps the address inside the row; zeroed in sstore()
        #pragma unroll
        for (int v = 0; v < NXV; v++) {
            px0[v] = *reinterpret_cast<const float4*>(a.x0 + xoff[v] + n);
            if (NX == 2) px1[v] = *reinterpret_cast<const float4*>(a.x1 + xoff[v] + n);
            if (NX == 1) mx[v] = xmbase[xmoff[v] + (k0 / KT) * mstep];
        }
        #pragma unroll
        for (int v = 0; v < NWV; v++) {
            pw[v] = *reinterpret_cast<const float4*>(a.w + woff[v] + n);
            if (NX == 1) mw[v] = wmbase[wmoff[v] + (k0 / KT) * mstep];
        }
    };
    auto fix = [&](float4& v, bool ok, uint32_t bits) {
        const float qnan = __builtin_nanf("");
        if (NX == 1) {
            bits = masked ? bits >> lc4 : 0xfu;
            v.x = (bits & 1u) ? v.x : qnan; v.y = (bits & 2u) ? v.y : qnan;
            v.z = (bits & 4u) ? v.z : qnan; v.w = (bits & 8u) ? v.w : qnan;
        }
        v.x = ok ? v.x : 0.f; v.y = ok ? v.y : 0.f; v.z = ok ? v.z : 0.f; v.w = ok ? v.w : 0.f;
    };
    // writes the staged chunk k0 to LDS (zeroing what lies outside the tensor / the slice)
    auto sstore = [&](int k0) {
        const bool in = k0 + lc4 < n_end;
        #pragma unroll
        for (int v = 0; v < NXV; v++) {
            int row = lrow + 32 * v;
            float4 l = px0[v], u = px1[v];
            if (NX == 2) {
                if (l.x > u.x) l.x = u.x = (l.x + u.x) * 0.5f;
                if (l.y > u.y) l.y = u.y = (l.y + u.y) * 0.5f;
                if (l.z > u.z) l.z = u.z = (l.z + u.z) * 0.5f;
                if (l.w > u.w) l.w = u.w = (l.w + u.w) * 0.5f;
                fix(u, ((okbits >> v) & 1u) && in, 0u);
            }
            fix(l, ((okbits >> v) & 1u) && in, NX == 1 ? mx[v] : 0u);
            if (NXV * 32 == BB || row < BB) {
                *reinterpret_cast<float4*>(&xs[0][row][lc4]) = l;
                if (NX == 2) *reinterpret_cast<float4*>(&xs[NX - 1][row][lc4]) = u;
            }
        }
        #pragma unroll
        for (int v = 0; v < NWV; v++) {
            int row = lrow + 32 * v;
            float4 t = pw[v];
            fix(t, ((okbits >> (8 + v)) & 1u) && in, NX == 1 ? mw[v] : 0u);
            if (NWV * 32 == BM || row < BM) *reinterpret_cast<float4*>(&ws[row][lc4]) = t;
        }
    };

    typename P::Acc acc[TB][TM];
    #pragma unroll
    for (int i = 0; i < TB; i++) {
        #pragma unroll
        for (int j = 0; j < TM; j++) {
            int r = r0 + tb + 16 * i, m = m0 + tm + 16 * j;
            size_t o = (size_t)(r * a.G + g) * a.COg + m;
            P::init(acc[i][j], a, o, r < a.R && m < a.COg, split);
        }
    }

    if (n_begin < n_end) gload(n_begin);
    for (int k0 = n_begin; k0 < n_end; k0 += KT) {
        sstore(k0);
        __syncthreads();
        if (k0 + KT < n_end) gload(k0 + KT);
        #pragma unroll
        for (int pass = 0; pass < P::PASSES; pass++) {
            #pragma unroll (pipe_unroll<P, TB, TM>())
            for (int n4 = 0; n4 < KT; n4 += 4) {
                float4 wv[TM];
                #pragma unroll
                for (int j = 0; j < TM; j++) wv[j] = *reinterpret_cast<const float4*>(&ws[tm + 16 * j][n4]);
                #pragma unroll
                for (int i = 0; i < TB; i++) {
                    float4 xl = *reinterpret_cast<const float4*>(&xs[0][tb + 16 * i][n4]);
                    float4 xu = (NX == 2) ? *reinterpret_cast<const float4*>(&xs[NX - 1][tb + 16 * i][n4]) : xl;
                    #pragma unroll
                    for (int j = 0; j < TM; j++) P::step4(acc[i][j], a, xl, xu, wv[j], k0 + n4, pass);
                }
            }
            #pragma unroll
            for (int i = 0; i < TB; i++) {
                #pragma unroll
                for (int j = 0; j < TM; j++) P::chunk_end(acc[i][j], a, pass, k0);
            }
        }
        __syncthreads();
    }

    #pragma unroll
    for (int i = 0; i < TB; i++) {
        #pragma unroll
        for (int j = 0; j < TM; j++) {
            int r = r0 + tb + 16 * i, m = m0 + tm + 16 * j;
            if (r < a.R && m < a.COg) P::store(acc[i][j], a, (size_t)(r * a.G + g) * a.COg + m, split);
        }
    }
}

// -------------------------------------------------------------------------------------------
// Pipelined variant for scalar loads: kept-channel index lists on either side (the weight element of input n
// is w[co_idx[m]][ci_idx[n]]), reduction lengths that are not a multiple of 4, unaligned rows, spatial
// positions (a row of the tile is one (sample, position) pair and its inputs lie HW floats apart).  Work-item t stages column t % 32 of the chunk for the rows t / 32 + 8 k, so a row of the input tile
// is one 128-byte segment when HW == 1 and the index of the column is looked up once.  As in fwd_kernel_pipe the loads of
// chunk k+1 (index, then the gathered weights) are in flight while chunk k is consumed.
// -------------------------------------------------------------------------------------------
template <class P, int TB, int TM>
__global__ void __launch_bounds__(256, (pipe_waves<P, TB, TM>())) fwd_kernel_lists(FwdArgs a) {
    if constexpr (P::GATED) { if (gate_closed(a.gate, a.gate_limit, a.gate_above)) return; }
    static_assert(P::NX == 1 && KT == 32, "one input tile, 32 columns per chunk");
    constexpr int BB = 16 * TB, BM = 16 * TM;
    constexpr int NXR = BB / 8, NWR = BM / 8;
    __shared__ __attribute__((aligned(16))) float xs[BB][LDP];
    __shared__ __attribute__((aligned(16))) float ws[BM][LDP];

    const int tid = threadIdx.x, tm = tid & 15, tb = tid >> 4;
    const int g = blockIdx.z % a.G, split = blockIdx.z / a.G;
    const int r0 = blockIdx.y * BB, m0 = blockIdx.x * BM;
    const int s = (r0 / a.HW) / kSubBatch;

    const int nchunks = (a.CIg + KT - 1) / KT;
    const int n_begin = (int)((long long)split * nchunks / a.nsplit) * KT;
    int n_end = (int)((long long)(split + 1) * nchunks / a.nsplit) * KT;
    if (n_end > a.CIg) n_end = a.CIg;

    const int col = tid & 31, lrow = tid >> 5;
    int xoff[NXR], woff[NWR];
    uint32_t okx = 0u, okw = 0u;
    #pragma unroll
    for (int k = 0; k < NXR; k++) {
        const int r = r0 + lrow + 8 * k;
        const bool ok = r < a.R;
        okx |= ok ? 1u << k : 0u;
        const int rr = ok ? r : r0, b = rr / a.HW, hw = rr - b * a.HW;
        xoff[k] = (b * a.G + g) * a.CIg * a.HW + hw;
    }
    #pragma unroll
    for (int k = 0; k < NWR; k++) {
        const int m = m0 + lrow + 8 * k;
        const bool ok = m < a.COg;
        okw |= ok ? 1u << k : 0u;
        const int mm = ok ? m : m0;
        const int wrow = a.co_idx ? a.co_idx[(s * a.G + g) * a.COg + mm] : mm;
        woff[k] = (g * a.W_COg + wrow) * a.W_CIg;
    }
    const int* cidx = a.ci_idx ? a.ci_idx + (size_t)(s * a.G + g) * a.CIg : nullptr;

    float px[NXR], pw[NWR];
    auto gload = [&](int k0) {
        int n = k0 + col;
        if (n >= n_end) n = n_begin;                  // a legal column; zeroed in sstore()
        const int wcol = cidx ? cidx[n] : n;
        #pragma unroll
        for (int k = 0; k < NXR; k++) px[k] = a.x0[xoff[k] + n * a.HW];
        #pragma unroll
        for (int k = 0; k < NWR; k++) pw[k] = a.w[woff[k] + wcol];
    };
    auto sstore = [&](int k0) {
        const bool in = k0 + col < n_end;
        #pragma unroll
        for (int k = 0; k < NXR; k++) xs[lrow + 8 * k][col] = (in && ((okx >> k) & 1u)) ? px[k] : 0.f;
        #pragma unroll
        for (int k = 0; k < NWR; k++) ws[lrow + 8 * k][col] = (in && ((okw >> k) & 1u)) ? pw[k] : 0.f;
    };

    typename P::Acc acc[TB][TM];
    #pragma unroll
    for (int i = 0; i < TB; i++) {
        #pragma unroll
        for (int j = 0; j < TM; j++) {
            int r = r0 + tb + 16 * i, m = m0 + tm + 16 * j;
            int b = r / a.HW, hw = r - b * a.HW;
            size_t o = ((size_t)(b * a.G + g) * a.COg + m) * a.HW + hw;
            P::init(acc[i][j], a, o, r < a.R && m < a.COg, split);
        }
    }

    if (n_begin < n_end) gload(n_begin);
    for (int k0 = n_begin; k0 < n_end; k0 += KT) {
        sstore(k0);
        __syncthreads();
        if (k0 + KT < n_end) gload(k0 + KT);
        #pragma unroll
        for (int pass = 0; pass < P::PASSES; pass++) {
            #pragma unroll (pipe_unroll<P, TB, TM>())
            for (int n4 = 0; n4 < KT; n4 += 4) {
                float4 wv[TM];
                #pragma unroll
                for (int j = 0; j < TM; j++) wv[j] = *reinterpret_cast<const float4*>(&ws[tm + 16 * j][n4]);
                #pragma unroll
                for (int i = 0; i < TB; i++) {
                    float4 xl = *reinterpret_cast<const float4*>(&xs[tb + 16 * i][n4]);
                    #pragma unroll
                    for (int j = 0; j < TM; j++) P::step4(acc[i][j], a, xl, xl, wv[j], k0 + n4, pass);
                }
            }
            #pragma unroll
            for (int i = 0; i < TB; i++) {
                #pragma unroll
                for (int j = 0; j < TM; j++) P::chunk_end(acc[i][j], a, pass, k0);
            }
        }
        __syncthreads();
    }

    #pragma unroll
    for (int i = 0; i < TB; i++) {
        #pragma unroll
        for (int j = 0; j < TM; j++) {
            int r = r0 + tb + 16 * i, m = m0 + tm + 16 * j;
            if (r < a.R && m < a.COg) {
                int b = r / a.HW, hw = r - b * a.HW;
                P::store(acc[i][j], a, ((size_t)(b * a.G + g) * a.COg + m) * a.HW + hw, split);
            }
        }
    }
}

}  // namespace sd
#include "fwd_direct.h"
namespace sd {

// host-side launcher; the caller has validated shapes
template <class P, int TB, int TM>
int launch_fwd_kernel(const FwdArgs& a, hipStream_t stream) {
    // exact dense tiles of the policies that opt in go through the LDS-direct kernel
    if constexpr (P::DIRECT && TB % 4 == 0 && TM % 4 == 0) {
        if (direct_ok<TB, TM, P::MASKABLE>(a)) return launch_fwd_direct<P, TB, TM>(a, stream);
    }
    dim3 grid((a.COg + 16 * TM - 1) / (16 * TM), (a.R + 16 * TB - 1) / (16 * TB), a.G * a.nsplit);
    if (a.fast_x && a.fast_w && (a.mask_mode != SD_MASK_FACTORED || a.xmask)) {
        note_forward_kernel("fwd_kernel_pipe", TB, TM);
        hipLaunchKernelGGL((fwd_kernel_pipe<P, TB, TM>), grid, dim3(256), 0, stream, a);
        return check_launch("fwd_kernel");
    }
    if constexpr (P::LISTS && TB == 2) {
        if (a.mask_mode != SD_MASK_FACTORED) {
            note_forward_kernel("fwd_kernel_lists", TB, TM);
            hipLaunchKernelGGL((fwd_kernel_lists<P, TB, TM>), grid, dim3(256), 0, stream, a);
            return check_launch("fwd_kernel");
        }
    }
    note_forward_kernel("fwd_kernel", TB, TM);
    hipLaunchKernelGGL((fwd_kernel<P, TB, TM>), grid, dim3(256), 0, stream, a);
    return check_launch("fwd_kernel");
}

template <class P, int TB, int TM>
int launch_fwd(const FwdArgs& a, hipStream_t stream) {
    forward_kernel_timer(stream, false);
    const int rc = launch_fwd_kernel<P, TB, TM>(a, stream);
    forward_kernel_timer(stream, true);
    return rc;
}

// -------------------------------------------------------------------------------------------
// policies.  step4 consumes inputs n .. n+3 of one (row, channel) pair.
// -------------------------------------------------------------------------------------------
struct PolicyBase {
    static constexpr int NX = 1;
    static constexpr int PASSES = 1;
    static constexpr int MIN_WAVES = 1;   // waves per SIMD the register budget must allow
    static constexpr int PIPE_WAVES = 2;  // same for the pipelined kernel
    static constexpr int UNROLL4 = 2;     // unroll factor of the loop over groups of four inputs
    static constexpr int PIPE_WAVES_TM4 = 0, UNROLL4_TM4 = 0;   // overrides for tiles of <= 4 channels (0: none)
    static constexpr int WIDE_TB = 4, WIDE_TM = 8;   // register tile of the large-batch launch of position kernels
    static constexpr bool LISTS = false;  // also built as fwd_kernel_lists (ops that accept kept-channel index lists)
    static constexpr bool DIRECT = false; // also built as fwd_kernel_direct (global -> LDS loads, exact dense tiles)
    static constexpr bool MASKABLE = false;  // fwd_kernel_direct is also built with the factored mask patched into LDS
    static constexpr bool GATED = false;  // the kernels honour FwdArgs::gate
    template <class A> static __device__ __forceinline__ void chunk_end(A&, const FwdArgs&, int, int) {}
    // Per-work-item state next to the per-output accumulators (fwd_kernel_direct only).  A policy with
    // HAS_TSTATE defines TState<N> (N = outputs per work-item), tinit, chunk_end_t and store_t, which then replace
    // chunk_end and store: idx = number of the output inside the register tile, kl = chunk number inside the
    // slice, c0 = first chunk of the slice.
    static constexpr bool HAS_TSTATE = false;
    template <int N> struct TState {};
};

// l-inf forward without indices (core/cuda/inf_dist_cuda.cu:17-107)
struct LinfNograd : PolicyBase {
    static constexpr bool GATED = true;   // one of two queued for a result when FwdArgs::gate is set
    static constexpr bool LISTS = true;
    static constexpr bool DIRECT = true;
    static constexpr bool MASKABLE = true;
    static constexpr int PIPE_WAVES = 3;
    static constexpr int MIN_WAVES = 3;
    static constexpr int UNROLL4 = 1;
    struct Acc { float v; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs&, size_t, bool, int split = 0) { A.v = kEps; }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs&, const float4& x, const float4&,
                                                 const float4& w, int, int) {
        float v = A.v;
        v = fmaxf(fmaxf(v, fabsf(x.x - w.x)), fabsf(x.y - w.y));
        v = fmaxf(fmaxf(v, fabsf(x.z - w.z)), fabsf(x.w - w.w));
        A.v = v;
    }
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) {
        // partial maxima are >= 1e-10 > 0, so their bit patterns order like integers
        if (a.nsplit > 1) atomicMax(reinterpret_cast<int*>(a.y0 + o), __float_as_int(A.v));
        else a.y0[o] = A.v;
    }
};

// the same kernel as one of two queued for a result, see FwdArgs::gate (first step of the general-p l-p forward)
struct LinfNogradGated : LinfNograd {
    static constexpr bool MASKABLE = false;
    static constexpr bool GATED = true;
};

// l-inf forward with arg-max index and sign (core/cuda/inf_dist_cuda.cu:110-212), without paying for
// index bookkeeping on every term: inside a chunk of KT inputs only the maximum
// is kept (one subtract per term, one 3-input max per two terms); at the end of the chunk the
// running (best, chunk index) pair is replaced only on a strictly larger maximum, so the lowest
// chunk attaining the final value survives.  The (best, chunk) pairs of the split-N slices are
// merged with a 64-bit atomic max on (value bits << 32 | ~chunk) and resolve_pos_kernel then
// rescans the one winning chunk of every output for the first input attaining the value.
__device__ __forceinline__ void store_chunk_winner(const FwdArgs& a, size_t o, float best, int cid, bool upper = false) {
    if (a.nsplit > 1) {
        if (cid >= 0) {
            unsigned long long key = ((unsigned long long)__float_as_uint(best) << 32) |
                                     (unsigned long long)(0xffffffffu - (uint32_t)cid);
            atomicMax((upper ? a.packed1 : a.packed0) + o, key);
        }
    } else if (upper) { a.y1[o] = best; a.p1[o] = cid; }
    else { a.y0[o] = best; a.p0[o] = cid; }
}

struct LinfChunk : PolicyBase {
    static constexpr bool GATED = true;   // one of two queued for a result when FwdArgs::gate is set
    static constexpr bool LISTS = true;
    static constexpr int PIPE_WAVES = 2;   // three accumulator registers per output: 2 x 8 outputs leave no room for more
    static constexpr int MIN_WAVES = 2;
    static constexpr int UNROLL4 = 2;
    // vector-load path: 4 x 4 (large batches) or 2 x 4 outputs per work-item in at most 128 registers, four
    // waves per SIMD; measured 7 % faster than 4 x 8 / 2 x 8 outputs at two waves although it reads a third more
    // LDS per term.  The gather kernel of the index lists keeps 2 x 8 at two waves (5 % faster there).
    static constexpr int WIDE_TB = 4, WIDE_TM = 4;
    static constexpr int PIPE_WAVES_TM4 = 4, UNROLL4_TM4 = 1;
    struct Acc { float best, cm; int cid; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs&, size_t, bool, int split = 0) { A.best = kEps; A.cm = 0.f; A.cid = -1; }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs&, const float4& x, const float4&,
                                                 const float4& w, int, int) {
        float v = A.cm;
        v = fmaxf(fmaxf(v, fabsf(x.x - w.x)), fabsf(x.y - w.y));
        v = fmaxf(fmaxf(v, fabsf(x.z - w.z)), fabsf(x.w - w.w));
        A.cm = v;
    }
    static __device__ __forceinline__ void chunk_end(Acc& A, const FwdArgs&, int, int k0) {
        if (A.cm > A.best) { A.best = A.cm; A.cid = k0 / KT; }
        A.cm = 0.f;
    }
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) { store_chunk_winner(a, o, A.best, A.cid); }
};

// LinfChunk for fwd_kernel_direct with the chunk numbers packed four to a register: the number of the winning chunk
// inside the slice needs 8 bits (at most 254 chunks per slice; 255 = none yet), so 4 x 8 outputs cost 64 + 8
// registers instead of 96 and fit four waves per SIMD without staging registers.
struct LinfChunkPacked : PolicyBase {
    static constexpr bool GATED = true;   // one of two queued for a result when FwdArgs::gate is set
    static constexpr bool DIRECT = true;
    static constexpr bool MASKABLE = true;
    static constexpr bool HAS_TSTATE = true;
    static constexpr int MAX_CHUNKS = 254;      // per slice
    struct Acc { float best, cm; };
    template <int N> struct TState { uint32_t cids[(N + 3) / 4]; };
    template <int N> static __device__ __forceinline__ void tinit(TState<N>& S) {
        #pragma unroll
        for (int k = 0; k < (N + 3) / 4; k++) S.cids[k] = 0xffffffffu;
    }
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs&, size_t, bool, int split = 0) { A.best = kEps; A.cm = 0.f; }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs&, const float4& x, const float4&,
                                                 const float4& w, int, int) {
        float v = A.cm;
        v = fmaxf(fmaxf(v, fabsf(x.x - w.x)), fabsf(x.y - w.y));
        v = fmaxf(fmaxf(v, fabsf(x.z - w.z)), fabsf(x.w - w.w));
        A.cm = v;
    }
    template <int N>
    static __device__ __forceinline__ void chunk_end_t(Acc& A, TState<N>& S, const FwdArgs&, int idx, int, int kl) {
        const bool win = A.cm > A.best;          // strictly larger: the lowest chunk attaining the value survives
        const int sh = 8 * (idx & 3);
        const uint32_t f = S.cids[idx >> 2];
        A.best = win ? A.cm : A.best;
        S.cids[idx >> 2] = win ? ((f & ~(0xffu << sh)) | ((uint32_t)kl << sh)) : f;
        A.cm = 0.f;
    }
    template <int N>
    static __device__ __forceinline__ void store_t(Acc& A, TState<N>& S, const FwdArgs& a, size_t o, int, int idx, int c0) {
        const uint32_t kl = (S.cids[idx >> 2] >> (8 * (idx & 3))) & 0xffu;
        store_chunk_winner(a, o, A.best, kl == 0xffu ? -1 : c0 + (int)kl);
    }
    static __device__ __forceinline__ void chunk_end(Acc&, const FwdArgs&, int, int) {}
    static __device__ __forceinline__ void store(Acc&, const FwdArgs&, size_t, int split = 0) {}
};

// |d| when the term's random byte is below the threshold (the term is kept), else 0.  Written as arithmetic on the
// sign of byte - t8 rather than as a compare and a select per term: the compiler still emits compares and selects from
// it, but schedules them 5 % faster than from the conditional expressions (2.12 -> 2.00 ms per 512 x 5120 x 5120 layer).
// Measured and not kept: 24-bit multiplies in the hash (full vector rate instead of a quarter: no change, the kernel is
// not bound by its multiplies) and the same masking forced through inline assembly (3 % slower).
__device__ __forceinline__ float masked_abs(float d, uint32_t byte, uint32_t t8) {
    const uint32_t keep = (uint32_t)(((int)byte - (int)t8) >> 31);
    return __uint_as_float(__float_as_uint(d) & keep & 0x7fffffffu);
}

// the per-term masked neuron with the same chunk tracking
struct MaskedTermChunk : PolicyBase {
    static constexpr int PIPE_WAVES = 2;   // hash-bound: timings were flat over 2..4 waves and 4x8 / 4x4 / 2x8 tiles
    static constexpr int MIN_WAVES = 2;
    struct Acc { float best, cm; int cid; uint32_t key; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs& a, size_t o, bool, int split = 0) {
        A.best = kEps; A.cm = 0.f; A.cid = -1; A.key = rng_row_key(a.seed, 0u, (uint32_t)o);
    }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs& a, const float4& x, const float4&,
                                                 const float4& w, int n, int) {
        const uint32_t word = rng_word(A.key, (uint32_t)n >> 2);
        float v = A.cm;
        v = fmaxf(fmaxf(v, masked_abs(x.x - w.x, word & 0xffu, a.t8)), masked_abs(x.y - w.y, (word >> 8) & 0xffu, a.t8));
        v = fmaxf(fmaxf(v, masked_abs(x.z - w.z, (word >> 16) & 0xffu, a.t8)), masked_abs(x.w - w.w, word >> 24, a.t8));
        A.cm = v;
    }
    static __device__ __forceinline__ void chunk_end(Acc& A, const FwdArgs&, int, int k0) {
        if (A.cm > A.best) { A.best = A.cm; A.cid = k0 / KT; }
        A.cm = 0.f;
    }
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) { store_chunk_winner(a, o, A.best, A.cid); }
};

// masked neuron without positions, independent draw per term: byte (n & 3) of
// word(key(output), n >> 2) < t8 keeps; dropped terms enter the maximum as 0
struct MaskedTermMax : PolicyBase {
    static constexpr int PIPE_WAVES = 2;   // hash-bound: timings were flat over 2..4 waves and 4x8 / 4x4 / 2x8 tiles
    static constexpr int MIN_WAVES = 2;
    struct Acc { float v; uint32_t key; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs& a, size_t o, bool, int split = 0) {
        A.v = kEps; A.key = rng_row_key(a.seed, 0u, (uint32_t)o);
    }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs& a, const float4& x, const float4&,
                                                 const float4& w, int n, int) {
        const uint32_t word = rng_word(A.key, (uint32_t)n >> 2);
        float v = A.v;
        v = fmaxf(fmaxf(v, masked_abs(x.x - w.x, word & 0xffu, a.t8)), masked_abs(x.y - w.y, (word >> 8) & 0xffu, a.t8));
        v = fmaxf(fmaxf(v, masked_abs(x.z - w.z, (word >> 16) & 0xffu, a.t8)), masked_abs(x.w - w.w, word >> 24, a.t8));
        A.v = v;
    }
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) {
        if (a.nsplit > 1) atomicMax(reinterpret_cast<int*>(a.y0 + o), __float_as_int(A.v));
        else a.y0[o] = A.v;
    }
};

// interval bounds, values only (core/cuda/bound_inf_dist_cuda.cu:15-118)
struct BoundNograd : PolicyBase {
    static constexpr bool DIRECT = true;
    static constexpr int PIPE_WAVES = 3;
    static constexpr int NX = 2;
    static constexpr int MIN_WAVES = 3;
    static constexpr int UNROLL4 = 1;
    struct Acc { float lo, hi; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs&, size_t, bool, int split = 0) { A.lo = -kEps; A.hi = kEps; }
    static __device__ __forceinline__ void term(Acc& A, float l, float u, float w) {
        float t1 = w - l, t2 = u - w;
        A.lo = fminf(fminf(A.lo, t1), t2);
        A.hi = fmaxf(fmaxf(A.hi, t1), t2);
    }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs&, const float4& l, const float4& u,
                                                 const float4& w, int, int) {
        term(A, l.x, u.x, w.x); term(A, l.y, u.y, w.y); term(A, l.z, u.z, w.z); term(A, l.w, u.w, w.w);
    }
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) {
        if (a.nsplit > 1) {
            atomicMax(reinterpret_cast<int*>(a.y0 + o), __float_as_int(-A.lo));
            atomicMax(reinterpret_cast<int*>(a.y1 + o), __float_as_int(A.hi));
        } else { a.y0[o] = -A.lo; a.y1[o] = A.hi; }
    }
};

// the same kernel as one of two queued for a result, see FwdArgs::gate
struct BoundNogradGated : BoundNograd {
    static constexpr bool GATED = true;
};

// interval bounds with indices (core/cuda/bound_inf_dist_cuda.cu:121-238), chunk-tracked like LinfChunk: the lower side tracks the largest
// -min(t1,t2) (a positive number once it passes 1e-10), the upper side the largest max(t1,t2);
// resolve_bound_kernel recovers the exact positions and branch bits
struct BoundChunk : PolicyBase {
    static constexpr bool GATED = true;   // one of two queued for a result when FwdArgs::gate is set
    static constexpr int NX = 2;
    static constexpr int PIPE_WAVES = 2;
    static constexpr int MIN_WAVES = 2;
    struct Acc { float lo, hi, cl, ch; int il, ih; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs&, size_t, bool, int split = 0) {
        A.lo = -kEps; A.hi = kEps; A.cl = 0.f; A.ch = 0.f; A.il = -1; A.ih = -1;
    }
    static __device__ __forceinline__ void term(Acc& A, float l, float u, float w) {
        float t1 = w - l, t2 = u - w;
        A.cl = fminf(fminf(A.cl, t1), t2);
        A.ch = fmaxf(fmaxf(A.ch, t1), t2);
    }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs&, const float4& l, const float4& u,
                                                 const float4& w, int, int) {
        term(A, l.x, u.x, w.x); term(A, l.y, u.y, w.y); term(A, l.z, u.z, w.z); term(A, l.w, u.w, w.w);
    }
    static __device__ __forceinline__ void chunk_end(Acc& A, const FwdArgs&, int, int k0) {
        if (A.cl < A.lo) { A.lo = A.cl; A.il = k0 / KT; }
        if (A.ch > A.hi) { A.hi = A.ch; A.ih = k0 / KT; }
        A.cl = 0.f; A.ch = 0.f;
    }
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) {
        store_chunk_winner(a, o, -A.lo, A.il, false);
        store_chunk_winner(a, o, A.hi, A.ih, true);
    }
};

// BoundChunk for the LDS-direct kernel: the numbers of the winning chunks inside the slice kept in 8 bits each, the
// lower and the upper bound's side by side (two outputs to a register; at most 254 chunks per slice, 255 = none), so
// that 4 x 4 outputs cost 64 + 8 registers and the tile fits four waves per SIMD next to no staging registers.  Same
// (value, chunk) pairs as BoundChunk, so the same resolve pass follows.
struct BoundChunkPacked : PolicyBase {
    static constexpr bool GATED = true;   // one of two queued for a result when FwdArgs::gate is set
    static constexpr bool DIRECT = true;
    static constexpr bool HAS_TSTATE = true;
    static constexpr int NX = 2;
    static constexpr int MAX_CHUNKS = 254;      // per slice
    struct Acc { float lo, hi, cl, ch; };
    template <int N> struct TState { uint32_t cids[(N + 1) / 2]; };   // per output: byte 0 lower, byte 1 upper (of its half word)
    template <int N> static __device__ __forceinline__ void tinit(TState<N>& S) {
        #pragma unroll
        for (int k = 0; k < (N + 1) / 2; k++) S.cids[k] = 0xffffffffu;
    }
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs&, size_t, bool, int split = 0) {
        A.lo = -kEps; A.hi = kEps; A.cl = 0.f; A.ch = 0.f;
    }
    static __device__ __forceinline__ void term(Acc& A, float l, float u, float w) {
        float t1 = w - l, t2 = u - w;
        A.cl = fminf(fminf(A.cl, t1), t2);
        A.ch = fmaxf(fmaxf(A.ch, t1), t2);
    }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs&, const float4& l, const float4& u,
                                                 const float4& w, int, int) {
        term(A, l.x, u.x, w.x); term(A, l.y, u.y, w.y); term(A, l.z, u.z, w.z); term(A, l.w, u.w, w.w);
    }
    template <int N>
    static __device__ __forceinline__ void chunk_end_t(Acc& A, TState<N>& S, const FwdArgs&, int idx, int, int kl) {
        const bool wl = A.cl < A.lo, wh = A.ch > A.hi;   // strictly better: the lowest chunk attaining a bound survives
        const int sh = 16 * (idx & 1);
        uint32_t f = S.cids[idx >> 1];
        A.lo = wl ? A.cl : A.lo;
        A.hi = wh ? A.ch : A.hi;
        f = wl ? ((f & ~(0xffu << sh)) | ((uint32_t)kl << sh)) : f;
        f = wh ? ((f & ~(0xffu << (sh + 8))) | ((uint32_t)kl << (sh + 8))) : f;
        S.cids[idx >> 1] = f;
        A.cl = 0.f; A.ch = 0.f;
    }
    template <int N>
    static __device__ __forceinline__ void store_t(Acc& A, TState<N>& S, const FwdArgs& a, size_t o, int, int idx, int c0) {
        const uint32_t f = S.cids[idx >> 1] >> (16 * (idx & 1));
        const uint32_t kl = f & 0xffu, kh = (f >> 8) & 0xffu;
        store_chunk_winner(a, o, -A.lo, kl == 0xffu ? -1 : c0 + (int)kl, false);
        store_chunk_winner(a, o, A.hi, kh == 0xffu ? -1 : c0 + (int)kh, true);
    }
    static __device__ __forceinline__ void chunk_end(Acc&, const FwdArgs&, int, int) {}
    static __device__ __forceinline__ void store(Acc&, const FwdArgs&, size_t, int split = 0) {}
};

// ---- sort neuron -------------------------------------------------------------------------
// res[] ascending (res[K-1] largest), slots start at 0.  A value v > res[0] is inserted above
// equal values: new[k] = clamp(v, res[k], res[k+1]), new[K-1] = max(res[K-1], v); the index
// array follows the same comparisons (core/cuda/sort_neuron.cu:73-77,176-185).
template <int K>
__device__ __forceinline__ void topk_insert_values(float (&res)[K], float v) {
    #pragma unroll
    for (int k = 0; k < K - 1; k++) res[k] = __builtin_amdgcn_fmed3f(res[k], v, res[k + 1]);
    res[K - 1] = __builtin_amdgcn_fmed3f(res[K - 1], v, __builtin_inff());   // max without the NaN-quieting moves of fmaxf
}
template <int K>
__device__ __forceinline__ void topk_insert(float (&res)[K], int (&idx)[K], float v, int p) {
    // (v and the entries are defined numbers here, so "v < res[k + 1]" of slot k is "not v >= res[k + 1]" of slot
    // k + 1: one comparison per slot serves both, and the values move as the median of (res[k], v, res[k + 1]))
    bool ge[K];
    #pragma unroll
    for (int k = 0; k < K; k++) ge[k] = v >= res[k];
    #pragma unroll
    for (int k = 0; k < K - 1; k++) {
        idx[k] = ge[k + 1] ? idx[k + 1] : (ge[k] ? p : idx[k]);
        res[k] = __builtin_amdgcn_fmed3f(res[k], v, res[k + 1]);   // = ge[k + 1] ? res[k + 1] : (ge[k] ? v : res[k])
    }
    idx[K - 1] = ge[K - 1] ? p : idx[K - 1];
    res[K - 1] = ge[K - 1] ? v : res[K - 1];
}
// y = (init + sum_j t_j c_j q) / (1 - c_K), largest first, every product rounded separately
template <int K>
__device__ __forceinline__ float geo_sum(const float (&res)[K], float q) {
    float ans = kEps, c = 1.f;
    #pragma unroll
    for (int k = K - 1; k >= 0; k--) { ans += res[k] * c * q; c *= 1.f - q; }
    return ans / (1.f - c);
}

template <int K>
struct SortNograd : PolicyBase {
    static constexpr bool GATED = true;   // one of two queued for a result when FwdArgs::gate is set
    struct Acc { float res[K]; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs&, size_t, bool, int split = 0) {
        #pragma unroll
        for (int k = 0; k < K; k++) A.res[k] = 0.f;
    }
    static __device__ __forceinline__ void term(Acc& A, float x, float w) {
        float v = fabsf(x - w);
        // wave-uniform test: inserting a value that does not exceed the smallest kept one changes nothing
        if (__builtin_amdgcn_ballot_w64(v > A.res[0]) != 0ull) topk_insert_values<K>(A.res, v);
    }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs&, const float4& x, const float4&,
                                                 const float4& w, int, int) {
        term(A, x.x, w.x); term(A, x.y, w.y); term(A, x.z, w.z); term(A, x.w, w.w);
    }
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) { a.y0[o] = geo_sum<K>(A.res, a.q); }
};

template <int K>
struct SortPos : PolicyBase {
    static constexpr bool GATED = true;   // one of two queued for a result when FwdArgs::gate is set
    struct Acc { float res[K]; int idx[K]; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs&, size_t, bool, int split = 0) {
        #pragma unroll
        for (int k = 0; k < K; k++) { A.res[k] = 0.f; A.idx[k] = 0; }
    }
    static __device__ __forceinline__ void term(Acc& A, float x, float w, int n) {
        float d = x - w, v = fabsf(d);
        if (v > A.res[0]) topk_insert<K>(A.res, A.idx, v, n | (d >= 0.f ? 0 : (int)kSign));
    }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs&, const float4& x, const float4&,
                                                 const float4& w, int n, int) {
        term(A, x.x, w.x, n); term(A, x.y, w.y, n + 1); term(A, x.z, w.z, n + 2); term(A, x.w, w.w, n + 3);
    }
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) {
        a.y0[o] = geo_sum<K>(A.res, a.q);
        size_t size = (size_t)a.B * a.G * a.COg * a.HW;
        #pragma unroll
        for (int k = K - 1; k >= 0; k--) a.p0[(size_t)(K - 1 - k) * size + o] = A.idx[k];
    }
};

// First pass of the two-level sort neuron.  The hot loop only keeps the maximum of |x - w| over a chunk of
// KT inputs (like LinfChunk); at the end of a chunk that maximum, with its low kKeyIdBits mantissa bits
// replaced by the chunk number, enters a sorted list of the K + kKeySlack largest such keys (branch-free
// 3-input medians on the integer patterns; all keys differ because the chunk numbers do).
// Why the list is enough: truncation is monotone, so the K-th largest truncated maximum is the truncation of
// the K-th largest maximum, and every term that can belong to the K largest terms lies in a chunk whose
// truncated maximum reaches that value.  Unless more than kKeySlack further chunks share that truncated
// value (then the smallest kept key still has it and the second pass scans every chunk instead), all those
// chunks are in the list; the second pass (sort_rows_kernel) looks at their K * KT or so candidates only.
// Keys go to p0 as K + kKeySlack planes of (channel, sample) layout.
constexpr int kKeyIdBits = 10;          // chunk numbers below 1024
constexpr int kKeySlack = 6;

__device__ __forceinline__ uint32_t umed3(uint32_t a, uint32_t b, uint32_t c) {
    uint32_t r;
    asm("v_med3_u32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

template <int KP>
__device__ __forceinline__ void key_insert(uint32_t (&key)[KP], uint32_t v) {
    #pragma unroll
    for (int k = 0; k < KP - 1; k++) key[k] = umed3(key[k], v, key[k + 1]);
    key[KP - 1] = key[KP - 1] > v ? key[KP - 1] : v;
}

template <int K>
struct SortChunkKeys : PolicyBase {
    static constexpr bool GATED = true;   // one of two queued for a result when FwdArgs::gate is set
    static constexpr int KP = K + kKeySlack;
    static constexpr int PIPE_WAVES = 2;
    static constexpr int MIN_WAVES = 2;
    struct Acc { float cm; uint32_t key[KP]; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs&, size_t, bool, int split = 0) {
        A.cm = 0.f;
        #pragma unroll
        for (int k = 0; k < KP; k++) A.key[k] = 0u;
    }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs&, const float4& x, const float4&,
                                                 const float4& w, int, int) {
        float v = A.cm;
        v = fmaxf(fmaxf(v, fabsf(x.x - w.x)), fabsf(x.y - w.y));
        v = fmaxf(fmaxf(v, fabsf(x.z - w.z)), fabsf(x.w - w.w));
        A.cm = v;
    }
    static __device__ __forceinline__ void chunk_end(Acc& A, const FwdArgs&, int, int k0) {
        const uint32_t v = (__float_as_uint(A.cm) & ~((1u << kKeyIdBits) - 1u)) | (uint32_t)(k0 / KT);
        A.cm = 0.f;
        key_insert<KP>(A.key, v);
    }
    // plane k, then output channel, then sample: the second pass reads one channel for consecutive samples
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) {
        const int channels = a.G * a.COg;                 // HW == 1 on this path
        const int b = (int)(o / channels), c = (int)(o - (size_t)b * channels);
        #pragma unroll
        for (int k = 0; k < KP; k++) a.p0[((size_t)k * channels + c) * a.B + b] = (int)A.key[k];
    }
};

// interval bounds of the sort neuron (core/cuda/sort_neuron.cu:216-314).  The lower side keeps
// the negated K most negative values of min(t1,t2), so both sides share the insertion routine.
template <int K>
struct BoundSort : PolicyBase {
    static constexpr bool GATED = true;   // one of two queued for a result when FwdArgs::gate is set
    static constexpr int NX = 2;
    struct Acc { float lo[K], hi[K]; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs&, size_t, bool, int split = 0) {
        #pragma unroll
        for (int k = 0; k < K; k++) { A.lo[k] = 0.f; A.hi[k] = 0.f; }
    }
    static __device__ __forceinline__ void term(Acc& A, float l, float u, float w) {
        float t1 = w - l, t2 = u - w;
        float nl = -fminf(t1, t2), hu = fmaxf(t1, t2);
        // one wave-uniform test for both lists: inserting a value that does not exceed the smallest kept one
        // leaves a list unchanged, so the insertions themselves need no lane mask
        if (__builtin_amdgcn_ballot_w64(nl > A.lo[0] || hu > A.hi[0]) != 0ull) {
            topk_insert_values<K>(A.lo, nl);
            topk_insert_values<K>(A.hi, hu);
        }
    }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs&, const float4& l, const float4& u,
                                                 const float4& w, int, int) {
        term(A, l.x, u.x, w.x); term(A, l.y, u.y, w.y); term(A, l.z, u.z, w.z); term(A, l.w, u.w, w.w);
    }
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) {
        a.y0[o] = geo_sum<K>(A.lo, a.q);
        a.y1[o] = geo_sum<K>(A.hi, a.q);
    }
};

// ---- l-p norm distance ---------------------------------------------------------------------
// a^ip for a >= 0 by multiply chains for ip = 1..8 (core/cuda/fast_pow.cuh:1-12), otherwise
// exp2(p log2 a) on the hardware transcendental units.
template <int IP>
__device__ __forceinline__ float pow_pos(float a, float p) {
    float t1;
    switch (IP) {
        case 0: return 1.f;
        case 1: return a;
        case 2: return a * a;
        case 3: return a * a * a;
        case 4: t1 = a * a; return t1 * t1;
        case 5: t1 = a * a; return a * t1 * t1;
        case 6: t1 = a * a; return t1 * t1 * t1;
        case 7: t1 = a * a; return a * t1 * t1 * t1;
        case 8: t1 = a * a; t1 = t1 * t1; return t1 * t1;
        default: return __builtin_amdgcn_exp2f(p * __builtin_amdgcn_logf(a));
    }
}

// s + a^ip for a >= 0: the last product of the chain and the sum are one fused multiply-add
template <int IP>
__device__ __forceinline__ float add_pow(float s, float a, float p) {
    float t1;
    switch (IP) {
        case 0: return s + 1.f;
        case 1: return s + a;
        case 2: return fmaf(a, a, s);
        case 3: return fmaf(a * a, a, s);
        case 4: t1 = a * a; return fmaf(t1, t1, s);
        case 5: t1 = a * a; return fmaf(t1 * t1, a, s);
        case 6: t1 = a * a; return fmaf(t1 * t1, t1, s);
        case 7: t1 = a * a; return fmaf(t1 * t1, t1 * a, s);
        case 8: t1 = a * a; t1 = t1 * t1; return fmaf(t1, t1, s);
        default: return s + __builtin_amdgcn_exp2f(p * __builtin_amdgcn_logf(a));
    }
}

// p <= 10: y = max(sum |d|^p, FLT_MIN)^(1/p)   (core/cuda/norm_dist_cuda.cu:163-259, no max)
template <int IP>
struct LpPlain : PolicyBase {
    static constexpr bool LISTS = true;
    static constexpr bool DIRECT = true;
    static constexpr int PIPE_WAVES = 3;
    static constexpr int MIN_WAVES = 3;
    struct Acc { float s; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs&, size_t, bool, int split = 0) { A.s = 0.f; }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs& a, const float4& x, const float4&,
                                                 const float4& w, int, int) {
        A.s = add_pow<IP>(A.s, fabsf(x.x - w.x), a.p);
        A.s = add_pow<IP>(A.s, fabsf(x.y - w.y), a.p);
        A.s = add_pow<IP>(A.s, fabsf(x.z - w.z), a.p);
        A.s = add_pow<IP>(A.s, fabsf(x.w - w.w), a.p);
    }
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) {
        if (a.nsplit > 1) a.part0[(size_t)split * a.part_stride + o] = A.s;   // summed by lp_finalize_kernel
        else a.y0[o] = powf(fmaxf(A.s, FLT_MIN), a.inv_p);
    }
};

// p > 10: running maximum M with rescaling, two passes over every LDS chunk
// (core/cuda/norm_dist_cuda.cu:36-160): y = M (sum (|d|/M)^p + (1e-10/M)^p)^(1/p).
template <int IP, bool FOLD = (IP < 0)>
struct LpOnline : PolicyBase {
    static constexpr bool LISTS = true;
    static constexpr int PIPE_WAVES = 3;
    static constexpr int MIN_WAVES = 3;
    static constexpr int PASSES = 2;
    // rinv = 1 / M; FOLD (general p) keeps c = p log2(1 / M) there instead, a term is exp2(p log2|d| + c) and the
    // rescaling factor of a new maximum is exp2(c_new - c_old) (see LpWithMax)
    struct Acc { float s, M, rinv, cm; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs& a, size_t, bool, int split = 0) {
        // the virtual term of size 1e-10 (res starts at 1 relative to M = 1e-10) belongs to slice 0 only
        A.s = split == 0 ? 1.f : 0.f; A.M = kEps; A.cm = 0.f;
        A.rinv = FOLD ? -a.p * __builtin_amdgcn_logf(kEps) : 1.f / kEps;
    }
    static __device__ __forceinline__ float term(const Acc& A, const FwdArgs& a, float d) {
        if (FOLD) return __builtin_amdgcn_exp2f(fmaf(a.p, __builtin_amdgcn_logf(fabsf(d)), A.rinv));
        return pow_pos<IP>(fabsf(d) * A.rinv, a.p);
    }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs& a, const float4& x, const float4&,
                                                 const float4& w, int, int pass) {
        if (pass == 0) {
            float v = A.cm;
            v = fmaxf(fmaxf(v, fabsf(x.x - w.x)), fabsf(x.y - w.y));
            v = fmaxf(fmaxf(v, fabsf(x.z - w.z)), fabsf(x.w - w.w));
            A.cm = v;
        } else {
            A.s += term(A, a, x.x - w.x);
            A.s += term(A, a, x.y - w.y);
            A.s += term(A, a, x.z - w.z);
            A.s += term(A, a, x.w - w.w);
        }
    }
    static __device__ __forceinline__ void chunk_end(Acc& A, const FwdArgs& a, int pass, int) {
        if (pass == 0) {
            if (A.cm > A.M) {
                if (FOLD) {
                    const float cn = -a.p * __builtin_amdgcn_logf(A.cm);
                    A.s *= __builtin_amdgcn_exp2f(cn - A.rinv);
                    A.rinv = cn;
                } else {
                    A.s *= __builtin_amdgcn_exp2f(a.p * __builtin_amdgcn_logf(A.M / A.cm));
                    A.rinv = 1.f / A.cm;
                }
                A.M = A.cm;
            }
            A.cm = 0.f;
        }
    }
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) {
        if (a.nsplit > 1) {
            a.part0[(size_t)split * a.part_stride + o] = A.s;
            a.part1[(size_t)split * a.part_stride + o] = A.M;
        } else a.y0[o] = powf(A.s, a.inv_p) * A.M;
    }
};

// caller-supplied maximum (core/cuda/norm_dist_cuda.cu:163-259 with has_max); also the second step of the
// general-p forward, whose first step is the l-inf kernel
template <int IP, bool FOLD = (IP < 0)>
struct LpWithMax : PolicyBase {
    static constexpr bool LISTS = true;
    static constexpr bool DIRECT = true;
    static constexpr bool GATED = true;
    static constexpr int PIPE_WAVES = 3;
    static constexpr int MIN_WAVES = 3;
    // rinv = 1 / maximum; FOLD (general p) keeps c = p log2(1 / maximum) instead, so that a term is
    // exp2(p log2|d| + c): one fused multiply-add in place of the scaling and the product (the rounding of
    // log2|d|, about 2.5e-7 absolute, reaches y divided by p times p, i.e. unchanged: far inside the 1e-5 bar)
    struct Acc { float s, rinv; };
    static __device__ __forceinline__ void init(Acc& A, const FwdArgs& a, size_t o, bool valid, int split = 0) {
        const float rinv = valid ? 1.f / a.aux[o] : 1.f;
        // the virtual term of size 1e-10 belongs to slice 0 only
        A.s = split == 0 ? __builtin_amdgcn_exp2f(a.p * __builtin_amdgcn_logf(kEps * rinv)) : 0.f;
        A.rinv = FOLD ? a.p * __builtin_amdgcn_logf(rinv) : rinv;
    }
    static __device__ __forceinline__ float term(const Acc& A, const FwdArgs& a, float d) {
        if (FOLD) return __builtin_amdgcn_exp2f(fmaf(a.p, __builtin_amdgcn_logf(fabsf(d)), A.rinv));
        return pow_pos<IP>(fabsf(d) * A.rinv, a.p);
    }
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs& a, const float4& x, const float4&,
                                                 const float4& w, int, int) {
        A.s += term(A, a, x.x - w.x);
        A.s += term(A, a, x.y - w.y);
        A.s += term(A, a, x.z - w.z);
        A.s += term(A, a, x.w - w.w);
    }
    static __device__ __forceinline__ void store(Acc& A, const FwdArgs& a, size_t o, int split = 0) {
        if (a.nsplit > 1) a.part0[(size_t)split * a.part_stride + o] = A.s;   // merged by lp_finalize_kernel
        else a.y0[o] = powf(A.s, a.inv_p) * a.aux[o];
    }
};

// Large p: a term whose ratio r to the scale is below skip_thr = (1e-6 / CI)^(1/p) contributes less than
// 1e-6 / CI to a sum that is at least 1, so all such terms together move the result by less than 1e-6 / p
// relative.  Nearly every term is of that kind once p reaches ~100, and the two transcendentals of r^p are
// the whole cost of the kernel: they are evaluated only when some lane of the wavefront holds a significant
// term (wave-uniform branches, first for the group of four inputs, then for each of them).
// The ratios are >= 0, where the bit patterns order like the values; an undefined ratio (an undefined input or
// weight) has a pattern above every number, so it counts as significant and reaches the sum as in the reference.
__device__ __forceinline__ void lp_add_significant(float& s, float r0, float r1, float r2, float r3, float p, float thr) {
    const int i0 = __builtin_bit_cast(int, r0), i1 = __builtin_bit_cast(int, r1);
    const int i2 = __builtin_bit_cast(int, r2), i3 = __builtin_bit_cast(int, r3), it = __builtin_bit_cast(int, thr);
    if (__builtin_amdgcn_ballot_w64(max(max(i0, i1), max(i2, i3)) > it) == 0ull) return;
    if (__builtin_amdgcn_ballot_w64(i0 > it) != 0ull) s += pow_pos<-1>(r0, p);
    if (__builtin_amdgcn_ballot_w64(i1 > it) != 0ull) s += pow_pos<-1>(r1, p);
    if (__builtin_amdgcn_ballot_w64(i2 > it) != 0ull) s += pow_pos<-1>(r2, p);
    if (__builtin_amdgcn_ballot_w64(i3 > it) != 0ull) s += pow_pos<-1>(r3, p);
}

struct LpWithMaxSkip : LpWithMax<-1, false> {   // the significance test needs the ratio itself
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs& a, const float4& x, const float4&,
                                                 const float4& w, int, int) {
        lp_add_significant(A.s, fabsf(x.x - w.x) * A.rinv, fabsf(x.y - w.y) * A.rinv, fabsf(x.z - w.z) * A.rinv,
                           fabsf(x.w - w.w) * A.rinv, a.p, a.skip_thr);
    }
};

struct LpOnlineSkip : LpOnline<-1, false> {
    static __device__ __forceinline__ void step4(Acc& A, const FwdArgs& a, const float4& x, const float4& xu,
                                                 const float4& w, int n, int pass) {
        if (pass == 0) LpOnline<-1, false>::step4(A, a, x, xu, w, n, pass);
        else lp_add_significant(A.s, fabsf(x.x - w.x) * A.rinv, fabsf(x.y - w.y) * A.rinv, fabsf(x.z - w.z) * A.rinv,
                                fabsf(x.w - w.w) * A.rinv, a.p, a.skip_thr);
    }
};

// -------------------------------------------------------------------------------------------
// resolve_pos_kernel: a wavefront owns 64 consecutive outputs.  Each lane first reads the winning
// (value, chunk) pair of its own output left by a chunk-tracking policy (from y/pos when the reduction
// was not split, else from the packed workspace) and posts the row offsets and keep information
// of that output in LDS.  The wavefront then walks its outputs two at a time, 32 lanes per output and
// one input of the winning chunk per lane, so that a chunk is fetched with one coalesced load per
// operand instead of one cache line per lane; a ballot finds the first kept input whose magnitude equals
// the value bit for bit, and the owner lane writes the final value and position.
// -------------------------------------------------------------------------------------------
struct ResolveSlot { int cid; float best; int xoff, woff, coff; uint32_t keep; int pad0, pad1; };

// keep bits of the 32 inputs of chunk `cid` of output `o` (input row xrow, weight row c) under the active mask mode
__device__ __forceinline__ uint32_t chunk_keep_bits(const FwdArgs& a, long long o, int xrow, int c, int cid, int nchunks) {
    if (a.mask_mode == SD_MASK_TERM) {
        const uint32_t key_t = rng_row_key(a.seed, 0u, (uint32_t)o);
        uint32_t keep = 0u;
        #pragma unroll
        for (int q4 = 0; q4 < KT / 4; q4++) {
            const uint32_t word = rng_word(key_t, (uint32_t)(cid * (KT / 4) + q4));
            #pragma unroll
            for (int c4 = 0; c4 < 4; c4++)
                if (((word >> (8 * c4)) & 0xffu) < a.t8) keep |= 1u << (q4 * 4 + c4);
        }
        return keep;
    }
    if (a.mask_mode == SD_MASK_FACTORED) {
        if (a.xmask) return a.xmask[(size_t)xrow * nchunks + cid] & a.wmask[(size_t)c * nchunks + cid];
        const uint32_t key_x = rng_row_key(a.seed, 1u, (uint32_t)xrow), key_w = rng_row_key(a.seed, 2u, (uint32_t)c);
        uint32_t keep = 0u;
        for (int k = 0; k < KT; k++) {
            const uint32_t n = (uint32_t)(cid * KT + k);
            if ((rng_word(key_x, n) >> 16) < a.t16 && (rng_word(key_w, n) >> 16) < a.t16) keep |= 1u << k;
        }
        return keep;
    }
    return 0xffffffffu;
}

// LISTS: the layer has kept-input index lists.  Without them an input's column is its number, and no load stands
// between the two operand loads of one output and those of the next, so that a wavefront has them all in flight.
template <bool PACKED, bool LISTS>
__global__ void __launch_bounds__(256) resolve_pos_kernel(FwdArgs a) {
    if (gate_closed(a.gate, a.gate_limit, a.gate_above)) return;   // one of two queued for the result
    __shared__ __attribute__((aligned(16))) ResolveSlot slots[4][64];
    const long long total = (long long)a.R * a.G * a.COg;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long long o_base = ((long long)blockIdx.x * 4 + wave) * 64;
    if (o_base >= total) return;                       // whole wavefront; no workgroup barrier below
    const long long o = o_base + lane;
    const bool mine = o < total;
    ResolveSlot me;
    me.cid = -1; me.best = kEps; me.xoff = me.woff = me.coff = 0; me.keep = 0u; me.pad0 = me.pad1 = 0;
    if (mine) {
        const int hw = (int)(o % a.HW);
        const long long t = o / a.HW;
        const int c = (int)(t % (a.G * a.COg));
        const int b = (int)(t / (a.G * a.COg));
        const int g = c / a.COg, m = c - g * a.COg;
        if (PACKED) {
            unsigned long long v = a.packed0[o];
            uint32_t low = (uint32_t)v;
            me.best = low ? __uint_as_float((uint32_t)(v >> 32)) : kEps;
            me.cid = low ? (int)(0xffffffffu - low) : -1;
        } else { me.best = a.y0[o]; me.cid = a.p0[o]; }
        if (me.cid >= 0) {
            const int s = b / kSubBatch;
            const int wrow = a.co_idx ? a.co_idx[(s * a.G + g) * a.COg + m] : m;
            me.woff = (g * a.W_COg + wrow) * a.W_CIg;
            me.xoff = (b * a.G + g) * a.CIg * a.HW + hw;
            me.coff = (s * a.G + g) * a.CIg;
            me.keep = chunk_keep_bits(a, o, (b * a.G + g) * a.HW + hw, c, me.cid, (a.CIg + KT - 1) / KT);
        }
    }
    slots[wave][lane] = me;
    __builtin_amdgcn_wave_barrier();                   // LDS operations of one wavefront complete in order

    // slots without a winning chunk keep offset 0 and keep bits 0: their loads hit element 0 and never match
    constexpr int U = 8;
    const int half = lane >> 5, l = lane & 31;
    int pos = 0;
    for (int it0 = 0; it0 < 32; it0 += U) {
        float d[U];
        bool cand[U];
        float best[U];
        #pragma unroll
        for (int u = 0; u < U; u++) {
            const ResolveSlot q = slots[wave][2 * (it0 + u) + half];
            int n = (q.cid < 0 ? 0 : q.cid) * KT + l;
            cand[u] = n < a.CIg && ((q.keep >> l) & 1u) != 0u;
            if (n >= a.CIg) n = 0;
            const int col = LISTS ? a.ci_idx[q.coff + n] : n;
            d[u] = a.x0[(size_t)q.xoff + (size_t)n * a.HW] - a.w[q.woff + col];
            best[u] = q.best;
        }
        #pragma unroll
        for (int u = 0; u < U; u++) {
            const unsigned long long hit = __ballot(cand[u] && fabsf(d[u]) == best[u]);
            const unsigned long long neg = __ballot(d[u] < 0.f);
            if ((lane >> 1) == it0 + u) {              // the two owner lanes of this step
                const uint32_t h32 = (lane & 1) ? (uint32_t)(hit >> 32) : (uint32_t)hit;
                const uint32_t n32 = (lane & 1) ? (uint32_t)(neg >> 32) : (uint32_t)neg;
                if (h32) {
                    const int first = __ffs((int)h32) - 1;
                    pos = (me.cid * KT + first) | (((n32 >> first) & 1u) ? (int)kSign : 0);
                }
            }
        }
    }
    if (mine) { a.y0[o] = me.best; a.p0[o] = pos; }
}

// Position resolve of the interval kernel: rescans the winning chunk of the lower and of the upper
// bound for the first input attaining the bound and rebuilds pos = n | (t1 <= t2 ? 0 : 1 << 31);
// a lower bound that never left its -1e-10 start keeps the 0xffffffff "no gradient" position.
// As resolve_pos_kernel: a wavefront owns 64 consecutive outputs, posts what the rescan needs in LDS and walks its
// outputs two at a time, 32 lanes per output and one input of the winning chunk per lane (coalesced 128-byte pieces
// of l, u and the weight row, for the lower and then for the upper bound); a ballot finds the first input whose term
// equals the bound bit for bit, a second one says which of its two terms it was.
struct ResolveBoundSlot { int cl, cu; float vl, vu; unsigned long long xoff, woff; };

template <bool PACKED>
__global__ void __launch_bounds__(256) resolve_bound_kernel(FwdArgs a) {
    __shared__ __attribute__((aligned(16))) ResolveBoundSlot slots[4][64];
    if (a.resolved != nullptr && *a.resolved != 0ull) return;   // (uniform over the launch)
    const long long total = (long long)a.R * a.G * a.COg;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long long o_base = ((long long)blockIdx.x * 4 + wave) * 64;
    if (o_base >= total) return;                       // whole wavefront; no workgroup barrier below
    const long long o = o_base + lane;
    const bool mine = o < total;
    ResolveBoundSlot me;
    me.cl = me.cu = -1; me.vl = me.vu = kEps; me.xoff = me.woff = 0ull;
    if (mine) {
        const int hw = (int)(o % a.HW);
        const long long t = o / a.HW;
        const int c = (int)(t % (a.G * a.COg));
        const int b = (int)(t / (a.G * a.COg));
        const int g = c / a.COg;
        if (PACKED) {
            const unsigned long long pl = a.packed0[o], pu = a.packed1[o];
            const uint32_t ll = (uint32_t)pl, lu = (uint32_t)pu;
            me.vl = ll ? __uint_as_float((uint32_t)(pl >> 32)) : kEps; me.cl = ll ? (int)(0xffffffffu - ll) : -1;
            me.vu = lu ? __uint_as_float((uint32_t)(pu >> 32)) : kEps; me.cu = lu ? (int)(0xffffffffu - lu) : -1;
        } else { me.vl = a.y0[o]; me.cl = a.p0[o]; me.vu = a.y1[o]; me.cu = a.p1[o]; }
        me.woff = (unsigned long long)c * a.CIg;
        me.xoff = ((unsigned long long)(b * a.G + g) * a.CIg) * a.HW + hw;
    }
    slots[wave][lane] = me;
    __builtin_amdgcn_wave_barrier();                   // LDS operations of one wavefront complete in order

    const int half = lane >> 5, l = lane & 31;
    uint32_t posl = kNanId, posu = 0u;
    constexpr int U = 4;
    for (int it0 = 0; it0 < 32; it0 += U) {
        float t1[U][2], t2[U][2], target[U][2];
        bool cand[U][2];
        int nn[U][2];
        #pragma unroll
        for (int u = 0; u < U; u++) {
            const ResolveBoundSlot q = slots[wave][2 * (it0 + u) + half];
            #pragma unroll
            for (int side = 0; side < 2; side++) {
                const int cid = side ? q.cu : q.cl;
                int n = (cid < 0 ? 0 : cid) * KT + l;
                cand[u][side] = cid >= 0 && n < a.CIg;
                if (n >= a.CIg) n = 0;
                float lv = a.x0[q.xoff + (size_t)n * a.HW], uv = a.x1[q.xoff + (size_t)n * a.HW];
                const float wv = a.w[q.woff + n];
                if (lv > uv) lv = uv = (lv + uv) * 0.5f;
                t1[u][side] = wv - lv; t2[u][side] = uv - wv;
                target[u][side] = side ? q.vu : q.vl;
                nn[u][side] = n;
            }
        }
        #pragma unroll
        for (int u = 0; u < U; u++) {
            #pragma unroll
            for (int side = 0; side < 2; side++) {
                const float v = side ? fmaxf(t1[u][side], t2[u][side]) : -fminf(t1[u][side], t2[u][side]);
                const unsigned long long hit = __ballot(cand[u][side] && v == target[u][side]);
                const unsigned long long second = __ballot(!(t1[u][side] <= t2[u][side]));
                if ((lane >> 1) == it0 + u) {          // the two owner lanes of this step
                    const uint32_t h32 = (lane & 1) ? (uint32_t)(hit >> 32) : (uint32_t)hit;
                    const uint32_t s32 = (lane & 1) ? (uint32_t)(second >> 32) : (uint32_t)second;
                    if (h32) {
                        const int first = __ffs((int)h32) - 1;
                        const int cid = side ? me.cu : me.cl;
                        const uint32_t found = (uint32_t)(cid * KT + first) | (((s32 >> first) & 1u) ? kSign : 0u);
                        if (side) posu = found; else posl = found;
                    }
                }
            }
        }
    }
    if (mine) {
        a.y0[o] = me.vl; a.y1[o] = me.vu;
        a.p0[o] = (int)posl; a.p1[o] = (int)posu;
    }
}

inline int launch_resolve_bound(const FwdArgs& a, hipStream_t stream) {
    long long total = (long long)a.R * a.G * a.COg;
    dim3 grid((unsigned)((total + 255) / 256));
    if (a.nsplit > 1) hipLaunchKernelGGL((resolve_bound_kernel<true>), grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((resolve_bound_kernel<false>), grid, dim3(256), 0, stream, a);
    return check_launch("resolve_bound_kernel");
}

inline int launch_resolve(const FwdArgs& a, hipStream_t stream) {
    long long total = (long long)a.R * a.G * a.COg;
    dim3 grid((unsigned)((total + 255) / 256));
    if (a.ci_idx) {
        if (a.nsplit > 1) hipLaunchKernelGGL((resolve_pos_kernel<true, true>), grid, dim3(256), 0, stream, a);
        else hipLaunchKernelGGL((resolve_pos_kernel<false, true>), grid, dim3(256), 0, stream, a);
    } else {
        if (a.nsplit > 1) hipLaunchKernelGGL((resolve_pos_kernel<true, false>), grid, dim3(256), 0, stream, a);
        else hipLaunchKernelGGL((resolve_pos_kernel<false, false>), grid, dim3(256), 0, stream, a);
    }
    return check_launch("resolve_pos_kernel");
}

}  // namespace sd

// Forward tile kernel whose operand tiles go from global memory straight into LDS (global_load_lds_dwordx4, the
// 128-bit LDS-direct load of gfx950) instead of through staging registers.
//
// Why: the tropical inner loop issues one LDS read per (TB + TM) / (TB * TM * 4) terms and 1.5 .. 4 vector
// instructions per term; at 4 x 8 outputs per work-item the LDS pipe and the vector ALUs of a compute unit are
// loaded about equally, and a larger register tile does not fit next to the 32 staging registers of the
// register-staged kernel (fwd_kernel_pipe) in the 128 registers that four waves per SIMD allow (three resident
// waves per SIMD issue at 3/4 of the rate of two or four).  Without staging registers 8 x 8 outputs of the
// one-accumulator policies and 4 x 8 of the interval policy fit in 128 registers.
//
// Layout: a chunk is KD = 16 inputs; a tile row is 64 bytes = four 16-byte slots.  One wave-wide load fills 16
// rows (lane l -> row l / 4, slot l % 4, 1024 contiguous bytes at the LDS address in M0).  Slot s of row r holds
// input group s ^ ((r / 4) % 4) -- the swizzle is applied to the global address of the lane.  The LDS has 64 banks of
// 4 bytes, i.e. sixteen 16-byte units per 256 bytes, and row r owns units 4 (r % 4) .. + 3: the four rows that share a
// unit group (r, r + 4, r + 8, r + 12) then read four different units, so the 128-bit reads of sixteen consecutive
// rows at one input group are conflict-free.
// Two LDS buffers: the loads of chunk k + 1 are in flight while chunk k is consumed, one barrier per chunk.
// Requirements (checked by the launcher): HW == 1, no index lists, no mask, CI / G a multiple of 32, rows and
// channels multiples of the tile, 16-byte aligned operands.  Everything else takes the register-staged kernels.
// Included by fwd_tile.h (which defines FwdArgs, KT and the policies) right before its launcher.
#pragma once

namespace sd {

constexpr int KD = 16;   // inputs per LDS-direct chunk

// One wave-wide 128-bit LDS-direct load: lane l moves 16 bytes from base + voff to LDS byte address lds + 16 l.
// Written as inline assembly on purpose: through the compiler builtin every later LDS read counts as possibly
// aliasing the load and is preceded by s_waitcnt vmcnt(0), which would expose the whole global latency once per
// chunk; here the kernel places its own waits (vmcnt(0) before the barrier that publishes a buffer).
__device__ __forceinline__ void load_group_to_lds(const float* base, uint32_t voff, uint32_t lds) {
    // the base is uniform, but under register pressure the compiler may hold it in vector registers: force a scalar pair
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    // (the builtin returns a signed int: widen through uint32_t, or the low half sign-extends into the high half)
    const uint64_t sb = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32)) << 32) |
                        (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b);
    base = reinterpret_cast<const float*>(sb);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds), "v"(voff), "s"(base) : "memory", "m0");
}

__device__ __forceinline__ uint32_t lds_address(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}

// slot of input group c (0..3) in tile row r
__device__ __forceinline__ int swz(int c, int r) { return c ^ ((r >> 2) & 3); }

template <class P, int TB, int TM, bool MASKED>
__global__ void __launch_bounds__(256, 4) fwd_kernel_direct(FwdArgs a) {
    if constexpr (P::GATED) { if (gate_closed(a.gate, a.gate_limit, a.gate_above)) return; }
    constexpr int BB = 16 * TB, BM = 16 * TM, NX = P::NX;
    constexpr int XG = BB / 16, WG = BM / 16;          // 16-row groups of one x tile / of the w tile
    constexpr int NG = NX * XG + WG;                    // wave-wide loads per chunk
    constexpr int GPW = NG / 4;                         // per wave
    static_assert(P::PASSES == 1, "single-pass policies only");
    static_assert(!MASKED || P::NX == 1, "the factored mask applies to one-input policies");
    __shared__ __attribute__((aligned(1024))) float tiles[2][NG * 16 * KD];

    const int tid = threadIdx.x, tm = tid & 15, tb = tid >> 4;
    const int wave = tid >> 6, lane = tid & 63, lr = lane >> 2, ls = lane & 3;
    const int g = blockIdx.z % a.G, split = blockIdx.z / a.G;
    const int r0 = blockIdx.y * BB, m0 = blockIdx.x * BM;

    const int nchunks = a.CIg / KT;
    const int n_begin = (int)((long long)split * nchunks / a.nsplit) * KT;
    const int n_end = (int)((long long)(split + 1) * nchunks / a.nsplit) * KT;

    // Loads of this wave (GPW per chunk, the same number for every wave).  One x tile: x groups wave + 4 u, then
    // w groups wave + 4 u.  Interval policies repair inverted intervals in LDS before the chunk is published, which
    // needs the lower and upper copy of a slot in the same lane: lower group q and upper group q are consecutive
    // loads of one wave.  LDS group order inside a buffer: lower x groups, upper x groups, w groups.
    static_assert(XG % 4 == 0 && WG % 4 == 0, "tile rows and channels must be multiples of 64");
    constexpr int XL = NX * XG / 4;                     // x loads per wave
    const int col = 4 * swz(ls, lr);
    // uniform bases of this workgroup's rows; per-lane byte offsets relative to them (they fit 32 bits: at most
    // 128 rows of the tile)
    const float* xbase0 = a.x0 + (size_t)(r0 * a.G + g) * a.CIg;
    const float* xbase1 = NX == 2 ? a.x1 + (size_t)(r0 * a.G + g) * a.CIg : xbase0;
    const float* wbase = a.w + (size_t)(g * a.W_COg + m0) * a.W_CIg;
    uint32_t goff[GPW];     // byte offset of this lane's 16 bytes at input 0
    #pragma unroll
    for (int v = 0; v < GPW; v++) {
        if (v < XL) {
            const int q = wave + 4 * (v / NX);
            goff[v] = (uint32_t)(((q * 16 + lr) * a.G * a.CIg + col) * 4);
        } else {
            const int q = wave + 4 * (v - XL);
            goff[v] = (uint32_t)(((q * 16 + lr) * a.W_CIg + col) * 4);
        }
    }
    // LDS group of load v (wave-uniform)
    auto lds_group = [&](int v) {
        if (v < XL) return (v % NX) * XG + wave + 4 * (v / NX);
        return NX * XG + wave + 4 * (v - XL);
    };
    const uint32_t lds0 = lds_address(&tiles[0][0]);

    auto issue = [&](int k0, int buf) {
        #pragma unroll
        for (int v = 0; v < GPW; v++) {
            const float* base = v >= XL ? wbase : ((v % NX) ? xbase1 : xbase0);
            load_group_to_lds(base + k0, goff[v],
                              __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)((buf * NG + lds_group(v)) * 16 * KD * 4)));
        }
    };
    // Factored mask: dropped inputs / weights become NaN in LDS (NaN never wins a maximum), from the keep-bit words
    // that build_masks_kernel left in the workspace (one 32-bit word per row and 32 inputs).  A lane patches the
    // slots it loaded itself, after its loads have landed and before the barrier publishes them.
    int moff[GPW];
    #pragma unroll
    for (int v = 0; v < GPW; v++) {
        if (!MASKED) moff[v] = 0;
        else if (v < XL) moff[v] = ((r0 + (wave + 4 * v) * 16 + lr) * a.G + g) * nchunks;
        else moff[v] = (g * a.COg + m0 + (wave + 4 * (v - XL)) * 16 + lr) * nchunks;
    }
    uint32_t mword[GPW];
    auto fetch_masks = [&](int k0) {       // words of the 32-input chunk that holds k0
        if (!MASKED) return;
        #pragma unroll
        for (int v = 0; v < GPW; v++) mword[v] = (v < XL ? a.xmask : a.wmask)[moff[v] + k0 / KT];
    };
    auto apply_masks = [&](int buf, int k0) {
        if (!MASKED) return;
        const float qnan = __builtin_nanf("");
        #pragma unroll
        for (int v = 0; v < GPW; v++) {
            float4* ps = reinterpret_cast<float4*>(&tiles[buf][lds_group(v) * 16 * KD + lane * 4]);
            float4 t = *ps;
            const uint32_t bits = mword[v] >> ((k0 & (KT - 1)) + col);
            t.x = (bits & 1u) ? t.x : qnan; t.y = (bits & 2u) ? t.y : qnan;
            t.z = (bits & 4u) ? t.z : qnan; t.w = (bits & 8u) ? t.w : qnan;
            *ps = t;
        }
    };

    // inverted intervals (lower > upper) become their midpoint (core/cuda/bound_inf_dist_cuda.cu:63); this lane
    // checks the slots it loaded itself, after its loads have landed and before the barrier publishes them
    auto repair = [&](int buf) {
        if (NX != 2) return;
        #pragma unroll
        for (int v = 0; v + 1 < XL; v += 2) {
            float4* pl = reinterpret_cast<float4*>(&tiles[buf][lds_group(v) * 16 * KD + lane * 4]);
            float4* pu = reinterpret_cast<float4*>(&tiles[buf][lds_group(v + 1) * 16 * KD + lane * 4]);
            float4 l = *pl, u = *pu;
            const bool bad = l.x > u.x || l.y > u.y || l.z > u.z || l.w > u.w;
            if (__builtin_amdgcn_ballot_w64(bad) != 0ull) {
                if (l.x > u.x) l.x = u.x = (l.x + u.x) * 0.5f;
                if (l.y > u.y) l.y = u.y = (l.y + u.y) * 0.5f;
                if (l.z > u.z) l.z = u.z = (l.z + u.z) * 0.5f;
                if (l.w > u.w) l.w = u.w = (l.w + u.w) * 0.5f;
                *pl = l; *pu = u;
            }
        }
    };

    typename P::Acc acc[TB][TM];
    typename P::template TState<TB * TM> tstate;
    if constexpr (P::HAS_TSTATE) P::tinit(tstate);
    #pragma unroll
    for (int i = 0; i < TB; i++) {
        #pragma unroll
        for (int j = 0; j < TM; j++) {
            const int r = r0 + tb + 16 * i, m = m0 + tm + 16 * j;
            P::init(acc[i][j], a, (size_t)(r * a.G + g) * a.COg + m, true, split);
        }
    }

    // read offsets (floats) of this work-item inside a buffer, without the slot
    const int xrow = tb * KD, wrow = (NX * XG * 16 + tm) * KD;
    const int xswz = (tb >> 2) & 3, wswz = (tm >> 2) & 3;

    auto compute = [&](int buf, int k0) {
        const float* T = tiles[buf];
        #pragma unroll 1
        for (int c = 0; c < KD / 4; c++) {
            float4 wv[TM];
            #pragma unroll
            for (int j = 0; j < TM; j++) wv[j] = *reinterpret_cast<const float4*>(&T[wrow + j * 16 * KD + 4 * (c ^ wswz)]);
            #pragma unroll
            for (int i = 0; i < TB; i++) {
                const float4 xl = *reinterpret_cast<const float4*>(&T[xrow + i * 16 * KD + 4 * (c ^ xswz)]);
                const float4 xu = (NX == 2) ? *reinterpret_cast<const float4*>(&T[xrow + (XG + i) * 16 * KD + 4 * (c ^ xswz)]) : xl;
                #pragma unroll
                for (int j = 0; j < TM; j++) P::step4(acc[i][j], a, xl, xu, wv[j], k0 + 4 * c, 0);
            }
        }
    };

    // waits until this wave's LDS-direct loads have landed; the empty statement keeps the compiler from moving the
    // LDS reads of the patch-up code above the wait (it does not know that the loads write LDS)
    auto landed = [&]() {
        __builtin_amdgcn_s_waitcnt(0x0f70);      // vmcnt(0)
        asm volatile("" ::: "memory");
    };

    // one iteration = one chunk of KT = 32 inputs = two LDS-direct sub-chunks (buffers 0 and 1)
    if (n_begin < n_end) { fetch_masks(n_begin); issue(n_begin, 0); }
    for (int k0 = n_begin; k0 < n_end; k0 += KT) {
        landed();
        repair(0);
        apply_masks(0, k0);
        __syncthreads();                          // buffer 0 complete; everyone is done reading buffer 1
        issue(k0 + KD, 1);
        compute(0, k0);
        landed();
        repair(1);
        apply_masks(1, k0 + KD);
        __syncthreads();                          // buffer 1 complete; everyone is done reading buffer 0
        if (k0 + KT < n_end) { fetch_masks(k0 + KT); issue(k0 + KT, 0); }
        compute(1, k0 + KD);
        #pragma unroll
        for (int i = 0; i < TB; i++) {
            #pragma unroll
            for (int j = 0; j < TM; j++) {
                if constexpr (P::HAS_TSTATE) P::chunk_end_t(acc[i][j], tstate, a, i * TM + j, k0, (k0 - n_begin) / KT);
                else P::chunk_end(acc[i][j], a, 0, k0);
            }
        }
    }

    #pragma unroll
    for (int i = 0; i < TB; i++) {
        #pragma unroll
        for (int j = 0; j < TM; j++) {
            const int r = r0 + tb + 16 * i, m = m0 + tm + 16 * j;
            const size_t o = (size_t)(r * a.G + g) * a.COg + m;
            if constexpr (P::HAS_TSTATE) P::store_t(acc[i][j], tstate, a, o, split, i * TM + j, n_begin / KT);
            else P::store(acc[i][j], a, o, split);
        }
    }
}

// true when the LDS-direct kernel with this tile can serve the call (the factored mask needs its keep-bit words and
// a policy that is built with the mask patch)
template <int TB, int TM, bool MASKABLE = true>
inline bool direct_ok(const FwdArgs& a) {
    const bool mask_ok = a.mask_mode < 0 || (MASKABLE && a.mask_mode == SD_MASK_FACTORED && a.xmask && a.wmask && !a.x1);
    // per-lane byte offsets are 32-bit and relative to the first row of the tile: 128 rows must stay below 4 GiB
    const bool offsets_ok = 128ll * a.G * a.CIg * 4 < (1ll << 32) && 128ll * a.W_CIg * 4 < (1ll << 32);
    return a.fast_x && a.fast_w && mask_ok && offsets_ok && !a.co_idx && !a.ci_idx && a.HW == 1 &&
           a.CIg % KT == 0 && a.R % (16 * TB) == 0 && a.COg % (16 * TM) == 0;
}

template <class P, int TB, int TM>
int launch_fwd_direct(const FwdArgs& a, hipStream_t stream) {
    dim3 grid(a.COg / (16 * TM), a.R / (16 * TB), a.G * a.nsplit);
    note_forward_kernel("fwd_kernel_direct", TB, TM);
    if constexpr (P::NX == 1 && P::MASKABLE) {
        if (a.mask_mode == SD_MASK_FACTORED) {
            hipLaunchKernelGGL((fwd_kernel_direct<P, TB, TM, true>), grid, dim3(256), 0, stream, a);
            return check_launch("fwd_kernel_direct");
        }
    }
    hipLaunchKernelGGL((fwd_kernel_direct<P, TB, TM, false>), grid, dim3(256), 0, stream, a);
    return check_launch("fwd_kernel_direct");
}

}  // namespace sd

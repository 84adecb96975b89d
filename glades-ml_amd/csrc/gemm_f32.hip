// fp32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32) for the canonical fp32 path:
// arbitrary M, N, K (bounds-checked, zero-filled tiles), either operand stored K-major or not,
// fused epilogues (bias + activation, activation-derivative product, plain scale).
//
// It realises the reference's three loop nests as matrix products over a whole batch:
//   forward   a_{l+1} = squash(W a_l + b)        network.cpp:466-516  -> C = A * W^T
//   back-prop e = W^T d                          network.cpp:660-662  -> C = D * W
//   gradient  dW = d (x) a, summed over the batch  node.cpp:278-292   -> C = D^T * A, with the
//             weight update (node.cpp:285-306 per batch: learning rate, momentum, both decays) and the
//             bias update (network.cpp:654-656 as a batch mean per output channel) in the epilogue
//
// Tile: 64 x 64 per workgroup of 8 wavefronts, K in slabs of 64.  Wavefront w owns the 32x32
// accumulator (w/2)%2, w%2 of the tile and half of every slab's K (w/4): these products are small
// (batch 512, layers ~1024 wide), so splitting K inside the workgroup is what gives all four SIMDs
// of a CU a matrix instruction stream; the two halves are added through LDS in a fixed order.
// A product whose 64 x 64 tiling leaves half of the compute units idle (128 workgroups or fewer)
// runs with 32 x 64 tiles instead: two 32x32 accumulators and a quarter of every slab's K per wavefront.
// Each operand keeps in LDS the orientation it has in global memory, so that staging never
// transposes: [k][row] for a K-major operand, [row][k] otherwise, both with pitch 68 (16-byte
// stores).  A lane of the 32x32x2 instruction supplies one row and one of the two k of an MFMA; here
// lane half lk takes k = 16*lk + i of its wavefront's half slab for MFMA i, so a [row][k] operand is
// fetched with four 16-byte reads per slab (a [k][row] operand with sixteen 4-byte reads).  Two LDS
// slabs per operand (slab kt feeds the matrix cores while slab kt+1 is written into the buffer slab kt-1
// has left) and two register sets holding the slabs after those on their way from memory: 68 KB of LDS,
// so that two workgroups share a compute unit and one's first loads, reduction and epilogue run under
// the other's K loop (with a third slab resting in LDS a workgroup had the unit to itself: the
// weight gradients of cfg3's step took 49 us instead of 37).

#include <cstring>

#include "ghip_internal.h"

#include <mutex>

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BN = 64, BK = 64, LDT = 64 + 4, NST = 2, NTHR = 512;

template <int UNITS>
struct Frag { float4 v[UNITS]; unsigned char ok[UNITS]; };  // ok: bit j = component j of the unit lies inside the operand

// Fetch this thread's UNITS float4 of a ROWS(row) x 64(k) operand tile (ROWS = UNITS * 32).
//   kmajor == 0: P is [rows][K]  (ld = row stride): unit u -> row = u/16, k = (u%16)*4 .. +3
//   kmajor == 1: P is [K][rows]  (ld = k stride):   unit u -> k = u/(ROWS/4), row = (u%(ROWS/4))*4 .. +3
// FAST: the minor extent is a multiple of 4 and rows are 16-byte aligned, so a unit is wholly
// inside or wholly outside the operand: one unconditional 16-byte load from a clamped address and
// a select, no control flow (loads inside branches are waited for where the branches join, which
// serialises the slab's fetch with its use).  Otherwise: four 4-byte loads, each from its own
// clamped address, and four selects -- still no control flow.
template <bool FAST, int UNITS>
__device__ __forceinline__ Frag<UNITS> fetch(const float* __restrict__ P, int ld, int kmajor, int r0, int k0, int R, int K, int t)
{
    Frag<UNITS> f;
    const int sh = (kmajor && UNITS == 1) ? 3 : 4;  // log2 of the units along the minor extent
#pragma unroll
    for (int i = 0; i < UNITS; ++i) {
        const int u = t + i * NTHR;
        const int major = u >> sh, minor = (u & ((1 << sh) - 1)) << 2;
        if constexpr (FAST) {
            const int mj = (kmajor ? k0 : r0) + major, mn = (kmajor ? r0 : k0) + minor;
            const bool ok = mj < (kmajor ? K : R) && mn < (kmajor ? R : K);
            // the value is not touched here: zeroing it now would wait for the load before the slab's MFMAs
            f.v[i] = *reinterpret_cast<const float4*>(P + (ok ? (long long)mj * ld + mn : 0ll));
            f.ok[i] = ok ? 15 : 0;
        } else {
            const int row = kmajor ? r0 + minor : r0 + major;
            const int k = kmajor ? k0 + major : k0 + minor;
            const long long base = kmajor ? (long long)k * ld + row : (long long)row * ld + k;
            float e[4];
            unsigned char m = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool ok = kmajor ? (k < K && row + j < R) : (row < R && k + j < K);
                e[j] = P[ok ? base + j : 0ll];
                m |= ok ? (1 << j) : 0;
            }
            f.v[i] = make_float4(e[0], e[1], e[2], e[3]);
            f.ok[i] = m;
        }
    }
    return f;
}

constexpr int SLAB = BK * LDT;  // floats of one operand slab (covers both orientations)
constexpr int PITCH_ROWS = 68;  // [row][k] orientation: 16-byte aligned rows; 16 lanes x 4 words step over all 64 banks

template <int UNITS>
__device__ __forceinline__ void stage(float* dst, const Frag<UNITS>& f, int kmajor, int t)
{
    const int sh = (kmajor && UNITS == 1) ? 3 : 4;
#pragma unroll
    for (int i = 0; i < UNITS; ++i) {
        const int u = t + i * NTHR;
        const int major = u >> sh, minor = (u & ((1 << sh) - 1)) << 2;
        const unsigned char m = f.ok[i];
        const float4 q = make_float4((m & 1) ? f.v[i].x : 0.0f, (m & 2) ? f.v[i].y : 0.0f, (m & 4) ? f.v[i].z : 0.0f,
                                     (m & 8) ? f.v[i].w : 0.0f);
        if (!kmajor) {
            *reinterpret_cast<float4*>(dst + major * PITCH_ROWS + minor) = q;   // row major, k minor .. +3
        } else {
            *reinterpret_cast<float4*>(dst + major * LDT + minor) = q;   // k major, row minor .. +3
        }
    }
}

// one tile (bx, by) of the product g
template <bool FAST, bool AKM, bool BKM, int BM>
__device__ __forceinline__ void gemm_f32_tile(const GemmF32Args& g, const int bx, const int by)
{
    constexpr int UA = BM * BK / 4 / NTHR, UB = BN * BK / 4 / NTHR;  // float4 units per thread and slab
    constexpr int SUBS = (BM / 32) * (BN / 32);  // 32x32 accumulators of the tile
    constexpr int KSPLIT = 8 / SUBS;             // wavefronts sharing one accumulator, each a part of every slab's K
    constexpr int KW = BK / KSPLIT;              // k per wavefront and slab
    extern __shared__ __attribute__((aligned(16))) float lds[];
    float* const As = lds;
    float* const Bs = lds + NST * SLAB;
    // word index of (k, row) in a slab: k * sk + row * sr
    constexpr int ska = AKM ? LDT : 1, sra = AKM ? 1 : PITCH_ROWS;
    constexpr int skb = BKM ? LDT : 1, srb = BKM ? 1 : PITCH_ROWS;
    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int bm = by * BM, bn = bx * BN;
    const int sub = w % SUBS, kpart = w / SUBS;
    const int wm = (sub >> 1) * 32, wn = (sub & 1) * 32, kh = kpart * KW;

    v16f acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
    const bool row_sums = g.epilogue == EPI_SGD && g.bias_w && bx == 0;
    float rs = 0.0f;  // this lane's share of the sum over K of its A row (the bias gradient)

    const int nk = (g.K + BK - 1) / BK;
    // Slab 0 goes straight to LDS; from then on slab kt+1 is staged at the end of iteration kt from
    // registers filled one iteration earlier, so a global load has a whole iteration to arrive
    // (two register sets, alternating: the loop body is written out for even and odd kt).  More sets
    // in flight bring nothing: an iteration is bounded by its LDS traffic and barriers, not by memory.
    Frag<UA> fa0, fa1;
    Frag<UB> fb0, fb1;
    {
        const Frag<UA> a0 = fetch<FAST, UA>(g.A, g.lda, AKM, bm, 0, g.M, g.K, t);
        const Frag<UB> b0 = fetch<FAST, UB>(g.B, g.ldb, BKM, bn, 0, g.N, g.K, t);
        // slab 1 (staged at the end of iteration 0) sets out before slab 0 is waited for
        fa0 = fetch<FAST, UA>(g.A, g.lda, AKM, bm, BK, g.M, g.K, t);      // past K: zeros
        fb0 = fetch<FAST, UB>(g.B, g.ldb, BKM, bn, BK, g.N, g.K, t);
        stage(As, a0, AKM, t);
        stage(Bs, b0, BKM, t);
    }
    __syncthreads();

    const int lr = lane & 31, lk = lane >> 5;
    auto iteration = [&](int kt, Frag<UA>& sa_, Frag<UB>& sb_, Frag<UA>& na_, Frag<UB>& nb_) {
        const int cur = kt % NST, nxt = (kt + 1) % NST;
        // slab kt+2 sets out now, into the register set that was staged one iteration ago
        na_ = fetch<FAST, UA>(g.A, g.lda, AKM, bm, (kt + 2) * BK, g.M, g.K, t);
        nb_ = fetch<FAST, UB>(g.B, g.ldb, BKM, bn, (kt + 2) * BK, g.N, g.K, t);
        // lane half lk supplies k = kh + (KW/2)*lk + i to MFMA i (any pairing works as long as A and B
        // agree): KW/2 consecutive k per lane, which a [row][k] operand delivers as 16-byte reads
        const float* pa = As + cur * SLAB + (kh + (KW / 2) * lk) * ska + (wm + lr) * sra;
        const float* pb = Bs + cur * SLAB + (kh + (KW / 2) * lk) * skb + (wn + lr) * srb;
        float av[KW / 2], bv[KW / 2];  // this wavefront's operand pairs of the slab, requested together
#pragma unroll
        for (int i = 0; i < KW / 2; ++i) { av[i] = pa[i * ska]; bv[i] = pb[i * skb]; }
        __builtin_amdgcn_sched_barrier(0);  // keep the reads together: sunk next to their MFMA each would be waited for alone
#pragma unroll
        for (int i = 0; i < KW / 2; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[i], acc, 0, 0, 0);
        if (row_sums) {
#pragma unroll
            for (int i = 0; i < KW / 2; ++i) rs += av[i];
        }
        // slab kt+1 (requested during iteration kt-1) into the buffer slab kt-1 has left
        stage(As + nxt * SLAB, sa_, AKM, t);
        stage(Bs + nxt * SLAB, sb_, BKM, t);
        // the wavefronts meet over LDS only (__syncthreads() would also drain the global loads just requested)
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };
    for (int kt = 0; kt < nk; kt += 2) {
        iteration(kt, fa0, fb0, fa1, fb1);
        if (kt + 1 < nk) iteration(kt + 1, fa1, fb1, fa0, fb0);
    }

    // the other K parts go to LDS ([wavefront][register][lane]) and are added, in order, by the first
    float* red = lds;
    float* rsum = lds + 8 * 16 * 64;  // behind the accumulators: [wavefront][lane]
    if (row_sums) rsum[w * 64 + lane] = rs;
    if (w >= SUBS) {
#pragma unroll
        for (int i = 0; i < 16; ++i) red[((w - SUBS) * 16 + i) * 64 + lane] = acc[i];
    }
    __syncthreads();
    if (w >= SUBS) return;
#pragma unroll
    for (int part = 1; part < KSPLIT; ++part) {
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] += red[(((part - 1) * SUBS + w) * 16 + i) * 64 + lane];
    }

    // bias: the wavefronts of the tile's first column of accumulators add the shares of a row (both lane
    // halves of every K part, in order) and apply the update
    if (row_sums && wn == 0 && lk == 0) {
        const int row = bm + wm + lr;
        if (row < g.M) {
            float sum = 0.0f;
#pragma unroll
            for (int part = 0; part < KSPLIT; ++part) {
                const float* q = rsum + (part * SUBS + sub) * 64 + lr;
                sum += q[0] + q[32];
            }
            const float d = g.lr * (sum * g.alpha) + g.mom * g.bias_v[row];
            g.bias_v[row] = d;
            g.bias_w[row] = g.bias_w[row] - d;
        }
    }

    // accumulator layout of the 32x32 tile: lane -> column lane%32; register i -> row
    // 8*(i/4) + 4*(lane/32) + i%4
    const int col = bn + wn + lr;
    if (col < g.N) {
        const float bias = (g.epilogue == EPI_BIAS_ACT && g.bias) ? g.bias[col] : 0.0f;
        // what the epilogue reads (activations for the derivative; weights and momentum for the update) is asked for in
        // one go, ahead of the first store: element by element, every load would wait out a round trip of its own
        float in0[16], in1[16];
        if (g.epilogue == EPI_SGD || g.epilogue == EPI_MUL_DER) {
            const float* s0 = g.epilogue == EPI_SGD ? g.C : g.aux;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int row = bm + wm + 8 * (i >> 2) + 4 * lk + (i & 3);
                in0[i] = row < g.M ? s0[(long long)row * g.ldc + col] : 0.0f;
            }
            if (g.epilogue == EPI_SGD)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int row = bm + wm + 8 * (i >> 2) + 4 * lk + (i & 3);
                    in1[i] = row < g.M ? g.V[(long long)row * g.ldc + col] : 0.0f;
                }
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int row = bm + wm + 8 * (i >> 2) + 4 * lk + (i & 3);
            if (row < g.M) {
                float v = acc[i];
                const long long idx = (long long)row * g.ldc + col;
                if (g.epilogue == EPI_BIAS_ACT) v = ghip_squash<false>(v + bias, g.act, g.act_param);
                else if (g.epilogue == EPI_MUL_DER) v = v * ghip_act_der_canon(in0[i], g.act, g.act_param);
                else if (g.epilogue == EPI_SGD) {
                    const float wgt = in0[i];
                    const float sg = (wgt > 0.0f) ? 1.0f : ((wgt < 0.0f) ? -1.0f : 0.0f);
                    const float grad = v * g.alpha + g.wd1 * sg + g.wd2 * wgt;
                    const float d = g.lr * grad + g.mom * in1[i];
                    g.V[idx] = d;
                    v = wgt - d;
                } else v = v * g.alpha;
                g.C[idx] = v;
            }
        }
    }
}

template <bool FAST, bool AKM, bool BKM, int BM>
__global__ void __launch_bounds__(NTHR) gemm_f32_kernel(GemmF32Args g)
{
    gemm_f32_tile<FAST, AKM, BKM, BM>(g, blockIdx.x, blockIdx.y);
}

// Several independent products of one kind in one launch (the weight gradients of a step): a workgroup finds
// its product by its index in the grid.  Products of this size are mostly a launch's fixed part, which is paid
// once here, and together their tiles fill the compute units that one of them alone leaves idle.
template <bool FAST, bool AKM, bool BKM, int BM>
__global__ void __launch_bounds__(NTHR) gemm_f32_group_kernel(GemmF32Group grp)
{
    int k = 0;
    while (k + 1 < grp.count && (int)blockIdx.x >= grp.first[k + 1]) ++k;
    const GemmF32Args g = grp.p[k];
    const int local = (int)blockIdx.x - grp.first[k];
    gemm_f32_tile<FAST, AKM, BKM, BM>(g, local % grp.gx[k], local / grp.gx[k]);
}

struct Variant { int bm; bool fast, akm, bkm; dim3 grid; };
Variant variant_of(const GemmF32Args& a)
{
    Variant v;
    // 64 x 64 tiles unless they would leave compute units without a workgroup
    const long long tiles64 = (long long)((a.N + BN - 1) / BN) * ((a.M + 63) / 64);
    v.bm = (tiles64 <= 128 && a.M > 32) ? 32 : 64;  // (up to 256: the grouped weight gradients 47 us instead of 37)
    // (32 x 32 tiles, 512 for cfg3's forward products so that two share a unit there too: 47 us for the two instead of 44)
    v.grid = dim3((a.N + BN - 1) / BN, (a.M + v.bm - 1) / v.bm);
    const bool a_fast = (a.lda % 4) == 0 && ((uintptr_t)a.A % 16) == 0 && ((a.a_kmajor ? a.M : a.K) % 4) == 0;
    const bool b_fast = (a.ldb % 4) == 0 && ((uintptr_t)a.B % 16) == 0 && ((a.b_kmajor ? a.N : a.K) % 4) == 0;
    v.fast = a_fast && b_fast;
    v.akm = a.a_kmajor != 0;
    v.bkm = a.b_kmajor != 0;
    return v;
}
constexpr size_t kLdsBytes = sizeof(float) * 2 * NST * SLAB;  // 69 632 B: above the 64 KiB default, two per compute unit

}  // namespace

hipError_t ghip_gemm_f32_group(const GemmF32Args* a, int count, hipStream_t s)
{
    if (count < 1 || count > GHIP_GEMM_F32_GROUP_MAX) return hipErrorInvalidValue;
    bool alike = count > 1;
    const Variant v0 = variant_of(a[0]);
    for (int k = 0; k < count; ++k) {
        if (a[k].M <= 0 || a[k].N <= 0 || a[k].K <= 0) return hipErrorInvalidValue;
        const Variant v = variant_of(a[k]);
        alike = alike && v.bm == v0.bm && v.fast == v0.fast && v.akm == v0.akm && v.bkm == v0.bkm;
    }
    if (!alike) {  // one launch each
        for (int k = 0; k < count; ++k) {
            hipError_t e = ghip_gemm_f32(a[k], s);
            if (e != hipSuccess) return e;
        }
        return hipSuccess;
    }
    GemmF32Group grp;
    memset(&grp, 0, sizeof(grp));
    grp.count = count;
    int blocks = 0;
    for (int k = 0; k < count; ++k) {
        const Variant v = variant_of(a[k]);
        grp.p[k] = a[k];
        grp.first[k] = blocks;
        grp.gx[k] = (int)v.grid.x;
        blocks += (int)(v.grid.x * v.grid.y);
    }
    grp.first[count] = blocks;
    typedef void (*kernel_t)(GemmF32Group);
#define GF32_ROW(F, BMV)                                                                                   \
    {{gemm_f32_group_kernel<F, false, false, BMV>, gemm_f32_group_kernel<F, false, true, BMV>},            \
     {gemm_f32_group_kernel<F, true, false, BMV>, gemm_f32_group_kernel<F, true, true, BMV>}}
    static const kernel_t table[2][2][2][2] = {{GF32_ROW(false, 64), GF32_ROW(true, 64)}, {GF32_ROW(false, 32), GF32_ROW(true, 32)}};
#undef GF32_ROW
    // once per process, whichever thread comes first (handles on several host threads launch side by side)
    static std::once_flag once;
    static hipError_t raised = hipSuccess;
    std::call_once(once, [] {
        for (int i = 0; i < 16 && raised == hipSuccess; ++i)
            raised = hipFuncSetAttribute((const void*)table[i >> 3][(i >> 2) & 1][(i >> 1) & 1][i & 1],
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
    });
    if (raised != hipSuccess) return raised;
    hipLaunchKernelGGL(table[v0.bm == 32][v0.fast][v0.akm ? 1 : 0][v0.bkm ? 1 : 0], dim3(blocks), dim3(NTHR), kLdsBytes, s, grp);
    return hipGetLastError();
}

hipError_t ghip_gemm_f32(const GemmF32Args& a, hipStream_t s)
{
    if (a.M <= 0 || a.N <= 0 || a.K <= 0) return hipErrorInvalidValue;
    const Variant v = variant_of(a);
    typedef void (*kernel_t)(GemmF32Args);
#define GF32_ROW(F, BMV)                                                                       \
    {{gemm_f32_kernel<F, false, false, BMV>, gemm_f32_kernel<F, false, true, BMV>},            \
     {gemm_f32_kernel<F, true, false, BMV>, gemm_f32_kernel<F, true, true, BMV>}}
    static const kernel_t table[2][2][2][2] = {{GF32_ROW(false, 64), GF32_ROW(true, 64)}, {GF32_ROW(false, 32), GF32_ROW(true, 32)}};
#undef GF32_ROW
    // once per process, whichever thread comes first (handles on several host threads launch side by side)
    static std::once_flag once;
    static hipError_t raised = hipSuccess;
    std::call_once(once, [] {
        for (int i = 0; i < 16 && raised == hipSuccess; ++i)
            raised = hipFuncSetAttribute((const void*)table[i >> 3][(i >> 2) & 1][(i >> 1) & 1][i & 1],
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
    });
    if (raised != hipSuccess) return raised;
    hipLaunchKernelGGL(table[v.bm == 32][v.fast][v.akm ? 1 : 0][v.bkm ? 1 : 0], v.grid, dim3(NTHR), kLdsBytes, s, a);
    return hipGetLastError();
}

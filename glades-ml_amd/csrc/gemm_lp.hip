// Low-precision GEMM for the wide canonical layers: C[M][N] = A[M][K] * B[N][K]^T with both
// operands K-contiguous, bf16 (v_mfma_f32_32x32x16_bf16) or e4m3 (v_mfma_scale_f32_32x32x64_f8f6f4
// with unit block scales), fp32 accumulation, fused epilogues.
//
// The three products of a training step are all brought to this one operand form by keeping
// transposed copies that the producing epilogues write for free (the GEMMs are compute bound
// by a factor of ~5 in HBM terms):
//   forward   H_{l+1} = squash(H_l W^T + b)   A = H_l [B][n_in],      B = W [n_out][n_in]
//   back-prop D_l = (D_{l+1} W) .* f'(H_l)    A = D_{l+1} [B][n_out], B = W^T [n_in][n_out]
//   gradient  G = D_{l+1}^T H_l               A = D^T [n_out][B],     B = H_l^T [n_in][B]
//             fused with the SGD + momentum + L1/L2 update of the fp32 master weights, which
//             also writes the bf16 W and W^T used by the next step.
//
// Tile: 256 x 256 x 128 bytes of K (64 bf16 / 128 e4m3) per workgroup of 8 wavefronts laid out
// 2 (M) x 4 (N); each wavefront owns 128 x 64 = 4 x 2 accumulators of 32x32 (128 VGPRs).
// LDS: two buffers of (256 + 256) rows x 128 B = 128 KiB.  Rows are 128 B, 16-byte chunks are
// XOR-swizzled with the row index so that both the row-wise stores and the per-lane 16-byte
// operand reads (32 consecutive rows, same logical chunk) spread over all banks.
// Workgroup ids are remapped so that each XCD (ids congruent mod 8 share an L2) walks a compact
// block of tiles.

#include "ghip_internal.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int TM = 256, TN = 256, TKB = 128, NT = 512;
constexpr int TILE_BYTES = 256 * TKB;  // one operand tile

__device__ __forceinline__ int swz(int row, int chunk) { return (row << 7) + (((chunk ^ row) & 7) << 4); }

__device__ __forceinline__ float lp_squash(float z, int act, float p) { return ghip_squash<false>(z, act, p); }

template <bool FP8, int EPI>
__global__ void __launch_bounds__(NT) gemm_lp_kernel(GemmLpArgs g)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    unsigned char* sA = lds;                    // [2][TILE_BYTES]
    unsigned char* sB = lds + 2 * TILE_BYTES;   // [2][TILE_BYTES]

    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int l31 = lane & 31, lh = lane >> 5;

    // ---- XCD-aware tile order: ids with equal (id % 8) run on one XCD; give each XCD a
    //      contiguous range of tile numbers, and walk tiles in column groups of 8 rows
    const int tiles_m = g.M / TM, tiles_n = g.N / TN;
    const int nb = tiles_m * tiles_n;
    int id = blockIdx.x;
    if ((nb & 7) == 0) id = (id & 7) * (nb >> 3) + (id >> 3);
    constexpr int GROUP = 8;
    const int per_group = GROUP * tiles_n;
    const int gidx = id / per_group;
    const int first_m = gidx * GROUP;
    const int gsize = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
    const int tm = first_m + (id % per_group) % gsize;
    const int tn = (id % per_group) / gsize;
    const int bm = tm * TM, bn = tn * TN;

    const long long ldk = FP8 ? (long long)g.K : (long long)g.K * 2;  // row pitch in bytes
    const unsigned char* gA = (const unsigned char*)g.A + (long long)bm * ldk;
    const unsigned char* gB = (const unsigned char*)g.B + (long long)bn * ldk;

    const int wm = (w >> 2) * 128, wn = (w & 3) * 64;

    v16f acc[4][2];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mi][ni][i] = 0.0f;

    v4i ra[4], rb[4];
    int lrow[4], lch[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int c = t + j * NT;
        lrow[j] = c >> 3;
        lch[j] = c & 7;
    }
    auto gload = [&](int kt) {
        const long long kb = (long long)kt * TKB;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            ra[j] = *reinterpret_cast<const v4i*>(gA + (long long)lrow[j] * ldk + kb + (lch[j] << 4));
            rb[j] = *reinterpret_cast<const v4i*>(gB + (long long)lrow[j] * ldk + kb + (lch[j] << 4));
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<v4i*>(sA + buf * TILE_BYTES + swz(lrow[j], lch[j])) = ra[j];
            *reinterpret_cast<v4i*>(sB + buf * TILE_BYTES + swz(lrow[j], lch[j])) = rb[j];
        }
    };

    const int nk = (int)(ldk / TKB);
    gload(0);
    lstore(0);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) gload(kt + 1);
        const unsigned char* a_base = sA + cur * TILE_BYTES;
        const unsigned char* b_base = sB + cur * TILE_BYTES;
        if (!FP8) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                v4i af[4], bf[2];
#pragma unroll
                for (int mi = 0; mi < 4; ++mi)
                    af[mi] = *reinterpret_cast<const v4i*>(a_base + swz(wm + mi * 32 + l31, ks * 2 + lh));
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    bf[ni] = *reinterpret_cast<const v4i*>(b_base + swz(wn + ni * 32 + l31, ks * 2 + lh));
#pragma unroll
                for (int mi = 0; mi < 4; ++mi)
#pragma unroll
                    for (int ni = 0; ni < 2; ++ni)
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(bf16x8, af[mi]), __builtin_bit_cast(bf16x8, bf[ni]), acc[mi][ni], 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                v8i af[4], bf[2];
#pragma unroll
                for (int mi = 0; mi < 4; ++mi) {
                    const int row = wm + mi * 32 + l31;
                    v4i lo = *reinterpret_cast<const v4i*>(a_base + swz(row, ks * 4 + lh * 2));
                    v4i hi = *reinterpret_cast<const v4i*>(a_base + swz(row, ks * 4 + lh * 2 + 1));
                    af[mi] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                }
#pragma unroll
                for (int ni = 0; ni < 2; ++ni) {
                    const int row = wn + ni * 32 + l31;
                    v4i lo = *reinterpret_cast<const v4i*>(b_base + swz(row, ks * 4 + lh * 2));
                    v4i hi = *reinterpret_cast<const v4i*>(b_base + swz(row, ks * 4 + lh * 2 + 1));
                    bf[ni] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                }
#pragma unroll
                for (int mi = 0; mi < 4; ++mi)
#pragma unroll
                    for (int ni = 0; ni < 2; ++ni)
                        acc[mi][ni] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                            af[mi], bf[ni], acc[mi][ni], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
            }
        }
        if (kt + 1 < nk) lstore(cur ^ 1);
        __syncthreads();
    }

    // ---- epilogue.  Accumulator layout of a 32x32 tile: lane -> column lane%32,
    //      register i -> row 8*(i/4) + 4*(lane/32) + i%4  (4 consecutive rows per register quad)
    const int M = g.M, N = g.N;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const int col = bn + wn + ni * 32 + l31;
            float cbias = 0.0f, cscale = 1.0f;
            if (EPI == LP_FWD_ACT || EPI == LP_FWD_F32) cbias = g.bias ? g.bias[col] : 0.0f;
            if (EPI == LP_FP8_ACT || EPI == LP_FP8_F32) cscale = g.col_scale[col];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int row0 = bm + wm + mi * 32 + 8 * q + 4 * lh;
                uint16_t hb[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int row = row0 + r;
                    const long long idx = (long long)row * N + col;
                    float v = acc[mi][ni][q * 4 + r];
                    if (EPI == LP_FWD_ACT) {
                        v = lp_squash(v + cbias, g.act, g.act_param);
                        hb[r] = ghip_f32_to_bf16(v);
                        ((uint16_t*)g.out)[idx] = hb[r];
                    } else if (EPI == LP_FWD_F32) {
                        ((float*)g.out)[idx] = lp_squash(v + cbias, g.act, g.act_param);
                    } else if (EPI == LP_DGRAD) {
                        v = v * ghip_act_der_canon(ghip_bf16_to_f32(g.aux[idx]), g.act, g.act_param);
                        hb[r] = ghip_f32_to_bf16(v);
                        ((uint16_t*)g.out)[idx] = hb[r];
                    } else if (EPI == LP_WGRAD_SGD) {
                        const float wv = g.master[idx];
                        const float sg = (wv > 0.0f) ? 1.0f : ((wv < 0.0f) ? -1.0f : 0.0f);
                        const float gr = v * g.gscale + g.wd1 * sg + g.wd2 * wv;
                        const float d = g.lr * gr + g.momf * g.mom[idx];
                        g.mom[idx] = d;
                        const float nw = wv - d;
                        g.master[idx] = nw;
                        hb[r] = ghip_f32_to_bf16(nw);
                        ((uint16_t*)g.out)[idx] = hb[r];
                    } else if (EPI == LP_FP8_ACT) {
                        v = lp_squash(__fmul_rn(v, __fmul_rn(g.row_scale[row], cscale)), g.act, g.act_param);
                        hb[r] = ghip_f32_to_bf16(v);
                        ((uint16_t*)g.out)[idx] = hb[r];
                        // row amax of the stored (bf16-rounded) values over this wavefront's 32 columns
                        float am = fabsf(ghip_bf16_to_f32(hb[r]));
#pragma unroll
                        for (int o = 16; o > 0; o >>= 1) am = fmaxf(am, __shfl_xor(am, o, 64));
                        if (l31 == 0) atomicMax(&g.row_amax_bits[row], __float_as_uint(am));
                    } else {  // LP_FP8_F32
                        v = lp_squash(__fmul_rn(v, __fmul_rn(g.row_scale[row], cscale)), g.act, g.act_param);
                        ((float*)g.out)[idx] = v;
                    }
                }
                if ((EPI == LP_FWD_ACT || EPI == LP_DGRAD || EPI == LP_WGRAD_SGD) && g.outT) {
                    uint2 pk;
                    pk.x = (uint32_t)hb[0] | ((uint32_t)hb[1] << 16);
                    pk.y = (uint32_t)hb[2] | ((uint32_t)hb[3] << 16);
                    *reinterpret_cast<uint2*>((uint16_t*)g.outT + (long long)col * M + row0) = pk;
                }
            }
        }
    }
}

template <bool FP8, int EPI>
hipError_t launch(const GemmLpArgs& a, hipStream_t s)
{
    const size_t lds = 4 * TILE_BYTES;
    static bool attr_done = false;
    if (!attr_done) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_lp_kernel<FP8, EPI>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_done = true;
    }
    const int nb = (a.M / TM) * (a.N / TN);
    hipLaunchKernelGGL((gemm_lp_kernel<FP8, EPI>), dim3(nb), dim3(NT), lds, s, a);
    return hipGetLastError();
}

}  // namespace

bool ghip_gemm_lp_shape_ok(int M, int N, int K, int fp8)
{
    const int kq = fp8 ? 128 : 64;
    return M > 0 && N > 0 && K > 0 && (M % TM) == 0 && (N % TN) == 0 && (K % kq) == 0;
}

hipError_t ghip_gemm_lp(const GemmLpArgs& a, hipStream_t s)
{
    if (!ghip_gemm_lp_shape_ok(a.M, a.N, a.K, a.fp8)) return hipErrorInvalidValue;
    if (!a.fp8) {
        switch (a.epilogue) {
        case LP_FWD_ACT: return launch<false, LP_FWD_ACT>(a, s);
        case LP_FWD_F32: return launch<false, LP_FWD_F32>(a, s);
        case LP_DGRAD: return launch<false, LP_DGRAD>(a, s);
        case LP_WGRAD_SGD: return launch<false, LP_WGRAD_SGD>(a, s);
        }
    } else {
        switch (a.epilogue) {
        case LP_FP8_ACT: return launch<true, LP_FP8_ACT>(a, s);
        case LP_FP8_F32: return launch<true, LP_FP8_F32>(a, s);
        }
    }
    return hipErrorInvalidValue;
}

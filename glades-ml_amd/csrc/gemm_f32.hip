// fp32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32) for the canonical fp32 path:
// arbitrary M, N, K (bounds-checked, zero-filled tiles), either operand stored K-major or not,
// fused epilogues (bias + activation, activation-derivative product, plain scale).
//
// It realises the reference's three loop nests as matrix products over a whole batch:
//   forward   a_{l+1} = squash(W a_l + b)        network.cpp:466-516  -> C = A * W^T
//   back-prop e = W^T d                          network.cpp:660-662  -> C = D * W
//   gradient  dW = d (x) a, summed over the batch  node.cpp:278-292   -> C = D^T * A
//
// Tile: 64 x 64 x 16 per workgroup of 4 wavefronts, each wavefront owns one 32x32 accumulator
// (16 VGPRs).  Operands are staged through LDS K-major ([k][row]) so that the per-lane operand
// fetch of the 32x32x2 instruction (lane -> row = lane%32, k = lane/32) reads 32 consecutive
// words: conflict free.  Two LDS buffers: the next K-slab is fetched from global memory into
// registers while the current one feeds the matrix cores.

#include "ghip_internal.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BM = 64, BN = 64, BK = 16, LDT = 64 + 4;

struct Frag { float v[4]; };

// Fetch this lane's 4 elements of a 64(row) x 16(k) operand tile.
//   kmajor == 0: P is [rows][K]  (ld = row stride): lane -> row = t/4, k = (t%4)*4 .. +3
//   kmajor == 1: P is [K][rows]  (ld = k stride):   lane -> k = t/16, row = (t%16)*4 .. +3
__device__ __forceinline__ Frag fetch(const float* __restrict__ P, int ld, int kmajor, int vec_ok,
                                      int r0, int k0, int R, int K, int t)
{
    Frag f;
    if (!kmajor) {
        const int row = r0 + (t >> 2), k = k0 + ((t & 3) << 2);
        const float* src = P + (long long)row * ld + k;
        if (row < R && k + 3 < K && vec_ok) {
            float4 q = *reinterpret_cast<const float4*>(src);
            f.v[0] = q.x; f.v[1] = q.y; f.v[2] = q.z; f.v[3] = q.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) f.v[j] = (row < R && k + j < K) ? src[j] : 0.0f;
        }
    } else {
        const int k = k0 + (t >> 4), row = r0 + ((t & 15) << 2);
        const float* src = P + (long long)k * ld + row;
        if (k < K && row + 3 < R && vec_ok) {
            float4 q = *reinterpret_cast<const float4*>(src);
            f.v[0] = q.x; f.v[1] = q.y; f.v[2] = q.z; f.v[3] = q.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) f.v[j] = (k < K && row + j < R) ? src[j] : 0.0f;
        }
    }
    return f;
}

__device__ __forceinline__ void stage(float (*dst)[LDT], const Frag& f, int kmajor, int t)
{
    if (!kmajor) {
        const int row = t >> 2, k = (t & 3) << 2;
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[k + j][row] = f.v[j];
    } else {
        const int k = t >> 4, row = (t & 15) << 2;
        *reinterpret_cast<float4*>(&dst[k][row]) = make_float4(f.v[0], f.v[1], f.v[2], f.v[3]);
    }
}

__global__ void __launch_bounds__(256) gemm_f32_kernel(GemmF32Args g)
{
    __shared__ __attribute__((aligned(16))) float As[2][BK][LDT];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK][LDT];
    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int bm = blockIdx.y * BM, bn = blockIdx.x * BN;
    const int wm = (w >> 1) * 32, wn = (w & 1) * 32;
    const int a_vec = ((g.lda & 3) == 0) && ((((uintptr_t)g.A) & 15) == 0);
    const int b_vec = ((g.ldb & 3) == 0) && ((((uintptr_t)g.B) & 15) == 0);

    v16f acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    Frag fa = fetch(g.A, g.lda, g.a_kmajor, a_vec, bm, 0, g.M, g.K, t);
    Frag fb = fetch(g.B, g.ldb, g.b_kmajor, b_vec, bn, 0, g.N, g.K, t);
    stage(As[0], fa, g.a_kmajor, t);
    stage(Bs[0], fb, g.b_kmajor, t);
    __syncthreads();

    const int nk = (g.K + BK - 1) / BK;
    const int lr = lane & 31, lk = lane >> 5;
    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) {
            fa = fetch(g.A, g.lda, g.a_kmajor, a_vec, bm, (kt + 1) * BK, g.M, g.K, t);
            fb = fetch(g.B, g.ldb, g.b_kmajor, b_vec, bn, (kt + 1) * BK, g.N, g.K, t);
        }
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            const float a = As[cur][kk + lk][wm + lr];
            const float b = Bs[cur][kk + lk][wn + lr];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
        }
        if (kt + 1 < nk) {
            stage(As[cur ^ 1], fa, g.a_kmajor, t);
            stage(Bs[cur ^ 1], fb, g.b_kmajor, t);
        }
        __syncthreads();
    }

    // accumulator layout of the 32x32 tile: lane -> column lane%32; register i -> row
    // 8*(i/4) + 4*(lane/32) + i%4
    const int col = bn + wn + lr;
    if (col < g.N) {
        const float bias = (g.epilogue == EPI_BIAS_ACT && g.bias) ? g.bias[col] : 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int row = bm + wm + 8 * (i >> 2) + 4 * lk + (i & 3);
            if (row < g.M) {
                float v = acc[i];
                const long long idx = (long long)row * g.ldc + col;
                if (g.epilogue == EPI_BIAS_ACT) v = ghip_squash<false>(v + bias, g.act, g.act_param);
                else if (g.epilogue == EPI_MUL_DER) v = v * ghip_act_der_canon(g.aux[idx], g.act, g.act_param);
                else v = v * g.alpha;
                g.C[idx] = v;
            }
        }
    }
}

}  // namespace

hipError_t ghip_gemm_f32(const GemmF32Args& a, hipStream_t s)
{
    if (a.M <= 0 || a.N <= 0 || a.K <= 0) return hipErrorInvalidValue;
    dim3 grid((a.N + BN - 1) / BN, (a.M + BM - 1) / BM);
    hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, s, a);
    return hipGetLastError();
}

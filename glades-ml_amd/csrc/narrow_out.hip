// The fp32 output layer when it is a few units wide (a classifier's 10 classes, a regressor's one
// value: NNInfo's OutputLayerInfo, outputlayerinfo.cpp:29).  Its three products are 1 % of a training
// step's arithmetic but, as 64-wide GEMM tiles that are 5/6 padding, a third of its time; here they
// are what they are: streams over the activations entering the layer, bound by memory latency.
//
//   forward   P[b][o] = squash(H[b][:] . W[o][:] + bias[o])
//   delta     D[b][:] = dLoss/dz of row b, with the loss and the metrics
//   backward  E[b][c] = (sum_o D[b][o] W[o][c]) * f'(H[b][c])
//             G_part[chunk][o][c] = sum_{b in chunk} D[b][o] H[b][c]
//   update    G = sum_chunk G_part (fixed order) -> the same fused SGD + momentum + L1/L2 step as
//             the GEMM's EPI_SGD epilogue, and the bias step from the column means of D
//
// A training step is two launches (forward + delta + backward per chunk of rows, then the update);
// inference uses the forward kernel alone.  The partial sums per chunk keep the reduction over the
// batch in a fixed order.

#include "ghip_internal.h"
#include "delta_row.h"

namespace {

constexpr int kMaxOut = 16;

// Sum of v[j] over the 64 lanes for every j < NP (NP a power of two <= 16), halving the number of
// live values at each of the first log2(NP) exchange steps.  Afterwards v[0] of lane L holds the
// total of output narrow_owner<NP>(L); lanes that differ only in their lowest bits hold copies.
template <int NP>
__device__ __forceinline__ void narrow_reduce(float (&v)[NP], int lane)
{
    int n = NP;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        if (n > 1) {
            const bool up = (lane & o) != 0;
#pragma unroll
            for (int i = 0; i < NP / 2; ++i) {
                if (i < n / 2) {
                    // the empty asm makes the two elements plain values: a select between two array
                    // elements is otherwise turned into one load at a lane-dependent index, which
                    // moves the whole array out of registers into scratch memory
                    float lo = v[i], hi = v[i + n / 2];
                    asm("" : "+v"(lo), "+v"(hi));
                    const float keep = up ? hi : lo;
                    const float send = up ? lo : hi;
                    v[i] = keep + __shfl_xor(send, o, 64);
                }
            }
            n >>= 1;
        } else {
            v[0] += __shfl_xor(v[0], o, 64);
        }
    }
}
template <int NP>
__device__ __forceinline__ int narrow_owner(int lane)
{
    int j = 0, n = NP;
#pragma unroll
    for (int o = 32; o > 0 && n > 1; o >>= 1) {
        n >>= 1;
        if (lane & o) j += n;
    }
    return j;
}
template <int NP> struct Log2 { static constexpr int value = 1 + Log2<NP / 2>::value; };
template <> struct Log2<1> { static constexpr int value = 0; };

// Inference: 4 rows per workgroup; wavefront w forms their dot products over the column slices w,
// w + 4, ... (256 columns each, so a weight is loaded once for the 4 rows and the row's loads are
// all in flight at once), the slices meet in LDS and wavefront w finishes row w.
template <int NP>
__global__ void __launch_bounds__(256) narrow_forward_kernel(NarrowOutArgs g)
{
    __shared__ float zpart[4][4][NP];
    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int n4 = g.ni >> 2;
    const int q0 = blockIdx.x * 4;
    const float4* const w4 = reinterpret_cast<const float4*>(g.W);
    const float4* const h4 = reinterpret_cast<const float4*>(g.H);
    float acc[4][NP];
#pragma unroll
    for (int rr = 0; rr < 4; ++rr)
#pragma unroll
        for (int j = 0; j < NP; ++j) acc[rr][j] = 0.0f;
    // rows past the batch repeat its last row, outputs past the last one repeat it: never stored
    for (int k = w * 64 + lane; k < n4; k += 256) {
        float4 h[4], wv[NP];
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) h[rr] = h4[(long long)(q0 + rr < g.B ? q0 + rr : g.B - 1) * n4 + k];
#pragma unroll
        for (int j = 0; j < NP; ++j) wv[j] = w4[(j < g.no ? j : g.no - 1) * n4 + k];
#pragma unroll
        for (int rr = 0; rr < 4; ++rr)
#pragma unroll
            for (int j = 0; j < NP; ++j)
                acc[rr][j] += (h[rr].x * wv[j].x + h[rr].y * wv[j].y) + (h[rr].z * wv[j].z + h[rr].w * wv[j].w);
    }
    constexpr int COPIES = 64 >> Log2<NP>::value;  // lanes holding one output's total
    const int own = narrow_owner<NP>(lane);
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
        narrow_reduce<NP>(acc[rr], lane);
        if ((lane & (COPIES - 1)) == 0) zpart[w][rr][own] = acc[rr][0];
    }
    __syncthreads();
    const int b = q0 + w;
    if (b < g.B && lane < g.no) {
        const float z = ((zpart[0][w][lane] + zpart[1][w][lane]) + (zpart[2][w][lane] + zpart[3][w][lane])) +
                        (g.bias ? g.bias[lane] : 0.0f);
        g.P[(long long)b * g.no + lane] = ghip_squash<false>(z, g.act, g.act_param);
    }
}

// Training step of the layer in one launch: a workgroup of 4 wavefronts takes a chunk of rows, 4 at
// a time.  Forward: wavefront w forms the dot products of the 4 rows over the column slices w, w+4,
// ... (256 columns each; a weight is loaded once for the 4 rows) and the slices meet in LDS.
// Output: wavefront w finishes row w (bias, activation, then loss / delta / metrics exactly as the
// output-delta kernel does) and leaves its deltas in LDS.  Backward: wavefront w walks its column
// slices again for the deltas of the layer below and the chunk's partial gradient (the
// activations and weights it asks for again are in this compute unit's cache).
template <int NP, bool kBelow>
__global__ void __launch_bounds__(256) narrow_train_kernel(NarrowOutArgs g, DeltaArgs da)
{
    __shared__ float zpart[4][4][NP];   // [slice owner][row of the group][output]
    __shared__ float dl[4][NP];         // [row of the group][output]
    __shared__ double red[4][3];
    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int n4 = g.ni >> 2;
    const int chunk = blockIdx.x;
    const int r0 = chunk * g.rows_per_chunk;
    const int r1 = (r0 + g.rows_per_chunk < g.B) ? r0 + g.rows_per_chunk : g.B;
    if (chunk == 0 && t < 4 && da.acc_clear) da.acc_clear[t] = 0.0;
    double loss = 0.0, accs = 0.0, corr = 0.0;
    // rows of W past the last output repeat it, rows of H past the chunk repeat its last row: their
    // sums are never used (zero deltas), and no load sits under a branch of its own
    // (addresses are formed where they are used: arrays of row pointers end up in scratch memory)
    const float4* const w4 = reinterpret_cast<const float4*>(g.W);
    const float4* const h4 = reinterpret_cast<const float4*>(g.H);
    auto wrow = [&](int j) { return (j < g.no ? j : g.no - 1) * n4; };
    constexpr int COPIES = 64 >> Log2<NP>::value;
    const int own = narrow_owner<NP>(lane);
    bool first = true;
    for (int q0 = r0; q0 < r1; q0 += 4, first = false) {
        auto hrow = [&](int rr) { return (long long)(q0 + rr < r1 ? q0 + rr : r1 - 1) * n4; };
        // this wavefront's row of targets travels while the dot products are formed
        const float yv = (q0 + w < r1) ? ghip_delta_target(da, q0 + w, lane) : 0.0f;
        // ---- forward
        float acc[4][NP];
#pragma unroll
        for (int rr = 0; rr < 4; ++rr)
#pragma unroll
            for (int j = 0; j < NP; ++j) acc[rr][j] = 0.0f;
        for (int k = w * 64 + lane; k < n4; k += 256) {
            float4 h[4], wv[NP];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) h[rr] = h4[hrow(rr) + k];
#pragma unroll
            for (int j = 0; j < NP; ++j) wv[j] = w4[wrow(j) + k];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr)
#pragma unroll
                for (int j = 0; j < NP; ++j)
                    acc[rr][j] += (h[rr].x * wv[j].x + h[rr].y * wv[j].y) + (h[rr].z * wv[j].z + h[rr].w * wv[j].w);
        }
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            narrow_reduce<NP>(acc[rr], lane);
            if ((lane & (COPIES - 1)) == 0) zpart[w][rr][own] = acc[rr][0];
        }
        __syncthreads();
        // ---- output, loss, delta: wavefront w has row q0 + w
        {
            const int b = q0 + w;
            float d = 0.0f;
            if (b < r1) {
                float v = -3.0e38f;
                if (lane < g.no) {
                    const float z = ((zpart[0][w][lane] + zpart[1][w][lane]) + (zpart[2][w][lane] + zpart[3][w][lane])) +
                                    (g.bias ? g.bias[lane] : 0.0f);
                    v = ghip_squash<false>(z, g.act, g.act_param);
                    g.P[(long long)b * g.no + lane] = v;
                }
                d = ghip_delta_row64(da, b, lane, v, yv, loss, accs, corr);
            }
            if (lane < NP) dl[w][lane] = (lane < g.no) ? d : 0.0f;
        }
        __syncthreads();
        // ---- backward
        for (int k = w * 64 + lane; k < n4; k += 256) {
            float4 h[4], wv[NP];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) h[rr] = h4[hrow(rr) + k];
            if (kBelow) {
#pragma unroll
                for (int j = 0; j < NP; ++j) wv[j] = w4[wrow(j) + k];
            }
            float4 pa[NP];
            if (!first) {
#pragma unroll
                for (int j = 0; j < NP; ++j)
                    pa[j] = reinterpret_cast<const float4*>(g.part + ((long long)chunk * g.no + (j < g.no ? j : g.no - 1)) * g.ni)[k];
            } else {
#pragma unroll
                for (int j = 0; j < NP; ++j) pa[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                float4 e = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int j = 0; j < NP; ++j) {
                    const float dj = dl[rr][j];
                    if (kBelow) { e.x += dj * wv[j].x; e.y += dj * wv[j].y; e.z += dj * wv[j].z; e.w += dj * wv[j].w; }
                    pa[j].x += dj * h[rr].x; pa[j].y += dj * h[rr].y; pa[j].z += dj * h[rr].z; pa[j].w += dj * h[rr].w;
                }
                if (kBelow && q0 + rr < r1) {
                    e.x *= ghip_act_der_canon(h[rr].x, g.act_below, g.act_below_param);
                    e.y *= ghip_act_der_canon(h[rr].y, g.act_below, g.act_below_param);
                    e.z *= ghip_act_der_canon(h[rr].z, g.act_below, g.act_below_param);
                    e.w *= ghip_act_der_canon(h[rr].w, g.act_below, g.act_below_param);
                    reinterpret_cast<float4*>(g.E + (long long)(q0 + rr) * g.ni)[k] = e;
                }
            }
#pragma unroll
            for (int j = 0; j < NP; ++j)
                if (j < g.no) reinterpret_cast<float4*>(g.part + ((long long)chunk * g.no + j) * g.ni)[k] = pa[j];
        }
        __syncthreads();  // the next group overwrites zpart and dl
    }
    // the chunk's three sums go to its own slot: the update kernel adds the slots up in order (every
    // workgroup adding to the same three doubles atomically takes longer than the rows themselves)
    if (lane == 0) { red[w][0] = loss; red[w][1] = accs; red[w][2] = corr; }
    __syncthreads();
    if (t < 3) g.metric_part[chunk * 4 + t] = (red[0][t] + red[1][t]) + (red[2][t] + red[3][t]);
}

// 64 weights per workgroup, 16 lanes of partial sums each; the last workgroup takes the bias.
constexpr int UPD_GROUPS = 16;
__global__ void __launch_bounds__(64 * UPD_GROUPS) narrow_update_kernel(NarrowOutArgs g)
{
    __shared__ float red[UPD_GROUPS][64];
    const int t = threadIdx.x, c = t & 63, grp = t >> 6;
    const long long nw = (long long)g.no * g.ni;
    if (blockIdx.x == gridDim.x - 1) {
        // bias: column means of D, rows dealt over the threads in a fixed pattern
        float sv[kMaxOut];
#pragma unroll
        for (int j = 0; j < kMaxOut; ++j) sv[j] = 0.0f;
        for (int r = t; r < g.B; r += 64 * UPD_GROUPS) {
            const float* d = g.D + (long long)r * g.no;
            float dv[kMaxOut];
#pragma unroll
            for (int j = 0; j < kMaxOut; ++j) dv[j] = d[j < g.no ? j : g.no - 1];
#pragma unroll
            for (int j = 0; j < kMaxOut; ++j) sv[j] += dv[j];
        }
        narrow_reduce<kMaxOut>(sv, c);
        if ((c & 3) == 0) red[grp][narrow_owner<kMaxOut>(c)] = sv[0];
        // loss, accuracy and correct count of the batch: the chunks' sums in chunk order
        if (grp == 1 && g.metric_part) {  // the second wavefront: two slots per lane, then across the lanes
            double m[3];
#pragma unroll
            for (int q = 0; q < 3; ++q) {
                const double lo = (c < g.chunks) ? g.metric_part[c * 4 + q] : 0.0;
                const double hi = (c + 64 < g.chunks) ? g.metric_part[(c + 64) * 4 + q] : 0.0;
                m[q] = lo + hi;
            }
#pragma unroll
            for (int q = 0; q < 3; ++q) {
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) m[q] += __shfl_xor(m[q], o, 64);
                if (c == 0) g.metric_acc[q] += m[q];
            }
        }
        __syncthreads();
        if (t < g.no && g.bias_w) {
            float sum = 0.0f;
#pragma unroll
            for (int q = 0; q < UPD_GROUPS; ++q) sum += red[q][t];
            const float d = g.lr * (sum * g.alpha) + g.mom * g.bias_v[t];
            g.bias_v[t] = d;
            g.bias_w[t] = g.bias_w[t] - d;
        }
        return;
    }
    const long long idx = (long long)blockIdx.x * 64 + c;   // weight index o * ni + column
    float wgt = 0.0f, vel = 0.0f;
    if (grp == 0 && idx < nw) { wgt = g.Wm[idx]; vel = g.V[idx]; }  // on their way while the chunks are added up
    float s = 0.0f;
    if (idx < nw) {
        // up to 8 chunks per lane (128 chunks at most): all loads first, then the sum in chunk order
        float pv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int ch = grp + i * UPD_GROUPS;
            pv[i] = g.part[(long long)(ch < g.chunks ? ch : grp % g.chunks) * nw + idx];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) s += (grp + i * UPD_GROUPS < g.chunks) ? pv[i] : 0.0f;
    }
    red[grp][c] = s;
    __syncthreads();
    if (grp == 0 && idx < nw) {
        float sum = 0.0f;
#pragma unroll
        for (int q = 0; q < UPD_GROUPS; ++q) sum += red[q][c];
        const float sg = (wgt > 0.0f) ? 1.0f : ((wgt < 0.0f) ? -1.0f : 0.0f);
        const float grad = sum * g.alpha + g.wd1 * sg + g.wd2 * wgt;
        const float d = g.lr * grad + g.mom * vel;
        g.V[idx] = d;
        g.Wm[idx] = wgt - d;
    }
}

}  // namespace

bool ghip_narrow_out_ok(int no, int ni)
{
    // rows longer than 8192 stay with the GEMM path: a chunk of rows is walked by 4 wavefronts only, and
    // the partial sums (up to 128 chunks x no x ni floats) would grow past 64 MB
    return no >= 1 && no <= kMaxOut && ni >= 4 && ni <= 8192 && (ni % 4) == 0;
}

static_assert(8 * UPD_GROUPS == 128, "narrow_update_kernel reads at most 8 chunks per lane");
void ghip_narrow_out_chunks(int B, int* chunks, int* rows_per_chunk)
{
    // up to 128 chunks of at least 4 rows: enough wavefronts to cover the chip at a batch of 512
    int want = (B + 3) / 4;
    if (want > 128) want = 128;
    if (want < 1) want = 1;
    const int rpc = (B + want - 1) / want;
    *rows_per_chunk = rpc;
    *chunks = (B + rpc - 1) / rpc;
}

static bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

hipError_t ghip_narrow_forward(const NarrowOutArgs& a, hipStream_t s)
{
    if (!ghip_narrow_out_ok(a.no, a.ni) || a.B < 1 || !aligned16(a.H) || !aligned16(a.W)) return hipErrorInvalidValue;
    const dim3 grid((a.B + 3) / 4), block(256);
    if (a.no <= 4) hipLaunchKernelGGL(narrow_forward_kernel<4>, grid, block, 0, s, a);
    else if (a.no <= 8) hipLaunchKernelGGL(narrow_forward_kernel<8>, grid, block, 0, s, a);
    else hipLaunchKernelGGL(narrow_forward_kernel<16>, grid, block, 0, s, a);
    return hipGetLastError();
}

hipError_t ghip_narrow_train(const NarrowOutArgs& a, const DeltaArgs& da, hipStream_t s)
{
    if (!ghip_narrow_out_ok(a.no, a.ni) || a.B < 1 || a.chunks < 1 || a.rows_per_chunk < 1 ||
        (long long)a.chunks * a.rows_per_chunk < a.B || !a.part || !a.metric_part || !a.P || !da.D || !da.acc || da.n != a.no || da.B != a.B ||
        da.P != a.P || da.Dbf || da.DbfT ||
        !aligned16(a.H) || !aligned16(a.W) || !aligned16(a.part) || (a.E && !aligned16(a.E)))
        return hipErrorInvalidValue;
    const dim3 grid(a.chunks), block(256);
#define NARROW_TRAIN(NP)                                                                         \
    do {                                                                                         \
        if (a.E) hipLaunchKernelGGL((narrow_train_kernel<NP, true>), grid, block, 0, s, a, da);    \
        else hipLaunchKernelGGL((narrow_train_kernel<NP, false>), grid, block, 0, s, a, da);       \
    } while (0)
    if (a.no <= 4) NARROW_TRAIN(4);
    else if (a.no <= 8) NARROW_TRAIN(8);
    else NARROW_TRAIN(16);
#undef NARROW_TRAIN
    return hipGetLastError();
}

hipError_t ghip_narrow_update(const NarrowOutArgs& a, hipStream_t s)
{
    if (!ghip_narrow_out_ok(a.no, a.ni) || a.chunks < 1 || a.chunks > 8 * UPD_GROUPS || !a.part || !a.Wm || !a.V || !a.D) return hipErrorInvalidValue;
    const long long nw = (long long)a.no * a.ni;
    const dim3 grid((unsigned)((nw + 63) / 64) + 1), block(64 * UPD_GROUPS);
    hipLaunchKernelGGL(narrow_update_kernel, grid, block, 0, s, a);
    return hipGetLastError();
}

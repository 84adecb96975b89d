// Canonical (batched) training and evaluation of a NARROW network as one persistent workgroup: every layer
// at most 64 wide, parameters, momentum, gradient accumulators and a chunk of rows' activations and deltas all
// in LDS, the batch loop, the pass over the table and the epoch loop inside the kernel.  Such networks (the
// reference's own test networks, network.cpp:171-195 is the epoch loop they run in) do a few thousand
// multiply-adds per row: as GEMM launches a step is seven launches of mostly fixed cost, here it is a few
// microseconds of one CU, and a whole schedule of epochs is ONE launch.
//
// A batch is walked in chunks of up to 64 rows.  Per chunk: forward (work item = (row, unit), rows fastest, so
// a wavefront shares a unit's weight row as LDS broadcasts and walks the activations at an odd pitch), output
// delta / loss / metrics with the row function the other canonical kernels use (a wavefront per row, a lane
// per output: the rules are stated once), back-propagation (item = (row, unit below)), and the gradient sums
// (item = a weight, which its thread owns for the whole launch: no reduction between threads, a fixed order of
// addition).  The update after the last chunk of a batch is the one of the GEMM path (gemm_f32.hip, EPI_SGD).

#include "delta_row.h"

#include <string.h>

#include <mutex>

namespace {

// lanes a row of n outputs takes in the row function: the power of two at or above n
template <int SEG, bool kTrain>
__device__ __forceinline__ void output_rows(const float* Y, const DeltaArgs& da, const float* AL, float* DL, int pitch,
                                            long long row0, int rc, int nL, int w, int NW, int lane,
                                            double& loss, double& accs, double& corr)
{
    constexpr int RPW = 64 / SEG;            // rows a wavefront finishes per call
    const int o = lane & (SEG - 1), sub = lane / SEG;
    for (int rb = w * RPW; rb < rc; rb += NW * RPW) {
        const int r = rb + sub;
        const bool live = r < rc && o < nL;
        const float v = live ? AL[r * pitch + o] : -3.0e38f;
        const float yv = live ? Y[(row0 + r) * nL + o] : 0.0f;
        double l1 = 0.0, a1 = 0.0, c1 = 0.0;
        const float d = ghip_delta_row_seg<SEG>(da, 0, lane, v, yv, l1, a1, c1);
        if (r < rc && o == 0) { loss += l1; accs += a1; corr += c1; }   // one lane per row keeps the row's figures
        if (kTrain && live) DL[r * pitch + o] = d;
    }
}

template <bool kTrain>
__global__ void __launch_bounds__(1024) canon_narrow_kernel(CanonNarrowArgs p)
{
    extern __shared__ float lds[];
    const int t = threadIdx.x, T = blockDim.x, lane = t & 63, w = t >> 6, NW = T >> 6;
    const int L = p.n_layers, RC = p.rows_per_chunk, rcsh = p.rc_shift;
    const int n0 = p.sizes[0], nL = p.sizes[L];
    __shared__ double red[16][3];
    __shared__ int stop_flag;

    for (int l = 0; l < L; ++l) {
        const int cnt = p.sizes[l] * p.sizes[l + 1], no = p.sizes[l + 1];
        for (int k = t; k < cnt; k += T) {
            lds[p.offW[l] + k] = p.W[l][k];
            if (kTrain) { lds[p.offVW[l] + k] = p.vW[l][k]; lds[p.offG[l] + k] = 0.0f; }
        }
        for (int k = t; k < no; k += T) {
            lds[p.offB[l] + k] = p.b[l][k];
            if (kTrain) { lds[p.offVB[l] + k] = p.vb[l][k]; lds[p.offGB[l] + k] = 0.0f; }
        }
    }
    if (t == 0) stop_flag = 0;
    __syncthreads();

    DeltaArgs da;
    da.P = nullptr; da.Y = nullptr; da.D = nullptr; da.Dbf = nullptr; da.DbfT = nullptr;
    da.B = 0; da.n = nL; da.ldp = 0; da.ldy = nL; da.ldd = 0;
    da.act = p.act[L - 1]; da.act_param = p.act_param[L - 1]; da.cost = p.cost;
    da.acc = nullptr; da.acc_clear = nullptr; da.cm = p.cm; da.store_p = 0;
    const bool softmax = p.act[L - 1] == GHIP_SOFTMAX;
    // a thread's place in the (row, unit) grids of the forward and backward phases: rows fastest, so that a
    // wavefront shares a unit (its weights are LDS broadcasts) and walks the rows at an odd pitch
    const int tr = t & (RC - 1), tg = t >> rcsh, NG = T >> rcsh;
    // a table that fits one chunk is staged once for all epochs, targets included
    const bool resident = p.n_rows <= RC && p.offY >= 0;
    auto stage_rows = [&](long long row0, int rc) {
        const float* src = p.X + row0 * n0;
        int r = t / n0, i = t - r * n0;              // one division per thread and chunk
        const int dr = T / n0, di = T - dr * n0;
        for (int k = t; k < rc * n0; k += T) {
            lds[p.offA[0] + r * p.pitchA[0] + i] = src[k];
            r += dr; i += di;
            if (i >= n0) { i -= n0; ++r; }
        }
    };
    if (resident) {
        stage_rows(0, (int)p.n_rows);
        for (int k = t; k < (int)p.n_rows * nL; k += T) lds[p.offY + k] = p.Y[k];
        __syncthreads();
    }
    const float* Yrows = resident ? lds + p.offY : p.Y;

    int ep = 0;
    for (; ep < p.n_epochs; ++ep) {
        double loss = 0.0, accs = 0.0, corr = 0.0;   // of the rows whose figures this lane keeps
        if (p.cm && p.reset_cm) {   // CMatrix::reset at the head of every epoch (network.cpp:183-185)
            for (int k = t; k < nL * nL; k += T) p.cm[k] = 0;
            __threadfence();
            __syncthreads();
        }
        for (long long r0 = 0; r0 < p.n_rows; r0 += p.batch) {
            const int bcount = (int)(p.n_rows - r0 < p.batch ? p.n_rows - r0 : p.batch);
            for (int c0 = 0; c0 < bcount; c0 += RC) {
                const int rc = bcount - c0 < RC ? bcount - c0 : RC;
                const long long row0 = r0 + c0;
                const int in_row0 = resident ? (int)row0 : 0;   // where the chunk's inputs start in the staged rows
                // ---- the chunk's rows (the table is read as it lies: consecutive lanes, consecutive floats)
                if (!resident) {
                    stage_rows(row0, rc);
                    __syncthreads();
                }
                // ---- forward
                for (int l = 0; l < L; ++l) {
                    const int ni = p.sizes[l], no = p.sizes[l + 1];
                    const float* Wl = lds + p.offW[l];
                    const float* Bl = lds + p.offB[l];
                    const float* ar = lds + p.offA[l] + ((l == 0 ? in_row0 : 0) + tr) * p.pitchA[l];
                    float* Aout = lds + p.offA[l + 1] + tr * p.pitchA[l + 1];
                    const bool raw = softmax && l == L - 1;   // the row function takes softmax's logits
                    const int act = p.act[l]; const float ap = p.act_param[l];
                    if (tr < rc)
                        for (int j = tg; j < no; j += NG) {
                            const float* wr = Wl + j * ni;
                            float z = 0.0f;
                            for (int i = 0; i < ni; ++i) z += wr[i] * ar[i];
                            z += Bl[j];
                            Aout[j] = raw ? z : ghip_squash<false>(z, act, ap);
                        }
                    __syncthreads();
                }
                // ---- output delta, loss, metrics: a wavefront finishes 64 / SEG rows per call
                {
                    const float* AL = lds + p.offA[L];
                    float* DL = lds + p.offD[L];
                    const int pl = p.pitchA[L];
                    if (nL <= 4) output_rows<4, kTrain>(Yrows, da, AL, DL, pl, row0, rc, nL, w, NW, lane, loss, accs, corr);
                    else if (nL <= 16) output_rows<16, kTrain>(Yrows, da, AL, DL, pl, row0, rc, nL, w, NW, lane, loss, accs, corr);
                    else output_rows<64, kTrain>(Yrows, da, AL, DL, pl, row0, rc, nL, w, NW, lane, loss, accs, corr);
                }
                if (kTrain) {
                    __syncthreads();
                    // ---- back-propagation: D_l = (D_{l+1} W_l) .* f'(A_l)
                    for (int l = L - 1; l >= 1; --l) {
                        const int ni = p.sizes[l], no = p.sizes[l + 1];
                        const float* Wl = lds + p.offW[l];
                        const float* dn = lds + p.offD[l + 1] + tr * p.pitchA[l + 1];
                        const float* al = lds + p.offA[l] + tr * p.pitchA[l];
                        float* dl = lds + p.offD[l] + tr * p.pitchA[l];
                        const int act = p.act[l - 1]; const float ap = p.act_param[l - 1];
                        if (tr < rc)
                            for (int i = tg; i < ni; i += NG) {
                                float e = 0.0f;
                                for (int j = 0; j < no; ++j) e += Wl[j * ni + i] * dn[j];
                                dl[i] = e * ghip_act_der_canon(al[i], act, ap);
                            }
                        __syncthreads();
                    }
                    // ---- gradient sums.  Networks of a few hundred weights: a wavefront per weight, lanes over the
                    // chunk's rows, one cross-lane sum (a thread per weight would leave most of the workgroup idle
                    // and walk the rows one after the other); larger ones: a thread per weight, which it owns for
                    // the whole launch.  Either way a weight's sum is formed in one fixed order.
                    for (int l = 0; l < L; ++l) {
                        const int ni = p.sizes[l], no = p.sizes[l + 1];
                        const float* Dn = lds + p.offD[l + 1];
                        const int pa = p.pitchA[l], pd = p.pitchA[l + 1];
                        const float* Al = lds + p.offA[l] + (l == 0 ? in_row0 : 0) * pa;
                        float* G = lds + p.offG[l];
                        float* GB = lds + p.offGB[l];
                        if (p.wave_per_weight) {
                            int j = w / ni, i = w - j * ni;        // weight k = w, w + NW, ...
                            const int dj = NW / ni, di = NW - dj * ni;
                            for (int k = w; k < no * ni; k += NW) {
                                float sm = 0.0f;
                                for (int r = lane; r < rc; r += 64) sm += Dn[r * pd + j] * Al[r * pa + i];
                                sm = ghip_wave_sum(sm);
                                if (lane == 0) G[k] += sm;
                                j += dj; i += di;
                                if (i >= ni) { i -= ni; ++j; }
                            }
                            for (int j2 = w; j2 < no; j2 += NW) {
                                float sm = 0.0f;
                                for (int r = lane; r < rc; r += 64) sm += Dn[r * pd + j2];
                                sm = ghip_wave_sum(sm);
                                if (lane == 0) GB[j2] += sm;
                            }
                        } else {
                            int j = t / ni, i = t - j * ni;
                            const int dj = T / ni, di = T - dj * ni;
                            for (int k = t; k < no * ni; k += T) {
                                float sm = G[k];
                                for (int r = 0; r < rc; ++r) sm += Dn[r * pd + j] * Al[r * pa + i];
                                G[k] = sm;
                                j += dj; i += di;
                                if (i >= ni) { i -= ni; ++j; }
                            }
                            for (int j2 = t; j2 < no; j2 += T) {
                                float sm = GB[j2];
                                for (int r = 0; r < rc; ++r) sm += Dn[r * pd + j2];
                                GB[j2] = sm;
                            }
                        }
                    }
                }
                __syncthreads();   // the next chunk overwrites activations and deltas
            }
            if (kTrain) {
                // ---- update: g = mean gradient + decays; d = lr g + mom V; V = d; W -= d (biases: no decay)
                const float alpha = 1.0f / (float)bcount;
                for (int l = 0; l < L; ++l) {
                    const int cnt = p.sizes[l] * p.sizes[l + 1], no = p.sizes[l + 1];
                    const float lr = p.lr[l], mom = p.mom[l], wd1 = p.wd1[l], wd2 = p.wd2[l];
                    for (int k = t; k < cnt; k += T) {
                        const float wgt = lds[p.offW[l] + k];
                        const float sg = (wgt > 0.0f) ? 1.0f : ((wgt < 0.0f) ? -1.0f : 0.0f);
                        const float grad = lds[p.offG[l] + k] * alpha + wd1 * sg + wd2 * wgt;
                        const float d = lr * grad + mom * lds[p.offVW[l] + k];
                        lds[p.offVW[l] + k] = d;
                        lds[p.offW[l] + k] = wgt - d;
                        lds[p.offG[l] + k] = 0.0f;
                    }
                    for (int j = t; j < no; j += T) {
                        const float d = lr * (lds[p.offGB[l] + j] * alpha) + mom * lds[p.offVB[l] + j];
                        lds[p.offVB[l] + j] = d;
                        lds[p.offB[l] + j] -= d;
                        lds[p.offGB[l] + j] = 0.0f;
                    }
                }
                __syncthreads();
            }
        }
        // ---- the epoch's figures: lanes, then wavefronts, added in a fixed order
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            loss += __shfl_xor(loss, o, 64); accs += __shfl_xor(accs, o, 64); corr += __shfl_xor(corr, o, 64);
        }
        if (lane == 0) { red[w][0] = loss; red[w][1] = accs; red[w][2] = corr; }
        __syncthreads();
        if (t == 0) {
            double a = 0.0, b = 0.0, c = 0.0;
            for (int k = 0; k < NW; ++k) { a += red[k][0]; b += red[k][1]; c += red[k][2]; }
            p.metrics[4 * ep + 0] = a; p.metrics[4 * ep + 1] = b; p.metrics[4 * ep + 2] = c; p.metrics[4 * ep + 3] = 0.0;
            const float accuracy = (float)(b / ((double)p.n_rows * nL));
            if (p.stop_accuracy > 0.0f && accuracy >= p.stop_accuracy) stop_flag = 1;
        }
        __syncthreads();
        if (stop_flag) { ++ep; break; }
    }
    if (kTrain) {
        for (int l = 0; l < L; ++l) {
            const int cnt = p.sizes[l] * p.sizes[l + 1], no = p.sizes[l + 1];
            for (int k = t; k < cnt; k += T) { p.W[l][k] = lds[p.offW[l] + k]; p.vW[l][k] = lds[p.offVW[l] + k]; }
            for (int k = t; k < no; k += T) { p.b[l][k] = lds[p.offB[l] + k]; p.vb[l][k] = lds[p.offVB[l] + k]; }
        }
    }
    if (t == 0) *p.epochs_run = ep;
    if (p.clear4 && t < 4) p.clear4[t] = 0.0;
}

constexpr size_t kLdsLimit = 160 * 1024 - 1024;   // the static part (reduction scratch) stays clear of the limit

}  // namespace

// Lays out the LDS block of a network (offsets in floats) and picks the rows per chunk; false if a layer is
// wider than 64 or the block does not fit next to at least 16 rows.
bool ghip_canon_narrow_plan(const int* sizes, int n_layers, int train, CanonNarrowArgs* out, size_t* lds_bytes)
{
    if (n_layers < 1 || n_layers > GHIP_MAX_LAYERS) return false;
    size_t off = 0;
    for (int l = 0; l <= n_layers; ++l)
        if (sizes[l] < 1 || sizes[l] > 64) return false;
    CanonNarrowArgs a;
    memset(&a, 0, sizeof(a));
    for (int l = 0; l < n_layers; ++l) {
        const size_t cnt = (size_t)sizes[l] * sizes[l + 1], no = (size_t)sizes[l + 1];
        a.offW[l] = (int)off; off += cnt;
        a.offB[l] = (int)off; off += no;
        if (train) {
            a.offVW[l] = (int)off; off += cnt;
            a.offVB[l] = (int)off; off += no;
            a.offG[l] = (int)off; off += cnt;
            a.offGB[l] = (int)off; off += no;
        }
    }
    size_t per_row = 0;
    for (int l = 0; l <= n_layers; ++l) per_row += (size_t)(sizes[l] | 1) * (train && l > 0 ? 2 : 1);
    int rc = 256;   // a power of two, at most a quarter of the workgroup: every row then has four threads or more
    while (rc >= 16 && (off + per_row * rc) * sizeof(float) > kLdsLimit) rc >>= 1;
    if (rc < 16) return false;
    size_t n_weights = 0;
    for (int l = 0; l < n_layers; ++l) n_weights += (size_t)sizes[l] * sizes[l + 1];
    a.wave_per_weight = n_weights <= 1024 ? 1 : 0;
    a.rc_shift = 0;
    while ((1 << a.rc_shift) < rc) ++a.rc_shift;
    for (int l = 0; l <= n_layers; ++l) {
        a.pitchA[l] = sizes[l] | 1;   // odd: a wavefront's lanes are rows
        a.offA[l] = (int)off; off += (size_t)a.pitchA[l] * rc;
        if (train && l > 0) { a.offD[l] = (int)off; off += (size_t)a.pitchA[l] * rc; }
    }
    // room for a chunk's targets: a table of at most one chunk then stays in LDS over the epochs
    a.offY = -1;
    if ((off + (size_t)rc * sizes[n_layers]) * sizeof(float) <= kLdsLimit) { a.offY = (int)off; off += (size_t)rc * sizes[n_layers]; }
    a.rows_per_chunk = rc;
    a.n_layers = n_layers;
    for (int l = 0; l <= n_layers; ++l) a.sizes[l] = sizes[l];
    if (out) *out = a;
    if (lds_bytes) *lds_bytes = off * sizeof(float);
    return true;
}

hipError_t ghip_canon_narrow_run(const CanonNarrowArgs& a, size_t lds_bytes, hipStream_t s)
{
    if (lds_bytes > kLdsLimit || a.n_rows < 1 || a.batch < 1 || a.n_epochs < 1 || !a.metrics || !a.epochs_run) return hipErrorInvalidValue;
    static std::once_flag once;
    static hipError_t raised = hipSuccess;
    std::call_once(once, [] {
        raised = hipFuncSetAttribute((const void*)canon_narrow_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsLimit);
        if (raised == hipSuccess)
            raised = hipFuncSetAttribute((const void*)canon_narrow_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsLimit);
    });
    if (raised != hipSuccess) return raised;
    if (a.train) hipLaunchKernelGGL(canon_narrow_kernel<true>, dim3(1), dim3(1024), lds_bytes, s, a);
    else hipLaunchKernelGGL(canon_narrow_kernel<false>, dim3(1), dim3(1024), lds_bytes, s, a);
    return hipGetLastError();
}

// Exact mode: the reference's per-sample sequential training as ONE persistent workgroup.
//
// Follows NNetwork::SGDHelper / ForwardPass / BackPropagation
// ("Backend/Machine Learning/Networks/network.cpp":399-668) and Node::getDelta / applyDeltas
// ("Backend/Machine Learning/State/node.cpp":278-307) for every row in order.  Samples are
// strictly sequential (the scalar layer bias and the weights change inside a "minibatch"), so
// the parallelism is inside a layer only:
//   forward      one lane per output node, inputs summed in ascending order (node.cpp:82-93)
//   edge update  one lane per edge (delta push, window sum, conditional apply)
//   back-prop    one lane per input node, outputs visited in ascending order with the
//                reference's doubling accumulator  e <- e + (e + d*w)   (network.cpp:660-662)
//   bias, loss   one wavefront / one designated lane, in the reference's visiting order
// Every fp32 operation is written as a separate round-to-nearest step in the reference's order, and
// the file is compiled with contraction off (the pragma below and -ffp-contract=off in the build):
// hipcc would otherwise fuse a product with the addition that follows it, also through the
// __fmul_rn / __fadd_rn helpers, which are plain operators.
//
// Dropout (the kDrop instantiation) takes the flags of every row from a table the host drew
// (LayerBuilder::scrambleDropout, "Backend/Machine Learning/State/LayerBuilder.cpp":497-523) and
// follows what the reference does with them: a dropped pair sets no edge activation and gets no
// delta, the output node is finalised regardless (a dropped hidden node becomes squash(bias)), a
// dropped pair still hands the output node's error accumulator down (without the derivative
// factor), and the accumulator of an output node is only cleared by a valid pair with the LAST
// input node -- so it can survive into the next row, the next epoch and the next call
// (network.cpp:480-516, 621-662).
//
// Weights, pending-delta sums and last deltas live in LDS for the whole call (3 floats per edge,
// rows padded to an odd stride so that lane-per-row and lane-per-column walks are both free of
// bank conflicts); networks too large for LDS keep them in global memory (L2 resident).

#pragma clang fp contract(off)

#include "ghip_internal.h"

namespace {

constexpr int kPrefetch = 4;  // values per lane of the next row held in registers
template <int V> struct IC { static constexpr int value = V; };

// The reference updates the scalar layer bias once per (input, output) pair (network.cpp:654-656):
// bias -= lr*d[o] for o = 0..n_out-1, repeated n_in times -- one dependent chain of n_in*n_out fp32
// subtractions whose rounding order must be kept.  The n_out values sit in NP registers (padded
// with zeros: b - 0 is exact), so a step is a single subtract with no memory access.
// With dropout only valid pairs take part: dropped output nodes (mo[k] != 0) subtract an exact zero
// and ni counts the valid input nodes.
template <int NP>
__device__ __forceinline__ float bias_chain(float b, const float* bs, int no, int ni, const int* mo = nullptr)
{
    float x[NP];
#pragma unroll
    for (int k = 0; k < NP; ++k) x[k] = (k < no && !(mo && mo[k])) ? bs[k] : 0.0f;
    // (short rounds are unrolled so that the chain, not the loop around it, sets the pace)
    constexpr int kRounds = NP >= 16 ? 1 : 16 / NP;
#pragma unroll kRounds
    for (int i = 0; i < ni; ++i) {
#pragma unroll
        for (int k = 0; k < NP; ++k) b = __fsub_rn(b, x[k]);
    }
    return b;
}

// A sequential fold z = step(z, x[i*xs], y[i*ys]) for i = 0..n-1 in that order, with the operands
// fetched from LDS eight steps at a time and one block ahead of the arithmetic (two register sets,
// alternating: a copy from one to the other would wait for the block just asked for).  Left to
// itself the compiler asks for two operands, waits for them, uses them, and asks for the next two: an
// LDS round trip per pair of steps, which is what a row's dot products then consist of.
template <typename Step>
__device__ __forceinline__ float fold8(float z, const float* x, int xs, const float* y, int ys, int n, Step step)
{
    constexpr int B = 8;
    const int nb = n / B;
    float xa[B], ya[B], xb[B], yb[B];
    auto fetch = [&](float (&xv)[B], float (&yv)[B], int blk) {
        const float* px = x + blk * B * xs;
        const float* py = y + blk * B * ys;
#pragma unroll
        for (int j = 0; j < B; ++j) { xv[j] = px[j * xs]; yv[j] = py[j * ys]; }
        __builtin_amdgcn_sched_barrier(0);
    };
    auto run = [&](const float (&xv)[B], const float (&yv)[B]) {
#pragma unroll
        for (int j = 0; j < B; ++j) z = step(z, xv[j], yv[j]);
        __builtin_amdgcn_sched_barrier(0);
    };
    if (nb > 0) {
        int b = 0;
        fetch(xa, ya, 0);
        // nothing else is outstanding when the loop is entered: with a scalar load possibly in flight
        // (they return out of order) the first wait inside the loop would be for everything
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        while (b + 2 < nb) {
            fetch(xb, yb, b + 1); run(xa, ya);
            fetch(xa, ya, b + 2); run(xb, yb);
            b += 2;
        }
        if (nb - b == 2) { fetch(xb, yb, b + 1); run(xa, ya); run(xb, yb); }
        else run(xa, ya);
    }
    // the last n % 8 steps: their operands asked for together (a loop would pay an LDS round trip per step,
    // which for the 4-input layer of a small network is the whole dot product); past the end the last pair is
    // read again and not used
    const int rem = n - nb * B;
    if (rem > 0) {
        float xv[B - 1], yv[B - 1];
#pragma unroll
        for (int j = 0; j < B - 1; ++j) {
            const int i = nb * B + (j < rem ? j : rem - 1);
            xv[j] = x[i * xs]; yv[j] = y[i * ys];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < B - 1; ++j)
            if (j < rem) z = step(z, xv[j], yv[j]);
    }
    return z;
}

// Inclusive scan over the 64 lanes of a wavefront with an associative op: shifts within the rows of 16 lanes,
// then the last lane of row 0 / 2 into rows 1 / 3 and the last lane of the lower half into the upper half.
// A lane without a source keeps `identity`.
template <typename Op>
__device__ __forceinline__ int wave_scan(int v, int identity, Op op)
{
    v = op(v, __builtin_amdgcn_update_dpp(identity, v, 0x111, 0xf, 0xf, false));  // row_shr:1
    v = op(v, __builtin_amdgcn_update_dpp(identity, v, 0x112, 0xf, 0xf, false));  // row_shr:2
    v = op(v, __builtin_amdgcn_update_dpp(identity, v, 0x114, 0xf, 0xf, false));  // row_shr:4
    v = op(v, __builtin_amdgcn_update_dpp(identity, v, 0x118, 0xf, 0xf, false));  // row_shr:8
    v = op(v, __builtin_amdgcn_update_dpp(identity, v, 0x142, 0xa, 0xf, false));  // row_bcast:15 into rows 1 and 3
    v = op(v, __builtin_amdgcn_update_dpp(identity, v, 0x143, 0xc, 0xf, false));  // row_bcast:31 into rows 2 and 3
    return v;
}

// The same chain without walking it, where that is provably the same.  While the bias stays in one
// binade [2^e, 2^(e+1)) its values are integers M in units of u = 2^(e-23), and b - x rounds to
// M - rn(x / u): the rounding does not depend on M unless x / u lies exactly half-way between two
// integers (a tie goes to the even M).  So with q_k = rn(x_k / u) the chain is integer arithmetic,
// which is associative: after n_in rounds M has moved by n_in * sum(q_k), and every intermediate
// value is i * sum(q) + (a prefix sum of q).  One wavefront, lane k holding x_k, checks with a
// prefix scan that no intermediate value leaves the binade (a value below 2^23 + 1 units could have
// been rounded on the finer grid underneath) and that there is no tie; if so it returns the result
// of the n_in * n_out subtractions exactly, otherwise it says no and the caller walks the chain.
// All 64 lanes call with the same b and n_in; xk is this lane's lr*d (0 past the last output).
__device__ __forceinline__ bool bias_chain_grid(float b, float xk, int ni, int lane, float* result)
{
    const unsigned int bits = __float_as_uint(b);
    const int ex = (int)((bits >> 23) & 0xffu);
    if (ex == 0 || ex == 255) return false;                 // zero, subnormal, infinite, not a number
    const long long m0 = (long long)((bits & 0x7fffffu) | 0x800000u);
    const bool neg = (bits >> 31) != 0;
    const long long M0 = neg ? -m0 : m0;
    // 1 / u = 2^(150 - ex) and u, as doubles: scaling a float by them is exact
    const double inv_u = __longlong_as_double((long long)(1023 + 150 - ex) << 52);
    const double u = __longlong_as_double((long long)(1023 - 150 + ex) << 52);
    const double t = (double)xk * inv_u;
    const bool in_range = fabs(t) <= 16777216.0;            // false for NaN too; 64 of them stay below 2^31
    const double q = __builtin_rint(t);                     // to nearest, ties to even
    const bool tie = fabs(t - q) == 0.5;
    if (__ballot(!in_range || tie) != 0ull) return false;
    const int qi = (int)q;
    // inclusive prefix sums over the lanes, their extremes, and the total: scans on the cross-lane data path
    // (a shuffle through LDS is a round trip of a hundred clocks per step, and this wavefront runs alone)
    const int pre = wave_scan(qi, 0, [](int a, int c) { return a + c; });
    const int pmin = __builtin_amdgcn_readlane(wave_scan(pre, 0x7fffffff, [](int a, int c) { return a < c ? a : c; }), 63);
    const int pmax = __builtin_amdgcn_readlane(wave_scan(pre, (int)0x80000000, [](int a, int c) { return a > c ? a : c; }), 63);
    const long long Q = (long long)__builtin_amdgcn_readlane(pre, 63);
    (void)lane;
    const long long span = (long long)(ni - 1) * Q;
    const long long lo = (span < 0 ? span : 0) + pmin;      // smallest and largest amount subtracted so far,
    const long long hi = (span > 0 ? span : 0) + pmax;      // over every step of every round
    const long long Mlo = M0 - hi, Mhi = M0 - lo;
    const long long kMin = (1ll << 23) + 1, kMax = (1ll << 24) - 1;
    const bool inside = neg ? (Mhi <= -kMin && Mlo >= -kMax) : (Mlo >= kMin && Mhi <= kMax);
    if (!inside) return false;
    *result = (float)((double)(M0 - (long long)ni * Q) * u);
    return true;
}
// chains shorter than this are walked: the check costs about as much as a few hundred subtractions
constexpr int kGridChainMin = 512;

// Barrier between the phases of a row.  With the state in LDS the phases only hand LDS data to one
// another, so the wait covers LDS operations alone: __syncthreads() would also wait for the global
// loads that prefetch the next row and for the confusion-matrix atomics, a trip to memory per row.
// With the state in global memory the full barrier stays.
// A workgroup of one wavefront (kWave) needs no barrier at all: its LDS operations execute in the order
// they were issued, so a value one lane stored is there when another lane's later load reads it.  What is
// left is a fence that keeps the compiler from moving memory operations across the hand-over.
template <bool kLds, bool kWave = false>
__device__ __forceinline__ void row_barrier()
{
    if (kWave) {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    } else if (kLds) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else __syncthreads();
}

// One workgroup per network: `p` describes the (shared) architecture, hyper-parameters and data
// table; with `multi` each workgroup b takes its own parameter / result pointers from multi[b]
// (the subnets of a MetaNetwork train at the same time, one per compute unit), without it the
// single network's pointers are the ones in `p`.
// kL: the number of layers where it is known at compile time (0: read from p).  With it the loops over the layers
// unroll, every p.x[l] becomes a fixed kernel-argument slot that is read once into a scalar register, and the
// per-layer code is laid out straight.  The arithmetic and its order are the same.
// kMaxT: the most threads a launch of this instantiation has: 1024, or 64 for the networks that one wavefront
// serves (below).  Instantiations for 256 and 512 threads, which may use two and four times the registers, gained
// nothing for one network and halved the networks a compute unit holds in a launch over many.
template <bool kLds, bool kDrop, int kL, int kMaxT>
__global__ void __launch_bounds__(kMaxT)
exact_kernel(ExactLaunch p, const ExactPointers* __restrict__ multi)
{
    extern __shared__ __align__(16) float smem[];
    const ExactPointers own = multi ? multi[blockIdx.x] : p.ptr;
    // one wavefront per network (the small networks: LDS-resident, at most 64 lanes of work per phase)
    constexpr bool kWave = kLds && kMaxT == 64;
    const int tid = threadIdx.x;
    const int T = kWave ? 64 : (int)blockDim.x;
    const int serial = T - 1;  // lane that carries the order-dependent scalar chains
    const int L = kL > 0 ? kL : p.n_layers;
    constexpr int kLayerUnroll = kL > 0 ? kL : 1;
    const int n0 = p.sizes[0];
    const int nout = p.sizes[L];
    const int S = p.state_floats;

    float* sW;
    float* sSum;
    float* sLast;
    float* nodes;
    if (kLds) {
        sW = smem;
        sSum = smem + S;
        sLast = smem + 2 * S;
        nodes = smem + 3 * S;
    } else {
        sW = own.W;
        sSum = own.wsum;
        sLast = own.wlast;
        nodes = smem;
    }
    float* sa = nodes;                      // node values, all layers
    float* sd = nodes + p.node_floats;      // d = errDer * derivative of the layer being updated
    float* sbase = nodes + 2 * p.node_floats;  // lr * d
    float* sy = nodes + 3 * p.node_floats;  // expected row
    float* sbias = sy + nout;               // GHIP_MAX_LAYERS scalars
    int* sflag = (int*)(sbias + GHIP_MAX_LAYERS);
    // dropout only: the row's flags (1 = dropped; output layer always 0) and the nodes' error
    // accumulators (Node::errorDer), which outlive the row
    // (predicted, expected) pairs of the rows since the last flush; their cost and accuracy terms
    // are computed a ring-full at a time, one lane each, and summed in visiting order afterwards
    const int cap = p.metric_cap;
    // the 2^(i/32) table of expf, so that a sigmoid costs an LDS read instead of a trip to memory
    // (8-byte aligned; found by index arithmetic: a pointer that went through an integer is a generic one to the
    // compiler, and a generic load also waits for every global load in flight, the next row's prefetch included)
    unsigned long long* sT = (unsigned long long*)(smem + ((((float*)(sflag + 4) - smem) + 1) & ~(ptrdiff_t)1));
    float* rp = (float*)(sT + 32);
    float* re = rp + cap;
    int fill = 0;
    int* sm = (int*)(re + cap);
    float* sE = (float*)(sm + p.node_floats);
    const int mask_len = p.aoff[L];  // flags of one row: the non-output layers side by side

    if (kDrop) {
        for (int k = tid; k < p.node_floats; k += T) {
            sm[k] = 0;
            sE[k] = own.errder[k];
        }
    }
    if (kLds) {
        for (int k = tid; k < S; k += T) {
            sW[k] = own.W[k];
            sSum[k] = own.wsum[k];
            sLast[k] = own.wlast[k];
        }
    }
    if (tid < GHIP_MAX_LAYERS) sbias[tid] = own.bias[tid];
    if (tid == 0) sflag[0] = 0;
    if (tid < 32) {
        const unsigned long long tab[32] = GLM_EXP2_TAB;
        sT[tid] = tab[tid];
    }

    const float data_size = (float)((unsigned)p.n_rows * (unsigned)nout);
    const float fmb = (float)p.mb;
    // (the single-wavefront instantiation is launched for layers of at most 64 nodes: one value per lane)
    constexpr int kPf = kWave ? 1 : kPrefetch;
    const bool small_row = kWave || ((n0 <= kPrefetch * T) && (nout <= kPrefetch * T));
    // chunks of T values a row and its targets really have (the rest of the kPf slots is skipped, not masked)
    const int nchunk = kWave ? 1 : ((n0 > nout ? n0 : nout) + T - 1) / T;

    // first row into registers
    float px[kPf], py[kPf];
#pragma unroll
    for (int j = 0; j < kPf; ++j) {
        int i = tid + j * T;
        px[j] = (small_row && i < n0) ? p.X[i] : 0.0f;
        py[j] = (small_row && i < nout) ? p.Y[i] : 0.0f;
    }
    __syncthreads();

    int ep = 0;
    for (; ep < p.n_epochs; ++ep) {
        float tot_err = 0.0f, tot_acc = 0.0f;
        long long correct = 0;
        const bool last_epoch = (ep == p.n_epochs - 1) || (p.stop_accuracy > 0.0f);
        if (own.cm) {  // CMatrix::reset at the head of every epoch (network.cpp:183-185)
            for (int k = tid; k < nout * nout; k += T) own.cm[k] = 0;
            __threadfence();
            __syncthreads();
        }
        int rmod = 0;  // r % mb
        for (long long r = 0; r < p.n_rows; ++r) {
            // ---- stage the row (prefetched) and start fetching the next one
            if (small_row) {
#pragma unroll
                for (int j = 0; j < kPf; ++j) {
                    if (j >= nchunk) break;
                    int i = tid + j * T;
                    if (i < n0) sa[i] = px[j];
                    if (i < nout) sy[i] = py[j];
                }
                long long rn = r + 1;
                if (rn == p.n_rows) rn = 0;
                const float* xn = p.X + rn * n0;
                const float* yn = p.Y + rn * nout;
#pragma unroll
                for (int j = 0; j < kPf; ++j) {
                    if (j >= nchunk) break;
                    int i = tid + j * T;
                    px[j] = (i < n0) ? xn[i] : 0.0f;
                    py[j] = (i < nout) ? yn[i] : 0.0f;
                }
            } else {
                for (int i = tid; i < n0; i += T) sa[i] = p.X[r * n0 + i];
                for (int i = tid; i < nout; i += T) sy[i] = p.Y[r * nout + i];
            }
            if (kDrop && own.masks) {
                const unsigned char* mr = own.masks + ((long long)ep * p.n_rows + r) * mask_len;
                for (int k = tid; k < mask_len; k += T) sm[k] = mr[k];
            }
            row_barrier<kLds, kWave>();

            // ---- ForwardPass (network.cpp:457-516)
#pragma unroll kLayerUnroll
            for (int l = 0; l < L; ++l) {
                const int ni = p.sizes[l], no = p.sizes[l + 1], ld = p.ld[l];
                const float* Wl = sW + p.woff[l];
                const float* ain = sa + p.aoff[l];
                float* aout = sa + p.aoff[l + 1];
                const int act = p.act[l];
                const float par = p.act_param[l];
                const float bl = sbias[l];
                const int* mi = sm + p.aoff[l];
                const int* mo = sm + p.aoff[l + 1];
                for (int o = tid; o < no; o += T) {
                    const float* w = Wl + o * ld;
                    float z = 0.0f;
                    if (kDrop) {
                        // the sum starts at +0 and never becomes -0, so adding +0 for a dropped
                        // pair leaves it as skipping the pair does
                        const bool vo = !mo[o];
#pragma unroll 8
                        for (int i = 0; i < ni; ++i)
                            z = __fadd_rn(z, (vo && !mi[i]) ? __fmul_rn(w[i], ain[i]) : 0.0f);
                    } else {
                        z = fold8(z, w, 1, ain, 1, ni, [](float acc, float wv, float av) { return __fadd_rn(acc, __fmul_rn(wv, av)); });
                    }
                    if (l != 0) z = __fadd_rn(z, bl);
                    const float a = ghip_squash<true>(z, act, par, (const uint64_t*)sT);
                    aout[o] = a;
                    if (l == L - 1) {
                        rp[fill + o] = a;
                        re[fill + o] = sy[o];
                    }
                    if (kWave) break;  // at most one node per lane there
                }
                row_barrier<kLds, kWave>();
            }
            fill += nout;
            const float* pred = sa + p.aoff[L];
            if (own.preds && last_epoch)
                for (int o = tid; o < nout; o += T) own.preds[r * nout + o] = pred[o];

            // ---- output metrics (network.cpp:519-559): the class of the row now, ...
            if (kWave) {
                // The scan "strictly greater than the best so far, starting from 0" ends on the first index that
                // holds the largest value above 0 (none: -1); a NaN never compares greater.  Across the lanes:
                // the maximum (the hardware's max ignores a NaN operand), then the lowest lane that holds it.
                const float pr = tid < nout ? pred[tid] : 0.0f, ex = tid < nout ? sy[tid] : 0.0f;
                auto fmax_op = [](int a, int c) { return __float_as_int(fmaxf(__int_as_float(a), __int_as_float(c))); };
                const float mp = __int_as_float(__builtin_amdgcn_readlane(wave_scan(__float_as_int(pr), 0, fmax_op), 63));
                const float my = __int_as_float(__builtin_amdgcn_readlane(wave_scan(__float_as_int(ex), 0, fmax_op), 63));
                const unsigned long long bp = __ballot(pr == mp && pr > 0.0f), by = __ballot(ex == my && ex > 0.0f);
                const int ip = bp ? __builtin_ctzll(bp) : -1, iy = by ? __builtin_ctzll(by) : -1;
                if (ip == iy) ++correct;   // every lane counts alike; lane `serial` reports
                if (tid == serial && own.cm && ip >= 0 && iy >= 0) atomicAdd(&own.cm[iy * nout + ip], 1);
            } else if (tid == serial) {
                float mp = 0.0f, my = 0.0f;
                int ip = -1, iy = -1;
                for (int o = 0; o < nout; ++o) {
                    const float pr = pred[o], ex = sy[o];
                    if (pr > mp) { mp = pr; ip = o; }
                    if (ex > my) { my = ex; iy = o; }
                }
                if (ip == iy) ++correct;
                // CMatrix::addResult (cmatrix.cpp:57-98): row = expected class, column = predicted
                if (own.cm && ip >= 0 && iy >= 0) atomicAdd(&own.cm[iy * nout + ip], 1);
            }
            // ... cost and accuracy once the ring is full: the terms in parallel (the logarithms of
            // the cost are the expensive part), the two running sums in visiting order by one lane.
            // The ring is written again only after the barriers that follow, so that lane is done.
            if (fill + nout > cap || r == p.n_rows - 1) {
                for (int k = tid; k < fill; k += T) {
                    const float pr = rp[k], ex = re[k];
                    rp[k] = ghip_cost<true>(ex, pr, data_size, p.cost);
                    re[k] = ghip_accuracy_term(pr, ex);
                }
                row_barrier<kLds, kWave>();
                if (tid == serial) {   // eight terms per LDS round trip
                    tot_err = fold8(tot_err, rp, 1, rp, 1, fill, [](float acc, float v, float) { return __fadd_rn(acc, v); });
                    tot_acc = fold8(tot_acc, re, 1, re, 1, fill, [](float acc, float v, float) { return __fadd_rn(acc, v); });
                }
                fill = 0;
            }

            if (p.train) {
                // output layer: errDer = 0 + costErrDer, derivative 1 (network.cpp:599-612)
                {
                    float* dl = sd + p.aoff[L];
                    float* bs = sbase + p.aoff[L];
                    const float lr = p.lr[L - 1];
                    for (int o = tid; o < nout; o += T) {
                        float e = __fadd_rn(0.0f, ghip_cost_der(sy[o], pred[o], p.cost));
                        dl[o] = e;
                        bs[o] = __fmul_rn(lr, e);
                        if (kDrop) sE[p.aoff[L] + o] = e;
                        if (kWave) break;
                    }
                }
                row_barrier<kLds, kWave>();
                const bool apply = rmod == 0;
#pragma unroll kLayerUnroll
                for (int Lo = L; Lo > 0; --Lo) {
                    const int l = Lo - 1;
                    const int ni = p.sizes[l], no = p.sizes[Lo], ld = p.ld[l];
                    float* Wl = sW + p.woff[l];
                    float* Sl = sSum + p.woff[l];
                    float* Ll = sLast + p.woff[l];
                    const float* ain = sa + p.aoff[l];
                    const float* dl = sd + p.aoff[Lo];
                    const float* bs = sbase + p.aoff[Lo];
                    const float lr = p.lr[l], mom = p.mom[l];
                    const float w1 = __fmul_rn(p.wd1[l], lr), w2 = __fmul_rn(p.wd2[l], lr);
                    const int* mi = sm + p.aoff[l];
                    const int* mo = sm + p.aoff[Lo];
                    const float* raw = sE + p.aoff[Lo];  // the out-layer's accumulators as they stand
                    // ---- per-edge delta push and conditional apply (node.cpp:278-307)
                    {
                        const int sh = p.tw_log2[l];
                        const int tw = 1 << sh;
                        // The last wavefront walks this layer's bias chain (below), which depends on nothing
                        // done here: where there are other wavefronts it starts on the chain at once and
                        // they share the edges (lane groups of at most a wavefront, so that they divide
                        // what is left).
                        const bool chain_apart = l != 0 && T >= 128 && tw <= 64;
                        const int Tp = chain_apart ? T - 64 : T;
                        const int i0 = tid & (tw - 1), o0 = tid >> sh, rpp = Tp >> sh;
                        if (tid < Tp) {
                        // an edge that sat out an applying row can hold more than mb pending deltas;
                        // applyDeltas reads the first mb only (node.cpp:299-301), so their number is kept
                        int* Cl = (kDrop && p.mb > 1) ? own.wcnt + p.woff[l] : nullptr;
                        if (!kDrop) {
                            // U edges of a lane at a time, their operands asked for together: four where a
                            // lane has several outputs per input column, one where it has at most one
                            // (the narrow layers of a small network, where three of four would be idle repeats
                            // and a lone wavefront pays for every instruction)
                            auto push = [&](auto uc) {
                                constexpr int U = decltype(uc)::value;
                                for (int i = i0; i < ni; i += tw) {
                                    const float a = ain[i];
                                    const float t1 = __fmul_rn(w1, fabsf(a));
                                    const float t2 = __fmul_rn(w2, a);
                                    for (int o = o0; o < no; o += U * rpp) {
                                        float bv[U], lv[U], sv[U];   // (the weight is only read by the row that applies)
                                        int kk[U];
#pragma unroll
                                        for (int j = 0; j < U; ++j) {
                                            const int oj = o + j * rpp;
                                            const int oc = oj < no ? oj : no - 1;  // past the end: a repeat that is not stored
                                            kk[j] = oc * ld + i;
                                            bv[j] = bs[oc]; lv[j] = Ll[kk[j]]; sv[j] = Sl[kk[j]];
                                        }
                                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                                        for (int j = 0; j < U; ++j) {
                                            if (o + j * rpp < no) {
                                                float dW = __fadd_rn(__fmul_rn(bv[j], a), __fmul_rn(mom, lv[j]));
                                                dW = __fadd_rn(dW, t1);
                                                dW = __fadd_rn(dW, t2);
                                                const float sn = __fadd_rn(sv[j], dW);
                                                if (apply) {
                                                    Wl[kk[j]] = __fsub_rn(Wl[kk[j]], __fdiv_rn(sn, fmb));
                                                    Sl[kk[j]] = 0.0f;
                                                    Ll[kk[j]] = 0.0f;
                                                } else {
                                                    Sl[kk[j]] = sn;
                                                    Ll[kk[j]] = dW;
                                                }
                                            }
                                        }
                                    }
                                }
                            };
                            if (no <= rpp) push(IC<1>{});
                            else push(IC<4>{});
                        } else
                        for (int i = i0; i < ni; i += tw) {
                            if (kDrop && mi[i]) continue;
                            const float a = ain[i];
                            const float t1 = __fmul_rn(w1, fabsf(a));
                            const float t2 = __fmul_rn(w2, a);
                            for (int o = o0; o < no; o += rpp) {
                                if (kDrop && mo[o]) continue;
                                const int k = o * ld + i;
                                float dW = __fadd_rn(__fmul_rn(bs[o], a), __fmul_rn(mom, Ll[k]));
                                dW = __fadd_rn(dW, t1);
                                dW = __fadd_rn(dW, t2);
                                float s = __fadd_rn(Sl[k], dW);
                                if (Cl) {
                                    const int c = Cl[k];
                                    if (c >= p.mb) s = Sl[k];
                                    Cl[k] = apply ? 0 : c + 1;
                                }
                                if (apply) {
                                    Wl[k] = __fsub_rn(Wl[k], __fdiv_rn(s, fmb));
                                    Sl[k] = 0.0f;
                                    Ll[k] = 0.0f;
                                } else {
                                    Sl[k] = s;
                                    Ll[k] = dW;
                                }
                            }
                        }
                        }
                    }
                    // ---- scalar bias of the in-layer (network.cpp:654-656)
                    // The n_in*n_out subtractions are one dependent chain; it runs in the last
                    // wavefront with the lr*d values held in registers (bias_chain below).
                    if ((tid >> 6) == (T >> 6) - 1 && l != 0) {
                        float b = sbias[l];
                        int nv = ni;  // input nodes taking part
                        const int* mk = nullptr;
                        if (kDrop) {
                            nv = 0;
                            for (int i = 0; i < ni; ++i) nv += mi[i] ? 0 : 1;
                            mk = mo;
                        }
                        bool walked = false;
                        if (p.bias_mode == GHIP_BIAS_SEQUENTIAL && no <= 64 && nv > 0 && (long long)nv * no >= kGridChainMin) {
                            const int k = tid & 63;
                            const float xk = (k < no && !(mk && mk[k])) ? bs[k] : 0.0f;
                            walked = bias_chain_grid(b, xk, nv, k, &b);
                        }
                        if (walked) {
                        } else if (p.bias_mode == GHIP_BIAS_SEQUENTIAL) {
                            if (no == 1) b = bias_chain<1>(b, bs, no, nv, mk);
                            else if (no == 2) b = bias_chain<2>(b, bs, no, nv, mk);
                            else if (no <= 4) b = bias_chain<4>(b, bs, no, nv, mk);
                            else if (no <= 8) b = bias_chain<8>(b, bs, no, nv, mk);
                            else if (no <= 16) b = bias_chain<16>(b, bs, no, nv, mk);
                            else if (no <= 32) b = bias_chain<32>(b, bs, no, nv, mk);
                            else if (no <= 64) b = bias_chain<64>(b, bs, no, nv, mk);
                            else {
                                for (int i = 0; i < nv; ++i) {
#pragma unroll 8
                                    for (int o = 0; o < no; ++o) b = __fsub_rn(b, (mk && mk[o]) ? 0.0f : bs[o]);
                                }
                            }
                        } else {
                            float s = 0.0f;
                            for (int o = 0; o < no; ++o) s = __fadd_rn(s, (mk && mk[o]) ? 0.0f : bs[o]);
                            b = __fsub_rn(b, __fmul_rn((float)nv, s));
                        }
                        if (tid == serial) sbias[l] = b;
                    }
                    row_barrier<kLds, kWave>();
                    // ---- error partials of the in-layer with the UPDATED weights
                    //      (network.cpp:660-662), then its own d and lr*d for the next round
                    if (l != 0) {
                        float* dn = sd + p.aoff[l];
                        float* bn = sbase + p.aoff[l];
                        const int actp = p.act[l - 1];
                        const float lrn = p.lr[l - 1];
                        for (int i = tid; i < ni; i += T) {
                            float e = 0.0f;
                            if (kDrop) {
                                // starts from what earlier rows left; a dropped pair hands down the
                                // out-node's accumulator without the derivative factor
                                e = sE[p.aoff[l] + i];
                                const bool di = mi[i] != 0;
#pragma unroll 8
                                for (int o = 0; o < no; ++o) {
                                    const float c = (di || mo[o]) ? raw[o] : dl[o];
                                    e = __fadd_rn(e, __fadd_rn(e, __fmul_rn(c, Wl[o * ld + i])));
                                }
                                sE[p.aoff[l] + i] = e;
                            } else {
                                e = fold8(e, dl, 1, Wl + i, ld, no,
                                          [](float acc, float dv, float wv) { return __fadd_rn(acc, __fadd_rn(acc, __fmul_rn(dv, wv))); });
                            }
                            // the reference always passes 0.01 here (network.cpp:617-618)
                            float d = __fmul_rn(e, ghip_act_der_ref(ain[i], actp, 0.01f));
                            dn[i] = d;
                            bn[i] = __fmul_rn(lrn, d);
                            if (kWave) break;
                        }
                        row_barrier<kLds, kWave>();
                    }
                    if (kDrop && Lo < L) {
                        // clearErrDer of the out-layer's nodes: only by a valid pair with the last
                        // input node (network.cpp:629-631)
                        if (!mi[ni - 1])
                            for (int o = tid; o < no; o += T)
                                if (!mo[o]) sE[p.aoff[Lo] + o] = 0.0f;
                        row_barrier<kLds, kWave>();
                    }
                }
            } else {
                row_barrier<kLds, kWave>();  // the metrics lane reads this row's outputs and targets: the next row waits
            }
            if (++rmod == p.mb) rmod = 0;
        }
        // ---- end of epoch (network.cpp:193-195, Terminator.cpp:73-74)
        if (tid == serial) {
            float acc = __fdiv_rn(tot_acc, __fmul_rn((float)(unsigned)p.n_rows, (float)(unsigned)nout));
            ghip_metrics* m = ((ghip_metrics*)own.metrics) + ep;
            m->loss = tot_err;
            m->accuracy = acc;
            m->correct = correct;
            if (own.cm && own.class_metrics) {  // network.cpp:218-224, read back through the atomics' path
                __threadfence();
                ghip_cmatrix_overall(own.cm, nout, own.class_metrics + 5 * ep);
            }
            if (p.stop_accuracy > 0.0f && acc >= p.stop_accuracy) sflag[0] = 1;
        }
        __syncthreads();
        if (sflag[0]) { ++ep; break; }
    }

    if (kLds) {
        for (int k = tid; k < S; k += T) {
            own.W[k] = sW[k];
            own.wsum[k] = sSum[k];
            own.wlast[k] = sLast[k];
        }
    }
    if (tid < GHIP_MAX_LAYERS) own.bias[tid] = sbias[tid];
    if (tid == 0) own.epochs_run[0] = ep;
    if (kDrop)
        for (int k = tid; k < p.node_floats; k += T) own.errder[k] = sE[k];
}

// ---------------------------------------------------------------- one wavefront per network
// The same rows, the same arithmetic in the same order, for the networks this is about most often: a few layers
// of at most 64 nodes, state in LDS, no dropout.  One wavefront runs alone on its SIMD and issues an instruction
// every other issue slot at best (each step of a row depends on the one before), so what a row costs is the
// number of instructions it executes.  Here that number is kept down: the layers are unrolled (kL of them), a
// lane owns one node of every layer and one column of edges, nothing is a loop that is known to run once, the
// layer biases and the row's targets stay in registers, the predicted class is found across the lanes, the kind
// of bias chain is decided once per launch, and there is no barrier: LDS operations of one wavefront execute
// in order.
template <int NP>
__device__ __forceinline__ float bias_chain_exact(float b, const float* bs, int ni)
{
    float x[NP];
#pragma unroll
    for (int k = 0; k < NP; ++k) x[k] = bs[k];
#pragma unroll 4
    for (int i = 0; i < ni; ++i) {
#pragma unroll
        for (int k = 0; k < NP; ++k) b = __fsub_rn(b, x[k]);
    }
    return b;
}

__device__ __forceinline__ void wave_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// kOcc: wavefronts per SIMD the register budget must allow.  2 (all the registers the code likes) is fastest for
// a launch that leaves SIMDs idle anyway; 4 costs one network 10 % and lets a launch over thousands of them
// keep four per SIMD, whose instructions fill each other's waiting slots.
template <int kL, int kOcc>
__global__ void __launch_bounds__(64, kOcc)
exact_wave_kernel(ExactLaunch p, const ExactPointers* __restrict__ multi)
{
    extern __shared__ __align__(16) float smem[];
    const ExactPointers own = multi ? multi[blockIdx.x] : p.ptr;
    const int lane = threadIdx.x;
    constexpr int L = kL;
    const int n0 = p.sizes[0];
    const int nout = p.sizes[L];
    const int S = p.state_floats;
    // the layout of exact_kernel's LDS-resident instantiation (ghip_exact_lds_bytes sizes it)
    float* sW = smem;
    float* sSum = smem + S;
    float* sLast = smem + 2 * S;
    float* nodes = smem + 3 * S;
    float* sa = nodes;
    float* sd = nodes + p.node_floats;
    float* sbase = nodes + 2 * p.node_floats;
    float* sy = nodes + 3 * p.node_floats;
    float* sbias = sy + nout;
    int* sflag = (int*)(sbias + GHIP_MAX_LAYERS);
    const int cap = p.metric_cap;
    // (8-byte aligned; found by index arithmetic: a pointer that went through an integer is a generic one to the
    // compiler, and a generic load also waits for every global load in flight, the next row's prefetch included)
    unsigned long long* sT = (unsigned long long*)(smem + ((((float*)(sflag + 4) - smem) + 1) & ~(ptrdiff_t)1));
    float* rp = (float*)(sT + 32);
    float* re = rp + cap;
    int fill = 0;

    for (int k = lane; k < S; k += 64) {
        sW[k] = own.W[k];
        sSum[k] = own.wsum[k];
        sLast[k] = own.wlast[k];
    }
    if (lane == 0) sflag[0] = 0;
    if (lane < 32) {
        const unsigned long long tab[32] = GLM_EXP2_TAB;
        sT[lane] = tab[lane];
    }
    float bias[kL];   // the scalar layer biases: every lane holds the same values
#pragma unroll
    for (int l = 0; l < kL; ++l) bias[l] = own.bias[l];

    // how layer l's bias chain is walked: 0 the closed form of the other bias mode, 1..8 / 16 / 32 / 64 that many
    // values per round held in registers; +128: first see whether the integer-grid shortcut applies
    int chain[kL];
#pragma unroll
    for (int l = 1; l < kL; ++l) {
        const int ni = p.sizes[l], no = p.sizes[l + 1];
        int c = 0;
        if (p.bias_mode == GHIP_BIAS_SEQUENTIAL) {
            c = no <= 8 ? no : (no <= 16 ? 16 : (no <= 32 ? 32 : 64));
            if ((long long)ni * no >= kGridChainMin) c += 128;
        }
        chain[l] = c;
    }

    const float data_size = (float)((unsigned)p.n_rows * (unsigned)nout);
    const float fmb = (float)p.mb;
    float px = lane < n0 ? p.X[lane] : 0.0f;
    float py = lane < nout ? p.Y[lane] : 0.0f;
    __syncthreads();

    int ep = 0;
    for (; ep < p.n_epochs; ++ep) {
        float tot_err = 0.0f, tot_acc = 0.0f;
        long long correct = 0;
        const bool last_epoch = (ep == p.n_epochs - 1) || (p.stop_accuracy > 0.0f);
        if (own.cm) {  // CMatrix::reset at the head of every epoch (network.cpp:183-185)
            for (int k = lane; k < nout * nout; k += 64) own.cm[k] = 0;
            __threadfence();
            __syncthreads();
        }
        int rmod = 0;  // r % mb
        for (long long r = 0; r < p.n_rows; ++r) {
            // ---- the row (fetched while the row before was worked on) and the request for the next one
            if (lane < n0) sa[lane] = px;
            const float yv = py;   // lane o: expected value of output o
            {
                long long rn = r + 1;
                if (rn == p.n_rows) rn = 0;
                px = lane < n0 ? p.X[rn * n0 + lane] : 0.0f;
                py = lane < nout ? p.Y[rn * nout + lane] : 0.0f;
            }
            wave_sync();

            // ---- ForwardPass (network.cpp:457-516)
            float pv = 0.0f;       // lane o: output o
#pragma unroll
            for (int l = 0; l < kL; ++l) {
                const int ni = p.sizes[l], no = p.sizes[l + 1], ld = p.ld[l];
                if (lane < no) {
                    float z = fold8(0.0f, sW + p.woff[l] + lane * ld, 1, sa + p.aoff[l], 1, ni,
                                    [](float acc, float wv, float av) { return __fadd_rn(acc, __fmul_rn(wv, av)); });
                    if (l != 0) z = __fadd_rn(z, bias[l]);
                    const float a = ghip_squash<true>(z, p.act[l], p.act_param[l], (const uint64_t*)sT);
                    sa[p.aoff[l + 1] + lane] = a;
                    if (l == kL - 1) {
                        rp[fill + lane] = a;
                        re[fill + lane] = yv;
                        pv = a;
                    }
                }
                wave_sync();
            }
            fill += nout;
            if (own.preds && last_epoch && lane < nout) own.preds[r * nout + lane] = pv;

            // ---- output metrics (network.cpp:519-559).  The scan "strictly greater than the best so far, starting
            // from 0" ends on the first index that holds the largest value above 0 (none: -1), and a NaN never
            // compares greater: across the lanes that is the maximum (the hardware's max passes over a NaN operand),
            // then the lowest lane that holds it.
            {
                const float pr = lane < nout ? pv : 0.0f, ex = lane < nout ? yv : 0.0f;
                auto fmax_op = [](int a, int c) { return __float_as_int(fmaxf(__int_as_float(a), __int_as_float(c))); };
                const float mp = __int_as_float(__builtin_amdgcn_readlane(wave_scan(__float_as_int(pr), 0, fmax_op), 63));
                const float my = __int_as_float(__builtin_amdgcn_readlane(wave_scan(__float_as_int(ex), 0, fmax_op), 63));
                const unsigned long long bp = __ballot(pr == mp && pr > 0.0f), by = __ballot(ex == my && ex > 0.0f);
                const int ip = bp ? __builtin_ctzll(bp) : -1, iy = by ? __builtin_ctzll(by) : -1;
                if (ip == iy) ++correct;
                // CMatrix::addResult (cmatrix.cpp:57-98): row = expected class, column = predicted
                if (lane == 63 && own.cm && ip >= 0 && iy >= 0) atomicAdd(&own.cm[iy * nout + ip], 1);
            }
            // cost and accuracy once the ring of (predicted, expected) pairs is full: the terms a lane each, the two
            // running sums in visiting order
            if (fill + nout > cap || r == p.n_rows - 1) {
                wave_sync();
                for (int k = lane; k < fill; k += 64) {
                    const float pr = rp[k], ex = re[k];
                    rp[k] = ghip_cost<true>(ex, pr, data_size, p.cost);
                    re[k] = ghip_accuracy_term(pr, ex);
                }
                wave_sync();
                // every lane walks the same two sums, eight terms per LDS round trip
                tot_err = fold8(tot_err, rp, 1, rp, 1, fill, [](float acc, float v, float) { return __fadd_rn(acc, v); });
                tot_acc = fold8(tot_acc, re, 1, re, 1, fill, [](float acc, float v, float) { return __fadd_rn(acc, v); });
                wave_sync();
                fill = 0;
            }

            if (p.train) {
                // output layer: errDer = 0 + costErrDer, derivative 1 (network.cpp:599-612)
                if (lane < nout) {
                    const float e = __fadd_rn(0.0f, ghip_cost_der(yv, pv, p.cost));
                    sd[p.aoff[L] + lane] = e;
                    sbase[p.aoff[L] + lane] = __fmul_rn(p.lr[L - 1], e);
                }
                wave_sync();
                const bool apply = rmod == 0;
#pragma unroll
                for (int Lo = kL; Lo > 0; --Lo) {
                    const int l = Lo - 1;
                    const int ni = p.sizes[l], no = p.sizes[Lo], ld = p.ld[l];
                    float* Wl = sW + p.woff[l];
                    float* Sl = sSum + p.woff[l];
                    float* Ll = sLast + p.woff[l];
                    const float* ain = sa + p.aoff[l];
                    const float* dl = sd + p.aoff[Lo];
                    const float* bs = sbase + p.aoff[Lo];
                    const float lr = p.lr[l], mom = p.mom[l];
                    const float w1 = __fmul_rn(p.wd1[l], lr), w2 = __fmul_rn(p.wd2[l], lr);
                    // ---- per-edge delta push and conditional apply (node.cpp:278-307): lane groups of tw lanes
                    //      walk a row of edges each (tw = the layer's width rounded up to a power of two)
                    {
                        const int sh = p.tw_log2[l];
                        const int i = lane & ((1 << sh) - 1), o0 = lane >> sh, rpp = 64 >> sh;
                        auto edge = [&](int k, float a, float t1, float t2, float bv, float lv, float sv) {
                            float dW = __fadd_rn(__fmul_rn(bv, a), __fmul_rn(mom, lv));
                            dW = __fadd_rn(dW, t1);
                            dW = __fadd_rn(dW, t2);
                            const float sn = __fadd_rn(sv, dW);
                            if (apply) {
                                Wl[k] = __fsub_rn(Wl[k], __fdiv_rn(sn, fmb));
                                Sl[k] = 0.0f;
                                Ll[k] = 0.0f;
                            } else {
                                Sl[k] = sn;
                                Ll[k] = dW;
                            }
                        };
                        if (no <= rpp) {
                            // one edge per lane: its four operands in one LDS round trip (an idle lane reads edge 0)
                            const bool mine = i < ni && o0 < no;
                            const int ic = mine ? i : 0, oc = mine ? o0 : 0, k = oc * ld + ic;
                            const float a = ain[ic], bv = bs[oc], lv = Ll[k], sv = Sl[k];
                            if (mine) edge(k, a, __fmul_rn(w1, fabsf(a)), __fmul_rn(w2, a), bv, lv, sv);
                        } else if (i < ni) {
                            const float a = ain[i];
                            const float t1 = __fmul_rn(w1, fabsf(a));
                            const float t2 = __fmul_rn(w2, a);
                            for (int o = o0; o < no; o += rpp) {
                                const int k = o * ld + i;
                                edge(k, a, t1, t2, bs[o], Ll[k], Sl[k]);
                            }
                        }
                    }
                    // ---- scalar bias of the in-layer (network.cpp:654-656): n_in rounds of n_out subtractions
                    if (l != 0) {
                        float b = bias[l];
                        int c = chain[l];
                        bool walked = false;
                        if (c & 128) {
                            walked = bias_chain_grid(b, lane < no ? bs[lane] : 0.0f, ni, lane, &b);
                            c &= 127;
                        }
                        if (!walked) {
                            switch (c) {
                            case 1: b = bias_chain_exact<1>(b, bs, ni); break;
                            case 2: b = bias_chain_exact<2>(b, bs, ni); break;
                            case 3: b = bias_chain_exact<3>(b, bs, ni); break;
                            case 4: b = bias_chain_exact<4>(b, bs, ni); break;
                            case 5: b = bias_chain_exact<5>(b, bs, ni); break;
                            case 6: b = bias_chain_exact<6>(b, bs, ni); break;
                            case 7: b = bias_chain_exact<7>(b, bs, ni); break;
                            case 8: b = bias_chain_exact<8>(b, bs, ni); break;
                            case 16: b = bias_chain<16>(b, bs, no, ni); break;
                            case 32: b = bias_chain<32>(b, bs, no, ni); break;
                            case 64: b = bias_chain<64>(b, bs, no, ni); break;
                            default: {
                                float sum = 0.0f;
                                for (int o = 0; o < no; ++o) sum = __fadd_rn(sum, bs[o]);
                                b = __fsub_rn(b, __fmul_rn((float)ni, sum));
                            }
                            }
                        }
                        bias[l] = b;
                    }
                    wave_sync();
                    // ---- error partials of the in-layer with the UPDATED weights (network.cpp:660-662), then its
                    //      own d and lr*d for the next round
                    if (l != 0) {
                        if (lane < ni) {
                            const float e = fold8(0.0f, dl, 1, Wl + lane, ld, no,
                                                  [](float acc, float dv, float wv) { return __fadd_rn(acc, __fadd_rn(acc, __fmul_rn(dv, wv))); });
                            // the reference always passes 0.01 here (network.cpp:617-618)
                            const float d = __fmul_rn(e, ghip_act_der_ref(ain[lane], p.act[l - 1], 0.01f));
                            sd[p.aoff[l] + lane] = d;
                            sbase[p.aoff[l] + lane] = __fmul_rn(p.lr[l - 1], d);
                        }
                        wave_sync();
                    }
                }
            }
            if (++rmod == p.mb) rmod = 0;
        }
        // ---- end of epoch (network.cpp:193-195, Terminator.cpp:73-74)
        if (lane == 63) {
            const float acc = __fdiv_rn(tot_acc, __fmul_rn((float)(unsigned)p.n_rows, (float)(unsigned)nout));
            ghip_metrics* m = ((ghip_metrics*)own.metrics) + ep;
            m->loss = tot_err;
            m->accuracy = acc;
            m->correct = correct;
            if (own.cm && own.class_metrics) {  // network.cpp:218-224, read back through the atomics' path
                __threadfence();
                ghip_cmatrix_overall(own.cm, nout, own.class_metrics + 5 * ep);
            }
            if (p.stop_accuracy > 0.0f && acc >= p.stop_accuracy) sflag[0] = 1;
        }
        __syncthreads();
        if (sflag[0]) { ++ep; break; }
    }

    for (int k = lane; k < S; k += 64) {
        own.W[k] = sW[k];
        own.wsum[k] = sSum[k];
        own.wlast[k] = sLast[k];
    }
    if (lane == 0) {
#pragma unroll
        for (int l = 0; l < kL; ++l) own.bias[l] = bias[l];
        own.epochs_run[0] = ep;
    }
}

// GMath::squash / activationErrDer / outputNodeCost / costErrDer over arrays, with exact mode's arithmetic
__global__ void gmath_eval_kernel(int fn, int kind, float param, const float* __restrict__ a, const float* __restrict__ b,
                                  float* __restrict__ out, long long n)
{
    for (long long k = (long long)blockIdx.x * blockDim.x + threadIdx.x; k < n; k += (long long)gridDim.x * blockDim.x) {
        float v = 0.0f;
        switch (fn) {
        case 0: v = ghip_squash<true>(a[k], kind, param); break;
        case 1: v = ghip_act_der_ref(a[k], kind, param); break;
        case 2: v = ghip_cost<true>(a[k], b[k], param, kind); break;
        case 3: v = ghip_cost_der(a[k], b[k], kind); break;
        }
        out[k] = v;
    }
}

// The bias chain of one row for n independent cases, a wavefront each: a[k] the bias before,
// b[64*k .. 64*k+63] the lr*d of the outputs (zeros past the last), n_in rounds.
// kind 0: one subtraction after the other; 1: the integer-grid shortcut where it applies, else the walk;
// 2: 1.0 where the shortcut applies, else 0.0.
__global__ void __launch_bounds__(256) bias_chain_eval_kernel(int kind, int ni, const float* __restrict__ a,
                                                              const float* __restrict__ b, float* __restrict__ out, long long n)
{
    const int lane = threadIdx.x & 63;
    const long long k = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (k >= n) return;
    float v = a[k];
    const float xk = b[k * 64 + lane];
    float fast = 0.0f;
    const bool ok = kind != 0 && ni > 0 && bias_chain_grid(v, xk, ni, lane, &fast);
    if (kind == 2) v = ok ? 1.0f : 0.0f;
    else if (ok) v = fast;
    else v = bias_chain<64>(v, b + k * 64, 64, ni);
    if (lane == 0) out[k] = v;
}

}  // namespace

hipError_t ghip_launch_bias_chain_eval(int kind, int ni, const float* a, const float* b, float* out, long long n, hipStream_t s)
{
    hipLaunchKernelGGL(bias_chain_eval_kernel, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, s, kind, ni, a, b, out, n);
    return hipGetLastError();
}

hipError_t ghip_launch_gmath_eval(int fn, int kind, float param, const float* a, const float* b, float* out, long long n,
                                  hipStream_t s)
{
    long long blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(gmath_eval_kernel, dim3((unsigned)blocks), dim3(256), 0, s, fn, kind, param, a, b, out, n);
    return hipGetLastError();
}

size_t ghip_exact_lds_bytes(const ExactLaunch& p, bool state_in_lds, bool dropout)
{
    size_t f = (size_t)3 * p.node_floats + p.sizes[p.n_layers] + GHIP_MAX_LAYERS + 4 + 2 + 64 + (size_t)2 * p.metric_cap;
    if (dropout) f += (size_t)2 * p.node_floats;
    if (state_in_lds) f += (size_t)3 * p.state_floats;
    return f * sizeof(float);
}

template <bool kLds, bool kDrop, int kL, int kMaxT>
static hipError_t launch_sized(const ExactLaunch& p, const ExactPointers* dev_multi, int count, int threads,
                               size_t lds_bytes, hipStream_t s)
{
    if (kLds) {
        hipError_t e = hipFuncSetAttribute((const void*)exact_kernel<kLds, kDrop, kL, kMaxT>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((exact_kernel<kLds, kDrop, kL, kMaxT>), dim3(count), dim3(threads), lds_bytes, s, p, dev_multi);
    return hipGetLastError();
}

template <bool kLds, bool kDrop, int kL>
static hipError_t launch_layers(const ExactLaunch& p, const ExactPointers* dev_multi, int count, int threads,
                                size_t lds_bytes, hipStream_t s)
{
    bool narrow = true;   // every layer fits the lanes of one wavefront
    for (int l = 0; l <= p.n_layers; ++l) narrow = narrow && p.sizes[l] <= 64;
    if constexpr (kL > 0 && kLds && !kDrop)
        if (threads == 64 && narrow) {
            // 256 compute units x 4 SIMDs x 2 wavefronts hold 2048 networks at the larger register budget
            const bool crowded = count > 2048;
            const void* fn = crowded ? (const void*)exact_wave_kernel<kL, 4> : (const void*)exact_wave_kernel<kL, 2>;
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
            if (e != hipSuccess) return e;
            if (crowded) hipLaunchKernelGGL((exact_wave_kernel<kL, 4>), dim3(count), dim3(64), lds_bytes, s, p, dev_multi);
            else hipLaunchKernelGGL((exact_wave_kernel<kL, 2>), dim3(count), dim3(64), lds_bytes, s, p, dev_multi);
            return hipGetLastError();
        }
    if constexpr (kL > 0 && kLds)
        if (threads == 64 && narrow) return launch_sized<kLds, kDrop, kL, 64>(p, dev_multi, count, threads, lds_bytes, s);
    return launch_sized<kLds, kDrop, kL, 1024>(p, dev_multi, count, threads, lds_bytes, s);
}

template <bool kLds, bool kDrop>
static hipError_t launch_variant(const ExactLaunch& p, const ExactPointers* dev_multi, int count, int threads,
                                 size_t lds_bytes, hipStream_t s)
{
    // the common depths have their own instantiation (one and two hidden layers)
    if (kLds && p.n_layers == 2) return launch_layers<kLds, kDrop, 2>(p, dev_multi, count, threads, lds_bytes, s);
    if (kLds && p.n_layers == 3) return launch_layers<kLds, kDrop, 3>(p, dev_multi, count, threads, lds_bytes, s);
    return launch_layers<kLds, kDrop, 0>(p, dev_multi, count, threads, lds_bytes, s);
}

hipError_t ghip_launch_exact(const ExactLaunch& p, const ExactPointers* dev_multi, int count, int threads, size_t lds_bytes,
                             hipStream_t s)
{
    if (p.dropout) {
        if (p.state_in_lds) return launch_variant<true, true>(p, dev_multi, count, threads, lds_bytes, s);
        return launch_variant<false, true>(p, dev_multi, count, threads, lds_bytes, s);
    }
    if (p.state_in_lds) return launch_variant<true, false>(p, dev_multi, count, threads, lds_bytes, s);
    return launch_variant<false, false>(p, dev_multi, count, threads, lds_bytes, s);
}

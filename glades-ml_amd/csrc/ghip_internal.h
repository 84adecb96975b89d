// Internal declarations shared by the HIP translation units of libglades_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/glades_hip.h"
#include "libm_exact.h"

#define GHIP_OUTLIER 0.046f  // knee of RELU / LEAKY in the reference (gmath.h:35, gmath.cpp:62-82)

// ---------------------------------------------------------------- element-wise device functions

// Reference GMath::squash (gmath.cpp:22-101).  kPrecise selects the routines that return, for every
// input, the float the reference's C library returns (libm_exact.h): exact mode is sequential and
// order-faithful, so with them nothing is left that could differ from the CPU path.  The fast fp32
// device routines serve the batched kernels.
template <bool kPrecise>
__device__ __forceinline__ float ghip_tanh(float z)
{
    if (kPrecise) return glm_tanhf(z);
    return tanhf(z);
}
// exp_tab: the table of glm_expf_tab where the caller keeps a copy close by (LDS), or NULL
template <bool kPrecise>
__device__ __forceinline__ float ghip_exp(float z, const uint64_t* exp_tab = nullptr)
{
    if (kPrecise) return exp_tab ? glm_expf_tab(z, exp_tab) : glm_expf(z);
    return expf(z);
}
template <bool kPrecise>
__device__ __forceinline__ float ghip_log(float z)
{
    if (kPrecise) return glm_logf(z);
    return logf(z);
}

template <bool kPrecise>
__device__ __forceinline__ float ghip_squash(float z, int act, float p, const uint64_t* exp_tab = nullptr)
{
    switch (act) {
    case GHIP_TANH: return ghip_tanh<kPrecise>(z);
    case GHIP_TANHP:
        if (z > 1.0f - p) return 1.0f;
        if (z < p - 1.0f) return -1.0f;
        return ghip_tanh<kPrecise>(z);
    case GHIP_SIGMOID: return __fdiv_rn(1.0f, __fadd_rn(1.0f, ghip_exp<kPrecise>(-z, exp_tab)));
    case GHIP_SIGMOIDP:
        if (z < p) return 0.01f;
        if (z > 1.0f - p) return 0.99f;
        return __fdiv_rn(1.0f, __fadd_rn(1.0f, ghip_exp<kPrecise>(-z, exp_tab)));
    case GHIP_RELU: return (z < GHIP_OUTLIER) ? 0.0f : z;
    case GHIP_LEAKY: return (z < GHIP_OUTLIER) ? __fmul_rn(p, z) : z;
    case GHIP_LINEAR: return __fmul_rn(p, z);
    case GHIP_STEP: return (z < p) ? 0.0f : 1.0f;
    }
    return 0.0f;
}

// Reference GMath::activationErrDer (gmath.cpp:182-245), in terms of the activation's output.
__device__ __forceinline__ float ghip_act_der_ref(float a, int act, float p)
{
    switch (act) {
    case GHIP_TANH:
    case GHIP_TANHP: return __fsub_rn(1.0f, __fmul_rn(a, a));
    case GHIP_SIGMOID:
    case GHIP_SIGMOIDP: return __fmul_rn(a, __fsub_rn(1.0f, a));
    case GHIP_RELU: return (a > 0.0f) ? 1.0f : 0.0f;
    case GHIP_LEAKY:
        if (a > 0.0f) return 1.0f;
        return (p < 0) ? p : -p;
    case GHIP_LINEAR: return p;
    case GHIP_STEP: return 0.0f;
    }
    return 1.0f;
}

// Canonical-mode derivative: the layer's own parameter, LEAKY slope = +param.
__device__ __forceinline__ float ghip_act_der_canon(float a, int act, float p)
{
    if (act == GHIP_LEAKY) return (a > 0.0f) ? 1.0f : p;
    return ghip_act_der_ref(a, act, p);
}

// Reference GMath::outputNodeCost (gmath.cpp:272-321)
template <bool kPrecise>
__device__ __forceinline__ float ghip_cost(float e, float p, float data_size, int cost)
{
    float c = 0.0f;
    switch (cost) {
    case GHIP_REGRESSION: {
        float d = __fsub_rn(e, p);
        c = __fdiv_rn(__fmul_rn(d, d), data_size);
        break;
    }
    case GHIP_CLASSIFICATION: {
        float t0 = __fmul_rn(e, ghip_log<kPrecise>(p));
        float t1 = __fmul_rn(__fsub_rn(1.0f, e), ghip_log<kPrecise>(__fsub_rn(1.0f, p)));
        c = __fdiv_rn(-__fadd_rn(t0, t1), data_size);
        break;
    }
    case GHIP_KL: c = __fdiv_rn(ghip_log<kPrecise>(__fdiv_rn(e, p)), data_size); break;
    }
    return c;
}

// Reference GMath::costErrDer (gmath.cpp:323-353)
__device__ __forceinline__ float ghip_cost_der(float e, float p, int cost)
{
    switch (cost) {
    case GHIP_REGRESSION: return __fmul_rn(2.0f, __fsub_rn(p, e));
    case GHIP_CLASSIFICATION:
        return __fdiv_rn(__fsub_rn(p, e), __fmul_rn(__fsub_rn(1.0f, p), p));
    case GHIP_KL: return -__fdiv_rn(e, p);
    }
    return 1.0f;
}

// Reference accuracy contribution (network.cpp:541-547 + gmath.cpp:252-270)
__device__ __forceinline__ float ghip_accuracy_term(float pred, float expect)
{
    float pe = __fsub_rn(pred, expect);
    if (pe < 0.0f) pe = -pe;
    if (pe > 1.0f) pe = 1.0f;
    float acc = __fmul_rn(__fsub_rn(1.0f, pe), 100.0f);
    return acc < 0.0f ? 0.0f : acc;
}

// Overall class metrics of the reference's confusion matrix (ML/GMath/cmatrix.cpp:100-132 for the
// per-class counts, :139-265 for the ratios): M is n x n, row = expected class, column = predicted.
// falsePositive[c] / falseNegative[r] collect the off-diagonal cells of column c / row r;
// truePositive[i] is the diagonal cell; trueNegative[i] is the sum of the OTHER classes' diagonal
// cells only.  Ratios are float, the overall figure is the mean over classes in class order (0/0
// gives NaN and stays).  out[0..4] = accuracy, precision, recall, specificity, F1 as fractions.
// Meant for one lane and a small n: O(n^2) reads.
__device__ inline void ghip_cmatrix_overall(const int* M, int n, float* out)
{
    // device-scope atomic loads: the counters are bumped with atomics, which live in L2
    auto at = [&](int idx) { return __hip_atomic_load(M + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
    int diag_sum = 0;
    for (int i = 0; i < n; ++i) diag_sum += at(i * n + i);
    float acc = 0.0f, pre = 0.0f, rec = 0.0f, spe = 0.0f, f1 = 0.0f;
    for (int i = 0; i < n; ++i) {
        int fp = 0, fn = 0;
        for (int k = 0; k < n; ++k)
            if (k != i) { fp += at(k * n + i); fn += at(i * n + k); }
        const int tp = at(i * n + i), tn = diag_sum - tp;
        const float truth = (float)(tp + tn), untruth = (float)(fp + fn);
        acc = __fadd_rn(acc, __fdiv_rn(truth, __fadd_rn(truth, untruth)));
        const float cp = __fdiv_rn((float)tp, (float)(tp + fp));
        const float cr = __fdiv_rn((float)tp, (float)(tp + fn));
        pre = __fadd_rn(pre, cp);
        rec = __fadd_rn(rec, cr);
        spe = __fadd_rn(spe, __fdiv_rn((float)tn, (float)(tn + fp)));
        f1 = __fadd_rn(f1, __fdiv_rn(__fmul_rn(__fmul_rn(2.0f, cr), cp), __fadd_rn(cr, cp)));
    }
    const float nn = (float)n;
    out[0] = __fdiv_rn(acc, nn); out[1] = __fdiv_rn(pre, nn); out[2] = __fdiv_rn(rec, nn);
    out[3] = __fdiv_rn(spe, nn); out[4] = __fdiv_rn(f1, nn);
}

// ---------------------------------------------------------------- bf16 helpers (bit level)

__device__ __forceinline__ uint16_t ghip_f32_to_bf16(float x)
{
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
// two at once with the hardware conversion (round to nearest even): low half = a, high half = b
__device__ __forceinline__ uint32_t ghip_f32x2_to_bf16x2(float a, float b)
{
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ float ghip_bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// OCP e4m3 (finite only) encode, round-to-nearest-even, saturating at 448.
__device__ __forceinline__ uint8_t ghip_f32_to_e4m3(float x)
{
    uint32_t u = __float_as_uint(x);
    uint8_t sign = (uint8_t)((u >> 31) << 7);
    float a = fabsf(x);
    if (a != a) return (uint8_t)(sign | 0x7f);
    if (a >= 448.0f) return (uint8_t)(sign | 0x7e);
    if (a < 0.015625f) return (uint8_t)(sign | (int)rintf(a * 512.0f));
    uint32_t ua = __float_as_uint(a);
    int ex = (int)(ua >> 23) - 127;
    // keep 3 mantissa bits, RNE on the 20 dropped bits
    uint32_t mant = ua & 0x7fffffu;
    uint32_t q = mant >> 20;
    uint32_t rem = mant & 0xfffffu;
    if (rem > 0x80000u || (rem == 0x80000u && (q & 1u))) ++q;
    if (q == 8) { q = 0; ++ex; }
    int code = ((ex + 7) << 3) | (int)q;
    if (code > 0x7e) code = 0x7e;
    return (uint8_t)(sign | code);
}

// Block-scaled e4m3 ("MX": an E8M0 power-of-two scale per 32 consecutive elements of a row).  The scale of a
// block is the power of two that brings its largest magnitude into (224, 448], the top binade of e4m3, so
// nothing saturates and the largest element keeps all three mantissa bits: with that magnitude
// 2^(E-127) (1 + M/128) in bf16 (bits amax15 = E << 7 | M) the E8M0 byte is E - 8, one more if 1 + M/128 > 1.75
// (256 (1 + M/128) would pass 448), never below 0 (magnitudes under 2^-119 then land under 256).
__device__ __forceinline__ int ghip_mx_scale_byte(unsigned int amax15)
{
    const int eb = (int)(amax15 >> 7) - 8 + ((amax15 & 0x7fu) > 96u ? 1 : 0);
    return eb < 0 ? 0 : eb;
}
// codes of 8 bf16 values (two per dword) over the scale 2^(eb - 127): the hardware's round-to-nearest-even conversion
__device__ __forceinline__ uint2 ghip_mx_quant8(unsigned int u0, unsigned int u1, unsigned int u2, unsigned int u3, int eb)
{
    const float inv = __uint_as_float((unsigned int)(254 - eb) << 23);   // 2^(127 - eb), exact
    uint2 q;
    int p = __builtin_amdgcn_cvt_pk_fp8_f32(__uint_as_float(u0 << 16) * inv, __uint_as_float(u0 & 0xffff0000u) * inv, 0, false);
    p = __builtin_amdgcn_cvt_pk_fp8_f32(__uint_as_float(u1 << 16) * inv, __uint_as_float(u1 & 0xffff0000u) * inv, p, true);
    q.x = (unsigned int)p;
    p = __builtin_amdgcn_cvt_pk_fp8_f32(__uint_as_float(u2 << 16) * inv, __uint_as_float(u2 & 0xffff0000u) * inv, 0, false);
    p = __builtin_amdgcn_cvt_pk_fp8_f32(__uint_as_float(u3 << 16) * inv, __uint_as_float(u3 & 0xffff0000u) * inv, p, true);
    q.y = (unsigned int)p;
    return q;
}
// largest 15-bit magnitude among 8 bf16 values (bf16 magnitudes order like their bit patterns)
__device__ __forceinline__ unsigned int ghip_bf16x8_amax15(unsigned int u0, unsigned int u1, unsigned int u2, unsigned int u3)
{
    unsigned int m = 0;
    const unsigned int w[4] = {u0, u1, u2, u3};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const unsigned int lo = w[d] & 0x7fffu, hi = (w[d] >> 16) & 0x7fffu;
        m = m > lo ? m : lo;
        m = m > hi ? m : hi;
    }
    return m;
}

// ---------------------------------------------------------------- exact mode (exact_kernel.hip)

// What differs between the networks of one launch: parameters, state and results.
struct ExactPointers {
    float* W;      // [state_floats] padded weights (global copy, read at start, written at end)
    float* wsum;   // pending-delta running sums
    float* wlast;  // last pending delta
    float* bias;   // [GHIP_MAX_LAYERS] scalar layer biases
    float* preds;  // n_rows x n_out or NULL
    float* metrics;// per epoch: loss, accuracy, correct
    int*   epochs_run;
    int*   cm;            // n_out x n_out confusion counters of the running epoch, or NULL
    float* class_metrics; // per epoch: overall accuracy, precision, recall, specificity, F1 (NULL with cm)
    // dropout launches only
    const unsigned char* masks; // n_epochs x n_rows x aoff[n_layers] flags (1 = dropped) or NULL = none dropped
    int*   wcnt;                // [state_floats] number of pending deltas per edge
    float* errder;              // [node_floats] the nodes' error accumulators between rows
};

struct ExactLaunch {
    int   n_layers;
    int   sizes[GHIP_MAX_LAYERS + 1];
    int   ld[GHIP_MAX_LAYERS];      // padded row stride of layer l in the state arrays (odd)
    int   woff[GHIP_MAX_LAYERS];    // offset of layer l in the state arrays
    int   aoff[GHIP_MAX_LAYERS + 1];// offset of layer l's node values in the node arrays
    int   tw_log2[GHIP_MAX_LAYERS]; // log2 of the lane group width used to walk layer l's edges
    float lr[GHIP_MAX_LAYERS], mom[GHIP_MAX_LAYERS], wd1[GHIP_MAX_LAYERS], wd2[GHIP_MAX_LAYERS];
    int   act[GHIP_MAX_LAYERS];
    float act_param[GHIP_MAX_LAYERS];
    int   mb, cost, bias_mode;
    int   state_floats;             // total padded floats of one state array
    int   node_floats;              // total node values
    int   n_epochs, train;
    float stop_accuracy;
    long long n_rows;
    const float* X;
    const float* Y;
    ExactPointers ptr;  // this network's own arrays (a launch over several networks passes a list instead)
    int    state_in_lds;
    int    metric_cap;  // outputs held back before their cost / accuracy terms are computed (>= sizes[n_layers])
    int    dropout;     // run the instantiation that reads flags and keeps accumulators / window lengths
};

// count workgroups = count networks; dev_multi (device memory, count entries) or NULL for the one network in p.ptr
hipError_t ghip_launch_exact(const ExactLaunch& p, const ExactPointers* dev_multi, int count, int threads, size_t lds_bytes,
                             hipStream_t s);
size_t ghip_exact_lds_bytes(const ExactLaunch& p, bool state_in_lds, bool dropout);
// fn 0 squash(a; kind, param), 1 activationErrDer(a; kind, param), 2 outputNodeCost(expected a, predicted b; cost
// kind, dataSize param), 3 costErrDer(expected a, predicted b; cost kind): device arrays of n floats
hipError_t ghip_launch_bias_chain_eval(int kind, int ni, const float* a, const float* b, float* out, long long n, hipStream_t s);
hipError_t ghip_launch_gmath_eval(int fn, int kind, float param, const float* a, const float* b, float* out, long long n,
                                  hipStream_t s);

// ---------------------------------------------------------------- canonical kernels

// C[M][N] (+epilogue) = A x B, fp32 via MFMA.  a_kmajor: A is stored [K][M] (else [M][K]);
// b_kmajor: B is stored [K][N] (else [N][K]).
enum GemmEpilogue {
    EPI_STORE = 0,        // C = acc * alpha
    EPI_BIAS_ACT = 1,     // C = squash(acc + bias[n])
    EPI_MUL_DER = 2,      // C = acc * act_der(aux[m][n])
    EPI_SGD = 3,          // C is the weight matrix: g = acc*alpha + wd1*sign(W) + wd2*W; d = lr*g + mom*V; V = d; W -= d
};
struct GemmF32Args {
    const float* A; const float* B; float* C;
    int M, N, K;
    int lda, ldb, ldc;
    int a_kmajor, b_kmajor;
    int epilogue;
    const float* bias;   // EPI_BIAS_ACT (may be NULL)
    const float* aux;    // EPI_MUL_DER: activations [M][N], ld = ldc
    int act; float act_param;
    float alpha;
    // EPI_SGD: momentum of C, hyper-parameters; with bias_w the kernel also sums its A operand over K
    // (A = delta^T: the bias gradient, times alpha) and updates bias_w / bias_v[M] the same way, no decay
    float* V;
    float lr, mom, wd1, wd2;
    float* bias_w; float* bias_v;
};
hipError_t ghip_gemm_f32(const GemmF32Args& a, hipStream_t s);
// out[r][c] = drop[r * ld_drop + c] ? 0 : X[r][c] (out may be X): a batch's rows, activations or deltas under its
// dropout flags
hipError_t ghip_mask_rows(const float* X, const uint8_t* drop, int ld_drop, int rows, int cols, float* out, hipStream_t s);
// up to GHIP_GEMM_F32_GROUP_MAX independent products in one launch where they run the same instantiation
// (tile height, operand orientations, alignment class), else one launch each
#define GHIP_GEMM_F32_GROUP_MAX 8
struct GemmF32Group { GemmF32Args p[GHIP_GEMM_F32_GROUP_MAX]; int first[GHIP_GEMM_F32_GROUP_MAX + 1]; int gx[GHIP_GEMM_F32_GROUP_MAX]; int count; };
hipError_t ghip_gemm_f32_group(const GemmF32Args* a, int count, hipStream_t s);

// ---------------------------------------------------------------- narrow fp32 output layer (narrow_out.hip)
// The products of a layer with at most 16 outputs as streams over its input activations H [B][ni]
// (ni a multiple of 4, rows 16-byte aligned) instead of padded GEMM tiles.
struct NarrowOutArgs {
    const float* H; const float* W; int B, ni, no;
    // forward: P [B][no] = squash(H W^T + bias)
    const float* bias; float* P; int act; float act_param;
    // backward: D [B][no] deltas of this layer; E [B][ni] = (D W) .* f'(H) or NULL (no layer below);
    // part [chunks][no][ni] receives the gradient summed over each chunk of rows_per_chunk rows
    const float* D; float* E; int act_below; float act_below_param;
    float* part; int chunks, rows_per_chunk;
    // metric_part [chunks][4] doubles: loss / accuracy / correct sums of each chunk, written by ghip_narrow_train;
    // ghip_narrow_update adds them (in chunk order) to metric_acc[0..2]
    double* metric_part; double* metric_acc;
    // update: G = sum of the chunks; the EPI_SGD step on Wm / V [no][ni] and on bias_w / bias_v [no] (may be NULL)
    float* Wm; float* V; float lr, mom, wd1, wd2, alpha; float* bias_w; float* bias_v;
};
bool ghip_narrow_out_ok(int no, int ni);
void ghip_narrow_out_chunks(int B, int* chunks, int* rows_per_chunk);
hipError_t ghip_narrow_forward(const NarrowOutArgs& a, hipStream_t s);

// softmax / output delta / metrics for fp32 logits-or-activations P[B][n] against Y[B][n].
// If act == SOFTMAX, P holds pre-softmax logits and is overwritten with probabilities.
// D (fp32, may be NULL) receives dL/dz; Dbf/DbfT (bf16 [B][n] and [n][B], may be NULL) too.
// acc: 4 doubles {loss sum, accuracy sum, correct count, unused}, atomically accumulated.
struct DeltaArgs {
    float* P; const float* Y; float* D; uint16_t* Dbf; uint16_t* DbfT;
    int B, n, ldp, ldy;
    int ldd;       // row pitch of Dbf in elements (0: n): the bf16 deltas of a padded low-precision network
    int act; float act_param; int cost;
    double* acc;
    double* acc_clear;  // 4 doubles set to zero by this launch (the next launch's accumulators), or NULL
    int* cm;       // n x n confusion counters (row expected, column predicted) or NULL
    int store_p;   // write the activated outputs (softmax probabilities) back into P
};
hipError_t ghip_output_delta(const DeltaArgs& a, hipStream_t s);
// forward of the narrow output layer, output delta / loss / metrics (as ghip_output_delta; da.P = a.P,
// da.D = the deltas a.D reads) and backward in one launch; ghip_narrow_update finishes the step
hipError_t ghip_narrow_train(const NarrowOutArgs& a, const DeltaArgs& da, hipStream_t s);
hipError_t ghip_narrow_update(const NarrowOutArgs& a, hipStream_t s);

// ---------------------------------------------------------------- narrow networks as one persistent workgroup (canon_narrow.hip)
// Canonical fp32 training or evaluation of a network whose layers are all at most 64 wide: n_epochs passes over
// rows [0, n_rows) of X / Y in batches of `batch` (the last one shorter), parameters and momentum read from and
// written back to W / b / vW / vb, per epoch four doubles in `metrics` (loss sum, accuracy-term sum, rows whose
// class agrees, 0) and the number of epochs run in *epochs_run (fewer than n_epochs if the mean accuracy term
// reached stop_accuracy > 0).  ghip_canon_narrow_plan fills the layout fields; the caller fills the rest.
struct CanonNarrowArgs {
    int   n_layers;
    int   sizes[GHIP_MAX_LAYERS + 1];
    int   act[GHIP_MAX_LAYERS]; float act_param[GHIP_MAX_LAYERS];
    float lr[GHIP_MAX_LAYERS], mom[GHIP_MAX_LAYERS], wd1[GHIP_MAX_LAYERS], wd2[GHIP_MAX_LAYERS];
    int   cost;
    const float* X; const float* Y; long long n_rows; int batch, n_epochs, train; float stop_accuracy;
    float* W[GHIP_MAX_LAYERS]; float* b[GHIP_MAX_LAYERS]; float* vW[GHIP_MAX_LAYERS]; float* vb[GHIP_MAX_LAYERS];
    int*  cm; int reset_cm;       // confusion counters (or NULL); cleared at the head of every epoch if reset_cm
    double* metrics; int* epochs_run;
    double* clear4;               // four doubles the launch sets to zero (the next metrics launch's accumulators), or NULL
    // layout of the workgroup's LDS block, in floats
    int rows_per_chunk, rc_shift;   // a power of two and its logarithm
    int wave_per_weight;            // gradient sums: a wavefront per weight (small networks) or a thread per weight
    int offW[GHIP_MAX_LAYERS], offB[GHIP_MAX_LAYERS], offVW[GHIP_MAX_LAYERS], offVB[GHIP_MAX_LAYERS], offG[GHIP_MAX_LAYERS], offGB[GHIP_MAX_LAYERS];
    int offA[GHIP_MAX_LAYERS + 1], offD[GHIP_MAX_LAYERS + 1], pitchA[GHIP_MAX_LAYERS + 1];
    int offY;                       // a chunk's targets, or -1 if they do not fit
};
bool ghip_canon_narrow_plan(const int* sizes, int n_layers, int train, CanonNarrowArgs* out, size_t* lds_bytes);
hipError_t ghip_canon_narrow_run(const CanonNarrowArgs& a, size_t lds_bytes, hipStream_t s);

hipError_t ghip_fill_f32(float* p, long long n, float v, hipStream_t s);
hipError_t ghip_fill_f64(double* p, long long n, double v, hipStream_t s);

// ---------------------------------------------------------------- low precision (gemm_lp.hip)

enum LpEpilogue {
    LP_FWD_ACT = 0,     // out bf16 [M][N] (+ transposed copy [N][M]) = squash(acc + bias[n])
    LP_FWD_F32 = 1,     // out fp32 [M][N] = squash(acc + bias[n])   (output layer; softmax logits use LINEAR 1)
    LP_DGRAD = 2,       // out bf16 (+T) = acc * act_der(aux bf16 [M][N])
    LP_WGRAD_SGD = 3,   // acc = batch-summed gradient tile [M=n_out][N=n_in]: fused update of
                        // fp32 master + momentum, writes bf16 W [M][N] and W^T [N][M]
    LP_FP8_ACT = 4,     // fp8 inference: v = squash(acc * rs[m] * cs[n]); bf16 out + row amax
    LP_FP8_F32 = 5,     // fp8 inference last layer: fp32 out = squash(acc * rs[m] * cs[n])
    // The same two with block-scaled activations (the MX form CDNA4's scaled MFMA takes): A comes with an E8M0
    // scale per row and 32 elements of K (a_scale) instead of one fp32 scale per row, and LP_FP8_ACT_MX leaves
    // its result as the next layer's A operand, e4m3 codes [M][N] + scales (out_scale), quantised in the epilogue.
    LP_FP8_ACT_MX = 6,  // v = squash(acc * cs[n]) -> bf16 rounding -> codes + block scales
    LP_FP8_F32_MX = 7,  // fp32 out = squash(acc * cs[n])
    LP_DGRAD_MASK = 8   // LP_DGRAD for a step derivative, from the sign bits in mask_in (chosen by ghip_gemm_lp; callers ask for LP_DGRAD)
};
struct GemmLpArgs {
    const void* A; const void* B;    // [M][K], [N][K], K contiguous; bf16 or e4m3
    int M, N, K;
    int lda, ldb;                     // row pitches of A and B in elements (0: K)
    // K-blocked operands: bytes between one stage's 128 bytes of a row and the next stage's (0: they follow
    // each other in the row).  With a pitch of 128 bytes and kstride = rows x 128 an operand lies as
    // [K bytes / 128][rows][128 bytes]: every stage of a tile is ONE contiguous block of memory instead of
    // 256 lines a row pitch apart.  The weight gradient's operands (activations and deltas transposed, K =
    // the batch) are kept that way: they come from HBM, where scattered lines cost a DRAM page each.
    long long kstrideA, kstrideB;
    int outT_blocked;                 // outT is written K-blocked for the product that will read it: [M / 64][N][64]
    int n_valid;                      // LP_FWD_ACT / LP_FP8_ACT: columns from here on are padding and are stored as 0 (0: none)
    int fp8;                          // 0: bf16 operands, 1: e4m3 operands
    int epilogue;
    void* out; void* outT;            // see LpEpilogue; outT may be NULL, and out for LP_DGRAD with outT (only the transposed copy is written)
    const float* bias;                // [N] or NULL
    const uint16_t* aux;              // LP_DGRAD: activations bf16 [M][N]
    // LP_FWD_ACT may leave, and LP_DGRAD take instead of aux, the signs of the stored activations (1 = positive), a bit
    // per element in the order of the computing workgroup's accumulators: M * N / 8 bytes.  For activations whose
    // derivative is a step (ReLU, leaky ReLU); both products then have to run the same tiling of [M][N].
    unsigned int* mask_out; const unsigned int* mask_in;
    float* colsum;                    // LP_DGRAD: if set, [M / tile_m][N] column sums of the stored deltas per tile row
    int act; float act_param;   // resolved into `ap` by ghip_gemm_lp
    struct ActForm {
        // forward:  v = z < thr ? a0*z + b0 : a1*z + b1;  if (trans) v = ta / (1 + exp(-tk*z)) + tb;
        //           v = z < clo ? vlo : v;  v = z > chi ? vhi : v
        float thr, a0, b0, a1, b1, tk, ta, tb, clo, vlo, chi, vhi;
        int trans;
        int plain;  // no transcendental part and no clamps: the first line is the whole activation
        // derivative in the output a:  step ? (a > 0 ? dhi : dlo) : c0 + c1*a + c2*a*a
        int step; float dhi, dlo, c0, c1, c2;
    } ap;
    // LP_WGRAD_SGD
    float* master; float* mom; float lr, momf, wd1, wd2, gscale;
    // fp8
    const float* row_scale; const float* col_scale; unsigned int* row_amax_bits;
    // block-scaled e4m3 activations: E8M0 bytes, stage-major: dword [k / 128][row] holds the scales of the four
    // 32-element blocks k..k+127 of that row; ld = dwords from one stage's rows to the next's (>= rows)
    const unsigned int* a_scale; int ld_scale;
    unsigned int* out_scale; int ld_out_scale;
};
hipError_t ghip_gemm_lp(const GemmLpArgs& a, hipStream_t s);
// The 256 x 256-tile weight gradients (LP_WGRAD_SGD, bf16) of up to GHIP_GEMM_LP_GROUP_MAX layers as one launch.
// ghip_gemm_lp_wgrad_plan lays out the launch's schedule for products of M[i] x N[i] outputs into `sched` (host
// memory, `cap` entries) and returns the number of workgroups, or -1 if a product takes the smaller tile; the
// launch takes that schedule in device memory.
#define GHIP_GEMM_LP_GROUP_MAX 8
int ghip_gemm_lp_wgrad_plan(const int* M, const int* N, int count, unsigned int* sched, int cap);
hipError_t ghip_gemm_lp_wgrad_group(const GemmLpArgs* a, int count, const unsigned int* dev_sched, int blocks, hipStream_t s);
bool ghip_gemm_lp_shape_ok(int M, int N, int K, int fp8);
int ghip_gemm_lp_tile_m(int M, int N);  // rows per tile the launcher picks for this product

// Transposed bf16 copies are K-blocked for the weight-gradient product (see GemmLpArgs::kstrideA):
// element (row r, column c) of a [rows][cols] source lies at ((r / 64) * cols + c) * 64 + r % 64 of dstT,
// i.e. dstT is [ceil(rows / 64)][cols][64].
hipError_t ghip_f32_to_bf16_2d(const float* src, uint16_t* dst, uint16_t* dstT, int rows, int cols, hipStream_t s);
// the same from a source of src_rows x src_cols (row pitch src_cols) into destinations of rows x cols: what lies
// outside the source is zero (the padded copy of a table)
hipError_t ghip_f32_to_bf16_2d_pad(const float* src, int src_rows, int src_cols, uint16_t* dst, uint16_t* dstT, int rows, int cols, hipStream_t s);
hipError_t ghip_bf16_transpose(const uint16_t* src, uint16_t* dstT, int rows, int cols, hipStream_t s);
// All bias updates of a bf16 step in one launch (a launch of its own per layer, between the products, costs the
// step its few microseconds plus the gap each time): per layer either the partial column sums the
// back-propagation product left ([tiles][n], a thread per channel adds them in order) or, for the output layer, the
// transposed deltas, K-blocked [rows / 64][n][64] (a wavefront per channel; rows past the batch are zero).
struct BiasStepArgs {
    struct Entry {
        const float* part; int tiles;      // partial sums [tiles][n], or NULL
        const uint16_t* DT; int rows;      // else delta^T, K-blocked, of `rows` batch rows (a multiple of 64)
        int n, batch;                      // channels; the divisor of the mean
        float* bias; float* vb; float lr, mom;
        int first_block;                   // this entry's first workgroup in the grid
    } e[GHIP_MAX_LAYERS];
    int count, blocks;
};
hipError_t ghip_bias_update_step(BiasStepArgs& a, hipStream_t s);   // fills first_block / blocks, launches
// per-row e4m3 quantisation: src fp32/bf16 [rows][cols]; scale = amax/448 (1 if row is zero).
// amax_bits: if non-NULL the row amax is taken from there (uint bits of a non-negative float)
// instead of being reduced from the row; with consume_amax the entry is set back to zero once read
// (ready for the next GEMM epilogue's atomic maxima).
hipError_t ghip_quant_rows_e4m3(const void* src, int src_is_bf16, int rows, int cols, uint8_t* q,
                                float* scale, unsigned int* amax_bits, int consume_amax, hipStream_t s);
hipError_t ghip_fill_u32(unsigned int* p, long long n, unsigned int v, hipStream_t s);
// Block-scaled e4m3 quantisation of bf16 rows (cols a multiple of 128, rows 16-byte aligned): codes [rows][cols]
// and the E8M0 scales stage-major, dword [c / 128][row] = the four blocks c..c+127 of that row (GemmLpArgs::a_scale)
hipError_t ghip_quant_rows_mx(const uint16_t* src, int rows, int cols, uint8_t* q, unsigned int* scale, int ld_scale, hipStream_t s);

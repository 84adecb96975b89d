// C ABI of libglades_hip.so (declared in include/glades_hip.h): the device-side network object
// and the host logic that strings the kernels together.

#include "ghip_internal.h"

#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <string>
#include <vector>

namespace {

thread_local std::string g_err;

int fail(int code, const char* fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_err = buf;
    return code;
}

#define HIP_TRY(expr)                                                                         \
    do {                                                                                      \
        hipError_t e__ = (expr);                                                              \
        if (e__ != hipSuccess)                                                                \
            return fail(GHIP_EHIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e__), __FILE__, __LINE__); \
    } while (0)

int g_device = -1;
int g_max_lds = 65536;

// Device memory of ghip_forward_noalloc, the one entry point that must not allocate: a header of
// accumulators (the softmax pass adds its row sums somewhere) and two halves that the hidden layers'
// activations alternate between.  Every GPU holds its own copy of the array until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress: the address kernels and
// copies get is the one that call returned for the current device, kept in g_scratch_ptr.
constexpr size_t kScratchHeader = 256;
constexpr size_t kScratchHalf = (size_t)GHIP_NOALLOC_MAX_ACTIVATIONS * sizeof(float);
constexpr size_t kScratchBytes = kScratchHeader + 2 * kScratchHalf;
constexpr int kMaxDevices = 16;
unsigned char* g_scratch_ptr[kMaxDevices] = {};

struct ProfRec { std::string name; hipEvent_t a, b; };
struct ProfAgg { std::string name; double ms; int64_t n; };

}  // namespace

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {

// Address of this device's copy of `scratch` (resolved once per device, with that device current).
int scratch_for_device(int device, unsigned char** out)
{
    if (device < 0 || device >= kMaxDevices) return fail(GHIP_EINVAL, "device %d: at most %d devices are supported", device, kMaxDevices);
    if (!g_scratch_ptr[device]) {
        void* p = nullptr;
        HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(GHIP_EHIP, "hipGetSymbolAddress returned no address for the scratch array");
        g_scratch_ptr[device] = (unsigned char*)p;
    }
    *out = g_scratch_ptr[device];
    return 0;
}

}  // namespace

struct ghip_net {
    ghip_net_spec spec;
    hipStream_t stream = nullptr;
    int L = 0;
    // Layer widths as the device holds them.  The bf16 / e4m3 products work on tiles of 256: there every width is
    // rounded up to a multiple of 256 and the units added are kept at zero (zero weights, zero bias, activation
    // stored as 0), so they change no result.  fp32: the widths of the spec.
    int ps[GHIP_MAX_LAYERS + 1] = {};
    int64_t table_rows = 0;   // rows the bf16 table holds: those of the dataset plus zero rows a padded last batch may read
    // dataset
    const float* dX = nullptr;
    const float* dY = nullptr;
    float* ownX = nullptr;
    float* ownY = nullptr;
    int64_t n_rows = 0;
    uint16_t* Xbf = nullptr;  // bf16 copy of the table (BF16 / FP8_INFER)
    uint16_t* XbfT = nullptr; // BF16 training: the same table transposed and K-blocked, [rows / 64][inputs][64]: the planes of a
                              // batch that starts on a multiple of 64 rows are the B operand of the first layer's weight
                              // gradient as they lie (nullptr: the batch is transposed per step)
    // exact
    ExactLaunch ex;
    int ex_threads = 64;
    size_t ex_lds = 0;
    float *exW = nullptr, *exSum = nullptr, *exLast = nullptr, *exBias = nullptr, *exPreds = nullptr;
    ghip_metrics* exMetrics = nullptr;
    int exMetricsCap = 0;
    int64_t exPredsCap = 0;
    int* exEpochs = nullptr;
    // dropout: flags of the coming epochs, window lengths, error accumulators; once a run has used
    // flags the accumulators may be non-zero between rows, so every later run keeps them too
    unsigned char* exMasks = nullptr;
    int exMaskEpochs = 0;
    int64_t exMasksCap = 0;
    int* exCnt = nullptr;
    float* exErr = nullptr;
    bool exDropState = false;
    // the launches without dropout do not keep window lengths: there every edge of a layer holds
    // the same number of pending deltas, noted here and written out when dropout state is first needed
    int exUniformCnt[GHIP_MAX_LAYERS] = {};
    size_t ex_lds_drop = 0;
    int ex_drop_in_lds = 0;
    ExactPointers* exMulti = nullptr;  // pointer list of a launch over several networks (held by the first one)
    int exMultiCap = 0;
    ghip_metrics* exMultiMetrics = nullptr;  // results of such a launch, all networks side by side: one copy back
    int* exMultiEpochs = nullptr;
    size_t exMultiMetricsCap = 0;
    int* cm = nullptr;              // confusion counters (both modes), n_out x n_out
    float* exClass = nullptr;       // exact mode: 5 floats per epoch of the last call
    int exClassCap = 0, exClassRan = 0;
    // canonical fp32 state (also the master copy for BF16 / the source for FP8)
    float* W[GHIP_MAX_LAYERS] = {};
    float* b[GHIP_MAX_LAYERS] = {};
    float* vW[GHIP_MAX_LAYERS] = {};
    float* vb[GHIP_MAX_LAYERS] = {};
    float* act[GHIP_MAX_LAYERS + 1] = {};
    float* dlt[GHIP_MAX_LAYERS + 1] = {};
    double* narrowMetrics = nullptr;  // and the loss / accuracy / correct sums per chunk
    bool passAcc = false;           // canonical mode: a pass over the table is running (ghip_net_run_epoch_canonical)
    bool amax_clean = false;        // e4m3 inference: every entry of amax_bits is zero
    float* narrowPart = nullptr;  // fp32 canonical, output layer at most 16 wide: partial gradient sums per chunk of rows
    float* stageX = nullptr;
    int cap_batch = 0;
    // narrow networks as one persistent workgroup (canon_narrow.hip): layout for training / for evaluation,
    // per-epoch figures of a launch over several epochs, the number of epochs it ran
    bool narrow_fit = false;
    CanonNarrowArgs narrowTrain, narrowEval;
    size_t narrowLdsTrain = 0, narrowLdsEval = 0;
    double* narrowEpochs = nullptr;
    int narrowEpochsCap = 0;
    int* narrowRan = nullptr;
    int canon_path = GHIP_CANON_PATH_AUTO;
    // metrics of a batch: three banks of 4 doubles.  A metrics launch adds into bank accBank^1 and
    // clears the bank the launch after it will use, so no separate clearing launch is needed; bank 2
    // takes the sums of launches whose metrics nobody reads.
    double* dAcc = nullptr;
    int accBank = 0;
    int last_batch = 0;
    // bf16
    uint16_t* Wh[GHIP_MAX_LAYERS] = {};
    uint16_t* WhT[GHIP_MAX_LAYERS] = {};
    uint16_t* H[GHIP_MAX_LAYERS + 1] = {};
    uint16_t* HT[GHIP_MAX_LAYERS + 1] = {};
    uint16_t* D[GHIP_MAX_LAYERS + 1] = {};
    uint16_t* DT[GHIP_MAX_LAYERS + 1] = {};
    float* csum[GHIP_MAX_LAYERS + 1] = {};  // per-tile-row column sums of D[l] (bias gradient partials)
    unsigned int* Hmask[GHIP_MAX_LAYERS + 1] = {};  // signs of H[l] where its activation's derivative is a step (ReLU, leaky): a bit per element
    float* logits = nullptr;
    bool shadow_dirty = true;
    // grouped weight-gradient launches: the layers of each group, its schedule (device) and number of workgroups
    // canonical mode's dropout: which of the epochs of flags in exMasks the coming pass uses (ghip_net_set_dropout_masks)
    int canMaskEpoch = 0;
    int wgGroups = 0;
    int wgCount[GHIP_MAX_LAYERS] = {};
    int wgLayer[GHIP_MAX_LAYERS][GHIP_GEMM_LP_GROUP_MAX] = {};
    unsigned int* wgSched[GHIP_MAX_LAYERS] = {};
    int wgBlocks[GHIP_MAX_LAYERS] = {};
    // fp8
    uint8_t* Wq[GHIP_MAX_LAYERS] = {};
    float* wscale[GHIP_MAX_LAYERS] = {};
    uint8_t* Aq[2] = {};
    float* ascale[2] = {};
    unsigned int* amax_bits = nullptr;
    uint16_t* Hq = nullptr;
    float* out8 = nullptr;
    bool quantized = false;
    // how activations are re-quantised between layers (ghip_net_set_fp8_activation_scaling)
    int fp8_act_mode = GHIP_FP8_ACT_BLOCK32;
    unsigned int* Asc[2] = {};   // block-scaled activations: E8M0 scales, stage-major [width / 128][cap_batch] dwords
    // profiling
    bool prof = false;
    std::vector<ProfRec> recs;
    std::vector<ProfAgg> aggs;
};

namespace {

template <typename T>
int dalloc(T** p, size_t count)
{
    if (count == 0) count = 1;
    hipError_t e = hipMalloc((void**)p, count * sizeof(T));
    if (e != hipSuccess) {
        *p = nullptr;
        return fail(GHIP_ENOMEM, "hipMalloc of %zu bytes failed: %s", count * sizeof(T), hipGetErrorString(e));
    }
    return 0;
}
#define TRY(expr) do { int r__ = (expr); if (r__ != 0) return r__; } while (0)

template <typename T>
void dfree(T*& p) { if (p) { (void)hipFree((void*)p); p = nullptr; } }

struct Scope {
    ghip_net* n; const char* name; hipEvent_t a = nullptr, b = nullptr;
    Scope(ghip_net* n_, const char* nm) : n(n_), name(nm)
    {
        if (n->prof) {
            (void)hipEventCreate(&a);
            (void)hipEventCreate(&b);
            (void)hipEventRecord(a, n->stream);
        }
    }
    ~Scope()
    {
        if (n->prof) {
            (void)hipEventRecord(b, n->stream);
            n->recs.push_back(ProfRec{name, a, b});
        }
    }
};
#define LAUNCH(net, name, expr)                                                                \
    do {                                                                                       \
        hipError_t e__;                                                                        \
        { Scope sc__(net, name); e__ = (expr); }                                               \
        if (e__ != hipSuccess) return fail(GHIP_EHIP, "%s: %s", name, hipGetErrorString(e__)); \
    } while (0)

void prof_collect(ghip_net* n)
{
    if (n->recs.empty()) return;
    (void)hipStreamSynchronize(n->stream);
    for (auto& r : n->recs) {
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, r.a, r.b) == hipSuccess) {
            bool found = false;
            for (auto& g : n->aggs)
                if (g.name == r.name) { g.ms += ms; g.n += 1; found = true; break; }
            if (!found) n->aggs.push_back(ProfAgg{r.name, ms, 1});
        }
        (void)hipEventDestroy(r.a);
        (void)hipEventDestroy(r.b);
    }
    n->recs.clear();
}

int pow2ceil(int v) { int p = 1; while (p < v) p <<= 1; return p; }
int pad256(int v) { return (v + 255) / 256 * 256; }
bool low_prec(const ghip_net* n) { return n->spec.mode == GHIP_MODE_CANONICAL && n->spec.dtype != GHIP_F32; }
// rows a batch occupies on the device: low-precision products take whole tiles of 256 rows; the rows added
// carry zero deltas, so they add nothing to a gradient, and their outputs are not read
int pad_batch(const ghip_net* n, int B) { return low_prec(n) ? pad256(B) : B; }
void set_padded_sizes(ghip_net* n)
{
    for (int l = 0; l <= n->spec.n_layers; ++l) n->ps[l] = low_prec(n) ? pad256(n->spec.sizes[l]) : n->spec.sizes[l];
}
// host <-> device copy of a rows x cols fp32 matrix whose device copy has row pitch dev_ld (>= cols)
hipError_t copy_matrix(float* dev, int dev_ld, float* host, int rows, int cols, bool to_device, hipStream_t st)
{
    if (to_device) return hipMemcpy2DAsync(dev, (size_t)dev_ld * 4, host, (size_t)cols * 4, (size_t)cols * 4, rows, hipMemcpyHostToDevice, st);
    return hipMemcpy2DAsync(host, (size_t)cols * 4, dev, (size_t)dev_ld * 4, (size_t)cols * 4, rows, hipMemcpyDeviceToHost, st);
}
int ilog2(int v) { int l = 0; while ((1 << l) < v) ++l; return l; }

bool is_canon(const ghip_net* n) { return n->spec.mode == GHIP_MODE_CANONICAL; }

int check_spec(const ghip_net_spec* s)
{
    if (!s) return fail(GHIP_EINVAL, "spec is NULL");
    if (s->n_layers < 1 || s->n_layers > GHIP_MAX_LAYERS) return fail(GHIP_EINVAL, "n_layers %d out of range", s->n_layers);
    for (int l = 0; l <= s->n_layers; ++l)
        if (s->sizes[l] < 1) return fail(GHIP_EINVAL, "layer %d has size %d", l, s->sizes[l]);
    if (s->cost < GHIP_REGRESSION || s->cost > GHIP_KL) return fail(GHIP_EINVAL, "unknown cost %d", s->cost);
    for (int l = 0; l < s->n_layers; ++l) {
        if (s->act[l] < GHIP_TANH || s->act[l] > GHIP_SOFTMAX) return fail(GHIP_EINVAL, "unknown activation %d", s->act[l]);
        if (s->act[l] == GHIP_SOFTMAX && (l != s->n_layers - 1 || s->mode != GHIP_MODE_CANONICAL))
            return fail(GHIP_EINVAL, "softmax is a canonical-mode output activation only");
    }
    if (s->mode == GHIP_MODE_EXACT) {
        // BATCH_FULL = 0 would be "row % 0" in the reference (nninfo.h:63, network.cpp:647)
        if (s->batch < 1) return fail(GHIP_EINVAL, "exact mode needs batch >= 1 (full batch = number of rows)");
        if (s->dtype != GHIP_F32) return fail(GHIP_EINVAL, "exact mode is fp32 only");
    } else if (s->mode == GHIP_MODE_CANONICAL) {
        if (s->dtype < GHIP_F32 || s->dtype > GHIP_FP8_INFER) return fail(GHIP_EINVAL, "unknown dtype %d", s->dtype);
    } else {
        return fail(GHIP_EINVAL, "unknown mode %d", s->mode);
    }
    return 0;
}

int setup_exact(ghip_net* n)
{
    ExactLaunch& e = n->ex;
    memset(&e, 0, sizeof(e));
    const ghip_net_spec& s = n->spec;
    e.n_layers = s.n_layers;
    int woff = 0, aoff = 0, max_edges = 0, max_nodes = 0;
    for (int l = 0; l <= s.n_layers; ++l) {
        e.sizes[l] = s.sizes[l];
        e.aoff[l] = aoff;
        aoff += s.sizes[l];
        if (s.sizes[l] > max_nodes) max_nodes = s.sizes[l];
    }
    for (int l = 0; l < s.n_layers; ++l) {
        e.ld[l] = s.sizes[l] | 1;
        e.woff[l] = woff;
        woff += e.ld[l] * s.sizes[l + 1];
        int edges = s.sizes[l] * s.sizes[l + 1];
        if (edges > max_edges) max_edges = edges;
        e.lr[l] = s.lr[l]; e.mom[l] = s.mom[l]; e.wd1[l] = s.wd1[l]; e.wd2[l] = s.wd2[l];
        e.act[l] = s.act[l]; e.act_param[l] = s.act_param[l];
    }
    e.state_floats = woff;
    e.node_floats = aoff;
    e.mb = s.batch; e.cost = s.cost; e.bias_mode = s.bias_mode;
    e.metric_cap = s.sizes[s.n_layers] > 128 ? s.sizes[s.n_layers] : 128;  // 1 KB: keeps two cfg2-sized networks per CU
    int T = pow2ceil((max_edges + 7) / 8);
    if (T < pow2ceil(max_nodes)) T = pow2ceil(max_nodes);
    if (T < 64) T = 64;
    if (T > 1024) T = 1024;
    if (const char* env = getenv("GHIP_EXACT_THREADS")) {
        int v = atoi(env);
        if (v == 64 || v == 128 || v == 256 || v == 512 || v == 1024) T = v;
    }
    n->ex_threads = T;
    for (int l = 0; l < s.n_layers; ++l) {
        int tw = pow2ceil(s.sizes[l]);
        if (tw > T) tw = T;
        e.tw_log2[l] = ilog2(tw);
    }
    size_t lds_full = ghip_exact_lds_bytes(e, true, false);
    e.state_in_lds = lds_full <= (size_t)g_max_lds ? 1 : 0;
    n->ex_lds = ghip_exact_lds_bytes(e, e.state_in_lds != 0, false);
    if (n->ex_lds > (size_t)g_max_lds)
        return fail(GHIP_EINVAL, "exact mode: layers too wide (%zu bytes of node state exceed LDS)", n->ex_lds);
    n->ex_drop_in_lds = ghip_exact_lds_bytes(e, true, true) <= (size_t)g_max_lds ? 1 : 0;
    n->ex_lds_drop = ghip_exact_lds_bytes(e, n->ex_drop_in_lds != 0, true);
    TRY(dalloc(&n->exW, (size_t)woff));
    TRY(dalloc(&n->exSum, (size_t)woff));
    TRY(dalloc(&n->exLast, (size_t)woff));
    TRY(dalloc(&n->exBias, GHIP_MAX_LAYERS));
    TRY(dalloc(&n->exEpochs, 1));
    TRY(dalloc(&n->exCnt, (size_t)woff));
    TRY(dalloc(&n->exErr, (size_t)aoff));
    HIP_TRY(hipMemsetAsync(n->exCnt, 0, sizeof(int) * woff, n->stream));
    HIP_TRY(hipMemsetAsync(n->exErr, 0, sizeof(float) * aoff, n->stream));
    HIP_TRY(hipMemsetAsync(n->exW, 0, sizeof(float) * woff, n->stream));
    HIP_TRY(hipMemsetAsync(n->exSum, 0, sizeof(float) * woff, n->stream));
    HIP_TRY(hipMemsetAsync(n->exLast, 0, sizeof(float) * woff, n->stream));
    HIP_TRY(hipMemsetAsync(n->exBias, 0, sizeof(float) * GHIP_MAX_LAYERS, n->stream));
    e.ptr.W = n->exW; e.ptr.wsum = n->exSum; e.ptr.wlast = n->exLast; e.ptr.bias = n->exBias; e.ptr.epochs_run = n->exEpochs;
    e.ptr.wcnt = n->exCnt; e.ptr.errder = n->exErr;
    return 0;
}

int setup_canon(ghip_net* n)
{
    const ghip_net_spec& s = n->spec;
    const int* ps = n->ps;
    for (int l = 0; l < s.n_layers; ++l) {
        size_t cnt = (size_t)ps[l] * ps[l + 1];
        TRY(dalloc(&n->W[l], cnt));
        TRY(dalloc(&n->b[l], (size_t)ps[l + 1]));
        HIP_TRY(hipMemsetAsync(n->W[l], 0, cnt * 4, n->stream));
        HIP_TRY(hipMemsetAsync(n->b[l], 0, (size_t)ps[l + 1] * 4, n->stream));
        if (s.dtype != GHIP_FP8_INFER) {
            TRY(dalloc(&n->vW[l], cnt));
            TRY(dalloc(&n->vb[l], (size_t)ps[l + 1]));
            HIP_TRY(hipMemsetAsync(n->vW[l], 0, cnt * 4, n->stream));
            HIP_TRY(hipMemsetAsync(n->vb[l], 0, (size_t)ps[l + 1] * 4, n->stream));
        }
        if (s.dtype == GHIP_BF16) {
            TRY(dalloc(&n->Wh[l], cnt));
            TRY(dalloc(&n->WhT[l], cnt));
        }
        if (s.dtype == GHIP_FP8_INFER) {
            TRY(dalloc(&n->Wq[l], cnt));
            TRY(dalloc(&n->wscale[l], (size_t)ps[l + 1]));
        }
    }
    if (s.dtype == GHIP_BF16) {
        // which weight gradients share a launch depends on the layers' sizes alone: laid out once
        int M[GHIP_GEMM_LP_GROUP_MAX], N[GHIP_GEMM_LP_GROUP_MAX];
        auto close_group = [&](int k) -> int {
            size_t cap = 0;
            for (int i = 0; i < n->wgCount[k]; ++i) cap += (size_t)(M[i] / 256) * (N[i] / 256);
            std::vector<unsigned int> sched(cap);
            const int blocks = ghip_gemm_lp_wgrad_plan(M, N, n->wgCount[k], sched.data(), (int)cap);
            if (blocks <= 0) return fail(GHIP_EINVAL, "no weight-gradient schedule for these layer sizes");
            TRY(dalloc(&n->wgSched[k], (size_t)blocks));
            HIP_TRY(hipMemcpy(n->wgSched[k], sched.data(), (size_t)blocks * sizeof(unsigned int), hipMemcpyHostToDevice));
            n->wgBlocks[k] = blocks;
            return 0;
        };
        int k = 0;
        for (int l = 0; l < s.n_layers; ++l) {
            if (ghip_gemm_lp_tile_m(ps[l + 1], ps[l]) != 256) continue;
            M[n->wgCount[k]] = ps[l + 1]; N[n->wgCount[k]] = ps[l];
            n->wgLayer[k][n->wgCount[k]++] = l;
            if (n->wgCount[k] == GHIP_GEMM_LP_GROUP_MAX) { TRY(close_group(k)); ++k; }
        }
        if (n->wgCount[k] > 0) { TRY(close_group(k)); ++k; }
        n->wgGroups = k;
    }
    if (s.dtype == GHIP_F32) {
        n->narrow_fit = ghip_canon_narrow_plan(s.sizes, s.n_layers, 1, &n->narrowTrain, &n->narrowLdsTrain) &&
                        ghip_canon_narrow_plan(s.sizes, s.n_layers, 0, &n->narrowEval, &n->narrowLdsEval);
        if (n->narrow_fit) TRY(dalloc(&n->narrowRan, 1));
    }
    TRY(dalloc(&n->dAcc, 16));  // two alternating banks per step, one for softmax-only launches, one per pass over the table
    HIP_TRY(hipMemsetAsync(n->dAcc, 0, 16 * sizeof(double), n->stream));
    return 0;
}

void free_batch_buffers(ghip_net* n)
{
    for (int l = 0; l <= GHIP_MAX_LAYERS; ++l) {
        dfree(n->act[l]); dfree(n->dlt[l]);
        if (l > 0) dfree(n->H[l]);
        dfree(n->HT[l]); dfree(n->D[l]); dfree(n->DT[l]); dfree(n->csum[l]); dfree(n->Hmask[l]);
    }
    dfree(n->stageX); dfree(n->logits); dfree(n->narrowPart); dfree(n->narrowMetrics);
    dfree(n->Aq[0]); dfree(n->Aq[1]); dfree(n->ascale[0]); dfree(n->ascale[1]);
    dfree(n->amax_bits); dfree(n->Hq); dfree(n->out8); dfree(n->Asc[0]); dfree(n->Asc[1]);
    n->cap_batch = 0;
}

// zeroed device memory (the padded parts of low-precision buffers are read and never written)
template <typename T>
int dalloc_zero(ghip_net* n, T** p, size_t count)
{
    TRY(dalloc(p, count));
    HIP_TRY(hipMemsetAsync(*p, 0, (count ? count : 1) * sizeof(T), n->stream));
    return 0;
}

int reserve_batch(ghip_net* n, int batch)
{
    const int B = pad_batch(n, batch);
    if (B <= n->cap_batch) return 0;
    (void)hipStreamSynchronize(n->stream);
    free_batch_buffers(n);
    const ghip_net_spec& s = n->spec;
    const int L = s.n_layers;
    const int* ps = n->ps;
    int maxw = 0;
    for (int l = 0; l <= L; ++l) if (ps[l] > maxw) maxw = ps[l];
    if (s.dtype == GHIP_F32) {
        TRY(dalloc(&n->stageX, (size_t)B * s.sizes[0]));
        TRY(dalloc(&n->act[0], (size_t)B * s.sizes[0]));   // a batch's rows under its dropout flags
        for (int l = 1; l <= L; ++l) {
            TRY(dalloc(&n->act[l], (size_t)B * s.sizes[l]));
            TRY(dalloc(&n->dlt[l], (size_t)B * s.sizes[l]));
        }
        if (ghip_narrow_out_ok(s.sizes[L], s.sizes[L - 1])) {
            // any batch up to B splits into at most this many chunks of rows (ghip_narrow_out_chunks)
            const int chunks = (B + 3) / 4 < 128 ? (B + 3) / 4 : 128;
            TRY(dalloc(&n->narrowPart, (size_t)chunks * s.sizes[L] * s.sizes[L - 1]));
            TRY(dalloc(&n->narrowMetrics, (size_t)chunks * 4));
        }
    } else if (s.dtype == GHIP_BF16) {
        TRY(dalloc(&n->stageX, (size_t)B * s.sizes[0]));
        TRY(dalloc_zero(n, &n->HT[0], (size_t)B * ps[0]));
        for (int l = 1; l <= L; ++l) {
            if (l < L) {
                TRY(dalloc_zero(n, &n->H[l], (size_t)B * ps[l]));
                TRY(dalloc_zero(n, &n->HT[l], (size_t)B * ps[l]));
                if ((s.act[l - 1] == GHIP_RELU || s.act[l - 1] == GHIP_LEAKY)) TRY(dalloc_zero(n, &n->Hmask[l], (size_t)B * ps[l] / 32));
            }
            // the output deltas are written for the units and rows the batch has; the rest of D[L] stays zero
            TRY(dalloc_zero(n, &n->D[l], (size_t)B * ps[l]));
            TRY(dalloc_zero(n, &n->DT[l], (size_t)B * ps[l]));
            if (l < L) TRY(dalloc(&n->csum[l], (size_t)((B + 127) / 128) * ps[l]));
        }
        TRY(dalloc_zero(n, &n->logits, (size_t)B * ps[L]));
    } else {
        TRY(dalloc(&n->stageX, (size_t)B * s.sizes[0]));
        TRY(dalloc_zero(n, &n->Aq[0], (size_t)B * maxw));
        TRY(dalloc_zero(n, &n->Aq[1], (size_t)B * maxw));
        TRY(dalloc(&n->ascale[0], (size_t)B));
        TRY(dalloc(&n->ascale[1], (size_t)B));
        TRY(dalloc(&n->amax_bits, (size_t)B));
        n->amax_clean = false;
        TRY(dalloc_zero(n, &n->Hq, (size_t)B * maxw));
        TRY(dalloc_zero(n, &n->out8, (size_t)B * ps[L]));
        TRY(dalloc_zero(n, &n->Asc[0], (size_t)B * (maxw / 128)));
        TRY(dalloc_zero(n, &n->Asc[1], (size_t)B * (maxw / 128)));
    }
    n->cap_batch = B;
    return 0;
}

// bf16 shadows W, W^T from the fp32 master (after ghip_net_set_params)
int refresh_shadows(ghip_net* n)
{
    if (!n->shadow_dirty) return 0;
    const ghip_net_spec& s = n->spec;
    for (int l = 0; l < s.n_layers; ++l)
        LAUNCH(n, "f32_to_bf16_transpose", ghip_f32_to_bf16_2d(n->W[l], n->Wh[l], n->WhT[l], n->ps[l + 1], n->ps[l], n->stream));
    n->shadow_dirty = false;
    return 0;
}

int out_act(const ghip_net_spec& s, int l, float* param)
{
    // the GEMM epilogue leaves softmax logits untouched (LINEAR with slope 1)
    if (s.act[l] == GHIP_SOFTMAX) { *param = 1.0f; return GHIP_LINEAR; }
    *param = s.act_param[l];
    return s.act[l];
}

// ---- canonical fp32 ----
// Dropout flags of canonical mode (fp32): per row of the table the node layers below the output side by side, 1 = dropped
// (the layout exact mode takes).  A dropped node's activation is stored as 0, so the layer above gets nothing from it,
// and its delta is 0 (network.cpp:476-480 carried over to batches; no rescaling, as in the reference).
int canon_nodes(const ghip_net* n)
{
    int t = 0;
    for (int l = 0; l < n->spec.n_layers; ++l) t += n->spec.sizes[l];
    return t;
}
bool canon_drop_on(const ghip_net* n) { return n->spec.mode == GHIP_MODE_CANONICAL && n->canMaskEpoch < n->exMaskEpochs; }
// the flags of table row `row0` in the epoch the coming pass uses, or NULL
const uint8_t* canon_drop(const ghip_net* n, int64_t row0)
{
    if (!canon_drop_on(n)) return nullptr;
    return n->exMasks + ((int64_t)n->canMaskEpoch * n->n_rows + row0) * canon_nodes(n);
}

// drop: the flags of the batch's first row (canon_drop) or NULL; with flags the batch's rows enter through act[0]
int forward_f32(ghip_net* n, const float* X, int B, int layers, const uint8_t* drop = nullptr)
{
    const ghip_net_spec& s = n->spec;
    const float* in = X;
    const int nodes = canon_nodes(n);
    int node0 = s.sizes[0];   // where the flags of layer l + 1's nodes start within a row's
    if (drop) {
        LAUNCH(n, "dropout_input", ghip_mask_rows(X, drop, nodes, B, s.sizes[0], n->act[0], n->stream));
        in = n->act[0];
    }
    for (int l = 0; l < layers; ++l) {
        GemmF32Args g;
        memset(&g, 0, sizeof(g));
        g.A = in; g.B = n->W[l]; g.C = n->act[l + 1];
        g.M = B; g.N = s.sizes[l + 1]; g.K = s.sizes[l];
        g.lda = s.sizes[l]; g.ldb = s.sizes[l]; g.ldc = s.sizes[l + 1];
        g.epilogue = EPI_BIAS_ACT; g.bias = n->b[l];
        g.act = out_act(s, l, &g.act_param);
        g.alpha = 1.0f;
        const uint8_t* const drop_out = (drop && l + 1 < s.n_layers) ? drop + node0 : nullptr;   // the flags of this layer's nodes
        node0 += s.sizes[l + 1];
        if (l == s.n_layers - 1 && ghip_narrow_out_ok(g.N, g.K) && ((uintptr_t)in % 16) == 0) {
            NarrowOutArgs a;
            memset(&a, 0, sizeof(a));
            a.H = in; a.W = n->W[l]; a.B = B; a.ni = g.K; a.no = g.N;
            a.bias = n->b[l]; a.P = n->act[l + 1]; a.act = g.act; a.act_param = g.act_param;
            LAUNCH(n, "narrow_out_forward", ghip_narrow_forward(a, n->stream));
        } else
            LAUNCH(n, "gemm_f32_forward", ghip_gemm_f32(g, n->stream));
        // (a pass of its own rather than a branch in the product's epilogue, which every network without flags would carry)
        if (drop_out) LAUNCH(n, "dropout_activations", ghip_mask_rows(n->act[l + 1], drop_out, nodes, B, s.sizes[l + 1], n->act[l + 1], n->stream));
        in = n->act[l + 1];
    }
    return 0;
}

// arguments of the output-delta step of one batch; moves on to the other bank of accumulators
DeltaArgs delta_args(ghip_net* n, float* P, const float* Y, float* D, uint16_t* Dbf, int B)
{
    const ghip_net_spec& s = n->spec;
    const int L = s.n_layers;
    const int bank = n->accBank ^ 1;
    DeltaArgs a;
    memset(&a, 0, sizeof(a));
    a.P = P; a.Y = Y; a.D = D; a.Dbf = Dbf; a.DbfT = nullptr;
    a.B = B; a.n = s.sizes[L]; a.ldp = n->ps[L]; a.ldy = s.sizes[L]; a.ldd = n->ps[L];
    a.act = s.act[L - 1]; a.act_param = s.act_param[L - 1]; a.cost = s.cost;
    a.acc = n->dAcc + 4 * bank; a.acc_clear = n->dAcc + 4 * (bank ^ 1);
    a.cm = n->cm;
    if (n->passAcc) {  // a whole pass adds up in its own bank, which nothing clears on the way
        a.acc = n->dAcc + 12; a.acc_clear = nullptr;
        return a;
    }
    n->accBank = bank;
    return a;
}

int output_delta_f32(ghip_net* n, float* P, const float* Y, float* D, uint16_t* Dbf, int B)
{
    const DeltaArgs a = delta_args(n, P, Y, D, Dbf, B);
    LAUNCH(n, "output_delta", ghip_output_delta(a, n->stream));
    return 0;
}

// ---- narrow canonical networks: one persistent workgroup ----
// Whether a pass in batches of `batch` goes to the one-workgroup kernel.  It runs on one CU, whose fp32 rate bounds
// it; the GEMM launches cost a fixed ~8 us each (7 to a step) and then use the whole chip.  Measured cross-over:
// about 2.5 10^5 multiply-adds per forward pass of a batch
// (13 us + 0.14 us per thousand of them against 50 us of launches).
bool use_narrow(const ghip_net* n, int batch)
{
    if (canon_drop_on(n)) return false;   // the flags are read by the launches' epilogues
    if (!n->narrow_fit || n->canon_path == GHIP_CANON_PATH_LAUNCHES) return false;
    if (n->canon_path == GHIP_CANON_PATH_ONE_WORKGROUP) return true;
    long long macs = 0;
    for (int l = 0; l < n->spec.n_layers; ++l) macs += (long long)n->spec.sizes[l] * n->spec.sizes[l + 1];
    return macs * batch <= 250000;
}

// n_epochs passes over rows [row0, row0 + rows) in batches of `batch`; per epoch 4 doubles at `metrics` (device)
int run_narrow(ghip_net* n, int64_t row0, int64_t rows, int batch, int n_epochs, int train, float stop_accuracy, int reset_cm,
               double* metrics, double* clear4 = nullptr)
{
    const ghip_net_spec& s = n->spec;
    const int L = s.n_layers;
    CanonNarrowArgs a = train ? n->narrowTrain : n->narrowEval;
    for (int l = 0; l < L; ++l) {
        a.act[l] = s.act[l]; a.act_param[l] = s.act_param[l];
        a.lr[l] = s.lr[l]; a.mom[l] = s.mom[l]; a.wd1[l] = s.wd1[l]; a.wd2[l] = s.wd2[l];
        a.W[l] = n->W[l]; a.b[l] = n->b[l]; a.vW[l] = n->vW[l]; a.vb[l] = n->vb[l];
    }
    a.cost = s.cost;
    a.X = n->dX + row0 * s.sizes[0]; a.Y = n->dY + row0 * s.sizes[L];
    a.n_rows = rows; a.batch = batch; a.n_epochs = n_epochs; a.train = train ? 1 : 0; a.stop_accuracy = stop_accuracy;
    a.cm = n->cm; a.reset_cm = reset_cm;
    a.metrics = metrics; a.epochs_run = n->narrowRan; a.clear4 = clear4;
    LAUNCH(n, train ? "canon_narrow_train" : "canon_narrow_eval",
           ghip_canon_narrow_run(a, train ? n->narrowLdsTrain : n->narrowLdsEval, n->stream));
    return 0;
}

int step_f32(ghip_net* n, int64_t row0, int B)
{
    if (use_narrow(n, B)) {
        // the kernel writes the batch's sums where the next reader expects them; the bank after it starts at zero
        const DeltaArgs da = delta_args(n, nullptr, nullptr, nullptr, nullptr, B);
        return run_narrow(n, row0, B, B, 1, 1, 0.0f, 0, da.acc, da.acc_clear);
    }
    const ghip_net_spec& s = n->spec;
    const int L = s.n_layers;
    const float* X = n->dX + row0 * s.sizes[0];
    const float* Y = n->dY + row0 * s.sizes[L];
    const uint8_t* drop = canon_drop(n, row0);
    const int nodes = canon_nodes(n);
    // an output layer of a few units: its forward, the output delta and its backward are one launch (without dropout
    // flags: that launch's backward does not read them)
    const bool narrow = !drop && n->narrowPart && ((uintptr_t)(L == 1 ? X : n->act[L - 1]) % 16) == 0;
    TRY(forward_f32(n, X, B, narrow ? L - 1 : L, drop));
    if (drop) X = n->act[0];   // the rows as the first layer saw them
    if (!narrow) TRY(output_delta_f32(n, n->act[L], Y, n->dlt[L], nullptr, B));
    // The weight gradients (with their updates) only need the deltas, which the back-propagation products
    // leave layer by layer, and write what those products read (the weights): so they wait until the
    // back-propagation below them is through and then run as one launch.
    GemmF32Args wgrads[GHIP_GEMM_F32_GROUP_MAX];
    int n_wgrads = 0;
    for (int l = L - 1; l >= 0; --l) {
        const int ni = s.sizes[l], no = s.sizes[l + 1];
        const float* Ain = (l == 0) ? X : n->act[l];
        GemmF32Args g;
        if (l == L - 1 && narrow) {
            // the launch leaves the outputs, the metrics, the deltas of this layer and of the layer below
            // and the gradient's partial sums; a second small kernel adds those up and updates
            NarrowOutArgs a;
            memset(&a, 0, sizeof(a));
            a.H = Ain; a.W = n->W[l]; a.B = B; a.ni = ni; a.no = no;
            a.bias = n->b[l]; a.P = n->act[l + 1]; a.act = out_act(s, l, &a.act_param);
            a.D = n->dlt[l + 1]; a.E = (l > 0) ? n->dlt[l] : nullptr;
            if (l > 0) { a.act_below = s.act[l - 1]; a.act_below_param = s.act_param[l - 1]; }
            a.part = n->narrowPart;
            ghip_narrow_out_chunks(B, &a.chunks, &a.rows_per_chunk);
            a.Wm = n->W[l]; a.V = n->vW[l]; a.lr = s.lr[l]; a.mom = s.mom[l]; a.wd1 = s.wd1[l]; a.wd2 = s.wd2[l];
            a.alpha = 1.0f / (float)B; a.bias_w = n->b[l]; a.bias_v = n->vb[l];
            const DeltaArgs da = delta_args(n, n->act[L], Y, n->dlt[L], nullptr, B);
            a.metric_part = n->narrowMetrics; a.metric_acc = da.acc;
            LAUNCH(n, "narrow_out_train", ghip_narrow_train(a, da, n->stream));
            LAUNCH(n, "narrow_out_update", ghip_narrow_update(a, n->stream));
            continue;
        }
        if (l > 0) {  // back-prop with the pre-update weights: E = D W, times f'(a_l)
            memset(&g, 0, sizeof(g));
            g.A = n->dlt[l + 1]; g.lda = no; g.a_kmajor = 0;
            g.B = n->W[l]; g.ldb = ni; g.b_kmajor = 1;
            g.C = n->dlt[l]; g.ldc = ni; g.M = B; g.N = ni; g.K = no;
            g.epilogue = EPI_MUL_DER; g.aux = n->act[l];
            g.act = s.act[l - 1]; g.act_param = s.act_param[l - 1]; g.alpha = 1.0f;
            LAUNCH(n, "gemm_f32_dgrad", ghip_gemm_f32(g, n->stream));
            if (drop) {
                int node0 = 0;
                for (int k = 0; k < l; ++k) node0 += s.sizes[k];
                LAUNCH(n, "dropout_deltas", ghip_mask_rows(n->dlt[l], drop + node0, nodes, B, ni, n->dlt[l], n->stream));
            }
        }
        // gradient D^T A / B and, in the same kernel's epilogue, the update of the weights (momentum,
        // both decays) and of the bias (batch mean of the delta = the row sums of the A operand)
        memset(&g, 0, sizeof(g));
        g.A = n->dlt[l + 1]; g.lda = no; g.a_kmajor = 1;
        g.B = Ain; g.ldb = ni; g.b_kmajor = 1;
        g.C = n->W[l]; g.ldc = ni; g.M = no; g.N = ni; g.K = B;
        g.epilogue = EPI_SGD; g.alpha = 1.0f / (float)B;
        g.V = n->vW[l]; g.lr = s.lr[l]; g.mom = s.mom[l]; g.wd1 = s.wd1[l]; g.wd2 = s.wd2[l];
        g.bias_w = n->b[l]; g.bias_v = n->vb[l];
        wgrads[n_wgrads++] = g;
        if (n_wgrads == GHIP_GEMM_F32_GROUP_MAX || l == 0) {
            LAUNCH(n, "gemm_f32_wgrad_sgd", ghip_gemm_f32_group(wgrads, n_wgrads, n->stream));
            n_wgrads = 0;
        }
    }
    return 0;
}

// ---- canonical bf16 ----
// X: the batch's rows in bf16 at pitch ps[0], pad_batch(batch) of them readable
// for_training: also leave the transposed activations the weight gradients read (a forward-only pass skips those stores)
int forward_bf16(ghip_net* n, const uint16_t* X, int batch, bool for_training = false)
{
    const ghip_net_spec& s = n->spec;
    const int L = s.n_layers;
    const int* ps = n->ps;
    const int B = pad_batch(n, batch);
    const uint16_t* in = X;
    for (int l = 0; l < L; ++l) {
        GemmLpArgs g;
        memset(&g, 0, sizeof(g));
        g.A = in; g.B = n->Wh[l]; g.M = B; g.N = ps[l + 1]; g.K = ps[l];
        g.fp8 = 0; g.bias = n->b[l];
        g.act = out_act(s, l, &g.act_param);
        if (l < L - 1) {
            g.epilogue = LP_FWD_ACT; g.out = n->H[l + 1]; g.outT = for_training ? n->HT[l + 1] : nullptr; g.outT_blocked = 1;
            g.mask_out = for_training ? n->Hmask[l + 1] : nullptr;
            g.n_valid = ps[l + 1] != s.sizes[l + 1] ? s.sizes[l + 1] : 0;
            LAUNCH(n, "gemm_bf16_forward", ghip_gemm_lp(g, n->stream));
        } else {
            g.epilogue = LP_FWD_F32; g.out = n->logits;
            LAUNCH(n, "gemm_bf16_forward_out", ghip_gemm_lp(g, n->stream));
        }
        in = n->H[l + 1];
    }
    return 0;
}

int step_bf16(ghip_net* n, int64_t row0, int batch)
{
    const ghip_net_spec& s = n->spec;
    const int L = s.n_layers;
    const int* ps = n->ps;
    const int B = pad_batch(n, batch);   // rows of every product; the means below divide by the batch's own count
    TRY(refresh_shadows(n));
    const uint16_t* X = n->Xbf + row0 * ps[0];
    const float* Y = n->dY + row0 * s.sizes[L];
    // the batch transposed: its columns of the transposed table where that is kept and the batch starts on a
    // cache line of it, a copy made now otherwise
    const bool inT = n->XbfT && (row0 % 64) == 0;
    if (!inT) LAUNCH(n, "bf16_transpose_input", ghip_bf16_transpose(X, n->HT[0], B, ps[0], n->stream));
    TRY(forward_bf16(n, X, batch, true));
    // rows past the batch carry zero deltas: an earlier, longer batch may have left its own there
    if (B != batch)
        LAUNCH(n, "fill_pad_delta", ghip_fill_u32((unsigned int*)(n->D[L] + (size_t)batch * ps[L]), (long long)(B - batch) * ps[L] / 2, 0u, n->stream));
    TRY(output_delta_f32(n, n->logits, Y, nullptr, n->D[L], batch));
    LAUNCH(n, "bf16_transpose_delta", ghip_bf16_transpose(n->D[L], n->DT[L], B, ps[L], n->stream));
    BiasStepArgs bias_args;
    memset(&bias_args, 0, sizeof(bias_args));
    GemmLpArgs wg[GHIP_MAX_LAYERS];
    for (int l = L - 1; l >= 0; --l) {
        const int ni = ps[l], no = ps[l + 1];
        GemmLpArgs g;
        if (l > 0) {
            memset(&g, 0, sizeof(g));
            g.A = n->D[l + 1]; g.B = n->WhT[l]; g.M = B; g.N = ni; g.K = no;
            g.ldb = 64; g.kstrideB = (long long)ni * 128;   // W^T is kept K-blocked: [n_out / 64][n_in][64]
            // (the first hidden layer's deltas have one reader, the first layer's weight gradient, which takes them transposed)
            g.epilogue = LP_DGRAD; g.out = l > 1 ? n->D[l] : nullptr; g.outT = n->DT[l]; g.outT_blocked = 1; g.aux = n->H[l]; g.colsum = n->csum[l];
            g.mask_in = n->Hmask[l];   // where the activation below is a ReLU: its signs as the forward product left them
            g.act = s.act[l - 1]; g.act_param = s.act_param[l - 1];
            LAUNCH(n, "gemm_bf16_dgrad", ghip_gemm_lp(g, n->stream));
        }
        // the layer's bias update: from the column sums the back-propagation product that made D[l+1] left, or
        // for the output layer from the transposed deltas; all of the step's in one launch after the products
        {
            BiasStepArgs::Entry& e = bias_args.e[bias_args.count++];
            if (l + 1 < L) { e.part = n->csum[l + 1]; e.tiles = B / ghip_gemm_lp_tile_m(B, no); }
            else { e.DT = n->DT[l + 1]; e.rows = B; }
            e.n = no; e.batch = batch; e.bias = n->b[l]; e.vb = n->vb[l]; e.lr = s.lr[l]; e.mom = s.mom[l];
        }
        memset(&g, 0, sizeof(g));
        // both operands K-blocked over the batch: [B / 64][nodes][64], a tile's stage one contiguous block
        g.A = n->DT[l + 1]; g.B = n->HT[l]; g.M = no; g.N = ni; g.K = B;
        g.lda = 64; g.kstrideA = (long long)no * 128;
        g.ldb = 64; g.kstrideB = (long long)ni * 128;
        if (l == 0 && inT) g.B = n->XbfT + (row0 / 64) * (long long)ni * 64;
        g.epilogue = LP_WGRAD_SGD; g.out = n->Wh[l]; g.outT = n->WhT[l]; g.outT_blocked = 1;
        g.master = n->W[l]; g.mom = n->vW[l];
        g.lr = s.lr[l]; g.momf = s.mom[l]; g.wd1 = s.wd1[l]; g.wd2 = s.wd2[l]; g.gscale = 1.0f / (float)batch;
        wg[l] = g;
    }
    // The weight gradients, with their updates, write what the back-propagation products read (W^T) and read
    // what those leave (the deltas), so they wait until that chain is through; first layer first, whose
    // deltas are the freshest.
    // the layers whose weight gradient takes the 256 x 256 tile run as one launch per group of 8, first layer first;
    // a narrower layer's (128 x 128 tiles, two workgroups to a CU) is a launch of its own
    for (int k = 0; k < n->wgGroups; ++k) {
        GemmLpArgs grp[GHIP_GEMM_LP_GROUP_MAX];
        for (int i = 0; i < n->wgCount[k]; ++i) grp[i] = wg[n->wgLayer[k][i]];
        LAUNCH(n, "gemm_bf16_wgrad_sgd", ghip_gemm_lp_wgrad_group(grp, n->wgCount[k], n->wgSched[k], n->wgBlocks[k], n->stream));
    }
    for (int l = 0; l < L; ++l)
        if (ghip_gemm_lp_tile_m(wg[l].M, wg[l].N) == 128) LAUNCH(n, "gemm_bf16_wgrad_sgd_t128", ghip_gemm_lp(wg[l], n->stream));
    LAUNCH(n, "bias_update_bf16", ghip_bias_update_step(bias_args, n->stream));
    return 0;
}

// ---- fp8 inference ----
// Xbf: the batch's rows in bf16 at pitch ps[0], pad_batch(batch) of them readable; dev_out has pitch ps[L]
int forward_fp8(ghip_net* n, const uint16_t* Xbf, int batch, float* dev_out)
{
    const ghip_net_spec& s = n->spec;
    const int L = s.n_layers;
    const int* ps = n->ps;
    const int B = pad_batch(n, batch);
    if (!n->quantized) return fail(GHIP_ESTATE, "call ghip_net_quantize_fp8 first");
    int cur = 0;
    if (n->fp8_act_mode == GHIP_FP8_ACT_BLOCK32) {
        // Block-scaled activations: every product's epilogue leaves the next product's A operand (e4m3 codes and an
        // E8M0 scale per row and 32 units), so between two layers nothing is written but that operand and nothing
        // runs but the products.
        const int ld = n->cap_batch;
        LAUNCH(n, "quant_rows_mx", ghip_quant_rows_mx(Xbf, B, ps[0], n->Aq[0], n->Asc[0], ld, n->stream));
        for (int l = 0; l < L; ++l) {
            GemmLpArgs g;
            memset(&g, 0, sizeof(g));
            g.A = n->Aq[cur]; g.B = n->Wq[l]; g.M = B; g.N = ps[l + 1]; g.K = ps[l];
            g.fp8 = 1; g.col_scale = n->wscale[l]; g.a_scale = n->Asc[cur]; g.ld_scale = ld;
            g.act = out_act(s, l, &g.act_param);
            if (l < L - 1) {
                g.epilogue = LP_FP8_ACT_MX; g.out = n->Aq[cur ^ 1]; g.out_scale = n->Asc[cur ^ 1]; g.ld_out_scale = ld;
                g.n_valid = ps[l + 1] != s.sizes[l + 1] ? s.sizes[l + 1] : 0;
                LAUNCH(n, "gemm_fp8_forward", ghip_gemm_lp(g, n->stream));
                cur ^= 1;
            } else {
                g.epilogue = LP_FP8_F32_MX; g.out = dev_out;
                LAUNCH(n, "gemm_fp8_forward_out", ghip_gemm_lp(g, n->stream));
            }
        }
        return 0;
    }
    LAUNCH(n, "quant_rows_e4m3", ghip_quant_rows_e4m3(Xbf, 1, B, ps[0], n->Aq[0], n->ascale[0], nullptr, 0, n->stream));
    // the row maxima start at zero and every re-quantisation puts the entries it has read back to
    // zero; they are only cleared here after a forward pass that stopped between the two
    if (!n->amax_clean) {
        LAUNCH(n, "fill_amax", ghip_fill_u32(n->amax_bits, n->cap_batch, 0u, n->stream));
        n->amax_clean = true;
    }
    for (int l = 0; l < L; ++l) {
        GemmLpArgs g;
        memset(&g, 0, sizeof(g));
        g.A = n->Aq[cur]; g.B = n->Wq[l]; g.M = B; g.N = ps[l + 1]; g.K = ps[l];
        g.fp8 = 1; g.row_scale = n->ascale[cur]; g.col_scale = n->wscale[l];
        g.act = out_act(s, l, &g.act_param);
        if (l < L - 1) {
            g.epilogue = LP_FP8_ACT; g.out = n->Hq; g.row_amax_bits = n->amax_bits;
            g.n_valid = ps[l + 1] != s.sizes[l + 1] ? s.sizes[l + 1] : 0;
            n->amax_clean = false;
            LAUNCH(n, "gemm_fp8_forward", ghip_gemm_lp(g, n->stream));
            LAUNCH(n, "requant_rows_e4m3", ghip_quant_rows_e4m3(n->Hq, 1, B, ps[l + 1], n->Aq[cur ^ 1], n->ascale[cur ^ 1],
                                                                n->amax_bits, 1, n->stream));
            n->amax_clean = true;
            cur ^= 1;
        } else {
            g.epilogue = LP_FP8_F32; g.out = dev_out;
            LAUNCH(n, "gemm_fp8_forward_out", ghip_gemm_lp(g, n->stream));
        }
    }
    return 0;
}

int fetch_metrics(ghip_net* n, ghip_metrics* m)
{
    double acc[4];
    HIP_TRY(hipMemcpyAsync(acc, n->dAcc + 4 * n->accBank, sizeof(acc), hipMemcpyDeviceToHost, n->stream));
    HIP_TRY(hipStreamSynchronize(n->stream));
    const int B = n->last_batch > 0 ? n->last_batch : 1;
    m->loss = (float)(acc[0] / (double)B);
    m->accuracy = (float)(acc[1] / ((double)B * n->spec.sizes[n->spec.n_layers]));
    m->correct = (int64_t)(acc[2] + 0.5);
    return 0;
}

}  // namespace

extern "C" {

const char* ghip_last_error(void) { return g_err.c_str(); }
const char* ghip_version(void) { return "glades-hip 0.1 (gfx950)"; }

int ghip_init(int device_ordinal)
{
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) return fail(GHIP_ENODEV, "no HIP device: %s", hipGetErrorString(e));
    if (device_ordinal < 0 || device_ordinal >= count) return fail(GHIP_EINVAL, "device %d of %d", device_ordinal, count);
    HIP_TRY(hipSetDevice(device_ordinal));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device_ordinal));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(GHIP_ENODEV, "device %d is %s; this library is built for gfx950 only", device_ordinal, prop.gcnArchName);
    int lds = 0;
    if (hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, device_ordinal) == hipSuccess && lds > 0)
        g_max_lds = lds;
    // The runtime completes its own set-up inside the first stream creation / allocation, and that
    // set-up draws from libc rand().  The reference's weight sampler and dropout read the same
    // stream, so it is done here: a caller who seeds rand() after this call finds the stream
    // untouched by the calls that follow.
    {
        hipStream_t s = nullptr;
        void* p = nullptr;
        HIP_TRY(hipStreamCreate(&s));
        HIP_TRY(hipMalloc(&p, 256));
        HIP_TRY(hipMemsetAsync(p, 0, 256, s));
        HIP_TRY(hipStreamSynchronize(s));
        HIP_TRY(hipFree(p));
        HIP_TRY(hipStreamDestroy(s));
    }
    g_device = device_ordinal;
    unsigned char* sp = nullptr;
    TRY(scratch_for_device(device_ordinal, &sp));
    return 0;
}

int ghip_gmath_eval(int fn, int kind, float param, const float* host_a, const float* host_b, float* host_out, int64_t n)
{
    if (fn < 0 || fn > 4 || !host_a || !host_out || n < 0 || (fn >= 2 && !host_b)) return fail(GHIP_EINVAL, "bad arguments");
    if (fn <= 1 && (kind < GHIP_TANH || kind > GHIP_STEP)) return fail(GHIP_EINVAL, "unknown activation %d", kind);
    if ((fn == 2 || fn == 3) && (kind < GHIP_REGRESSION || kind > GHIP_KL)) return fail(GHIP_EINVAL, "unknown cost %d", kind);
    if (fn == 4 && (kind < 0 || kind > 2 || !(param >= 0.0f && param <= 1.0e6f))) return fail(GHIP_EINVAL, "bias chain: kind 0..2, rounds 0..1e6");
    const size_t bn = (fn == 4) ? (size_t)n * 64 : (size_t)n;  // floats of host_b
    if (n == 0) return 0;
    if (g_device < 0) TRY(ghip_init(0));
    HIP_TRY(hipSetDevice(g_device));
    float *a = nullptr, *b = nullptr, *o = nullptr;
    int rc = dalloc(&a, (size_t)n);
    if (rc == 0) rc = dalloc(&o, (size_t)n);
    if (rc == 0 && fn >= 2) rc = dalloc(&b, bn);
    hipError_t e = hipSuccess;
    if (rc == 0) e = hipMemcpy(a, host_a, (size_t)n * 4, hipMemcpyHostToDevice);
    if (rc == 0 && e == hipSuccess && b) e = hipMemcpy(b, host_b, bn * 4, hipMemcpyHostToDevice);
    if (rc == 0 && e == hipSuccess)
        e = (fn == 4) ? ghip_launch_bias_chain_eval(kind, (int)param, a, b, o, n, 0) : ghip_launch_gmath_eval(fn, kind, param, a, b, o, n, 0);
    if (rc == 0 && e == hipSuccess) e = hipMemcpy(host_out, o, (size_t)n * 4, hipMemcpyDeviceToHost);
    dfree(a); dfree(b); dfree(o);
    if (rc != 0) return rc;
    if (e != hipSuccess) return fail(GHIP_EHIP, "gmath_eval: %s", hipGetErrorString(e));
    return 0;
}

int ghip_net_create(const ghip_net_spec* spec, ghip_net** out)
{
    if (!out) return fail(GHIP_EINVAL, "out is NULL");
    *out = nullptr;
    if (g_device < 0) TRY(ghip_init(0));
    HIP_TRY(hipSetDevice(g_device));  // the calling thread may be a fresh one (one host thread per MetaNetwork subnet)
    TRY(check_spec(spec));
    ghip_net* n = new ghip_net();
    n->spec = *spec;
    n->L = spec->n_layers;
    set_padded_sizes(n);
    hipError_t e = hipStreamCreate(&n->stream);
    if (e != hipSuccess) { delete n; return fail(GHIP_EHIP, "hipStreamCreate: %s", hipGetErrorString(e)); }
    int r = (spec->mode == GHIP_MODE_EXACT) ? setup_exact(n) : setup_canon(n);
    if (r != 0) { std::string keep = g_err; ghip_net_destroy(n); g_err = keep; return r; }
    *out = n;
    return 0;
}

int ghip_net_destroy(ghip_net* n)
{
    if (!n) return 0;
    if (n->stream) (void)hipStreamSynchronize(n->stream);
    prof_collect(n);
    free_batch_buffers(n);
    dfree(n->ownX); dfree(n->ownY); dfree(n->Xbf); dfree(n->XbfT);
    dfree(n->exW); dfree(n->exSum); dfree(n->exLast); dfree(n->exBias); dfree(n->exPreds);
    dfree(n->exMetrics); dfree(n->exEpochs); dfree(n->cm); dfree(n->exClass); dfree(n->exMulti);
    dfree(n->exMasks); dfree(n->exCnt); dfree(n->exErr); dfree(n->exMultiMetrics); dfree(n->exMultiEpochs);
    for (int l = 0; l < GHIP_MAX_LAYERS; ++l) {
        dfree(n->W[l]); dfree(n->b[l]); dfree(n->vW[l]); dfree(n->vb[l]);
        dfree(n->Wh[l]); dfree(n->WhT[l]); dfree(n->Wq[l]); dfree(n->wscale[l]);
    }
    dfree(n->dAcc); dfree(n->narrowEpochs); dfree(n->narrowRan);
    for (auto& p : n->wgSched) dfree(p);
    if (n->stream) (void)hipStreamDestroy(n->stream);
    delete n;
    return 0;
}

int ghip_net_set_params(ghip_net* n, int layer, const float* host_W, const float* host_bias, int bias_len)
{
    if (!n || layer < 0 || layer >= n->L) return fail(GHIP_EINVAL, "bad net or layer");
    const ghip_net_spec& s = n->spec;
    const int ni = s.sizes[layer], no = s.sizes[layer + 1];
    if (s.mode == GHIP_MODE_EXACT) {
        if (bias_len != 0 && bias_len != 1) return fail(GHIP_EINVAL, "exact mode bias is one scalar per layer");
        if (host_W) {
            const int ld = n->ex.ld[layer];
            std::vector<float> pad((size_t)ld * no, 0.0f);
            for (int o = 0; o < no; ++o) memcpy(&pad[(size_t)o * ld], host_W + (size_t)o * ni, sizeof(float) * ni);
            HIP_TRY(hipMemcpyAsync(n->exW + n->ex.woff[layer], pad.data(), pad.size() * 4, hipMemcpyHostToDevice, n->stream));
            HIP_TRY(hipMemsetAsync(n->exSum + n->ex.woff[layer], 0, pad.size() * 4, n->stream));
            HIP_TRY(hipMemsetAsync(n->exLast + n->ex.woff[layer], 0, pad.size() * 4, n->stream));
            HIP_TRY(hipMemsetAsync(n->exCnt + n->ex.woff[layer], 0, pad.size() * 4, n->stream));
            n->exUniformCnt[layer] = 0;
            HIP_TRY(hipStreamSynchronize(n->stream));
        }
        if (host_bias && bias_len == 1) {
            HIP_TRY(hipMemcpyAsync(n->exBias + layer, host_bias, 4, hipMemcpyHostToDevice, n->stream));
            HIP_TRY(hipStreamSynchronize(n->stream));
        }
        return 0;
    }
    if (bias_len != 0 && bias_len != no) return fail(GHIP_EINVAL, "canonical bias has one entry per output channel (%d), got %d", no, bias_len);
    const int pni = n->ps[layer];
    const size_t cnt = (size_t)pni * n->ps[layer + 1];
    if (host_W) {
        if (pni == ni) HIP_TRY(hipMemcpyAsync(n->W[layer], host_W, (size_t)ni * no * 4, hipMemcpyHostToDevice, n->stream));
        else HIP_TRY(copy_matrix(n->W[layer], pni, const_cast<float*>(host_W), no, ni, true, n->stream));
        if (n->vW[layer]) HIP_TRY(hipMemsetAsync(n->vW[layer], 0, cnt * 4, n->stream));
        n->shadow_dirty = true;
        n->quantized = false;
    }
    if (host_bias && bias_len == no) HIP_TRY(hipMemcpyAsync(n->b[layer], host_bias, (size_t)no * 4, hipMemcpyHostToDevice, n->stream));
    else if (host_W) HIP_TRY(hipMemsetAsync(n->b[layer], 0, (size_t)no * 4, n->stream));
    if (n->vb[layer]) HIP_TRY(hipMemsetAsync(n->vb[layer], 0, (size_t)no * 4, n->stream));
    HIP_TRY(hipStreamSynchronize(n->stream));
    return 0;
}

int ghip_net_get_params(ghip_net* n, int layer, float* host_W, float* host_bias, int bias_len)
{
    if (!n || layer < 0 || layer >= n->L) return fail(GHIP_EINVAL, "bad net or layer");
    const ghip_net_spec& s = n->spec;
    const int ni = s.sizes[layer], no = s.sizes[layer + 1];
    HIP_TRY(hipStreamSynchronize(n->stream));
    if (s.mode == GHIP_MODE_EXACT) {
        if (host_W) {
            const int ld = n->ex.ld[layer];
            std::vector<float> pad((size_t)ld * no);
            HIP_TRY(hipMemcpy(pad.data(), n->exW + n->ex.woff[layer], pad.size() * 4, hipMemcpyDeviceToHost));
            for (int o = 0; o < no; ++o) memcpy(host_W + (size_t)o * ni, &pad[(size_t)o * ld], sizeof(float) * ni);
        }
        if (host_bias && bias_len >= 1) HIP_TRY(hipMemcpy(host_bias, n->exBias + layer, 4, hipMemcpyDeviceToHost));
        return 0;
    }
    if (host_W) {
        if (n->ps[layer] == ni) HIP_TRY(hipMemcpy(host_W, n->W[layer], (size_t)ni * no * 4, hipMemcpyDeviceToHost));
        else {
            HIP_TRY(copy_matrix(n->W[layer], n->ps[layer], host_W, no, ni, false, n->stream));
            HIP_TRY(hipStreamSynchronize(n->stream));
        }
    }
    if (host_bias) {
        if (bias_len != no) return fail(GHIP_EINVAL, "bias_len %d != %d", bias_len, no);
        HIP_TRY(hipMemcpy(host_bias, n->b[layer], (size_t)no * 4, hipMemcpyDeviceToHost));
    }
    return 0;
}

// direction 0: device -> host, 1: host -> device
static int move_state(ghip_net* n, int layer, float* a, float* b, int to_device)
{
    if (!n || layer < 0 || layer >= n->L) return fail(GHIP_EINVAL, "bad net or layer");
    const ghip_net_spec& s = n->spec;
    const int ni = s.sizes[layer], no = s.sizes[layer + 1];
    HIP_TRY(hipStreamSynchronize(n->stream));
    if (s.mode == GHIP_MODE_EXACT) {
        const int ld = n->ex.ld[layer];
        float* dev[2] = {n->exSum + n->ex.woff[layer], n->exLast + n->ex.woff[layer]};
        float* host[2] = {a, b};
        std::vector<float> pad((size_t)ld * no, 0.0f);
        for (int k = 0; k < 2; ++k) {
            if (!host[k]) continue;
            if (to_device) {
                for (int o = 0; o < no; ++o) memcpy(&pad[(size_t)o * ld], host[k] + (size_t)o * ni, sizeof(float) * ni);
                HIP_TRY(hipMemcpy(dev[k], pad.data(), pad.size() * 4, hipMemcpyHostToDevice));
            } else {
                HIP_TRY(hipMemcpy(pad.data(), dev[k], pad.size() * 4, hipMemcpyDeviceToHost));
                for (int o = 0; o < no; ++o) memcpy(host[k] + (size_t)o * ni, &pad[(size_t)o * ld], sizeof(float) * ni);
            }
        }
        return 0;
    }
    if (s.dtype == GHIP_FP8_INFER) return fail(GHIP_ESTATE, "an inference-only network has no optimiser state");
    if (a && n->ps[layer] != ni) {
        HIP_TRY(copy_matrix(n->vW[layer], n->ps[layer], a, no, ni, to_device != 0, n->stream));
        HIP_TRY(hipStreamSynchronize(n->stream));
    } else if (a)
        HIP_TRY(to_device ? hipMemcpy(n->vW[layer], a, (size_t)ni * no * 4, hipMemcpyHostToDevice)
                          : hipMemcpy(a, n->vW[layer], (size_t)ni * no * 4, hipMemcpyDeviceToHost));
    if (b) HIP_TRY(to_device ? hipMemcpy(n->vb[layer], b, (size_t)no * 4, hipMemcpyHostToDevice)
                             : hipMemcpy(b, n->vb[layer], (size_t)no * 4, hipMemcpyDeviceToHost));
    return 0;
}

int ghip_net_get_state(ghip_net* n, int layer, float* host_a, float* host_b) { return move_state(n, layer, host_a, host_b, 0); }
int ghip_net_set_state(ghip_net* n, int layer, const float* host_a, const float* host_b)
{
    return move_state(n, layer, const_cast<float*>(host_a), const_cast<float*>(host_b), 1);
}

int ghip_net_set_dropout_masks(ghip_net* n, const uint8_t* host_masks, int n_epochs)
{
    if (!n) return fail(GHIP_EINVAL, "bad net");
    HIP_TRY(hipSetDevice(g_device));
    if (n->spec.mode != GHIP_MODE_EXACT && n->spec.dtype != GHIP_F32)
        return fail(GHIP_ESTATE, "dropout flags are taken in exact mode and by fp32 networks in canonical mode");
    n->canMaskEpoch = 0;
    if (!host_masks) {
        n->exMaskEpochs = 0;
        return 0;
    }
    if (n_epochs < 1) return fail(GHIP_EINVAL, "bad arguments");
    if (!n->dX || !n->dY) return fail(GHIP_ESTATE, "no dataset (the flags are per row of the table)");
    const int64_t len = (int64_t)n_epochs * n->n_rows * canon_nodes(n);
    for (int64_t k = 0; k < len; ++k)
        if (host_masks[k] > 1) return fail(GHIP_EINVAL, "flag %lld is %d, not 0 or 1", (long long)k, (int)host_masks[k]);
    // a layer with every node dropped would never finalise the next layer (Layer::lastValidPath,
    // ML/State/layer.cpp:168-183); the reference redraws such a layer (layer.cpp:114-133)
    {
        const uint8_t* m = host_masks;
        for (int64_t row = 0; row < (int64_t)n_epochs * n->n_rows; ++row)
            for (int l = 0; l < n->L; ++l) {
                int valid = 0;
                for (int i = 0; i < n->spec.sizes[l]; ++i) valid += m[i] ? 0 : 1;
                if (!valid) return fail(GHIP_EINVAL, "row %lld drops every node of layer %d", (long long)row, l);
                m += n->spec.sizes[l];
            }
    }
    HIP_TRY(hipStreamSynchronize(n->stream));
    if (len > n->exMasksCap) {
        dfree(n->exMasks);
        TRY(dalloc(&n->exMasks, (size_t)len));
        n->exMasksCap = len;
    }
    HIP_TRY(hipMemcpy(n->exMasks, host_masks, (size_t)len, hipMemcpyHostToDevice));
    n->exMaskEpochs = n_epochs;
    return 0;
}

// Window lengths of a network that has only run without dropout: the same for every edge of a layer.
static int materialize_counts(ghip_net* n)
{
    if (n->exDropState) return 0;
    HIP_TRY(hipStreamSynchronize(n->stream));
    for (int l = 0; l < n->L; ++l) {
        std::vector<int32_t> pad((size_t)n->ex.ld[l] * n->spec.sizes[l + 1], n->exUniformCnt[l]);
        HIP_TRY(hipMemcpy(n->exCnt + n->ex.woff[l], pad.data(), pad.size() * 4, hipMemcpyHostToDevice));
    }
    return 0;
}

// direction 0: device -> host, 1: host -> device
static int move_dropout_state(ghip_net* n, int layer, int32_t* counts, float* errder, int to_device)
{
    if (!n || layer < 0 || layer >= n->L) return fail(GHIP_EINVAL, "bad net or layer");
    if (n->spec.mode != GHIP_MODE_EXACT) return fail(GHIP_ESTATE, "dropout state belongs to exact mode");
    HIP_TRY(hipSetDevice(g_device));
    const int ni = n->spec.sizes[layer], no = n->spec.sizes[layer + 1], ld = n->ex.ld[layer];
    HIP_TRY(hipStreamSynchronize(n->stream));
    TRY(materialize_counts(n));
    if (counts) {
        std::vector<int32_t> pad((size_t)ld * no, 0);
        int* dev = n->exCnt + n->ex.woff[layer];
        if (to_device) {
            for (int o = 0; o < no; ++o) memcpy(&pad[(size_t)o * ld], counts + (size_t)o * ni, sizeof(int32_t) * ni);
            HIP_TRY(hipMemcpy(dev, pad.data(), pad.size() * 4, hipMemcpyHostToDevice));
        } else {
            HIP_TRY(hipMemcpy(pad.data(), dev, pad.size() * 4, hipMemcpyDeviceToHost));
            for (int o = 0; o < no; ++o) memcpy(counts + (size_t)o * ni, &pad[(size_t)o * ld], sizeof(int32_t) * ni);
        }
    }
    if (errder) {
        float* dev = n->exErr + n->ex.aoff[layer + 1];
        HIP_TRY(to_device ? hipMemcpy(dev, errder, (size_t)no * 4, hipMemcpyHostToDevice)
                          : hipMemcpy(errder, dev, (size_t)no * 4, hipMemcpyDeviceToHost));
    }
    if (to_device) n->exDropState = true;
    return 0;
}

int ghip_net_get_dropout_state(ghip_net* n, int layer, int32_t* host_counts, float* host_errder)
{
    return move_dropout_state(n, layer, host_counts, host_errder, 0);
}
int ghip_net_set_dropout_state(ghip_net* n, int layer, const int32_t* host_counts, const float* host_errder)
{
    return move_dropout_state(n, layer, const_cast<int32_t*>(host_counts), const_cast<float*>(host_errder), 1);
}

static int make_bf16_table(ghip_net* n)
{
    const ghip_net_spec& s = n->spec;
    if (s.mode != GHIP_MODE_CANONICAL || s.dtype == GHIP_F32) return 0;
    dfree(n->Xbf);
    dfree(n->XbfT);
    const int n0 = s.sizes[0], pn0 = n->ps[0];
    // a last batch that is not a multiple of 256 rows reads on into rows of zeros
    n->table_rows = (n->n_rows + 255 + 63) / 64 * 64;
    TRY(dalloc(&n->Xbf, (size_t)n->table_rows * pn0));
    HIP_TRY(hipMemsetAsync(n->Xbf + (size_t)n->n_rows * pn0, 0, (size_t)(n->table_rows - n->n_rows) * pn0 * 2, n->stream));
    // Training reads each batch transposed as well (the weight gradient of the first layer runs over the
    // batch): the whole table is kept that way, in planes of 64 rows.  A table too large for that is
    // transposed batch by batch.
    const size_t bytesT = (size_t)pn0 * (size_t)n->table_rows * 2;
    if (s.dtype == GHIP_BF16 && n->n_rows >= 64 && bytesT <= ((size_t)16 << 30)) {
        if (hipMalloc((void**)&n->XbfT, bytesT) != hipSuccess) { n->XbfT = nullptr; (void)hipGetLastError(); }
        else HIP_TRY(hipMemsetAsync(n->XbfT + (size_t)(n->n_rows / 64) * pn0 * 64, 0, (size_t)(n->table_rows / 64 - n->n_rows / 64) * pn0 * 128, n->stream));
    }
    // convert in slabs of rows to keep the grid small
    const int64_t slab = 65536;
    for (int64_t r = 0; r < n->n_rows; r += slab) {
        const int rows = (int)((n->n_rows - r) < slab ? (n->n_rows - r) : slab);
        LAUNCH(n, "f32_to_bf16_table", ghip_f32_to_bf16_2d_pad(n->dX + r * n0, rows, n0, n->Xbf + r * pn0,
                                                              n->XbfT ? n->XbfT + (r / 64) * pn0 * 64 : nullptr, rows, pn0, n->stream));
    }
    return 0;
}

int ghip_net_set_dataset(ghip_net* n, const float* host_X, const float* host_Y, int64_t n_rows)
{
    if (!n || !host_X || n_rows <= 0) return fail(GHIP_EINVAL, "bad dataset arguments");
    const ghip_net_spec& s = n->spec;
    HIP_TRY(hipSetDevice(g_device));
    HIP_TRY(hipStreamSynchronize(n->stream));
    n->exMaskEpochs = 0;  // dropout flags are per row of the table they were set for
    dfree(n->ownX); dfree(n->ownY);
    const size_t nx = (size_t)n_rows * s.sizes[0], ny = (size_t)n_rows * s.sizes[s.n_layers];
    TRY(dalloc(&n->ownX, nx));
    HIP_TRY(hipMemcpy(n->ownX, host_X, nx * 4, hipMemcpyHostToDevice));
    if (host_Y) {
        TRY(dalloc(&n->ownY, ny));
        HIP_TRY(hipMemcpy(n->ownY, host_Y, ny * 4, hipMemcpyHostToDevice));
    }
    n->dX = n->ownX; n->dY = n->ownY; n->n_rows = n_rows;
    return make_bf16_table(n);
}

int ghip_net_set_dataset_device(ghip_net* n, const float* dev_X, const float* dev_Y, int64_t n_rows)
{
    if (!n || !dev_X || n_rows <= 0) return fail(GHIP_EINVAL, "bad dataset arguments");
    HIP_TRY(hipSetDevice(g_device));
    HIP_TRY(hipStreamSynchronize(n->stream));
    n->exMaskEpochs = 0;
    dfree(n->ownX); dfree(n->ownY);
    n->dX = dev_X; n->dY = dev_Y; n->n_rows = n_rows;
    return make_bf16_table(n);
}

// buffers of one network for a call of n_epochs epochs; fills ptr
static int exact_prepare(ghip_net* n, int n_epochs, bool want_preds, bool own_metrics, ExactPointers* ptr)
{
    const int nout = n->spec.sizes[n->L];
    if (own_metrics && n_epochs > n->exMetricsCap) {
        HIP_TRY(hipStreamSynchronize(n->stream));
        dfree(n->exMetrics);
        TRY(dalloc(&n->exMetrics, (size_t)n_epochs));
        n->exMetricsCap = n_epochs;
    }
    if (want_preds && n->n_rows * nout > n->exPredsCap) {
        HIP_TRY(hipStreamSynchronize(n->stream));
        dfree(n->exPreds);
        TRY(dalloc(&n->exPreds, (size_t)n->n_rows * nout));
        n->exPredsCap = n->n_rows * nout;
    }
    *ptr = n->ex.ptr;
    ptr->masks = nullptr;
    if (n->exMaskEpochs > 0) {
        if (n_epochs > n->exMaskEpochs)
            return fail(GHIP_EINVAL, "%d epochs asked for, dropout flags for %d", n_epochs, n->exMaskEpochs);
        ptr->masks = n->exMasks;
    }
    ptr->preds = want_preds ? n->exPreds : nullptr;
    ptr->metrics = (float*)n->exMetrics;
    ptr->cm = n->cm;
    ptr->class_metrics = nullptr;
    if (n->cm && nout <= 64) {
        if (n_epochs > n->exClassCap) {
            HIP_TRY(hipStreamSynchronize(n->stream));
            dfree(n->exClass);
            TRY(dalloc(&n->exClass, (size_t)n_epochs * 5));
            n->exClassCap = n_epochs;
        }
        ptr->class_metrics = n->exClass;
    }
    n->exClassRan = 0;
    return 0;
}

int ghip_net_run_epochs_exact(ghip_net* n, int n_epochs, int train, float stop_accuracy,
                              ghip_metrics* host_metrics, int* epochs_run, float* host_preds)
{
    if (!n || n_epochs < 1) return fail(GHIP_EINVAL, "bad arguments");
    HIP_TRY(hipSetDevice(g_device));
    if (n->spec.mode != GHIP_MODE_EXACT) return fail(GHIP_ESTATE, "network is not in exact mode");
    if (!n->dX || !n->dY) return fail(GHIP_ESTATE, "no dataset");
    const int nout = n->spec.sizes[n->L];
    ExactLaunch e = n->ex;
    TRY(exact_prepare(n, n_epochs, host_preds != nullptr, true, &e.ptr));
    e.X = n->dX; e.Y = n->dY; e.n_rows = n->n_rows;
    e.n_epochs = n_epochs; e.train = train ? 1 : 0; e.stop_accuracy = stop_accuracy;
    size_t lds = n->ex_lds;
    if (e.ptr.masks || n->exDropState) {
        TRY(materialize_counts(n));
        e.dropout = 1;
        e.state_in_lds = n->ex_drop_in_lds;
        lds = n->ex_lds_drop;
        n->exDropState = true;
        n->exMaskEpochs = 0;  // flags are used once
    }
    else if (e.train) {
        // rows after the last applying one each pushed a delta (network.cpp:647-651)
        for (int l = 0; l < n->L; ++l) n->exUniformCnt[l] = (int)((n->n_rows - 1) % n->spec.batch);
    }
    LAUNCH(n, e.dropout ? "exact_epochs_dropout" : "exact_epochs", ghip_launch_exact(e, nullptr, 1, n->ex_threads, lds, n->stream));
    int ran = 0;
    HIP_TRY(hipMemcpyAsync(&ran, n->exEpochs, sizeof(int), hipMemcpyDeviceToHost, n->stream));
    HIP_TRY(hipStreamSynchronize(n->stream));
    if (epochs_run) *epochs_run = ran;
    n->exClassRan = e.ptr.class_metrics ? ran : 0;
    if (host_metrics && ran > 0) HIP_TRY(hipMemcpy(host_metrics, n->exMetrics, sizeof(ghip_metrics) * ran, hipMemcpyDeviceToHost));
    if (host_preds) HIP_TRY(hipMemcpy(host_preds, n->exPreds, sizeof(float) * n->n_rows * nout, hipMemcpyDeviceToHost));
    return 0;
}

int ghip_net_run_epochs_exact_multi(ghip_net* const* nets, int count, int n_epochs, int train, float stop_accuracy,
                                    ghip_metrics* host_metrics, int* epochs_run)
{
    if (!nets || count < 1 || n_epochs < 1) return fail(GHIP_EINVAL, "bad arguments");
    HIP_TRY(hipSetDevice(g_device));
    ghip_net* lead = nets[0];
    {
        std::vector<const ghip_net*> sorted(nets, nets + count);
        std::sort(sorted.begin(), sorted.end());
        for (int k = 1; k < count; ++k)
            if (sorted[k] && sorted[k] == sorted[k - 1]) return fail(GHIP_EINVAL, "a network appears twice in the list");
    }
    for (int k = 0; k < count; ++k) {
        ghip_net* n = nets[k];
        if (!n) return fail(GHIP_EINVAL, "network %d is NULL", k);
        if (n->spec.mode != GHIP_MODE_EXACT) return fail(GHIP_ESTATE, "network %d is not in exact mode", k);
        if (!n->dX || !n->dY) return fail(GHIP_ESTATE, "network %d has no dataset", k);
        // one launch = one architecture, one schedule, one table: everything but the parameters is shared
        if (memcmp(&n->spec, &lead->spec, sizeof(ghip_net_spec)) != 0) return fail(GHIP_EINVAL, "network %d differs from network 0 in its specification", k);
        if (n->n_rows != lead->n_rows) return fail(GHIP_EINVAL, "network %d has a table of another length", k);
    }
    std::vector<ExactPointers> list(count);
    for (int k = 0; k < count; ++k) TRY(exact_prepare(nets[k], n_epochs, false, false, &list[k]));
    // every network's earlier work (on its own stream) is done before lead's stream touches its arrays
    if (count > 1) HIP_TRY(hipDeviceSynchronize());
    if (count > lead->exMultiCap) {
        HIP_TRY(hipStreamSynchronize(lead->stream));
        dfree(lead->exMulti); dfree(lead->exMultiEpochs);
        TRY(dalloc(&lead->exMulti, (size_t)count));
        TRY(dalloc(&lead->exMultiEpochs, (size_t)count));
        lead->exMultiCap = count;
    }
    if ((size_t)count * n_epochs > lead->exMultiMetricsCap) {
        HIP_TRY(hipStreamSynchronize(lead->stream));
        dfree(lead->exMultiMetrics);
        TRY(dalloc(&lead->exMultiMetrics, (size_t)count * n_epochs));
        lead->exMultiMetricsCap = (size_t)count * n_epochs;
    }
    // every network writes its results into its slot of one array: two copies back instead of two per network
    for (int k = 0; k < count; ++k) {
        list[k].metrics = (float*)(lead->exMultiMetrics + (size_t)k * n_epochs);
        list[k].epochs_run = lead->exMultiEpochs + k;
    }
    HIP_TRY(hipMemcpyAsync(lead->exMulti, list.data(), sizeof(ExactPointers) * count, hipMemcpyHostToDevice, lead->stream));
    ExactLaunch e = lead->ex;
    // each network reads its own copy of the table (identical content is the caller's business: the
    // reference trains every subnet of a MetaNetwork on the same DataInput, ML/main.cpp:137-160)
    e.X = lead->dX; e.Y = lead->dY; e.n_rows = lead->n_rows;
    e.n_epochs = n_epochs; e.train = train ? 1 : 0; e.stop_accuracy = stop_accuracy;
    size_t lds = lead->ex_lds;
    bool any_drop = false;
    for (int k = 0; k < count; ++k) any_drop = any_drop || list[k].masks || nets[k]->exDropState;
    if (any_drop) {
        e.dropout = 1;
        e.state_in_lds = lead->ex_drop_in_lds;
        lds = lead->ex_lds_drop;
        for (int k = 0; k < count; ++k) {
            TRY(materialize_counts(nets[k]));
            nets[k]->exDropState = true;
            nets[k]->exMaskEpochs = 0;
        }
    } else if (e.train) {
        for (int k = 0; k < count; ++k)
            for (int l = 0; l < lead->L; ++l) nets[k]->exUniformCnt[l] = (int)((lead->n_rows - 1) % lead->spec.batch);
    }
    LAUNCH(lead, any_drop ? "exact_epochs_multi_dropout" : "exact_epochs_multi",
           ghip_launch_exact(e, lead->exMulti, count, lead->ex_threads, lds, lead->stream));
    std::vector<int> ran(count);
    std::vector<ghip_metrics> all(host_metrics ? (size_t)count * n_epochs : 0);
    HIP_TRY(hipMemcpyAsync(ran.data(), lead->exMultiEpochs, sizeof(int) * count, hipMemcpyDeviceToHost, lead->stream));
    if (host_metrics)
        HIP_TRY(hipMemcpyAsync(all.data(), lead->exMultiMetrics, sizeof(ghip_metrics) * all.size(), hipMemcpyDeviceToHost, lead->stream));
    HIP_TRY(hipStreamSynchronize(lead->stream));
    for (int k = 0; k < count; ++k) {
        if (epochs_run) epochs_run[k] = ran[k];
        nets[k]->exClassRan = list[k].class_metrics ? ran[k] : 0;
        if (host_metrics && ran[k] > 0)
            memcpy(host_metrics + (size_t)k * n_epochs, all.data() + (size_t)k * n_epochs, sizeof(ghip_metrics) * ran[k]);
    }
    return 0;
}

int ghip_net_train_step(ghip_net* n, int64_t row0, int batch, ghip_metrics* host_metrics)
{
    if (!n || batch < 1 || row0 < 0) return fail(GHIP_EINVAL, "bad arguments");
    HIP_TRY(hipSetDevice(g_device));
    if (!is_canon(n)) return fail(GHIP_ESTATE, "network is not in canonical mode");
    if (n->spec.dtype == GHIP_FP8_INFER) return fail(GHIP_ESTATE, "fp8 networks are inference only");
    if (!n->dX || !n->dY) return fail(GHIP_ESTATE, "no dataset");
    if (row0 + batch > n->n_rows) return fail(GHIP_EINVAL, "rows [%lld,%lld) exceed the table (%lld rows)", (long long)row0, (long long)(row0 + batch), (long long)n->n_rows);
    TRY(reserve_batch(n, batch));
    n->last_batch = batch;
    if (n->spec.dtype == GHIP_F32) TRY(step_f32(n, row0, batch));
    else TRY(step_bf16(n, row0, batch));
    if (host_metrics) return fetch_metrics(n, host_metrics);
    return 0;
}

int ghip_net_run_epoch_canonical(ghip_net* n, int batch, int train, ghip_metrics* host_metrics)
{
    if (!n || batch < 1 || !host_metrics) return fail(GHIP_EINVAL, "bad arguments");
    HIP_TRY(hipSetDevice(g_device));
    if (!is_canon(n)) return fail(GHIP_ESTATE, "network is not in canonical mode");
    if (!n->dX || !n->dY) return fail(GHIP_ESTATE, "no dataset");
    const ghip_net_spec& s = n->spec;
    const int L = s.n_layers;
    if (train && s.dtype == GHIP_FP8_INFER) return fail(GHIP_ESTATE, "fp8 networks are inference only");
    const int64_t N = n->n_rows;
    if (batch > N) batch = (int)N;
    TRY(reserve_batch(n, batch));
    if (s.dtype == GHIP_BF16) TRY(refresh_shadows(n));
    if (s.dtype == GHIP_F32 && use_narrow(n, batch)) {
        // the whole pass is one launch
        TRY(run_narrow(n, 0, N, batch, 1, train, 0.0f, 0, n->dAcc + 12));
        n->last_batch = (int)(N % batch ? N % batch : batch);
        double acc[4];
        HIP_TRY(hipMemcpyAsync(acc, n->dAcc + 12, sizeof(acc), hipMemcpyDeviceToHost, n->stream));
        HIP_TRY(hipStreamSynchronize(n->stream));
        host_metrics->loss = (float)(acc[0] / (double)N);
        host_metrics->accuracy = (float)(acc[1] / ((double)N * s.sizes[L]));
        host_metrics->correct = (int64_t)(acc[2] + 0.5);
        return 0;
    }
    LAUNCH(n, "fill_pass_metrics", ghip_fill_f64(n->dAcc + 12, 4, 0.0, n->stream));
    n->passAcc = true;
    int rc = 0;
    for (int64_t r0 = 0; r0 < N && rc == 0; r0 += batch) {
        const int b = (int)(N - r0 < batch ? N - r0 : batch);
        if (train) {
            rc = (s.dtype == GHIP_F32) ? step_f32(n, r0, b) : step_bf16(n, r0, b);
        } else {
            float* P = nullptr;
            if (s.dtype == GHIP_F32) { rc = forward_f32(n, n->dX + r0 * s.sizes[0], b, L, canon_drop(n, r0)); P = n->act[L]; }
            else if (s.dtype == GHIP_BF16) { rc = forward_bf16(n, n->Xbf + r0 * n->ps[0], b); P = n->logits; }
            else { rc = forward_fp8(n, n->Xbf + r0 * n->ps[0], b, n->out8); P = n->out8; }
            if (rc == 0) rc = output_delta_f32(n, P, n->dY + r0 * s.sizes[L], nullptr, nullptr, b);
        }
        n->last_batch = b;
    }
    n->passAcc = false;
    if (rc != 0) return rc;
    if (canon_drop_on(n)) ++n->canMaskEpoch;   // the next pass takes the next epoch's flags; past the last, none
    double acc[4];
    HIP_TRY(hipMemcpyAsync(acc, n->dAcc + 12, sizeof(acc), hipMemcpyDeviceToHost, n->stream));
    HIP_TRY(hipStreamSynchronize(n->stream));
    host_metrics->loss = (float)(acc[0] / (double)N);
    host_metrics->accuracy = (float)(acc[1] / ((double)N * s.sizes[L]));
    host_metrics->correct = (int64_t)(acc[2] + 0.5);
    return 0;
}

int ghip_net_run_epochs_canonical(ghip_net* n, int batch, int n_epochs, int train, float stop_accuracy,
                                  ghip_metrics* host_metrics, int* epochs_run)
{
    if (!n || batch < 1 || n_epochs < 1 || !host_metrics) return fail(GHIP_EINVAL, "bad arguments");
    HIP_TRY(hipSetDevice(g_device));
    if (!is_canon(n)) return fail(GHIP_ESTATE, "network is not in canonical mode");
    if (!n->dX || !n->dY) return fail(GHIP_ESTATE, "no dataset");
    const ghip_net_spec& s = n->spec;
    const int64_t N = n->n_rows;
    if (batch > N) batch = (int)N;
    if (canon_drop_on(n) && n_epochs > n->exMaskEpochs - n->canMaskEpoch)
        return fail(GHIP_EINVAL, "%d epochs asked for, dropout flags for %d", n_epochs, n->exMaskEpochs - n->canMaskEpoch);
    if (s.dtype == GHIP_F32 && use_narrow(n, batch)) {
        // narrow network: the epochs are one launch, the stop condition is looked at on the device
        if (n_epochs > n->narrowEpochsCap) {
            (void)hipStreamSynchronize(n->stream);
            dfree(n->narrowEpochs);
            TRY(dalloc(&n->narrowEpochs, (size_t)4 * n_epochs));
            n->narrowEpochsCap = n_epochs;
        }
        TRY(run_narrow(n, 0, N, batch, n_epochs, train, stop_accuracy, n->cm ? 1 : 0, n->narrowEpochs));
        n->last_batch = (int)(N % batch ? N % batch : batch);
        int ran = 0;
        HIP_TRY(hipMemcpyAsync(&ran, n->narrowRan, sizeof(int), hipMemcpyDeviceToHost, n->stream));
        HIP_TRY(hipStreamSynchronize(n->stream));
        if (ran < 0 || ran > n_epochs) return fail(GHIP_EHIP, "the kernel reports %d epochs", ran);
        std::vector<double> acc((size_t)4 * (ran > 0 ? ran : 1));
        if (ran > 0) HIP_TRY(hipMemcpy(acc.data(), n->narrowEpochs, sizeof(double) * 4 * ran, hipMemcpyDeviceToHost));
        for (int e = 0; e < ran; ++e) {
            host_metrics[e].loss = (float)(acc[4 * e] / (double)N);
            host_metrics[e].accuracy = (float)(acc[4 * e + 1] / ((double)N * s.sizes[s.n_layers]));
            host_metrics[e].correct = (int64_t)(acc[4 * e + 2] + 0.5);
        }
        if (epochs_run) *epochs_run = ran;
        return 0;
    }
    int ran = 0;
    for (int e = 0; e < n_epochs; ++e) {
        if (n->cm) TRY(ghip_net_confusion_reset(n));   // CMatrix::reset at the head of every epoch (network.cpp:183-185)
        TRY(ghip_net_run_epoch_canonical(n, batch, train, host_metrics + e));
        ++ran;
        if (stop_accuracy > 0.0f && host_metrics[e].accuracy >= stop_accuracy) break;
    }
    if (epochs_run) *epochs_run = ran;
    return 0;
}

int ghip_net_set_canonical_path(ghip_net* n, int path)
{
    if (!n || !is_canon(n)) return fail(GHIP_EINVAL, "not a canonical network");
    if (path != GHIP_CANON_PATH_AUTO && path != GHIP_CANON_PATH_LAUNCHES && path != GHIP_CANON_PATH_ONE_WORKGROUP)
        return fail(GHIP_EINVAL, "unknown path %d", path);
    if (path == GHIP_CANON_PATH_ONE_WORKGROUP && !n->narrow_fit)
        return fail(GHIP_EINVAL, "the one-workgroup kernel takes fp32 networks whose layers are at most 64 wide and fit its LDS");
    n->canon_path = path;
    return 0;
}

int ghip_net_last_metrics(ghip_net* n, ghip_metrics* m)
{
    if (!n || !m) return fail(GHIP_EINVAL, "bad arguments");
    if (!is_canon(n)) return fail(GHIP_ESTATE, "network is not in canonical mode");
    return fetch_metrics(n, m);
}

static int forward_any(ghip_net* n, const float* dev_X32, const uint16_t* dev_Xbf, int batch, float** result)
{
    const ghip_net_spec& s = n->spec;
    const int L = s.n_layers;
    if (s.dtype == GHIP_F32) {
        TRY(forward_f32(n, dev_X32, batch, n->spec.n_layers));
        if (s.act[L - 1] == GHIP_SOFTMAX) {
            DeltaArgs a;
            memset(&a, 0, sizeof(a));
            a.P = n->act[L]; a.B = batch; a.n = s.sizes[L]; a.ldp = s.sizes[L]; a.ldy = s.sizes[L];
            a.act = GHIP_SOFTMAX; a.cost = s.cost; a.acc = n->dAcc + 8; a.store_p = 1;
            LAUNCH(n, "softmax", ghip_output_delta(a, n->stream));
        }
        *result = n->act[L];
    } else if (s.dtype == GHIP_BF16) {
        TRY(refresh_shadows(n));
        TRY(forward_bf16(n, dev_Xbf, batch));
        if (s.act[L - 1] == GHIP_SOFTMAX) {
            DeltaArgs a;
            memset(&a, 0, sizeof(a));
            a.P = n->logits; a.B = batch; a.n = s.sizes[L]; a.ldp = n->ps[L]; a.ldy = s.sizes[L];
            a.act = GHIP_SOFTMAX; a.cost = s.cost; a.acc = n->dAcc + 8; a.store_p = 1;
            LAUNCH(n, "softmax", ghip_output_delta(a, n->stream));
        }
        *result = n->logits;
    } else {
        TRY(forward_fp8(n, dev_Xbf, batch, n->out8));
        *result = n->out8;
    }
    return 0;
}

int ghip_net_forward(ghip_net* n, const float* host_X, int batch, float* host_out)
{
    if (!n || !host_X || !host_out || batch < 1) return fail(GHIP_EINVAL, "bad arguments");
    HIP_TRY(hipSetDevice(g_device));
    if (!is_canon(n)) return fail(GHIP_ESTATE, "network is not in canonical mode");
    const ghip_net_spec& s = n->spec;
    TRY(reserve_batch(n, batch));
    HIP_TRY(hipMemcpyAsync(n->stageX, host_X, (size_t)batch * s.sizes[0] * 4, hipMemcpyHostToDevice, n->stream));
    uint16_t* xbf = nullptr;
    if (s.dtype != GHIP_F32) {
        // the bf16 copy of the staged rows goes to a buffer the forward pass only overwrites after
        // having consumed it (transposed-input buffer for bf16, activation scratch for fp8)
        xbf = (s.dtype == GHIP_BF16) ? n->HT[0] : n->Hq;
        LAUNCH(n, "f32_to_bf16_input", ghip_f32_to_bf16_2d_pad(n->stageX, batch, s.sizes[0], xbf, nullptr, pad_batch(n, batch), n->ps[0], n->stream));
    }
    float* res = nullptr;
    TRY(forward_any(n, n->stageX, xbf, batch, &res));
    const int nout = s.sizes[s.n_layers];
    if (n->ps[s.n_layers] == nout) HIP_TRY(hipMemcpyAsync(host_out, res, (size_t)batch * nout * 4, hipMemcpyDeviceToHost, n->stream));
    else HIP_TRY(copy_matrix(res, n->ps[s.n_layers], host_out, batch, nout, false, n->stream));
    HIP_TRY(hipStreamSynchronize(n->stream));
    return 0;
}

int ghip_net_forward_resident(ghip_net* n, int64_t row0, int batch, float* dev_out)
{
    if (!n || batch < 1 || row0 < 0) return fail(GHIP_EINVAL, "bad arguments");
    HIP_TRY(hipSetDevice(g_device));
    if (!is_canon(n)) return fail(GHIP_ESTATE, "network is not in canonical mode");
    if (!n->dX) return fail(GHIP_ESTATE, "no dataset");
    if (row0 + batch > n->n_rows) return fail(GHIP_EINVAL, "rows exceed the table");
    const ghip_net_spec& s = n->spec;
    TRY(reserve_batch(n, batch));
    float* res = nullptr;
    TRY(forward_any(n, n->dX + row0 * s.sizes[0], n->Xbf ? n->Xbf + row0 * n->ps[0] : nullptr, batch, &res));
    const int nout = s.sizes[s.n_layers];
    if (dev_out && n->ps[s.n_layers] == nout) HIP_TRY(hipMemcpyAsync(dev_out, res, (size_t)batch * nout * 4, hipMemcpyDeviceToDevice, n->stream));
    else if (dev_out)
        HIP_TRY(hipMemcpy2DAsync(dev_out, (size_t)nout * 4, res, (size_t)n->ps[s.n_layers] * 4, (size_t)nout * 4, batch, hipMemcpyDeviceToDevice, n->stream));
    return 0;
}

int ghip_forward_noalloc(const ghip_net_spec* spec, const float* const* dev_W, const float* const* dev_bias,
                         const float* dev_X, int batch, float* dev_out, void* hip_stream)
{
    if (check_spec(spec)) return GHIP_EINVAL;
    if (!dev_W || !dev_bias || !dev_X || !dev_out || batch < 1) return fail(GHIP_EINVAL, "bad arguments");
    if (spec->mode != GHIP_MODE_CANONICAL || spec->dtype != GHIP_F32)
        return fail(GHIP_EINVAL, "ghip_forward_noalloc is the canonical fp32 forward only");
    const int L = spec->n_layers;
    for (int l = 0; l < L; ++l)
        if (!dev_W[l] || !dev_bias[l]) return fail(GHIP_EINVAL, "layer %d: weights or biases are NULL", l);
    // the kernels' 16-byte accesses: a pointer off that grid would quietly take the slow variants
    bool aligned = (((uintptr_t)dev_X | (uintptr_t)dev_out) % 16) == 0;
    for (int l = 0; l < L; ++l) aligned = aligned && (((uintptr_t)dev_W[l] | (uintptr_t)dev_bias[l]) % 16) == 0;
    if (!aligned) return fail(GHIP_EINVAL, "ghip_forward_noalloc takes 16-byte aligned device pointers");
    for (int l = 1; l < L; ++l)
        if ((int64_t)batch * spec->sizes[l] > (int64_t)GHIP_NOALLOC_MAX_ACTIVATIONS)
            return fail(GHIP_EINVAL, "batch %d x hidden layer %d of %d units = %lld activations: the fixed scratch of this entry point "
                        "holds %lld per layer; use ghip_net_forward_resident or a smaller batch",
                        batch, l, spec->sizes[l], (long long)batch * spec->sizes[l], (long long)GHIP_NOALLOC_MAX_ACTIVATIONS);
    int device = -1;
    HIP_TRY(hipGetDevice(&device));
    unsigned char* sp = nullptr;
    TRY(scratch_for_device(device, &sp));
    // A network object on the stack that owns nothing: the caller's parameters, the caller's stream,
    // hidden activations in the two halves of the scratch array, the last layer straight into dev_out.
    ghip_net n;
    n.spec = *spec;
    n.L = L;
    set_padded_sizes(&n);
    n.stream = (hipStream_t)hip_stream;
    for (int l = 0; l < L; ++l) {
        n.W[l] = const_cast<float*>(dev_W[l]);
        n.b[l] = const_cast<float*>(dev_bias[l]);
        n.act[l + 1] = (l == L - 1) ? dev_out : (float*)(sp + kScratchHeader + (size_t)(l & 1) * kScratchHalf);
    }
    // the softmax pass adds its row sums into accumulators nobody reads: they need no clearing
    n.dAcc = (double*)sp;
    float* res = nullptr;
    TRY(forward_any(&n, dev_X, nullptr, batch, &res));
    return 0;
}

int ghip_net_eval_resident(ghip_net* n, int64_t row0, int batch, ghip_metrics* host_metrics)
{
    if (!n || batch < 1 || row0 < 0 || !host_metrics) return fail(GHIP_EINVAL, "bad arguments");
    HIP_TRY(hipSetDevice(g_device));
    if (!is_canon(n)) return fail(GHIP_ESTATE, "network is not in canonical mode");
    if (!n->dX || !n->dY) return fail(GHIP_ESTATE, "no dataset");
    if (row0 + batch > n->n_rows) return fail(GHIP_EINVAL, "rows exceed the table");
    const ghip_net_spec& s = n->spec;
    TRY(reserve_batch(n, batch));
    const int L = s.n_layers;
    float* P = nullptr;
    if (s.dtype == GHIP_F32) { TRY(forward_f32(n, n->dX + row0 * s.sizes[0], batch, L, canon_drop(n, row0))); P = n->act[L]; }
    else if (s.dtype == GHIP_BF16) { TRY(refresh_shadows(n)); TRY(forward_bf16(n, n->Xbf + row0 * n->ps[0], batch)); P = n->logits; }
    else { TRY(forward_fp8(n, n->Xbf + row0 * n->ps[0], batch, n->out8)); P = n->out8; }
    TRY(output_delta_f32(n, P, n->dY + row0 * s.sizes[L], nullptr, nullptr, batch));
    n->last_batch = batch;
    return fetch_metrics(n, host_metrics);
}

int ghip_net_confusion_enable(ghip_net* n, int enable)
{
    if (!n) return fail(GHIP_EINVAL, "net is NULL");
    HIP_TRY(hipStreamSynchronize(n->stream));
    dfree(n->cm);
    if (!enable) return 0;
    const int nout = n->spec.sizes[n->L];
    if (nout > 8192) return fail(GHIP_EINVAL, "confusion matrix of %d classes is not supported", nout);
    TRY(dalloc(&n->cm, (size_t)nout * nout));
    HIP_TRY(hipMemsetAsync(n->cm, 0, sizeof(int) * (size_t)nout * nout, n->stream));
    return 0;
}

int ghip_net_confusion_reset(ghip_net* n)
{
    if (!n) return fail(GHIP_EINVAL, "net is NULL");
    if (!n->cm) return fail(GHIP_ESTATE, "confusion matrix is not enabled");
    const int nout = n->spec.sizes[n->L];
    LAUNCH(n, "fill_confusion", ghip_fill_u32((unsigned int*)n->cm, (long long)nout * nout, 0u, n->stream));
    return 0;
}

int ghip_net_confusion_get(ghip_net* n, int32_t* host_matrix, int64_t len)
{
    if (!n || !host_matrix) return fail(GHIP_EINVAL, "bad arguments");
    if (!n->cm) return fail(GHIP_ESTATE, "confusion matrix is not enabled");
    const int64_t nout = n->spec.sizes[n->L];
    if (len != nout * nout) return fail(GHIP_EINVAL, "matrix has %lld cells, caller gave room for %lld", (long long)(nout * nout), (long long)len);
    HIP_TRY(hipMemcpyAsync(host_matrix, n->cm, sizeof(int32_t) * len, hipMemcpyDeviceToHost, n->stream));
    HIP_TRY(hipStreamSynchronize(n->stream));
    return 0;
}

int ghip_net_class_metrics(ghip_net* n, int epoch, ghip_class_metrics* out)
{
    if (!n || !out) return fail(GHIP_EINVAL, "bad arguments");
    if (n->spec.mode != GHIP_MODE_EXACT) return fail(GHIP_ESTATE, "per-epoch class metrics are an exact-mode figure");
    if (epoch < 0 || epoch >= n->exClassRan)
        return fail(GHIP_EINVAL, "epoch %d of %d with class metrics (enable the confusion matrix before the run; n_out <= 64)", epoch, n->exClassRan);
    HIP_TRY(hipMemcpyAsync(out, n->exClass + 5 * epoch, sizeof(float) * 5, hipMemcpyDeviceToHost, n->stream));
    HIP_TRY(hipStreamSynchronize(n->stream));
    return 0;
}

int ghip_net_quantize_fp8(ghip_net* n, float* const* host_scales, uint8_t* const* host_codes)
{
    if (!n) return fail(GHIP_EINVAL, "net is NULL");
    const ghip_net_spec& s = n->spec;
    if (!is_canon(n) || s.dtype != GHIP_FP8_INFER) return fail(GHIP_ESTATE, "network was not created with GHIP_FP8_INFER");
    for (int l = 0; l < s.n_layers; ++l)
        LAUNCH(n, "quant_weights_e4m3", ghip_quant_rows_e4m3(n->W[l], 0, n->ps[l + 1], n->ps[l], n->Wq[l], n->wscale[l], nullptr, 0, n->stream));
    HIP_TRY(hipStreamSynchronize(n->stream));
    n->quantized = true;
    for (int l = 0; l < s.n_layers; ++l) {
        if (host_scales && host_scales[l]) HIP_TRY(hipMemcpy(host_scales[l], n->wscale[l], (size_t)s.sizes[l + 1] * 4, hipMemcpyDeviceToHost));
        if (host_codes && host_codes[l])
            HIP_TRY(hipMemcpy2D(host_codes[l], (size_t)s.sizes[l], n->Wq[l], (size_t)n->ps[l], (size_t)s.sizes[l], s.sizes[l + 1], hipMemcpyDeviceToHost));
    }
    return 0;
}

int ghip_net_set_fp8_activation_scaling(ghip_net* n, int mode)
{
    if (!n || n->spec.mode != GHIP_MODE_CANONICAL || n->spec.dtype != GHIP_FP8_INFER) return fail(GHIP_EINVAL, "not an e4m3 inference network");
    if (mode != GHIP_FP8_ACT_PER_TOKEN && mode != GHIP_FP8_ACT_BLOCK32) return fail(GHIP_EINVAL, "unknown activation scaling %d", mode);
    n->fp8_act_mode = mode;
    return 0;
}

int ghip_quantize_rows_e4m3_block32(const float* host_x, int64_t rows, int cols, uint8_t* host_codes, uint8_t* host_scales)
{
    if (!host_x || !host_codes || !host_scales || rows <= 0 || rows > (1 << 24) || cols <= 0) return fail(GHIP_EINVAL, "bad arguments");
    const int pc = (cols + 127) / 128 * 128, nblk = (cols + 31) / 32, R = (int)rows;
    float* dx = nullptr; uint16_t* dbf = nullptr; uint8_t* dq = nullptr; unsigned int* dsc = nullptr;
    std::vector<unsigned int> sc((size_t)(pc / 128) * R);
    int rc = 0;
    auto run = [&]() -> int {
        TRY(dalloc(&dx, (size_t)R * cols)); TRY(dalloc(&dbf, (size_t)R * pc)); TRY(dalloc(&dq, (size_t)R * pc)); TRY(dalloc(&dsc, sc.size()));
        HIP_TRY(hipMemcpy(dx, host_x, (size_t)R * cols * sizeof(float), hipMemcpyHostToDevice));
        HIP_TRY(ghip_f32_to_bf16_2d_pad(dx, R, cols, dbf, nullptr, R, pc, nullptr));
        HIP_TRY(ghip_quant_rows_mx(dbf, R, pc, dq, dsc, R, nullptr));
        HIP_TRY(hipMemcpy2D(host_codes, (size_t)cols, dq, (size_t)pc, (size_t)cols, (size_t)R, hipMemcpyDeviceToHost));
        HIP_TRY(hipMemcpy(sc.data(), dsc, sc.size() * sizeof(unsigned int), hipMemcpyDeviceToHost));
        return 0;
    };
    rc = run();
    dfree(dx); dfree(dbf); dfree(dq); dfree(dsc);
    if (rc) return rc;
    for (int r = 0; r < R; ++r)
        for (int b = 0; b < nblk; ++b) host_scales[(size_t)r * nblk + b] = (uint8_t)(sc[(size_t)(b / 4) * R + r] >> (8 * (b % 4)));
    return 0;
}

int ghip_net_sync(ghip_net* n)
{
    if (!n) return fail(GHIP_EINVAL, "net is NULL");
    HIP_TRY(hipStreamSynchronize(n->stream));
    return 0;
}

int ghip_net_profile(ghip_net* n, int enable)
{
    if (!n) return fail(GHIP_EINVAL, "net is NULL");
    prof_collect(n);
    n->prof = enable != 0;
    return 0;
}
int ghip_net_profile_count(ghip_net* n)
{
    if (!n) return fail(GHIP_EINVAL, "net is NULL");
    prof_collect(n);
    return (int)n->aggs.size();
}
int ghip_net_profile_entry(ghip_net* n, int index, char* name, int name_len, double* total_ms, int64_t* launches)
{
    if (!n) return fail(GHIP_EINVAL, "net is NULL");
    prof_collect(n);
    if (index < 0 || index >= (int)n->aggs.size()) return fail(GHIP_EINVAL, "profile index out of range");
    const ProfAgg& g = n->aggs[index];
    if (name && name_len > 0) { strncpy(name, g.name.c_str(), name_len - 1); name[name_len - 1] = 0; }
    if (total_ms) *total_ms = g.ms;
    if (launches) *launches = g.n;
    return 0;
}
int ghip_net_profile_reset(ghip_net* n)
{
    if (!n) return fail(GHIP_EINVAL, "net is NULL");
    prof_collect(n);
    n->aggs.clear();
    return 0;
}

}  // extern "C"

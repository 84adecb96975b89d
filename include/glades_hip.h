/*
 * glades_hip.h -- C ABI of the MI355X (gfx950) dense feed-forward path for Glades.
 *
 * The reference (Gattic/glades-ml) has no plugin or FFI interface: its boundary for this
 * path is the C++ class API (NNInfo / NNetwork / Terminator / DataInput / glades::train).
 * These entry points are what a binding of that API to the GPU needs; each one names the
 * reference code it stands in for ("ML/" = "Backend/Machine Learning/").  The C++ mirror of
 * the class API that sits on top of this header is glades-ml_amd/host/glades.h.
 *
 * Conventions: every function returns 0 on success and a negative GHIP_E* code on failure
 * (no exceptions, nothing is thrown across the boundary); ghip_last_error() gives the
 * message of the calling thread's last failure.  Pointers named host_* are host memory the
 * caller owns; pointers named dev_* are device memory the caller owns and keeps alive while
 * the network uses it.  Everything else on the device is owned by the handle.  A handle owns
 * one HIP stream; calls on one handle must not overlap (same as the reference: single
 * threaded per network); different handles are independent.
 *
 * Matrices are dense row-major.  Weights of weight-layer l are [sizes[l+1]][sizes[l]]
 * (row o = the incoming edges of node o, the reference's Node::edges order, node.h:45).
 */
#ifndef GLADES_HIP_H
#define GLADES_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GHIP_MAX_LAYERS 16

/* activation ids = ML/GMath/gmath.h:43-50; SOFTMAX (canonical mode, output layer only) is an
 * extension the reference does not have */
enum { GHIP_TANH = 0, GHIP_TANHP = 1, GHIP_SIGMOID = 2, GHIP_SIGMOIDP = 3, GHIP_LINEAR = 4,
       GHIP_RELU = 5, GHIP_LEAKY = 6, GHIP_STEP = 7, GHIP_SOFTMAX = 8 };
/* cost ids = ML/GMath/gmath.h:38-40 */
enum { GHIP_REGRESSION = 0, GHIP_CLASSIFICATION = 1, GHIP_KL = 2 };

enum {
    GHIP_MODE_EXACT = 0,     /* the reference's per-sample sequential semantics, quirk for quirk
                                (ML/Networks/network.cpp:399-668) */
    GHIP_MODE_CANONICAL = 1  /* batched training: reference forward, true dL/dz backward,
                                per-channel bias, momentum across steps */
};
enum {
    GHIP_F32 = 0,       /* fp32 storage and arithmetic */
    GHIP_BF16 = 1,      /* canonical only: bf16 weights/activations, fp32 accumulate, fp32 master */
    GHIP_FP8_INFER = 2  /* canonical, forward only: e4m3 weights (per-output-channel scale) and
                           e4m3 activations (per-row scale), fp32 accumulate */
};
enum { GHIP_BIAS_SEQUENTIAL = 0, /* exact mode: repeat "bias -= lr*delta" once per (input, output)
                                    pair in the reference's order (network.cpp:654-656) */
       GHIP_BIAS_CLOSED_FORM = 1 /* exact mode: bias -= n_in * sum_o(lr*delta_o), one rounding
                                    instead of n_in*n_out; faster, not bit-faithful */ };

#define GHIP_EINVAL   (-1)  /* bad argument / unsupported shape for the chosen dtype */
#define GHIP_ENOMEM   (-2)
#define GHIP_EHIP     (-3)  /* a HIP runtime call failed */
#define GHIP_ESTATE   (-4)  /* call order: no dataset, wrong mode, ... */
#define GHIP_ENODEV   (-5)  /* no usable gfx950 device */

typedef struct ghip_net ghip_net;

/* Resolved hyper-parameters: what NNInfo's index-shifted getters return for weight layer l
 * (ML/Structure/nninfo.cpp:240-373: index 0 reads the input row, index k the hidden row k-1). */
typedef struct {
    int   n_layers;                    /* weight layers = hidden layers + 1, 1..GHIP_MAX_LAYERS */
    int   sizes[GHIP_MAX_LAYERS + 1];  /* sizes[0] features ... sizes[n_layers] outputs */
    float lr[GHIP_MAX_LAYERS];
    float mom[GHIP_MAX_LAYERS];
    float wd1[GHIP_MAX_LAYERS];
    float wd2[GHIP_MAX_LAYERS];
    int   act[GHIP_MAX_LAYERS];        /* activation producing layer l+1 */
    float act_param[GHIP_MAX_LAYERS];
    int   batch;                       /* NNInfo::getBatchSize(); exact mode needs >= 1 */
    int   cost;                        /* NNInfo::getOutputType() */
    int   mode;                        /* GHIP_MODE_* */
    int   dtype;                       /* GHIP_F32 / GHIP_BF16 / GHIP_FP8_INFER */
    int   bias_mode;                   /* GHIP_BIAS_* (exact mode) */
} ghip_net_spec;

/* Per-epoch (exact) or per-step (canonical) figures.
 * exact:     loss = overallTotalError, accuracy = overallTotalAccuracy (network.cpp:533-547,194-195)
 * canonical: loss = mean per-sample loss, accuracy = the same 0..100 measure over the batch
 * correct = rows whose argmax equals the label's under the reference rule (gmath.cpp:412-455) */
typedef struct {
    float   loss;
    float   accuracy;
    int64_t correct;
} ghip_metrics;

/* Selects the device and checks that it is a gfx950.  Stands in for glades::init()
 * (ML/main.cpp:51-56) as the once-per-process set-up call.  It also makes the HIP runtime finish
 * its own lazy set-up (first stream, first allocation), which draws from libc rand(): seed rand()
 * AFTER this call and the stream the reference's weight sampler (ML/State/node.cpp:241-276) and
 * dropout (ML/State/layer.cpp:102-134) read stays reproducible. */
int ghip_init(int device_ordinal);

/* The element-wise functions of the path over arrays, with exact mode's arithmetic (what one row of
 * the persistent kernel applies to one node), for callers and tests that want them on their own:
 * fn 0  GMath::squash(a[k], kind, param)                       ML/GMath/gmath.cpp:22-101
 * fn 1  GMath::activationErrDer(a[k], kind, param)             ML/GMath/gmath.cpp:182-245
 * fn 2  GMath::outputNodeCost(expected a[k], predicted b[k], dataSize = param, cost kind)  :272-321
 * fn 3  GMath::costErrDer(expected a[k], predicted b[k], cost kind)                        :323-353
 * fn 4  the scalar layer bias after one row's back-propagation (ML/Networks/network.cpp:654-656: bias -= lr*d[o]
 *       once per (input, output) pair, outputs innermost): a[k] the bias before, host_b[64*k .. 64*k+63] the
 *       lr*d of up to 64 outputs (zeros past the last), param = number of input nodes (rounds).
 *       kind 0 walks the n_in * 64 subtractions; kind 1 is what the persistent kernel does: an
 *       integer-arithmetic shortcut where it is provably the same float, else the walk; kind 2 returns
 *       1.0 where that shortcut applies, else 0.0
 * kind is an activation id for fn 0/1 and a cost id for fn 2/3; host_b is unused for fn 0/1.  tanh, exp
 * and log return the floats of the reference platform's C library (GNU libc 2.35), bit for bit. */
int ghip_gmath_eval(int fn, int kind, float param, const float* host_a, const float* host_b, float* host_out, int64_t n);

/* Builds the device-side network: replaces LayerBuilder::build (ML/State/LayerBuilder.cpp:54-98)
 * minus the weight sampling, which stays with the caller (ghip_net_set_params). */
int ghip_net_create(const ghip_net_spec* spec, ghip_net** out);
int ghip_net_destroy(ghip_net* net);

/* Weight / bias transfer: replaces Node::setEdgeWeight / getEdgeWeight (ML/State/node.cpp:60-66,
 * 142-148) and Layer::setBiasWeight / getBiasWeight (ML/State/layer.cpp:52-74).
 * exact mode:     bias_len is 0 or 1; the scalar is the bias of layer `layer` (added to layer
 *                 layer+1; ignored for layer 0, network.cpp:501-502).
 * canonical mode: bias_len is 0 or sizes[layer+1] (per output channel).
 * host_W may be NULL in get to fetch the bias only.  Setting parameters clears momentum. */
int ghip_net_set_params(ghip_net* net, int layer, const float* host_W, const float* host_bias, int bias_len);
int ghip_net_get_params(ghip_net* net, int layer, float* host_W, float* host_bias, int bias_len);

/* What a checkpoint needs beyond the parameters, so that a restored network continues exactly as the
 * original would have (the reference's NNetwork::save writes the NNInfo table only and leaves the
 * weights to a stub, ML/Networks/network.cpp:714-743, so there is no reference format to follow).
 * exact mode:     a = pending-delta running sums, b = last pending delta, each sizes[layer+1] x
 *                 sizes[layer] row-major: the content of the reference's Edge::prevDelta windows
 *                 (ML/State/edge.cpp:54-101), which survive from one epoch into the next.
 * canonical mode: a = weight momentum (previous update) sizes[layer+1] x sizes[layer],
 *                 b = bias momentum sizes[layer+1].
 * Either pointer may be NULL.  ghip_net_set_params clears this state: set the parameters first.
 * Exact mode: the windows' lengths are implied for a network that has never run with dropout (every
 * edge of a layer holds the same number of entries); one that has carries them separately, see
 * ghip_net_get_dropout_state. */
int ghip_net_get_state(ghip_net* net, int layer, float* host_a, float* host_b);
int ghip_net_set_state(ghip_net* net, int layer, const float* host_a, const float* host_b);

/* Dropout (exact mode): replaces LayerBuilder::scrambleDropout (ML/State/LayerBuilder.cpp:497-523)
 * as the source of the per-row flags and Layer::possiblePath / lastValidPath
 * (ML/State/layer.cpp:136-183) as their readers.  The caller draws the flags -- the reference draws
 * them from libc rand() (Layer::generateDropout, ML/State/layer.cpp:102-134), a stream that lives on
 * the host -- and hands over n_epochs x n_rows x (sizes[0] + ... + sizes[n_layers-1]) bytes: for
 * every epoch and row the node layers 0..n_layers-1 side by side, 1 = dropped.  The next
 * ghip_net_run_epochs_exact / _multi call (train or test: the reference scrambles in both,
 * ML/Networks/network.cpp:407-411) consumes them and must not ask for more epochs; later calls run
 * without dropout until flags are set again.  A row that drops every node of a layer is refused
 * (the reference redraws such a layer).  Needs the table (ghip_net_set_dataset) first.
 * NULL forgets flags that were set.
 * Canonical mode, fp32 networks: the same flags in the same layout.  A dropped node's activation is taken as 0 by
 * the layer above (the reference skips every edge that leaves it, ML/Networks/network.cpp:476-480, and rescales
 * nothing) and it gets no delta, in training and test passes alike.  Every pass of ghip_net_run_epoch_canonical /
 * ghip_net_run_epochs_canonical uses up one epoch of flags (a call may not ask for more epochs than are left);
 * ghip_net_train_step and ghip_net_eval_resident read the flags of their rows in the epoch that is next, without
 * using it up; ghip_net_forward* never drop.  Past the last epoch of flags the network runs without dropout.
 * bf16 / e4m3 networks refuse flags. */
int ghip_net_set_dropout_masks(ghip_net* net, const uint8_t* host_masks, int n_epochs);
/* What dropout leaves behind between rows, for checkpoints: the number of pending deltas of every
 * edge of weight layer `layer` (Edge::prevDelta.size(), ML/State/edge.cpp:64-67; sizes[layer+1] x
 * sizes[layer]: an edge that sat out an applying row keeps its window, and Node::applyDeltas reads
 * the first minibatchSize entries only, ML/State/node.cpp:294-307) and the error accumulators of
 * the nodes of layer `layer`+1 (Node::errorDer, cleared only by a valid pair with the last input
 * node, ML/Networks/network.cpp:629-631; sizes[layer+1]).  Either pointer may be NULL. */
int ghip_net_get_dropout_state(ghip_net* net, int layer, int32_t* host_counts, float* host_errder);
int ghip_net_set_dropout_state(ghip_net* net, int layer, const int32_t* host_counts, const float* host_errder);

/* Uploads the training table once: replaces LayerBuilder::buildInputLayers
 * (ML/State/LayerBuilder.cpp:100-190) and DataInput::getTrainRow / getTrainExpectedRow
 * (ML/DataObjects/DataInput.h:39-40).  X is N x sizes[0], Y is N x sizes[n_layers]. */
int ghip_net_set_dataset(ghip_net* net, const float* host_X, const float* host_Y, int64_t n_rows);
/* Same, for tables already resident in device memory (fp32); nothing is copied. */
int ghip_net_set_dataset_device(ghip_net* net, const float* dev_X, const float* dev_Y, int64_t n_rows);

/* Exact mode: n_epochs passes over the rows in order, each row = SGDHelper
 * (ML/Networks/network.cpp:399-455: ForwardPass :457-575, BackPropagation :577-668), one kernel
 * launch for the whole call.  train = 0 is the RUN_TEST pass (forward and metrics only).
 * stop_accuracy > 0 ends the call after the first epoch whose accuracy reaches it
 * (Terminator::triggered, ML/State/Terminator.cpp:73-74).  host_metrics receives one entry per
 * epoch run (n_epochs entries of room); *epochs_run says how many.  host_preds (may be NULL)
 * receives the last epoch's predictions, n_rows x sizes[n_layers]. */
int ghip_net_run_epochs_exact(ghip_net* net, int n_epochs, int train, float stop_accuracy,
                              ghip_metrics* host_metrics, int* epochs_run, float* host_preds);

/* The same for `count` networks of one specification and one table length at once, one workgroup
 * each: the subnets of a MetaNetwork, which the reference trains one after the other on the same
 * DataInput (ML/main.cpp:137-160, ML/Networks/metanetwork.cpp:216-251).  Narrow networks are bound
 * by the latency of their sequential rows, so the device's answer is many of them side by side.
 * All networks use the table of nets[0] (the caller has given every one the same data).
 * host_metrics: count x n_epochs entries, row k for nets[k]; epochs_run: count entries.
 * Every network stops on its own when it reaches stop_accuracy. */
int ghip_net_run_epochs_exact_multi(ghip_net* const* nets, int count, int n_epochs, int train, float stop_accuracy,
                                    ghip_metrics* host_metrics, int* epochs_run);

/* Canonical mode: one pass over the whole resident table in batches [k*batch, (k+1)*batch) (the last
 * one shorter and averaged over its true size), every step enqueued back to back and one
 * synchronisation at the end: the body of NNetwork::run's epoch loop (ML/Networks/network.cpp:171-191:
 * SGDHelper for every row, then the epoch's error and accuracy) for batched training.  train != 0:
 * forward, backward and update per batch; 0: forward and metrics only.  host_metrics: the pass's mean
 * per-sample loss, its accuracy and its count of rows whose predicted class is the expected one
 * (accumulated on the device over all batches).  ghip_net_last_metrics afterwards still refers to the
 * last ghip_net_train_step. */
int ghip_net_run_epoch_canonical(ghip_net* net, int batch, int train, ghip_metrics* host_metrics);

/* Canonical mode: up to n_epochs such passes, the epoch loop of NNetwork::run
 * (Backend/Machine Learning/Networks/network.cpp:171-195) with the Terminator's accuracy condition
 * (State/Terminator.cpp:63-78): host_metrics[e] receives epoch e's figures, *epochs_run how many were run;
 * the loop ends early once an epoch's accuracy reaches stop_accuracy (> 0).  The confusion counters, if
 * enabled, restart at the head of every epoch (network.cpp:183-185).  An fp32 network whose layers are all at
 * most 64 wide runs the whole call as ONE launch of one persistent workgroup (parameters, momentum and a
 * chunk of rows' activations in LDS; see ghip_net_set_canonical_path); other networks run pass by pass. */
int ghip_net_run_epochs_canonical(ghip_net* net, int batch, int n_epochs, int train, float stop_accuracy,
                                  ghip_metrics* host_metrics, int* epochs_run);

/* Canonical fp32 networks: which kernels train and evaluate them.  No reference counterpart.
 *   GHIP_CANON_PATH_AUTO (default): the one-workgroup kernel where it applies (every layer at most 64 wide,
 *     state fits the LDS) and the work of a batch is small enough for one CU to beat a step's seven launches;
 *   GHIP_CANON_PATH_LAUNCHES: always the GEMM / streaming launches;
 *   GHIP_CANON_PATH_ONE_WORKGROUP: always the one-workgroup kernel (refused where it does not apply).
 * Results agree to fp32 summation order either way. */
#define GHIP_CANON_PATH_AUTO          0
#define GHIP_CANON_PATH_LAUNCHES      1
#define GHIP_CANON_PATH_ONE_WORKGROUP 2
int ghip_net_set_canonical_path(ghip_net* net, int path);

/* Canonical mode: one training step (forward, backward, update) on rows [row0, row0+batch) of
 * the resident table.  host_metrics may be NULL (then the call does not synchronise). */
int ghip_net_train_step(ghip_net* net, int64_t row0, int batch, ghip_metrics* host_metrics);
/* Metrics of the most recent ghip_net_train_step (synchronises). */
int ghip_net_last_metrics(ghip_net* net, ghip_metrics* host_metrics);

/* Canonical mode forward of `batch` rows: the reference forward (network.cpp:457-516) as GEMMs.
 * host_X: batch x sizes[0] fp32, host_out: batch x sizes[n_layers] fp32. */
int ghip_net_forward(ghip_net* net, const float* host_X, int batch, float* host_out);
/* Forward of rows [row0,row0+batch) of the resident table; the result stays on the device and
 * dev_out (fp32, batch x sizes[n_layers], may be NULL) receives a device-to-device copy. */
int ghip_net_forward_resident(ghip_net* net, int64_t row0, int batch, float* dev_out);

/* No counterpart in the reference.  The canonical fp32 forward (as ghip_net_forward_resident: same
 * kernels, same results bit for bit) for callers that cannot allocate device memory: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It takes no handle and calls
 * no allocating routine: parameters, inputs and outputs are the caller's device memory (dev_W[l]:
 * sizes[l+1] x sizes[l] row-major, dev_bias[l]: sizes[l+1], dev_X: batch x sizes[0], dev_out: batch x
 * sizes[n_layers], all fp32, 16-byte aligned: other pointers are refused with GHIP_EINVAL), and the
 * hidden layers' activations live in a fixed
 * array in the library's device image (2 x GHIP_NOALLOC_MAX_ACTIVATIONS floats + 256 bytes = 32 MiB
 * per GPU, held until the process ends).  batch x sizes[l] of every hidden layer l must not exceed
 * GHIP_NOALLOC_MAX_ACTIVATIONS; larger requests are refused with GHIP_EINVAL.  spec: mode
 * GHIP_MODE_CANONICAL, dtype GHIP_F32.  The work is queued on hip_stream (a hipStream_t; NULL = the
 * null stream) of the calling thread's current device and the call does not wait for it.  All
 * calls on one GPU share that GPU's array: calls that overlap in time on one GPU race. */
#define GHIP_NOALLOC_MAX_ACTIVATIONS (4 * 1024 * 1024)
int ghip_forward_noalloc(const ghip_net_spec* spec, const float* const* dev_W, const float* const* dev_bias,
                         const float* dev_X, int batch, float* dev_out, void* hip_stream);

/* Canonical mode RUN_TEST pass (network.cpp:109-112,372-373) on rows [row0,row0+batch) of the
 * resident table: forward and metrics, no parameter changes. */
int ghip_net_eval_resident(ghip_net* net, int64_t row0, int batch, ghip_metrics* host_metrics);

/* Confusion matrix on the device: replaces CMatrix::addResult per sample (ML/GMath/cmatrix.cpp:57-98,
 * called from network.cpp:420-423) with counters the kernels that already compute both argmaxes
 * bump, so no prediction leaves the device for it.  n_out x n_out int32, row = expected class,
 * column = predicted class, both under the argmax rule of gmath.cpp:412-455 (a row with no
 * positive entry has no class and counts nowhere).
 * enable != 0 allocates and zeroes the counters; 0 frees them.
 * exact mode: the counters restart at every epoch (CMatrix::reset, network.cpp:183-185), so after
 *   ghip_net_run_epochs_exact they hold the last epoch run; ghip_net_class_metrics returns the
 *   overall accuracy / precision / recall / specificity / F1 of epoch `epoch` of that call
 *   (CMatrix::updateResultParams + getOverall*, cmatrix.cpp:100-265; network.cpp:218-224), as
 *   fractions, computed on the device at the epoch's end (n_out <= 64).
 * canonical mode: ghip_net_train_step / ghip_net_eval_resident add to the counters until
 *   ghip_net_confusion_reset. */
typedef struct {
    float accuracy, precision, recall, specificity, f1;
} ghip_class_metrics;
int ghip_net_confusion_enable(ghip_net* net, int enable);
int ghip_net_confusion_reset(ghip_net* net);
int ghip_net_confusion_get(ghip_net* net, int32_t* host_matrix, int64_t len);
int ghip_net_class_metrics(ghip_net* net, int epoch, ghip_class_metrics* host_out);

/* GHIP_FP8_INFER: quantises the current fp32 weights to e4m3 with one fp32 scale per output
 * channel (scale = amax(row)/448).  host_scales[l] (may be NULL) receives sizes[l+1] scales and
 * host_codes[l] (may be NULL) the sizes[l+1]*sizes[l] code bytes.  No reference counterpart (the
 * reference is fp32 only); checked against its fp32 forward on the dequantised weights. */
int ghip_net_quantize_fp8(ghip_net* net, float* const* host_scales, uint8_t* const* host_codes);

/* GHIP_FP8_INFER: how the activations are re-quantised to e4m3 between layers.  No reference counterpart.
 *   GHIP_FP8_ACT_BLOCK32 (default): every token (row) gets a power-of-two (E8M0) scale per 32 consecutive
 *     units, the block format gfx950's scaled MFMA takes as it is; the producing product's epilogue writes
 *     the codes and scales, so nothing runs between two layers' products.  Scale of a block = the power of
 *     two that brings its largest magnitude into (224, 448].
 *   GHIP_FP8_ACT_PER_TOKEN: one fp32 scale per token (row amax / 448) for the whole row; the product writes
 *     bf16 activations and row maxima, a second kernel re-quantises the rows.
 * Both quantise the bf16-rounded activations. */
#define GHIP_FP8_ACT_PER_TOKEN 0
#define GHIP_FP8_ACT_BLOCK32   1
int ghip_net_set_fp8_activation_scaling(ghip_net* net, int mode);

/* The GHIP_FP8_ACT_BLOCK32 quantiser on its own (what the products' epilogues apply between layers): host_x
 * [rows][cols] fp32 is rounded to bf16 and quantised on the device; host_codes [rows][cols] receives the
 * e4m3 codes, host_scales [rows][ceil(cols / 32)] the E8M0 bytes (value 2^(byte - 127)). */
int ghip_quantize_rows_e4m3_block32(const float* host_x, int64_t rows, int cols, uint8_t* host_codes, uint8_t* host_scales);

/* Blocks until everything queued on the handle's stream has finished. */
int ghip_net_sync(ghip_net* net);

/* Per-kernel timing with HIP events on the handle's stream.  While enabled, every kernel launch
 * of this handle is bracketed by events and accumulated under its name. */
int ghip_net_profile(ghip_net* net, int enable);
int ghip_net_profile_count(ghip_net* net);
int ghip_net_profile_entry(ghip_net* net, int index, char* name, int name_len, double* total_ms,
                           int64_t* launches);
int ghip_net_profile_reset(ghip_net* net);

const char* ghip_last_error(void);
const char* ghip_version(void);

#ifdef __cplusplus
}
#endif
#endif

/*
 * glades_oracle.h -- CPU restatement of the Glades dense feed-forward hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP path is compared
 * with (tests, the smoke check, the CPU-baseline leg of the benchmark).  The product
 * library never links, loads or calls it.
 *
 * Two semantics are restated (citations are to files under the reference tree,
 * "ML/" = "Backend/Machine Learning/"):
 *
 *  exact mode     the reference's per-sample sequential algorithm, quirk for quirk:
 *                 ML/Networks/network.cpp:457-575 (ForwardPass), :577-668
 *                 (BackPropagation), ML/State/node.cpp:82-93,278-307 (activation sum,
 *                 getDelta, applyDeltas), ML/State/edge.cpp:54-101 (delta window),
 *                 ML/GMath/gmath.cpp:22-101,182-353 (squash, derivatives, costs).
 *  canonical mode textbook minibatch training whose forward is the reference forward
 *                 (per-channel bias vector; an all-equal vector reproduces the
 *                 reference's scalar layer bias) and whose backward is true dL/dz
 *                 back-propagation with heavy-ball momentum across steps.
 *
 * Pinning status of each function (what, other than re-reading the source, says it
 * is right):
 *   go_squash / go_act_der / go_cost / go_cost_der / go_percent_error
 *       pinned: bit-compared with the reference's own compiled gmath.cpp over a grid
 *       (oracle/_ref harness, fixture tests/golden/gmath_grid.npz) and closed forms.
 *   go_ref_xavier_layer
 *       pinned: bit-compared with the reference's compiled Layer::initWeights /
 *       Node::initWeights under the same srand() seed (fixture xavier_*.npz).
 *   go_exact_*  (per-edge arithmetic: activation sum, getDelta, applyDeltas window,
 *       bias update, error accumulator)
 *       pinned: bit-compared with a harness that runs the reference's compiled
 *       Node/Edge/Layer/GMath objects through the network.cpp loop nest, plus
 *       closed forms (doubling accumulator pattern, n_in*lr*sum(delta) bias step,
 *       online-SGD reduction for a 1-node next layer).
 *       The loop NEST itself (network.cpp:457-668, LayerBuilder.cpp:269-336) cannot
 *       be compiled here (it needs the un-vendored shmea library); its order is
 *       restated from the source text in both the harness and this file:
 *       for that ordering alone -- parity unpinned by execution.
 *   go_dropout_draw / the dropout branches of go_exact_*  (layer.cpp:102-183, network.cpp:480-488,
 *       621-662)  pinned: the flags, the rand() stream position afterwards and the trained state
 *       are bit-compared with the reference's compiled Layer::generateDropout / possiblePath /
 *       lastValidPath and Node/Edge objects run through the same harness (fixtures
 *       tests/golden/dropout_*.npz); the loop nest is restated as above.
 *   go_canon_*  no counterpart in the reference (the reference has no batched
 *       training, softmax or per-channel bias): pinned against torch autograd +
 *       torch.optim.SGD and finite differences; forward pinned against go_exact
 *       forward (bit-exact for equal parameters, with and without dropout flags);
 *       go_canon_set_drop pinned by torch autograd through the masked network.
 *   go_cmatrix_*  ML/GMath/cmatrix.cpp needs the un-vendored shmea containers and cannot be
 *       compiled here: restated from the source text -- parity unpinned by execution; pinned
 *       by hand-computed matrices, the perfect-classifier closed form and brute force on
 *       tiny inputs (tests/test_oracle_cmatrix.py).
 *   go_bf16_* / go_e4m3_*  format conversions: pinned against torch's bf16 /
 *       float8_e4m3fn casts, exhaustive over all 256 e4m3 codes.
 */
#ifndef GLADES_ORACLE_H
#define GLADES_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GO_MAX_LAYERS 16

/* activation ids: ML/GMath/gmath.h:43-50; SOFTMAX is an extension (canonical only) */
enum { GO_TANH = 0, GO_TANHP = 1, GO_SIGMOID = 2, GO_SIGMOIDP = 3, GO_LINEAR = 4,
       GO_RELU = 5, GO_LEAKY = 6, GO_STEP = 7, GO_SOFTMAX = 8 };
/* cost ids: ML/GMath/gmath.h:38-40 */
enum { GO_REGRESSION = 0, GO_CLASSIFICATION = 1, GO_KL = 2 };

typedef struct {
    int   n_layers;                 /* weight layers = hidden layers + 1 */
    int   sizes[GO_MAX_LAYERS + 1]; /* sizes[0] = features ... sizes[n_layers] = outputs */
    float lr[GO_MAX_LAYERS];        /* hyper-parameters of weight layer l (the reference's */
    float mom[GO_MAX_LAYERS];       /* NNInfo getters with index l, nninfo.cpp:240-373)     */
    float wd1[GO_MAX_LAYERS];
    float wd2[GO_MAX_LAYERS];
    int   act[GO_MAX_LAYERS];       /* activation producing layer l+1 */
    float act_param[GO_MAX_LAYERS];
    int   batch;                    /* minibatchSize (exact) / informational (canonical) */
    int   cost;                     /* GO_REGRESSION / GO_CLASSIFICATION / GO_KL */
} go_spec;

typedef struct {
    float   loss;      /* exact: overallTotalError of the epoch; canonical: mean per-sample loss */
    float   accuracy;  /* reference accuracy 0..100 (network.cpp:541-547,194-195) */
    int64_t correct;   /* rows whose argmax (gmath.cpp:412-455 rule) equals the label's */
} go_metrics;

/* ---- element-wise (gmath.cpp) ---- */
float go_squash(float z, int act, float param);
float go_act_der(float a, int act, float param);
float go_cost(float expect, float pred, float data_size, int cost);
float go_cost_der(float expect, float pred, int cost);
float go_percent_error(float pred, float expect);
/* the four functions above over arrays: fn 0 squash(a), 1 act_der(a), 2 cost(expect a, pred b, data_size
   param), 3 cost_der(expect a, pred b); kind = activation or cost id */
void  go_eval(int fn, int kind, float param, const float* a, const float* b, float* out, int64_t n);
int   go_argmax_ref(const float* v, int n);  /* -1 when no element is > 0 */

/* confusion matrix, ML/GMath/cmatrix.cpp: M is n x n int32 row-major (row expected, column predicted) */
void go_cmatrix_add(int n, int32_t* M, const float* expected, const float* predicted);
void go_cmatrix_params(int n, const int32_t* M, int32_t* tp, int32_t* tn, int32_t* fp, int32_t* fn);
/* out[6]: overall accuracy, precision, recall, specificity, F1, false alarm (fractions) */
void go_cmatrix_overall(int n, const int32_t* tp, const int32_t* tn, const int32_t* fp, const int32_t* fn, float* out);

/* ---- the reference's weight sampler (layer.cpp:196-217, node.cpp:241-276); uses libc rand() ---- */
void  go_ref_xavier_layer(int fan_in, int n_out, int act_type, float* W /* n_out*fan_in */);

/* ---- exact mode ---- */
typedef struct go_exact go_exact;
go_exact* go_exact_create(const go_spec* spec);
void  go_exact_destroy(go_exact* n);
void  go_exact_set_weights(go_exact* n, int layer, const float* W);
void  go_exact_get_weights(const go_exact* n, int layer, float* W);
void  go_exact_set_bias(go_exact* n, int layer, float b);   /* scalar bias of layer `layer` (>=1) */
float go_exact_get_bias(const go_exact* n, int layer);
/* window state (running sum of the edge's pending deltas and the last one pushed) */
void  go_exact_get_window(const go_exact* n, int layer, float* sum, float* last);
/* one epoch over rows 0..N-1 in order. train=0: forward + metrics only.
   preds (N*n_out) may be NULL. */
void  go_exact_epoch(go_exact* n, const float* X, const float* Y, int64_t N, int train,
                     go_metrics* m, float* preds);

/* dropout: flags for one epoch, N rows x go_exact_mask_len() bytes (1 = dropped), the node layers
   0..n_layers-1 of a row side by side; NULL = nothing dropped.  The pointer is kept, not copied. */
int   go_exact_mask_len(const go_exact* n);
void  go_exact_set_dropout(go_exact* n, const uint8_t* masks);
/* draws one epoch's flags with libc rand() in the reference's order (layer.cpp:102-134,
   LayerBuilder.cpp:497-523, network.cpp:407-411); p[l] = probability of node layer l */
void  go_dropout_draw(const go_spec* s, const float* p, int64_t N, uint8_t* masks);
/* what dropout leaves behind between rows: pending-delta counts per edge and the error
   accumulators of a hidden layer's nodes */
void  go_exact_get_pending(const go_exact* n, int layer, int32_t* cnt);
void  go_exact_get_errder(const go_exact* n, int layer, float* e);

/* ---- canonical mode ---- */
typedef struct go_canon go_canon;
go_canon* go_canon_create(const go_spec* spec);
void  go_canon_destroy(go_canon* n);
void  go_canon_set_params(go_canon* n, int layer, const float* W, const float* bias /* n_out or NULL=0 */);
void  go_canon_get_params(const go_canon* n, int layer, float* W, float* bias);
void  go_canon_get_momentum(const go_canon* n, int layer, float* vW, float* vb);
/* forward of B rows; out = B*n_out activations of the last layer */
void  go_canon_forward(go_canon* n, const float* X, int64_t B, float* out);
/* one training step on B rows (forward, backward, update) */
void  go_canon_step(go_canon* n, const float* X, const float* Y, int64_t B, go_metrics* m);
/* gradients of the last go_canon_step (batch-mean, before decay) for gradient checks */
void  go_canon_get_grads(const go_canon* n, int layer, float* gW, float* gb);
/* mean per-sample loss of a batch without touching parameters */
double go_canon_loss(go_canon* n, const float* X, const float* Y, int64_t B);
/* dropout flags for the rows of the calls that follow, [B][sizes[0] + ... + sizes[n_layers-1]] bytes, 1 = dropped
   (the caller keeps them alive; NULL: none).  A dropped node's activation is taken as 0 by the layer above and
   it gets no delta (layer.cpp:102-134, network.cpp:476-480 carried over to batches; no rescaling). */
void  go_canon_set_drop(go_canon* n, const uint8_t* flags);
void  go_set_threads(int t);
/* canonical mode: 1 = every sum is walked from its far end (same mathematics, another order of fp32 addition) */
void  go_set_sum_order(int reversed);

/* ---- low-precision formats ---- */
uint16_t go_bf16_from_f32(float x);           /* round-to-nearest-even, NaN kept quiet */
float    go_bf16_to_f32(uint16_t h);
uint8_t  go_e4m3_from_f32(float x);           /* OCP e4m3fn, RNE, saturating to +-448 */
float    go_e4m3_to_f32(uint8_t b);
/* per-row symmetric quantisation: scale[r] = amax(row)/448 (1 when the row is all zero),
   q = e4m3(x / scale) */
void  go_e4m3_quant_rows(const float* x, int64_t rows, int64_t cols, uint8_t* q, float* scale);
/* forward of the quantised inference pipeline: weights e4m3 + per-output-channel scale,
   activations re-quantised per row before every layer, fp32 accumulation,
   activation act[l] after each layer; X is fp32 (already rounded to bf16 by the caller) */
void  go_fp8_forward(const go_spec* spec, const uint8_t* const* Wq, const float* const* wscale,
                     const float* X, int64_t B, float* out);

/* the same with block-scaled activations: an E8M0 byte per row and 32 consecutive columns, [rows][ceil(cols/32)],
   value 2^(byte-127) = the power of two that brings the block's largest magnitude into (224, 448]; no reference
   counterpart.  Pinned by tests/test_oracle_formats.py against torch's float8_e4m3fn casts and the rule's
   defining inequalities. */
void  go_e4m3_quant_rows_block32(const float* x, int64_t rows, int64_t cols, uint8_t* q, uint8_t* scale);
void  go_fp8_forward_block32(const go_spec* spec, const uint8_t* const* Wq, const float* const* wscale,
                             const float* X, int64_t B, float* out);

#ifdef __cplusplus
}
#endif
#endif

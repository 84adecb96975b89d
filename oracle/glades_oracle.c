/*
 * glades_oracle.c -- CPU restatement of the Glades dense feed-forward hot path.
 * TEST INFRASTRUCTURE ONLY (see glades_oracle.h).  Plain C, fp32 arithmetic written
 * so that the compiler can neither fuse multiply-add nor re-associate: build with
 * -ffp-contract=off and without -ffast-math.
 *
 * "ML/" = "Backend/Machine Learning/" in the reference tree.
 */
#include "glades_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define OUTLIER 0.046f /* ML/GMath/gmath.h:35 */

/* ------------------------------------------------------------------ element-wise */

/* ML/GMath/gmath.cpp:22-101.  tanh/exp on a float argument resolve to the float
 * overloads in the reference's C++ (tanhf/expf). */
float go_squash(float z, int act, float p)
{
    switch (act) {
    case GO_TANH: return tanhf(z);
    case GO_TANHP:
        if (z > 1.0f - p) return 1.0f;
        if (z < p - 1.0f) return -1.0f;
        return tanhf(z);
    case GO_SIGMOID: return 1.0f / (1.0f + expf(-z));
    case GO_SIGMOIDP:
        if (z < p) return 0.01f;
        if (z > 1.0f - p) return 0.99f;
        return 1.0f / (1.0f + expf(-z));
    case GO_RELU: return (z < OUTLIER) ? 0.0f : z;
    case GO_LEAKY: return (z < OUTLIER) ? p * z : z;
    case GO_LINEAR: return p * z;
    case GO_STEP: return (z < p) ? 0.0f : 1.0f;
    }
    return 0.0f;
}

/* ML/GMath/gmath.cpp:182-245: derivative expressed in the activation's OUTPUT. */
float go_act_der(float a, int act, float p)
{
    switch (act) {
    case GO_TANH:
    case GO_TANHP: return 1.0f - (a * a);
    case GO_SIGMOID:
    case GO_SIGMOIDP: return a * (1.0f - a);
    case GO_RELU: return (a > 0.0f) ? 1.0f : 0.0f;
    case GO_LEAKY:
        if (a > 0.0f) return 1.0f;
        return (p < 0) ? p : -p;
    case GO_LINEAR: return p;
    case GO_STEP: return 0.0f;
    }
    return 1.0f;
}

/* ML/GMath/gmath.cpp:272-321 */
float go_cost(float e, float p, float data_size, int cost)
{
    float c = 0.0f;
    switch (cost) {
    case GO_REGRESSION: {
        float d = e - p;
        c = d * d;
        c /= data_size;
        break;
    }
    case GO_CLASSIFICATION:
        c = -((e * logf(p)) + ((1 - e) * logf(1 - p)));
        c /= data_size;
        break;
    case GO_KL:
        c = logf(e / p);
        c /= data_size;
        break;
    }
    return c;
}

/* ML/GMath/gmath.cpp:323-353 */
float go_cost_der(float e, float p, int cost)
{
    switch (cost) {
    case GO_REGRESSION: return 2.0f * (p - e);
    case GO_CLASSIFICATION: return (p - e) / ((1 - p) * p);
    case GO_KL: return -(e / p);
    }
    return 1.0f;
}

/* ML/GMath/gmath.cpp:252-270 */
float go_percent_error(float pred, float expect)
{
    float pe = pred - expect;
    if (pe < 0.0f) pe = -pe;
    if (pe > 1.0f) pe = 1.0f;
    return pe;
}

/* ML/GMath/gmath.cpp:412-455: strictly-greater scan starting from max = 0 */
int go_argmax_ref(const float* v, int n)
{
    float mx = 0.0f;
    int idx = -1;
    for (int i = 0; i < n; ++i)
        if (v[i] > mx) { mx = v[i]; idx = i; }
    return idx;
}

/* ------------------------------------------------------------------ confusion matrix */

/* ML/GMath/cmatrix.cpp:57-98: both vectors go through the argmax rule above (a 0/1 vector with
 * at most one 1); for the expected class i (if any) row i gains the predicted 0/1 vector, i.e.
 * M[i][j] += 1 for the predicted class j (if any).  Row = expected, column = predicted. */
void go_cmatrix_add(int n, int32_t* M, const float* expected, const float* predicted)
{
    const int i = go_argmax_ref(expected, n);
    const int j = go_argmax_ref(predicted, n);
    if (i >= 0 && j >= 0) M[(int64_t)i * n + j] += 1;
}

/* ML/GMath/cmatrix.cpp:100-132, starting from the zeroed lists reset() leaves (:285-298).
 * Off-diagonal cells feed falsePositive[col] and falseNegative[row]; a diagonal cell sets
 * truePositive[row] and is ADDED to trueNegative of every other class, so trueNegative[i] is the
 * sum of the other classes' diagonal cells only (off-diagonal cells never count as negatives). */
void go_cmatrix_params(int n, const int32_t* M, int32_t* tp, int32_t* tn, int32_t* fp, int32_t* fn)
{
    for (int i = 0; i < n; ++i) tp[i] = tn[i] = fp[i] = fn[i] = 0;
    for (int row = 0; row < n; ++row)
        for (int col = 0; col < n; ++col) {
            const int32_t v = M[(int64_t)row * n + col];
            if (row != col) {
                fp[col] += v;
                fn[row] += v;
            } else {
                for (int itr = 0; itr < n; ++itr) {
                    if (itr == row) tp[itr] = v;
                    else tn[itr] += v;
                }
            }
        }
}

/* ML/GMath/cmatrix.cpp:139-265: per-class ratios in float, overall = mean over the classes
 * accumulated in class order (0/0 gives NaN and poisons the mean, as in the reference).
 * out[0..5] = accuracy, precision, recall, specificity, F1, false alarm (fractions, not percent) */
void go_cmatrix_overall(int n, const int32_t* tp, const int32_t* tn, const int32_t* fp, const int32_t* fn, float* out)
{
    float acc = 0.0f, pre = 0.0f, rec = 0.0f, spe = 0.0f, f1 = 0.0f, fa = 0.0f;
    for (int i = 0; i < n; ++i) {
        const float truth = (float)(tp[i] + tn[i]);
        const float untruth = (float)(fp[i] + fn[i]);
        acc += truth / (truth + untruth);
        const float cp = ((float)tp[i]) / ((float)(tp[i] + fp[i]));
        const float cr = ((float)tp[i]) / ((float)(tp[i] + fn[i]));
        pre += cp;
        rec += cr;
        spe += ((float)tn[i]) / ((float)(tn[i] + fp[i]));
        fa += ((float)fp[i]) / ((float)(tn[i] + fp[i]));
        f1 += (2.0f * cr * cp) / (cr + cp);
    }
    const float nn = (float)n;
    out[0] = acc / nn; out[1] = pre / nn; out[2] = rec / nn; out[3] = spe / nn; out[4] = f1 / nn; out[5] = fa / nn;
}

/* ------------------------------------------------------------------ init sampler */

/* ML/GMath/gmath.cpp:355-405 (Acklam).  log/sqrt on float arguments are the float
 * overloads in the reference; the rational part is evaluated in double. */
static float norm_inv_cdf(float x)
{
    const double a1 = -39.69683028665376, a2 = 220.9460984245205, a3 = -275.9285104469687,
                 a4 = 138.3577518672690, a5 = -30.66479806614716, a6 = 2.506628277459239;
    const double b1 = -54.47609879822406, b2 = 161.5858368580409, b3 = -155.6989798598866,
                 b4 = 66.80131188771972, b5 = -13.280681552885721;
    const double c1 = -0.007784894002430293, c2 = -0.3223964580411365, c3 = -2.400758277161838,
                 c4 = -2.549732539343734, c5 = 4.374664141464968, c6 = 2.938163982698783;
    const double d1 = 0.007784695709041462, d2 = 0.3224671290700398, d3 = 2.445134137142996,
                 d4 = 3.754408661907416;
    float p_low = 0.02452;
    float p_high = 1 - p_low;
    if (x < p_low) {
        double q = sqrtf(-2 * logf(x));
        return (float)((((((c1 * q + c2) * q + c3) * q + c4) * q + c5) * q + c6) /
                       ((((d1 * q + d2) * q + d3) * q + d4) * q + 1));
    } else if (x < p_high) {
        double q = x - 0.5;
        double r = q * q;
        return (float)(((((((a1 * r + a2) * r + a3) * r + a4) * r + a5) * r + a6) * q) /
                       (((((b1 * r + b2) * r + b3) * r + b4) * r + b5) * r + 1));
    } else {
        double q = sqrtf(-2 * logf(1 - x));
        return (float)(-(((((c1 * q + c2) * q + c3) * q + c4) * q + c5) * q + c6) /
                       ((((d1 * q + d2) * q + d3) * q + d4) * q + 1));
    }
}

/* ML/GMath/gmath.cpp:407-410 */
static float normal_pdf(float z)
{
    return (float)((1 / sqrt(6.2831853)) * expf(-(z * z) / 2));
}

/* ML/State/layer.cpp:196-217 (table) + ML/State/node.cpp:241-276 (rejection loop).
 * Both INIT_XAVIER and INIT_POSXAVIER take this path, so every weight is >= 0. */
void go_ref_xavier_layer(int fan_in, int n_out, int act_type, float* W)
{
    enum { NL = 2048 };
    static float zigg[NL + 1];
    float cdf = 1.0;
    for (unsigned i = 1; i < NL; i++) {
        cdf = cdf - (1 / ((float)NL * 2));
        zigg[i] = norm_inv_cdf(cdf);
    }
    zigg[0] = zigg[1];
    zigg[NL] = 0;

    float std_dev;
    if (act_type != GO_RELU) std_dev = sqrtf(1 / (float)fan_in);
    else std_dev = sqrtf(2 / (float)fan_in);

    for (int o = 0; o < n_out; ++o)
        for (int i = 0; i < fan_in; ++i) {
            int accepted = 0;
            float x = 0.0f;
            while (!accepted) {
                int layer = rand() % 2048;
                x = rand() / (RAND_MAX / zigg[layer]);
                if (layer == 0) continue;
                else if (x < zigg[layer + 1]) accepted = 1;
                else if (x > zigg[layer + 1]) {
                    float randU = rand() / RAND_MAX; /* integer division, as written */
                    float y = normal_pdf(zigg[layer]) +
                              randU * (normal_pdf(zigg[layer - 1] - normal_pdf(zigg[layer])));
                    if (y < normal_pdf(x)) accepted = 1;
                }
            }
            W[(size_t)o * fan_in + i] = x * std_dev;
        }
}

/* the element-wise functions over arrays: fn 0 squash, 1 act_der, 2 cost(expected a, predicted b,
   data_size param), 3 cost_der(expected a, predicted b) */
void go_eval(int fn, int kind, float param, const float* a, const float* b, float* out, int64_t n)
{
#pragma omp parallel for schedule(static)
    for (int64_t k = 0; k < n; ++k) {
        switch (fn) {
        case 0: out[k] = go_squash(a[k], kind, param); break;
        case 1: out[k] = go_act_der(a[k], kind, param); break;
        case 2: out[k] = go_cost(a[k], b[k], param, kind); break;
        default: out[k] = go_cost_der(a[k], b[k], kind); break;
        }
    }
}

/* ------------------------------------------------------------------ exact mode */

struct go_exact {
    go_spec s;
    float* W[GO_MAX_LAYERS];     /* [n_out][n_in] row-major: the incoming edges of node o */
    float* wsum[GO_MAX_LAYERS];  /* running sum of the edge's pending deltas (edge.cpp window) */
    float* wlast[GO_MAX_LAYERS]; /* last pending delta, 0 when the window is empty */
    float  bias[GO_MAX_LAYERS];  /* scalar bias of layer l, added to layer l+1 (l >= 1) */
    float* a[GO_MAX_LAYERS + 1]; /* node values */
    float* e[GO_MAX_LAYERS + 1]; /* node error accumulators */
    int32_t* wcnt[GO_MAX_LAYERS]; /* number of pending deltas of the edge (Edge::prevDelta.size()) */
    const uint8_t* masks;        /* dropout flags of the coming epoch, N rows x mask_len, or NULL */
    int mask_len, moff[GO_MAX_LAYERS + 1];
};

go_exact* go_exact_create(const go_spec* spec)
{
    go_exact* n = (go_exact*)calloc(1, sizeof(go_exact));
    n->s = *spec;
    for (int l = 0; l < spec->n_layers; ++l) {
        size_t cnt = (size_t)spec->sizes[l] * spec->sizes[l + 1];
        n->W[l] = (float*)calloc(cnt, sizeof(float));
        n->wsum[l] = (float*)calloc(cnt, sizeof(float));
        n->wlast[l] = (float*)calloc(cnt, sizeof(float));
        n->wcnt[l] = (int32_t*)calloc(cnt, sizeof(int32_t));
        n->moff[l] = n->mask_len;
        n->mask_len += spec->sizes[l];
    }
    for (int l = 0; l <= spec->n_layers; ++l) {
        n->a[l] = (float*)calloc(spec->sizes[l], sizeof(float));
        n->e[l] = (float*)calloc(spec->sizes[l], sizeof(float));
    }
    return n;
}

void go_exact_destroy(go_exact* n)
{
    if (!n) return;
    for (int l = 0; l < n->s.n_layers; ++l) { free(n->W[l]); free(n->wsum[l]); free(n->wlast[l]); free(n->wcnt[l]); }
    for (int l = 0; l <= n->s.n_layers; ++l) { free(n->a[l]); free(n->e[l]); }
    free(n);
}

void go_exact_set_weights(go_exact* n, int l, const float* W)
{ memcpy(n->W[l], W, sizeof(float) * n->s.sizes[l] * n->s.sizes[l + 1]); }
void go_exact_get_weights(const go_exact* n, int l, float* W)
{ memcpy(W, n->W[l], sizeof(float) * n->s.sizes[l] * n->s.sizes[l + 1]); }
void go_exact_set_bias(go_exact* n, int l, float b) { n->bias[l] = b; }
float go_exact_get_bias(const go_exact* n, int l) { return n->bias[l]; }
void go_exact_get_window(const go_exact* n, int l, float* sum, float* last)
{
    size_t cnt = (size_t)n->s.sizes[l] * n->s.sizes[l + 1];
    memcpy(sum, n->wsum[l], cnt * sizeof(float));
    memcpy(last, n->wlast[l], cnt * sizeof(float));
}

/* Layer::possiblePath (layer.cpp:136-150): nodes of the output layer are never dropped. */
static int valid_node(const go_exact* n, const uint8_t* m, int layer, int i)
{
    if (!m || layer >= n->s.n_layers) return 1;
    return !m[n->moff[layer] + i];
}

/* network.cpp:457-575 for one row; m = the row's dropout flags or NULL. */
static void exact_forward(go_exact* n, const float* x, const float* y, int64_t N,
                          float* tot_err, float* tot_acc, const uint8_t* m)
{
    const go_spec* s = &n->s;
    const int H1 = s->n_layers;
    memcpy(n->a[0], x, sizeof(float) * s->sizes[0]);
    for (int l = 0; l < H1; ++l) {
        const int ni = s->sizes[l], no = s->sizes[l + 1];
        const float* W = n->W[l];
        for (int o = 0; o < no; ++o) {
            float z = 0.0f; /* node.cpp:82-93: sum of edge activations, i ascending */
            for (int i = 0; i < ni; ++i) {
                /* network.cpp:480-488: a dropped pair sets no edge activation */
                if (!(valid_node(n, m, l, i) && valid_node(n, m, l + 1, o))) continue;
                float ea = W[(size_t)o * ni + i] * n->a[l][i]; /* network.cpp:485-487 */
                z += ea;
            }
            /* network.cpp:491-516 runs at the last valid input node for EVERY output node: a dropped
               output node still becomes squash(bias) */
            if (l != 0) z += n->bias[l]; /* network.cpp:501-502 */
            n->a[l + 1][o] = go_squash(z, s->act[l], s->act_param[l]);
            if (l == H1 - 1) { /* network.cpp:519-559 */
                float pred = n->a[l + 1][o], expect = y[o];
                float data_size = (float)((unsigned)N * (unsigned)no);
                float c = go_cost(expect, pred, data_size, s->cost);
                *tot_err += c;
                float acc = (1.0f - go_percent_error(pred, expect)) * 100.0f;
                if (acc < 0.0f) acc = 0.0f;
                *tot_acc += acc;
            }
        }
    }
}

/* network.cpp:577-668 for one row `r`; node.cpp:278-307 inlined; m = the row's dropout flags or NULL. */
static void exact_backward(go_exact* n, const float* y, int64_t r, const uint8_t* m)
{
    const go_spec* s = &n->s;
    const int H1 = s->n_layers;
    const int mb = s->batch;
    for (int L = H1; L > 0; --L) {
        const int l = L - 1; /* weight layer; hyper-parameter row of the in-layer */
        const int ni = s->sizes[l], no = s->sizes[L];
        float* W = n->W[l];
        float* ws = n->wsum[l];
        float* wl = n->wlast[l];
        int32_t* wc = n->wcnt[l];
        const float lr = s->lr[l], mom = s->mom[l], wd1 = s->wd1[l], wd2 = s->wd2[l];
        for (int i = 0; i < ni; ++i) {
            const float ain = n->a[l][i];
            for (int o = 0; o < no; ++o) {
                float der = 1.0f;
                if (L == H1) { /* output layer: clearErrDer + adjustErrDer(costErrDer) */
                    n->e[L][o] = 0;
                    n->e[L][o] += go_cost_der(y[o], n->a[L][o], s->cost);
                } else {
                    der = go_act_der(n->a[L][o], s->act[l], 0.01f); /* network.cpp:616-618 */
                }
                /* network.cpp:621-625 */
                const int dropout = !(valid_node(n, m, l, i) && valid_node(n, m, L, o));
                float d = n->e[L][o];
                size_t k = (size_t)o * ni + i;
                if (!dropout) {
                    d *= der;
                    if (i == ni - 1) n->e[L][o] = 0;
                    float base = lr * d;
                    /* node.cpp:285-288 */
                    float dW = ((base * ain) + (mom * wl[k]) + (wd1 * lr * fabsf(ain)) +
                                (wd2 * lr * ain));
                    /* node.cpp:299-301 sums the window's first minibatchSize entries from 0; an edge
                       that sat out an applying row can hold more than that */
                    if (wc[k] < mb) ws[k] += dW;
                    wc[k] += 1;
                    wl[k] = dW;
                    if ((r % mb) == 0) { /* network.cpp:647-651 */
                        float dsum = ws[k];
                        dsum /= mb;
                        W[k] = W[k] - dsum;
                        ws[k] = 0.0f;
                        wl[k] = 0.0f;
                        wc[k] = 0;
                    }
                    if (l != 0) n->bias[l] = n->bias[l] - base; /* network.cpp:654-656 */
                }
                /* network.cpp:660-662 + node.cpp:173-176: runs for dropped pairs too, with the
                   accumulator of the output node taken as it stands (no derivative factor) */
                float cin = n->e[l][i] + (d * W[k]);
                n->e[l][i] += cin;
            }
        }
    }
    /* the accumulators of the row's own input nodes are never read again */
    memset(n->e[0], 0, sizeof(float) * s->sizes[0]);
}

void go_exact_epoch(go_exact* n, const float* X, const float* Y, int64_t N, int train,
                    go_metrics* m, float* preds)
{
    const go_spec* s = &n->s;
    const int nf = s->sizes[0], no = s->sizes[s->n_layers];
    float tot_err = 0.0f, tot_acc = 0.0f;
    int64_t correct = 0;
    for (int64_t r = 0; r < N; ++r) {
        const float* x = X + r * nf;
        const float* y = Y + r * no;
        const uint8_t* m = n->masks ? n->masks + (size_t)r * n->mask_len : NULL;
        exact_forward(n, x, y, N, &tot_err, &tot_acc, m);
        const float* p = n->a[s->n_layers];
        if (preds) memcpy(preds + r * no, p, sizeof(float) * no);
        if (go_argmax_ref(p, no) == go_argmax_ref(y, no)) ++correct;
        if (train) exact_backward(n, y, r, m);
    }
    tot_acc /= ((float)(unsigned)N) * ((float)(unsigned)no); /* network.cpp:194-195 */
    if (m) { m->loss = tot_err; m->accuracy = tot_acc; m->correct = correct; }
}

/* ---- dropout (layer.cpp:102-134, LayerBuilder.cpp:497-523) ---- */

int go_exact_mask_len(const go_exact* n) { return n->mask_len; }
void go_exact_set_dropout(go_exact* n, const uint8_t* masks) { n->masks = masks; }
void go_exact_get_pending(const go_exact* n, int l, int32_t* cnt)
{ memcpy(cnt, n->wcnt[l], sizeof(int32_t) * n->s.sizes[l] * n->s.sizes[l + 1]); }
void go_exact_get_errder(const go_exact* n, int layer, float* e)
{ memcpy(e, n->e[layer], sizeof(float) * n->s.sizes[layer]); }

/* Layer::generateDropout: one dart rand()%100+1 per node, node dropped when dart <= int(p*100);
   the whole layer is drawn again while every node came out dropped; a rate below 0 or from 100
   up draws nothing and leaves the flags as they are. */
static void draw_layer(float p, int n, uint8_t* flag)
{
    int rate = p * 100.0f;
    if (rate < 0) return;
    if (rate >= 100) return;
    int all_dropped;
    do {
        all_dropped = 1;
        for (int i = 0; i < n; ++i) {
            int dropped = 0;
            int dart = (rand() % 100) + 1;
            if (dart <= rate) dropped = 1;
            else all_dropped = 0;
            flag[i] = (uint8_t)dropped;
        }
    } while (all_dropped);
}

/* One epoch's flags in the order SGDHelper draws them (network.cpp:407-411): for every row, the
   row's input layer, then each hidden layer.  p[l] is the probability of node layer l (0 = input);
   masks is N x sum(sizes[0..n_layers-1]) bytes, 1 = dropped, and must hold the previous row's flags
   of the hidden layers and the previous epoch's flags of the row's input layer on entry for layers
   whose rate draws nothing (all zero for a fresh network). */
void go_dropout_draw(const go_spec* s, const float* p, int64_t N, uint8_t* masks)
{
    int len = 0;
    for (int l = 0; l < s->n_layers; ++l) len += s->sizes[l];
    for (int64_t r = 0; r < N; ++r) {
        uint8_t* m = masks + (size_t)r * len;
        int off = 0;
        for (int l = 0; l < s->n_layers; ++l) {
            draw_layer(p[l], s->sizes[l], m + off);
            off += s->sizes[l];
        }
    }
}

/* ------------------------------------------------------------------ canonical mode */

static int g_threads = 1;
void go_set_threads(int t) { g_threads = t > 0 ? t : 1; }
/* canonical mode only: walk every sum (a unit's inputs, a unit's outputs, a weight's batch rows) from the far end.
   Same mathematics, another order of fp32 addition: what a second implementation may legitimately differ by. */
static int g_reverse = 0;
void go_set_sum_order(int reversed) { g_reverse = reversed ? 1 : 0; }

struct go_canon {
    go_spec s;
    float* W[GO_MAX_LAYERS];  float* b[GO_MAX_LAYERS];
    float* vW[GO_MAX_LAYERS]; float* vb[GO_MAX_LAYERS]; /* previous step's applied delta */
    float* gW[GO_MAX_LAYERS]; float* gb[GO_MAX_LAYERS];
    float* a[GO_MAX_LAYERS + 1]; /* [B][n] activations */
    float* d[GO_MAX_LAYERS + 1]; /* [B][n] deltas (dL/dz) */
    int64_t cap;
    const uint8_t* drop;         /* go_canon_set_drop: the coming batch's flags, or NULL */
};

go_canon* go_canon_create(const go_spec* spec)
{
    go_canon* n = (go_canon*)calloc(1, sizeof(go_canon));
    n->s = *spec;
    for (int l = 0; l < spec->n_layers; ++l) {
        size_t cnt = (size_t)spec->sizes[l] * spec->sizes[l + 1];
        n->W[l] = (float*)calloc(cnt, 4); n->vW[l] = (float*)calloc(cnt, 4);
        n->gW[l] = (float*)calloc(cnt, 4);
        n->b[l] = (float*)calloc(spec->sizes[l + 1], 4);
        n->vb[l] = (float*)calloc(spec->sizes[l + 1], 4);
        n->gb[l] = (float*)calloc(spec->sizes[l + 1], 4);
    }
    return n;
}

static void canon_free_acts(go_canon* n)
{
    for (int l = 0; l <= n->s.n_layers; ++l) { free(n->a[l]); free(n->d[l]); n->a[l] = n->d[l] = 0; }
    n->cap = 0;
}

void go_canon_destroy(go_canon* n)
{
    if (!n) return;
    canon_free_acts(n);
    for (int l = 0; l < n->s.n_layers; ++l) {
        free(n->W[l]); free(n->vW[l]); free(n->gW[l]); free(n->b[l]); free(n->vb[l]); free(n->gb[l]);
    }
    free(n);
}

static void canon_reserve(go_canon* n, int64_t B)
{
    if (B <= n->cap) return;
    canon_free_acts(n);
    for (int l = 0; l <= n->s.n_layers; ++l) {
        n->a[l] = (float*)malloc(sizeof(float) * B * n->s.sizes[l]);
        n->d[l] = (float*)malloc(sizeof(float) * B * n->s.sizes[l]);
    }
    n->cap = B;
}

void go_canon_set_params(go_canon* n, int l, const float* W, const float* bias)
{
    size_t cnt = (size_t)n->s.sizes[l] * n->s.sizes[l + 1];
    memcpy(n->W[l], W, cnt * 4);
    if (bias) memcpy(n->b[l], bias, 4 * n->s.sizes[l + 1]);
    else memset(n->b[l], 0, 4 * n->s.sizes[l + 1]);
}
void go_canon_get_params(const go_canon* n, int l, float* W, float* bias)
{
    if (W) memcpy(W, n->W[l], 4 * (size_t)n->s.sizes[l] * n->s.sizes[l + 1]);
    if (bias) memcpy(bias, n->b[l], 4 * n->s.sizes[l + 1]);
}
void go_canon_get_momentum(const go_canon* n, int l, float* vW, float* vb)
{
    if (vW) memcpy(vW, n->vW[l], 4 * (size_t)n->s.sizes[l] * n->s.sizes[l + 1]);
    if (vb) memcpy(vb, n->vb[l], 4 * n->s.sizes[l + 1]);
}
void go_canon_get_grads(const go_canon* n, int l, float* gW, float* gb)
{
    if (gW) memcpy(gW, n->gW[l], 4 * (size_t)n->s.sizes[l] * n->s.sizes[l + 1]);
    if (gb) memcpy(gb, n->gb[l], 4 * n->s.sizes[l + 1]);
}

#define TB 16 /* batch rows handled together so the inner loop vectorises without re-association */

/* z[b][o] = sum_i W[o][i]*a[b][i] (i ascending, product rounded before the add) + bias[o] */
__attribute__((target_clones("avx2", "default")))
static void canon_layer_forward(const float* W, const float* bias, const float* A, float* Z,
                                int64_t B, int ni, int no)
{
    int64_t nblk = (B + TB - 1) / TB;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t blk = 0; blk < nblk; ++blk) {
        int64_t b0 = blk * TB;
        int nb = (int)((B - b0) < TB ? (B - b0) : TB);
        float* At = (float*)malloc(sizeof(float) * (size_t)ni * TB);
        for (int i = 0; i < ni; ++i)
            for (int t = 0; t < TB; ++t) At[(size_t)i * TB + t] = (t < nb) ? A[(b0 + t) * ni + i] : 0.0f;
        for (int o = 0; o < no; ++o) {
            float acc[TB];
            for (int t = 0; t < TB; ++t) acc[t] = 0.0f;
            const float* w = W + (size_t)o * ni;
            for (int i0 = 0; i0 < ni; ++i0) {
                const int i = g_reverse ? ni - 1 - i0 : i0;
                const float wi = w[i];
                const float* at = At + (size_t)i * TB;
                for (int t = 0; t < TB; ++t) { float pr = wi * at[t]; acc[t] += pr; }
            }
            const float bo = bias[o];
            for (int t = 0; t < nb; ++t) Z[(b0 + t) * no + o] = acc[t] + bo;
        }
        free(At);
    }
}

static void canon_activate(const go_spec* s, int l, float* Z, int64_t B)
{
    const int no = s->sizes[l + 1];
    const int act = s->act[l];
    const float p = s->act_param[l];
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t b = 0; b < B; ++b) {
        float* z = Z + b * no;
        if (act == GO_SOFTMAX) {
            float mx = z[0];
            for (int o = 1; o < no; ++o) if (z[o] > mx) mx = z[o];
            float sum = 0.0f;
            for (int o = 0; o < no; ++o) { z[o] = expf(z[o] - mx); sum += z[o]; }
            for (int o = 0; o < no; ++o) z[o] = z[o] / sum;
        } else {
            for (int o = 0; o < no; ++o) z[o] = go_squash(z[o], act, p);
        }
    }
}

/* Dropout in canonical mode.  The flags are the reference's: one per row and node of the input and hidden
 * layers (Layer::generateDropout, layer.cpp:102-134), and a dropped node feeds nothing on: the reference skips
 * every edge that leaves it (possiblePath, network.cpp:476-480), with no rescaling of the others.  Batched, that
 * is the node's activation taken as 0 by the layer above; back-propagation through the same function gives the
 * dropped node no delta, so the weights into it and its bias get no gradient from that row. */
static int canon_nodes(const go_spec* s)
{
    int t = 0;
    for (int l = 0; l < s->n_layers; ++l) t += s->sizes[l];
    return t;
}
static void canon_drop(const go_canon* n, int l, float* A, int64_t B)
{
    if (!n->drop) return;
    const go_spec* s = &n->s;
    const int nodes = canon_nodes(s), nl = s->sizes[l];
    int off = 0;
    for (int k = 0; k < l; ++k) off += s->sizes[k];
    for (int64_t b = 0; b < B; ++b)
        for (int i = 0; i < nl; ++i)
            if (n->drop[b * nodes + off + i]) A[b * nl + i] = 0.0f;
}
void go_canon_set_drop(go_canon* n, const uint8_t* flags) { n->drop = flags; }

static void canon_forward_all(go_canon* n, const float* X, int64_t B)
{
    const go_spec* s = &n->s;
    canon_reserve(n, B);
    memcpy(n->a[0], X, sizeof(float) * B * s->sizes[0]);
    canon_drop(n, 0, n->a[0], B);
    for (int l = 0; l < s->n_layers; ++l) {
        canon_layer_forward(n->W[l], n->b[l], n->a[l], n->a[l + 1], B, s->sizes[l], s->sizes[l + 1]);
        canon_activate(s, l, n->a[l + 1], B);
        if (l + 1 < s->n_layers) canon_drop(n, l + 1, n->a[l + 1], B);
    }
}

void go_canon_forward(go_canon* n, const float* X, int64_t B, float* out)
{
    canon_forward_all(n, X, B);
    memcpy(out, n->a[n->s.n_layers], sizeof(float) * B * n->s.sizes[n->s.n_layers]);
}

/* canonical derivative: the reference's output-expressed forms with the layer's own
 * parameter (LEAKY slope = +param). */
static inline float canon_act_der(float a, int act, float p)
{
    if (act == GO_LEAKY) return (a > 0.0f) ? 1.0f : p;
    return go_act_der(a, act, p);
}

/* per-sample loss = sum over outputs (no 1/data_size); delta = dLoss/dz */
static double canon_output_delta(const go_spec* s, const float* P, const float* Y, float* D,
                                 int64_t B, go_metrics* m)
{
    const int L = s->n_layers, no = s->sizes[L];
    const int act = s->act[L - 1];
    const float par = s->act_param[L - 1];
    double loss = 0.0, acc = 0.0;
    int64_t correct = 0;
    for (int64_t b = 0; b < B; ++b) {
        const float* p = P + b * no;
        const float* y = Y + b * no;
        float* d = D ? D + b * no : 0;
        for (int o = 0; o < no; ++o) {
            float c;
            if (act == GO_SOFTMAX) c = -(y[o] * logf(p[o] > 1e-30f ? p[o] : 1e-30f));
            else c = go_cost(y[o], p[o], 1.0f, s->cost);
            if (!(act == GO_SOFTMAX && y[o] == 0.0f)) loss += c;
            if (d) {
                if (act == GO_SOFTMAX ||
                    ((act == GO_SIGMOID || act == GO_SIGMOIDP) && s->cost == GO_CLASSIFICATION))
                    d[o] = p[o] - y[o];
                else
                    d[o] = go_cost_der(y[o], p[o], s->cost) * canon_act_der(p[o], act, par);
            }
            float a = (1.0f - go_percent_error(p[o], y[o])) * 100.0f;
            if (a < 0.0f) a = 0.0f;
            acc += a;
        }
        if (go_argmax_ref(p, no) == go_argmax_ref(y, no)) ++correct;
    }
    if (m) {
        m->loss = (float)(loss / (double)B);
        m->accuracy = (float)(acc / ((double)B * no));
        m->correct = correct;
    }
    return loss / (double)B;
}

double go_canon_loss(go_canon* n, const float* X, const float* Y, int64_t B)
{
    canon_forward_all(n, X, B);
    return canon_output_delta(&n->s, n->a[n->s.n_layers], Y, 0, B, 0);
}

/* E[b][i] = sum_o D[b][o]*W[o][i] (o ascending) */
__attribute__((target_clones("avx2", "default")))
static void canon_dgrad(const float* W, const float* D, float* E, int64_t B, int ni, int no)
{
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t b = 0; b < B; ++b) {
        float* e = E + b * ni;
        for (int i = 0; i < ni; ++i) e[i] = 0.0f;
        for (int o0 = 0; o0 < no; ++o0) {
            const int o = g_reverse ? no - 1 - o0 : o0;
            const float dv = D[b * no + o];
            const float* w = W + (size_t)o * ni;
            for (int i = 0; i < ni; ++i) { float pr = dv * w[i]; e[i] += pr; }
        }
    }
}

/* G[o][i] = (sum_b D[b][o]*A[b][i]) / B  (b ascending);  gb[o] = (sum_b D[b][o]) / B */
__attribute__((target_clones("avx2", "default")))
static void canon_wgrad(const float* D, const float* A, float* G, float* gb, int64_t B, int ni, int no)
{
    const float invB = 1.0f / (float)B;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int o = 0; o < no; ++o) {
        float* g = G + (size_t)o * ni;
        for (int i = 0; i < ni; ++i) g[i] = 0.0f;
        float sb = 0.0f;
        for (int64_t b0 = 0; b0 < B; ++b0) {
            const int64_t b = g_reverse ? B - 1 - b0 : b0;
            const float dv = D[b * no + o];
            const float* a = A + b * ni;
            for (int i = 0; i < ni; ++i) { float pr = dv * a[i]; g[i] += pr; }
            sb += dv;
        }
        for (int i = 0; i < ni; ++i) g[i] = g[i] * invB;
        gb[o] = sb * invB;
    }
}

static inline float sgnf(float w) { return (w > 0.0f) ? 1.0f : ((w < 0.0f) ? -1.0f : 0.0f); }

void go_canon_step(go_canon* n, const float* X, const float* Y, int64_t B, go_metrics* m)
{
    const go_spec* s = &n->s;
    const int L = s->n_layers;
    canon_forward_all(n, X, B);
    canon_output_delta(s, n->a[L], Y, n->d[L], B, m);
    for (int l = L - 1; l >= 0; --l) {
        const int ni = s->sizes[l], no = s->sizes[l + 1];
        canon_wgrad(n->d[l + 1], n->a[l], n->gW[l], n->gb[l], B, ni, no);
        if (l > 0) { /* uses the pre-update weights */
            canon_dgrad(n->W[l], n->d[l + 1], n->d[l], B, ni, no);
            const int act = s->act[l - 1];
            const float par = s->act_param[l - 1];
            float* d = n->d[l];
            const float* a = n->a[l];
#pragma omp parallel for num_threads(g_threads) schedule(static)
            for (int64_t k = 0; k < B * ni; ++k) d[k] = d[k] * canon_act_der(a[k], act, par);
            canon_drop(n, l, d, B);
        }
        /* delta_t = lr*(g + wd1*sign(W) + wd2*W) + mom*delta_{t-1};  W -= delta_t */
        const float lr = s->lr[l], mom = s->mom[l], wd1 = s->wd1[l], wd2 = s->wd2[l];
        float* W = n->W[l]; float* vW = n->vW[l]; const float* gW = n->gW[l];
        const int64_t cnt = (int64_t)ni * no;
#pragma omp parallel for num_threads(g_threads) schedule(static)
        for (int64_t k = 0; k < cnt; ++k) {
            float g = gW[k] + wd1 * sgnf(W[k]) + wd2 * W[k];
            float dl = lr * g + mom * vW[k];
            vW[k] = dl;
            W[k] = W[k] - dl;
        }
        for (int o = 0; o < no; ++o) { /* biases: momentum, no decay */
            float dl = lr * n->gb[l][o] + mom * n->vb[l][o];
            n->vb[l][o] = dl;
            n->b[l][o] = n->b[l][o] - dl;
        }
    }
}

/* ------------------------------------------------------------------ low precision */

static inline uint32_t f2u(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
static inline float u2f(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }

uint16_t go_bf16_from_f32(float x)
{
    uint32_t u = f2u(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40); /* quiet NaN */
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
float go_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* OCP FP8 E4M3 (finite-only variant: bias 7, max 448, 0x7f = NaN) */
float go_e4m3_to_f32(uint8_t b)
{
    int sign = b >> 7, e = (b >> 3) & 0xf, mnt = b & 7;
    float v;
    if (e == 0xf && mnt == 7) return NAN;
    if (e == 0) v = ldexpf((float)mnt, -9);
    else v = ldexpf(1.0f + (float)mnt / 8.0f, e - 7);
    return sign ? -v : v;
}

uint8_t go_e4m3_from_f32(float x)
{
    uint8_t sign = (uint8_t)((f2u(x) >> 31) << 7);
    float a = fabsf(x);
    if (a != a) return (uint8_t)(sign | 0x7f);
    if (a >= 448.0f) return (uint8_t)(sign | 0x7e); /* saturate */
    if (a < 0.015625f) { /* below the smallest normal 2^-6: multiples of 2^-9 */
        int q = (int)rintf(a * 512.0f);
        return (uint8_t)(sign | q); /* q == 8 is exactly the smallest normal's code */
    }
    int ex;
    float fr = frexpf(a, &ex); /* a = fr * 2^ex, fr in [0.5,1) */
    float mant = fr * 2.0f;    /* [1,2) */
    ex -= 1;
    int q = (int)rintf((mant - 1.0f) * 8.0f); /* ties to even */
    if (q == 8) { q = 0; ex += 1; }
    int code = ((ex + 7) << 3) | q;
    if (code > 0x7e) code = 0x7e;
    return (uint8_t)(sign | code);
}

void go_e4m3_quant_rows(const float* x, int64_t rows, int64_t cols, uint8_t* q, float* scale)
{
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* xr = x + r * cols;
        float amax = 0.0f;
        for (int64_t c = 0; c < cols; ++c) { float a = fabsf(xr[c]); if (a > amax) amax = a; }
        float sc = (amax > 0.0f) ? amax / 448.0f : 1.0f;
        scale[r] = sc;
        for (int64_t c = 0; c < cols; ++c) q[r * cols + c] = go_e4m3_from_f32(xr[c] / sc);
    }
}

/* Block-scaled e4m3 ("MX"): one E8M0 power-of-two scale per row and 32 consecutive columns.  No reference
 * counterpart (the reference is fp32); the rule is this build's: the scale is the power of two that brings
 * the block's largest magnitude amax into (224, 448] -- byte = E - 8 for amax = 2^(E-127) m, m in [1, 2), one more
 * if 256 m would pass 448 (m > 1.75), never below 0 -- and the codes are e4m3(x / scale), round to nearest even.
 * scale bytes: [rows][ceil(cols / 32)]. */
void go_e4m3_quant_rows_block32(const float* x, int64_t rows, int64_t cols, uint8_t* q, uint8_t* scale)
{
    const int64_t nblk = (cols + 31) / 32;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t b = 0; b < nblk; ++b) {
            const int64_t c0 = b * 32, c1 = c0 + 32 < cols ? c0 + 32 : cols;
            float amax = 0.0f;
            for (int64_t c = c0; c < c1; ++c) { float a = fabsf(x[r * cols + c]); if (a > amax) amax = a; }
            const uint32_t u = f2u(amax);
            int eb = (int)(u >> 23) - 8 + ((u & 0x7fffffu) > 0x600000u ? 1 : 0); /* mantissa field above .75 */
            if (eb < 0) eb = 0;
            scale[r * nblk + b] = (uint8_t)eb;
            const float sc = ldexpf(1.0f, eb - 127);
            for (int64_t c = c0; c < c1; ++c) q[r * cols + c] = go_e4m3_from_f32(x[r * cols + c] / sc);
        }
}

/* go_fp8_forward with block-scaled activations: between layers the bf16-rounded activations are quantised by
 * go_e4m3_quant_rows_block32; a product is sum over blocks of 2^(byte-127) * (sum over the block of code values
 * times weight code values), times the output channel's weight scale. */
void go_fp8_forward_block32(const go_spec* s, const uint8_t* const* Wq, const float* const* wscale,
                            const float* X, int64_t B, float* out)
{
    static float lut[256];
    for (int i = 0; i < 256; ++i) lut[i] = go_e4m3_to_f32((uint8_t)i);
    int maxw = 0;
    for (int l = 0; l <= s->n_layers; ++l) if (s->sizes[l] > maxw) maxw = s->sizes[l];
    float* cur = (float*)malloc(sizeof(float) * B * maxw);
    float* nxt = (float*)malloc(sizeof(float) * B * maxw);
    uint8_t* q = (uint8_t*)malloc((size_t)B * maxw);
    uint8_t* xs = (uint8_t*)malloc((size_t)B * ((maxw + 31) / 32));
    memcpy(cur, X, sizeof(float) * B * s->sizes[0]);
    for (int l = 0; l < s->n_layers; ++l) {
        const int ni = s->sizes[l], no = s->sizes[l + 1], nblk = (ni + 31) / 32;
        go_e4m3_quant_rows_block32(cur, B, ni, q, xs);
        float* wf = (float*)malloc(sizeof(float) * (size_t)ni * no);
        for (size_t k = 0; k < (size_t)ni * no; ++k) wf[k] = lut[Wq[l][k]];
#pragma omp parallel for num_threads(g_threads) schedule(static)
        for (int64_t b = 0; b < B; ++b) {
            float* xf = (float*)malloc(sizeof(float) * ni);
            for (int i = 0; i < ni; ++i) xf[i] = lut[q[b * ni + i]] * ldexpf(1.0f, (int)xs[b * nblk + i / 32] - 127);
            for (int o = 0; o < no; ++o) {
                const float* w = wf + (size_t)o * ni;
                float acc = 0.0f;
                for (int i = 0; i < ni; ++i) { float pr = w[i] * xf[i]; acc += pr; }
                float v = acc * wscale[l][o];
                v = go_squash(v, s->act[l], s->act_param[l]);
                if (l + 1 < s->n_layers) v = go_bf16_to_f32(go_bf16_from_f32(v));
                nxt[b * no + o] = v;
            }
            free(xf);
        }
        free(wf);
        float* t = cur; cur = nxt; nxt = t;
    }
    memcpy(out, cur, sizeof(float) * B * s->sizes[s->n_layers]);
    free(cur); free(nxt); free(q); free(xs);
}

void go_fp8_forward(const go_spec* s, const uint8_t* const* Wq, const float* const* wscale,
                    const float* X, int64_t B, float* out)
{
    static float lut[256];
    for (int i = 0; i < 256; ++i) lut[i] = go_e4m3_to_f32((uint8_t)i);
    int maxw = 0;
    for (int l = 0; l <= s->n_layers; ++l) if (s->sizes[l] > maxw) maxw = s->sizes[l];
    float* cur = (float*)malloc(sizeof(float) * B * maxw);
    float* nxt = (float*)malloc(sizeof(float) * B * maxw);
    uint8_t* q = (uint8_t*)malloc((size_t)B * maxw);
    float* xs = (float*)malloc(sizeof(float) * B);
    memcpy(cur, X, sizeof(float) * B * s->sizes[0]);
    for (int l = 0; l < s->n_layers; ++l) {
        const int ni = s->sizes[l], no = s->sizes[l + 1];
        go_e4m3_quant_rows(cur, B, ni, q, xs);
        float* wf = (float*)malloc(sizeof(float) * (size_t)ni * no);
        for (size_t k = 0; k < (size_t)ni * no; ++k) wf[k] = lut[Wq[l][k]];
#pragma omp parallel for num_threads(g_threads) schedule(static)
        for (int64_t b = 0; b < B; ++b) {
            float* xf = (float*)malloc(sizeof(float) * ni);
            for (int i = 0; i < ni; ++i) xf[i] = lut[q[b * ni + i]];
            for (int o = 0; o < no; ++o) {
                const float* w = wf + (size_t)o * ni;
                float acc = 0.0f;
                for (int i = 0; i < ni; ++i) { float pr = w[i] * xf[i]; acc += pr; }
                float v = acc * (xs[b] * wscale[l][o]);
                v = go_squash(v, s->act[l], s->act_param[l]);
                if (l + 1 < s->n_layers) v = go_bf16_to_f32(go_bf16_from_f32(v));
                nxt[b * no + o] = v;
            }
            free(xf);
        }
        free(wf);
        float* t = cur; cur = nxt; nxt = t;
    }
    memcpy(out, cur, sizeof(float) * B * s->sizes[s->n_layers]);
    free(cur); free(nxt); free(q); free(xs);
}

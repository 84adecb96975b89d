/*
 * ref_harness.cpp -- drives the REFERENCE's own compiled State/GMath objects.
 * TEST INFRASTRUCTURE ONLY; built into oracle/_ref/ (never committed, never shipped as
 * product).  It is compiled against the reference headers where they lie and linked with
 * the reference's node.cpp, edge.cpp, layer.cpp, Terminator.cpp and gmath.cpp, which need
 * no external library (the one GList-based helper in gmath.cpp is dropped by
 * --gc-sections because nothing here calls it).
 *
 * What is the reference's code here: every Node / Edge / Layer / GMath / Terminator call.
 * What is NOT: the loop nest in run_case(), which restates
 * "Backend/Machine Learning/Networks/network.cpp":457-575 (ForwardPass) and :577-668
 * (BackPropagation) and the index lookup of State/LayerBuilder.cpp:269-336, because
 * network.cpp / LayerBuilder.cpp need the un-vendored shmea library and cannot be linked.
 *
 * Usage:
 *   ref_harness gmath  <out.bin>                      grid of element-wise functions
 *   ref_harness xavier <seed> <fan_in> <n_out> <act> <out.bin>
 *   ref_harness xavierseq <seed> <out.bin> <fan_in> <n_out> <act> [<fan_in> <n_out> <act> ...]
 *       the layers one after the other under ONE srand(seed), then rand() % 65536 as a float
 *   ref_harness train  <case.bin> <out.bin>           see tests/golden/make_golden.py
 *   ref_harness term   <out.bin>                      Terminator truth table
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>

#include "Backend/Machine Learning/GMath/gmath.h"
#include "Backend/Machine Learning/State/Terminator.h"
#include "Backend/Machine Learning/State/edge.h"
#include "Backend/Machine Learning/State/layer.h"
#include "Backend/Machine Learning/State/node.h"

using namespace glades;

static void wr(FILE* f, const void* p, size_t n) { fwrite(p, 1, n, f); }
static void wrf(FILE* f, float v) { wr(f, &v, 4); }

static int do_gmath(const char* out)
{
    FILE* f = fopen(out, "wb");
    if (!f) return 1;
    /* z grid x 8 activations x 3 params: squash, then activationErrDer of that output */
    static const float params[3] = {0.0f, 0.01f, 0.1f};
    int nz = 0;
    for (float z = -6.0f; z <= 6.0f; z += 0.0625f) ++nz;
    int32_t hdr[2] = {nz, 3};
    wr(f, hdr, 8);
    for (int act = 0; act < 8; ++act)
        for (int p = 0; p < 3; ++p) {
            if (act == GMath::LEAKY && params[p] > 0.1f) continue;
            for (float z = -6.0f; z <= 6.0f; z += 0.0625f) {
                float a = GMath::squash(z, act, params[p]);
                float d = GMath::activationErrDer(a, act, params[p]);
                wrf(f, z); wrf(f, a); wrf(f, d);
            }
        }
    /* cost grid: expectation x prediction x 3 costs */
    static const float es[6] = {0.0f, 0.01f, 0.25f, 0.5f, 0.99f, 1.0f};
    for (int c = 0; c < 3; ++c)
        for (int ei = 0; ei < 6; ++ei)
            for (float p = 0.03125f; p < 1.0f; p += 0.03125f) {
                wrf(f, es[ei]); wrf(f, p);
                wrf(f, GMath::outputNodeCost(es[ei], p, 12.0f, c));
                wrf(f, GMath::costErrDer(es[ei], p, c));
                wrf(f, GMath::PercentError(p * 3.0f - 1.0f, es[ei], 0.0f));
            }
    fclose(f);
    return 0;
}

static int do_xavier(int seed, int fan_in, int n_out, int act, const char* out)
{
    srand(seed);
    Layer layer(Layer::HIDDEN_TYPE);
    layer.initWeights(fan_in, n_out, Node::INIT_XAVIER, act);
    FILE* f = fopen(out, "wb");
    if (!f) return 1;
    for (int o = 0; o < n_out; ++o)
        for (int i = 0; i < fan_in; ++i) wrf(f, layer[o]->getEdgeWeight(i));
    fclose(f);
    return 0;
}

static int do_xavier_seq(int seed, const char* out, int n, char** spec)
{
    srand(seed);
    FILE* f = fopen(out, "wb");
    if (!f) return 1;
    for (int k = 0; k + 2 < n; k += 3) {
        const int fan_in = atoi(spec[k]), n_out = atoi(spec[k + 1]), act = atoi(spec[k + 2]);
        Layer layer(Layer::HIDDEN_TYPE);
        layer.initWeights(fan_in, n_out, Node::INIT_XAVIER, act);
        for (int o = 0; o < n_out; ++o)
            for (int i = 0; i < fan_in; ++i) wrf(f, layer[o]->getEdgeWeight(i));
    }
    wrf(f, (float)(rand() % 65536));
    fclose(f);
    return 0;
}

static int do_term(const char* out)
{
    FILE* f = fopen(out, "wb");
    if (!f) return 1;
    static const int64_t ts[3] = {0, 7, 10}, es[3] = {0, 5, 100000};
    static const float as[3] = {0.0f, 95.0f, 50.5f};
    for (int a = 0; a < 3; ++a)
        for (int b = 0; b < 3; ++b)
            for (int c = 0; c < 3; ++c) {
                Terminator t;
                t.setTimestamp(ts[a]); t.setEpoch(es[b]); t.setAccuracy(as[c]);
                for (int64_t now = 68; now < 72; ++now)
                    for (int64_t ep = 4; ep < 7; ++ep)
                        for (float acc = 40.0f; acc < 100.0f; acc += 27.75f) {
                            int32_t rec[7] = {(int32_t)ts[a], (int32_t)es[b], (int32_t)as[c] * 2,
                                              (int32_t)now, (int32_t)ep, (int32_t)(acc * 4),
                                              t.triggered(now, ep, acc) ? 1 : 0};
                            rec[2] = (int32_t)(as[c] * 2);
                            wr(f, rec, sizeof(rec));
                        }
            }
    fclose(f);
    return 0;
}

struct Case {
    int32_t n_layers;
    std::vector<int32_t> sizes;
    int32_t batch, cost, N, epochs;
    std::vector<float> lr, mom, wd1, wd2, act_param;
    std::vector<int32_t> act;
};

static int do_train(const char* in, const char* out)
{
    FILE* f = fopen(in, "rb");
    if (!f) return 1;
    Case c;
    int32_t magic = 0;
    if (fread(&magic, 4, 1, f) != 1 || magic != 0x474c4144) return 2;
    if (fread(&c.n_layers, 4, 1, f) != 1) return 2;
    c.sizes.resize(c.n_layers + 1);
    if (fread(&c.sizes[0], 4, c.n_layers + 1, f) != (size_t)c.n_layers + 1) return 2;
    int32_t h4[4];
    if (fread(h4, 4, 4, f) != 4) return 2;
    c.batch = h4[0]; c.cost = h4[1]; c.N = h4[2]; c.epochs = h4[3];
    c.lr.resize(c.n_layers); c.mom.resize(c.n_layers); c.wd1.resize(c.n_layers);
    c.wd2.resize(c.n_layers); c.act_param.resize(c.n_layers); c.act.resize(c.n_layers);
    for (int l = 0; l < c.n_layers; ++l) {
        float p[4];
        if (fread(p, 4, 4, f) != 4) return 2;
        c.lr[l] = p[0]; c.mom[l] = p[1]; c.wd1[l] = p[2]; c.wd2[l] = p[3];
        if (fread(&c.act[l], 4, 1, f) != 1) return 2;
        if (fread(&c.act_param[l], 4, 1, f) != 1) return 2;
    }
    const int H1 = c.n_layers;
    /* layers[0] is rebuilt per row as the input layer; layers[1..H1] are hidden/output */
    std::vector<Layer*> layers(H1 + 1);
    for (int L = 1; L <= H1; ++L) {
        Layer* ly = new Layer(L == H1 ? Layer::OUTPUT_TYPE : Layer::HIDDEN_TYPE);
        for (int o = 0; o < c.sizes[L]; ++o) {
            Node* nd = new Node();
            std::vector<Edge*> edges;
            for (int i = 0; i < c.sizes[L - 1]; ++i) {
                float w;
                if (fread(&w, 4, 1, f) != 1) return 2;
                edges.push_back(new Edge(i, w));
            }
            nd->setEdges(edges);
            ly->addNode(nd);
        }
        layers[L] = ly;
    }
    for (int l = 0; l < H1; ++l) {
        float b;
        if (fread(&b, 4, 1, f) != 1) return 2;
        if (l >= 1) layers[l]->setBiasWeight(b);
    }
    const int nf = c.sizes[0], no = c.sizes[H1];
    std::vector<float> X((size_t)c.N * nf), Y((size_t)c.N * no);
    if (fread(&X[0], 4, X.size(), f) != X.size()) return 2;
    if (fread(&Y[0], 4, Y.size(), f) != Y.size()) return 2;
    /* optional trailer: srand() seed and one dropout probability per non-output layer */
    int32_t seed = 0;
    std::vector<float> pdrop(H1, 0.0f);
    const bool with_dropout = fread(&seed, 4, 1, f) == 1;
    if (with_dropout && fread(&pdrop[0], 4, H1, f) != (size_t)H1) return 2;
    fclose(f);
    std::vector<float> flags; /* every row's flags of every epoch, in drawing order */
    if (with_dropout) srand((unsigned)seed);

    /* one input Layer per row, as LayerBuilder::buildInputLayers does */
    std::vector<Layer*> inputLayers(c.N);
    for (int r = 0; r < c.N; ++r) {
        Layer* ly = new Layer(Layer::INPUT_TYPE, false);
        for (int i = 0; i < nf; ++i) {
            Node* nd = new Node();
            nd->setWeight(X[(size_t)r * nf + i]);
            ly->addNode(nd);
        }
        inputLayers[r] = ly;
    }

    FILE* fo = fopen(out, "wb");
    if (!fo) return 1;
    std::vector<float> preds((size_t)c.N * no);
    Terminator term;
    term.setEpoch(c.epochs);
    int epochs = 0;
    const int minibatchSize = c.batch;
    while (true) {
        float overallTotalError = 0.0f, overallTotalAccuracy = 0.0f;
        for (unsigned int r = 0; r < (unsigned)c.N; ++r) {
            layers[0] = inputLayers[r];
            /* scrambleDropout (LayerBuilder.cpp:497-523): the row's input layer, then the hidden
               layers; with p = 0 the flags stay false and only rand() is consumed */
            for (int L = 0; L < H1; ++L) layers[L]->generateDropout(pdrop[L]);
            if (with_dropout)
                for (int L = 0; L < H1; ++L)
                    for (unsigned i = 0; i < layers[L]->size(); ++i)
                        flags.push_back(layers[L]->possiblePath(i) ? 0.0f : 1.0f);
            /* ---- ForwardPass ---- */
            for (int cl = 0; cl < H1; ++cl) {
                Layer* inL = layers[cl];
                Layer* outL = layers[cl + 1];
                for (unsigned o = 0; o < outL->size(); ++o)
                    for (unsigned i = 0; i < inL->size(); ++i) {
                        Node* inN = inL->getNode(i);
                        Node* outN = (*outL)[o];
                        bool dropout = !(inL->possiblePath(i) && outL->possiblePath(o));
                        if (!dropout) {
                            float ea = outN->getEdgeWeight(i) * inN->getWeight();
                            outN->setActivation(i, ea);
                        }
                        if (i == inL->lastValidPath()) {
                            float z = outN->getActivation();
                            outN->clearActivation();
                            if (inL->getType() != Layer::INPUT_TYPE) z += inL->getBiasWeight();
                            float a = GMath::squash(z, c.act[cl], c.act_param[cl]);
                            outN->setWeight(a);
                            if (outL->getType() == Layer::OUTPUT_TYPE) {
                                float prediction = outN->getWeight();
                                float expectation = Y[(size_t)r * no + o];
                                preds[(size_t)r * no + o] = prediction;
                                float dataSize = (float)((unsigned)c.N * outL->size());
                                float cost = GMath::outputNodeCost(expectation, prediction, dataSize, c.cost);
                                overallTotalError += cost;
                                float pe = GMath::PercentError(prediction, expectation, cost);
                                float accuracy = (1.0f - pe) * 100.0f;
                                if (accuracy < 0.0f) accuracy = 0.0f;
                                overallTotalAccuracy += accuracy;
                            }
                        }
                    }
            }
            /* ---- BackPropagation ---- */
            for (int cl = H1; cl > 0; --cl) {
                Layer* inL = layers[cl - 1];
                Layer* outL = layers[cl];
                const int hp = cl - 1;
                for (unsigned i = 0; i < inL->size(); ++i)
                    for (unsigned o = 0; o < outL->size(); ++o) {
                        Node* inN = inL->getNode(i);
                        Node* outN = (*outL)[o];
                        float der = 1.0f;
                        if (outL->getType() == Layer::OUTPUT_TYPE) {
                            float prediction = outN->getWeight();
                            float expectation = Y[(size_t)r * no + o];
                            outN->clearErrDer();
                            outN->adjustErrDer(GMath::costErrDer(expectation, prediction, c.cost));
                        } else if (outL->getType() == Layer::HIDDEN_TYPE) {
                            der = GMath::activationErrDer(outN->getWeight(), c.act[hp], 0.01f);
                        }
                        bool dropout = !(inL->possiblePath(i) && outL->possiblePath(o));
                        float d = outN->getErrDer();
                        if (!dropout) {
                            d *= der;
                            if (i == inL->size() - 1) outN->clearErrDer();
                            float lr = c.lr[hp], mom = c.mom[hp], wd1 = c.wd1[hp], wd2 = c.wd2[hp];
                            float base = lr * d;
                            outN->getDelta(i, base, inN->getWeight(), lr, mom, wd1, wd2);
                            if ((r % minibatchSize) == 0) {
                                outN->applyDeltas(i, minibatchSize);
                                outN->clearPrevDeltas(i);
                            }
                            if (inL->getType() != Layer::INPUT_TYPE)
                                inL->setBiasWeight(inL->getBiasWeight() - base);
                        }
                        float cin = inN->getErrDer() + (d * outN->getEdgeWeight(i));
                        inN->adjustErrDer(cin);
                    }
            }
        }
        ++epochs;
        overallTotalAccuracy /= ((float)(unsigned)c.N) * ((float)(unsigned)no);
        wrf(fo, overallTotalError);
        wrf(fo, overallTotalAccuracy);
        if (term.triggered(1, epochs, -1.0f)) break;
    }
    for (int L = 1; L <= H1; ++L)
        for (int o = 0; o < c.sizes[L]; ++o)
            for (int i = 0; i < c.sizes[L - 1]; ++i) wrf(fo, (*layers[L])[o]->getEdgeWeight(i));
    for (int l = 0; l < H1; ++l) wrf(fo, l >= 1 ? layers[l]->getBiasWeight() : 0.0f);
    wr(fo, &preds[0], preds.size() * 4);
    /* window state: number of pending deltas, their ordered sum from 0, and the last one */
    for (int L = 1; L <= H1; ++L)
        for (int o = 0; o < c.sizes[L]; ++o)
            for (int i = 0; i < c.sizes[L - 1]; ++i) {
                std::vector<float> pd = (*layers[L])[o]->getPrevDeltas(i);
                float s = 0.0f;
                /* the entries applyDeltas would read (node.cpp:299-301: the first minibatchSize) */
                for (size_t k = 0; k < pd.size() && k < (size_t)minibatchSize; ++k) s += pd[k];
                wrf(fo, s);
                wrf(fo, pd.empty() ? 0.0f : pd.back());
            }
    if (with_dropout) {
        wr(fo, &flags[0], flags.size() * 4);
        /* what is left behind between rows: window lengths and the hidden nodes' accumulators */
        for (int L = 1; L <= H1; ++L)
            for (int o = 0; o < c.sizes[L]; ++o)
                for (int i = 0; i < c.sizes[L - 1]; ++i)
                    wrf(fo, (float)(*layers[L])[o]->getPrevDeltas(i).size());
        for (int L = 1; L < H1; ++L)
            for (int o = 0; o < c.sizes[L]; ++o) wrf(fo, (*layers[L])[o]->getErrDer());
        wrf(fo, (float)(rand() % 65536)); /* where the rand() stream stands afterwards */
    }
    fclose(fo);
    return 0;
}

int main(int argc, char** argv)
{
    if (argc >= 3 && !strcmp(argv[1], "gmath")) return do_gmath(argv[2]);
    if (argc >= 7 && !strcmp(argv[1], "xavierseq"))
        return do_xavier_seq(atoi(argv[2]), argv[3], argc - 4, argv + 4);
    if (argc >= 7 && !strcmp(argv[1], "xavier"))
        return do_xavier(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), argv[6]);
    if (argc >= 4 && !strcmp(argv[1], "train")) return do_train(argv[2], argv[3]);
    if (argc >= 3 && !strcmp(argv[1], "term")) return do_term(argv[2]);
    fprintf(stderr, "usage: see the header of ref_harness.cpp\n");
    return 64;
}

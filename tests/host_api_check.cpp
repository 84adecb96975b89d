// Driver for the C++ class API (glades-ml_amd/host/glades.h), used by tests/test_host_api.py.
// Written the way the reference's own unit test drives a network
// ("unit-tests/Backend/Machine Learning/nn-test.cpp":27-75): build / load an NNInfo, set the
// Terminator, glades::train(&network, dataInput), read accuracy and epochs.
//
//   host_api_check xavier <seed> <fan_in> <n_out> <act> <out.bin>        (no GPU needed)
//   host_api_check nninfo <table.csv> <resaved.csv>                      (no GPU needed)
//   host_api_check cmatrix <n> <pairs.bin> <out.bin>                     (no GPU needed)
//   host_api_check train  <case.bin> <out.bin> <stop_epoch> <stop_accuracy> <mode>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <vector>

#include "glades.h"

using namespace glades;

static int do_xavier(int seed, int fi, int no, int act, const char* out)
{
    srand(seed);
    std::vector<float> W((size_t)fi * no);
    xavierLayer(fi, no, act, W.data());
    FILE* f = fopen(out, "wb");
    if (!f) return 1;
    fwrite(W.data(), 4, W.size(), f);
    fclose(f);
    return 0;
}

static int do_nninfo(const char* path, const char* resave)
{
    NNetwork net;
    if (!net.load(path)) { printf("load failed\n"); return 1; }
    NNInfo* s = net.getNNInfo();
    printf("hidden %d out %u type %d batch %d\n", s->numHiddenLayers(), s->getOutputLayerSize(), s->getOutputType(), s->getBatchSize());
    for (int i = 0; i <= s->numHiddenLayers() + 1; ++i)
        printf("idx %d lr %f mom %f wd1 %f wd2 %f p %f act %d par %f\n", i, s->getLearningRate(i), s->getMomentumFactor(i),
               s->getWeightDecay1(i), s->getWeightDecay2(i), s->getPDropout(i), s->getActivationType(i), s->getActivationParam(i));
    for (int i = 0; i < s->numHiddenLayers(); ++i) printf("hsize %d %d\n", i, s->getHiddenLayerSize(i));
    return net.save(resave) ? 0 : 2;
}

// pairs.bin: rows of n (expected, predicted) float pairs, interleaved as NNetwork's results list holds them
static int do_cmatrix(int n, const char* in, const char* out)
{
    FILE* f = fopen(in, "rb");
    if (!f) return 1;
    CMatrix cm;
    cm.build(n);
    std::vector<float> row(2 * n);
    while (fread(row.data(), 4, row.size(), f) == row.size()) cm.addResult(row);
    fclose(f);
    cm.updateResultParams();
    FILE* fo = fopen(out, "wb");
    if (!fo) return 1;
    for (int r = 0; r < n; ++r)
        for (int c = 0; c < n; ++c) { float v = (float)cm.getCell(r, c); fwrite(&v, 4, 1, fo); }
    float ov[6] = {cm.getOverallAccuracy(), cm.getOverallPrecision(), cm.getOverallRecall(), cm.getOverallSpecificity(),
                   cm.getOverallF1Score(), cm.getOverallFalseAlarm()};
    fwrite(ov, 4, 6, fo);
    fclose(fo);
    return 0;
}

static int do_train(const char* in, const char* out, long stop_epoch, float stop_acc, int mode)
{
    FILE* f = fopen(in, "rb");
    if (!f) return 1;
    int32_t magic, nl;
    if (fread(&magic, 4, 1, f) != 1 || fread(&nl, 4, 1, f) != 1 || magic != 0x474c4144) return 2;
    std::vector<int32_t> sizes(nl + 1);
    if (fread(sizes.data(), 4, nl + 1, f) != (size_t)nl + 1) return 2;
    int32_t h4[4];
    if (fread(h4, 4, 4, f) != 4) return 2;
    const int batch = h4[0], cost = h4[1], N = h4[2];
    std::vector<float> lr(nl), mom(nl), wd1(nl), wd2(nl), par(nl);
    std::vector<int32_t> act(nl);
    for (int l = 0; l < nl; ++l) {
        float p[4];
        if (fread(p, 4, 4, f) != 4 || fread(&act[l], 4, 1, f) != 1 || fread(&par[l], 4, 1, f) != 1) return 2;
        lr[l] = p[0]; mom[l] = p[1]; wd1[l] = p[2]; wd2[l] = p[3];
    }
    std::vector<std::vector<float> > W(nl);
    for (int l = 0; l < nl; ++l) {
        W[l].resize((size_t)sizes[l] * sizes[l + 1]);
        if (fread(W[l].data(), 4, W[l].size(), f) != W[l].size()) return 2;
    }
    std::vector<float> bias(nl);
    if (fread(bias.data(), 4, nl, f) != (size_t)nl) return 2;
    std::vector<float> X((size_t)N * sizes[0]), Y((size_t)N * sizes[nl]);
    if (fread(X.data(), 4, X.size(), f) != X.size() || fread(Y.data(), 4, Y.size(), f) != Y.size()) return 2;
    fclose(f);

    // skeleton rows: the input row carries weight layer 0's hyper-parameters, hidden row k those of
    // weight layer k (ML/Structure/nninfo.cpp:240-373)
    InputLayerInfo* il = new InputLayerInfo(batch, lr[0], mom[0], wd1[0], wd2[0], 0.0f, act[0], par[0]);
    std::vector<HiddenLayerInfo*> hidden;
    for (int k = 1; k < nl; ++k) hidden.push_back(new HiddenLayerInfo(sizes[k], lr[k], mom[k], wd1[k], wd2[k], 0.0f, act[k], par[k]));
    OutputLayerInfo* ol = new OutputLayerInfo(sizes[nl], cost);
    NNInfo info("check", il, hidden, ol);

    glades::init();
    DenseInput di(X.data(), Y.data(), N, sizes[0], sizes[nl]);
    NNetwork net(&info);
    net.setMode(mode);
    for (int l = 0; l < nl; ++l) {
        net.setWeights(l, W[l]);
        if (mode == NNetwork::MODE_EXACT) net.setBias(l, std::vector<float>(1, bias[l]));
    }
    net.terminator.setEpoch(stop_epoch);
    net.terminator.setAccuracy(stop_acc);
    if (!(net.getAccuracy() < 95.0f)) return 3;  // the reference test's own pre-training assertion
    MetaNetwork* meta = glades::train(&net, &di);
    if (!meta || meta->size() != 1) return 4;
    if (!net.getLastError().empty()) { fprintf(stderr, "error: %s\n", net.getLastError().c_str()); return 5; }
    const int trained = net.getEpochs();
    const float acc = net.getAccuracy(), loss = net.getLoss();
    std::vector<float> results = net.getResults();
    // the class figures of the last training epoch (network.cpp:218-224) and the matrix behind them
    const CMatrix& cm = net.getConfusionMatrix();
    std::vector<float> tail(1, (float)cm.size());
    if (cm.size() > 0) {
        const float five[5] = {net.getClassAccuracy(), net.getClassPrecision(), net.getClassRecall(), net.getClassSpecificity(), net.getClassF1()};
        tail.insert(tail.end(), five, five + 5);
        for (unsigned int r = 0; r < cm.size(); ++r)
            for (unsigned int c = 0; c < cm.size(); ++c) tail.push_back((float)cm.getCell(r, c));
    }
    glades::test(&net, &di);   // RUN_TEST pass: one more epoch counted, parameters untouched
    FILE* fo = fopen(out, "wb");
    if (!fo) return 1;
    float head[6] = {(float)trained, acc, loss, (float)net.getEpochs(), net.getAccuracy(), (float)results.size()};
    fwrite(head, 4, 6, fo);
    fwrite(results.data(), 4, results.size(), fo);
    for (int l = 0; l < nl; ++l) {
        std::vector<float> w = net.getWeights(l);
        fwrite(w.data(), 4, w.size(), fo);
    }
    for (int l = 0; l < nl; ++l) {
        std::vector<float> b = net.getBias(l);
        fwrite(b.data(), 4, b.size(), fo);
    }
    fwrite(tail.data(), 4, tail.size(), fo);
    fclose(fo);
    delete meta;
    return 0;
}

int main(int argc, char** argv)
{
    if (argc >= 7 && !strcmp(argv[1], "xavier")) return do_xavier(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), argv[6]);
    if (argc >= 4 && !strcmp(argv[1], "nninfo")) return do_nninfo(argv[2], argv[3]);
    if (argc >= 5 && !strcmp(argv[1], "cmatrix")) return do_cmatrix(atoi(argv[2]), argv[3], argv[4]);
    if (argc >= 7 && !strcmp(argv[1], "train")) return do_train(argv[2], argv[3], atol(argv[4]), (float)atof(argv[5]), atoi(argv[6]));
    fprintf(stderr, "usage: see the header of host_api_check.cpp\n");
    return 64;
}

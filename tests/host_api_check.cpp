// Driver for the C++ class API (glades-ml_amd/host/glades.h), used by tests/test_host_api.py.
// Written the way the reference's own unit test drives a network
// ("unit-tests/Backend/Machine Learning/nn-test.cpp":27-75): build / load an NNInfo, set the
// Terminator, glades::train(&network, dataInput), read accuracy and epochs.
//
//   host_api_check xavier <seed> <fan_in> <n_out> <act> <out.bin>        (no GPU needed)
//   host_api_check initseq <seed> <n_feat> <n_out> <output type> <out.bin> <input-row act> [<hidden size> <hidden-row act> ...]   (no GPU needed)
//   host_api_check randpos <case.bin> <seed> <epochs> <k subnets> <concurrent 0|1> <out.bin>
//   host_api_check nninfo <table.csv> <resaved.csv>                      (no GPU needed)
//   host_api_check cmatrix <n> <pairs.bin> <out.bin>                     (no GPU needed)
//   host_api_check ohe                                                   (no GPU needed)
//   host_api_check numberinput <file.csv> <minmax|zscore> <out.bin>      (no GPU needed)
//   host_api_check traincsv <file.csv> <nninfo table> <stop_epoch> <stop_accuracy> <seed> <out.bin> [case.bin with the initial weights]
//   host_api_check checkpoint <case.bin> <mode> <E1> <E2> <file.ckpt> <out.bin>
//   host_api_check meta <case.bin> <mode> <k subnets> <epochs> <out.bin>
//   host_api_check train  <case.bin> <out.bin> <stop_epoch> <stop_accuracy> <mode>
//   host_api_check dropout <case.bin> <seed> <E1> <E2> <file.ckpt> <out.bin> <rate of the input row> <rates of the hidden rows ...>
//   host_api_check dropoutcanon <case.bin> <seed> <epochs> <out.bin> <rates as above>      (canonical mode)
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include <vector>

#include "glades.h"

// writes a float array; an empty one (whose data() may be null) writes nothing
static void put(const std::vector<float>& v, FILE* f) { if (!v.empty()) fwrite(v.data(), 4, v.size(), f); }

using namespace glades;

static int do_xavier(int seed, int fi, int no, int act, const char* out)
{
    srand(seed);
    std::vector<float> W((size_t)fi * no);
    xavierLayer(fi, no, act, W.data());
    FILE* f = fopen(out, "wb");
    if (!f) return 1;
    put(W, f);
    fclose(f);
    return 0;
}

// the whole network's initial weights in the reference's sampling order, then rand() % 65536
static int do_initseq(int seed, int nFeat, int nOut, int outType, const char* out, int n, char** spec)
{
    std::vector<HiddenLayerInfo*> hidden;
    for (int k = 1; k + 1 < n; k += 2) hidden.push_back(new HiddenLayerInfo(atoi(spec[k]), 0.01f, 0.0f, 0.0f, 0.0f, 0.0f, atoi(spec[k + 1]), 0.0f));
    NNInfo info("seq", new InputLayerInfo(1, 0.01f, 0.0f, 0.0f, 0.0f, 0.0f, atoi(spec[0]), 0.0f), hidden, new OutputLayerInfo(nOut, outType));
    srand(seed);
    std::vector<std::vector<float> > W;
    std::string err;
    if (!sampleInitialWeights(&info, nFeat, nOut, W, &err)) { printf("refused: %s\n", err.c_str()); return 7; }
    FILE* f = fopen(out, "wb");
    if (!f) return 1;
    for (size_t l = 0; l < W.size(); ++l) put(W[l], f);
    const float next = (float)(rand() % 65536);
    fwrite(&next, 4, 1, f);
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

// the editing methods of NNInfo (nninfo.cpp:436-703) on a loaded table; prints the table after every step
static int do_nnedit(const char* path)
{
    NNetwork net;
    if (!net.load(path)) return 1;
    NNInfo* s = net.getNNInfo();
    auto dump = [&](const char* what) {
        printf("-- %s\n", what);
        const NNTable t = s->toTable();
        for (size_t r = 0; r < t.size(); ++r) {
            for (size_t c = 0; c < t[r].size(); ++c) printf("%s%g", c ? "," : "", t[r][c]);
            printf("\n");
        }
    };
    dump("loaded");
    s->setPInput(0.25f); s->setPDropout(1, 0.5f); s->setWeightDecay1(2, 0.125f);
    s->setWeightDecay2(0, 0.75f); s->setWeightDecay2(1, 0.0625f); s->setWeightDecay2(2, 0.03125f);
    dump("rates");
    s->copyHiddenLayer(1, 0);
    dump("copy 1 <- 0");
    s->resizeHiddenLayers(4);
    s->setLearningRate(3, 0.5f);   // hidden row 2 only: the new rows are separate objects
    dump("resize 4");
    s->removeHiddenLayer(0);
    s->resizeHiddenLayers(2);
    dump("remove 0, resize 2");
    printf("input size %d hidden %d p %g/%g\n", s->getInputLayerSize(), s->numHiddenLayers(), s->getPInput(), s->getPDropout(0));
    s->print();
    return 0;
}

// NNetwork::save() / load(name) / glades::saveNeuralNetwork through the database folder of the working
// directory (the caller runs this in a scratch directory), getLearningCurve, getCurrentTimeMilliseconds
static int do_db(const char* table)
{
    if (glades::doesDatabaseExist()) return 1;
    NNetwork net;
    if (!net.load(table)) return 2;
    net.getNNInfo()->setName("saved-net");
    if (!glades::saveNeuralNetwork(&net) || !glades::doesDatabaseExist()) return 3;
    NNetwork again;
    if (!again.load("saved-net")) return 4;           // no such path: looked up in database/neuralnetworks/
    if (again.getName() != "saved-net") return 5;
    if (again.getNNInfo()->toTable() != net.getNNInfo()->toTable()) return 6;
    NNetwork none;
    if (none.load("no-such-net") || none.save() || glades::saveNeuralNetwork(NULL)) return 7;
    // MetaNetwork's constructors and look-ups (metanetwork.cpp:30-214)
    {
        MetaNetwork byInfo(net.getNNInfo(), 3);
        if (byInfo.size() != 3 || byInfo.getName() != "saved-net" || byInfo.getCollectionType() != MetaNetwork::ONE_TO_MANY) return 9;
        if (byInfo.getSubnet(0) == byInfo.getSubnet(1) || byInfo.getSubnet(2)->getNNInfo() != net.getNNInfo()) return 10;
        MetaNetwork byName("meta", "saved-net", 2);
        if (byName.size() != 2 || byName.getSubnetName(1) != "saved-net" || byName.getSubnetByName("saved-net") != byName.getSubnet(0)) return 11;
        if (byName.getSubnetByName("other") || byName.getSubnetName(5) != "") return 12;
        byName.addSubnet(std::string("no-such-net"));
        byName.addSubnet(std::string(""));
        if (byName.size() != 2 || byName.getCollectionType() != MetaNetwork::ONE_TO_MANY) return 13;
        MetaNetwork one("solo");
        one.setName("renamed");
        if (one.size() != 0 || one.getName() != "renamed" || one.getCollectionType() != MetaNetwork::ONE_TO_ONE) return 14;
    }
    const int64_t t0 = net.getCurrentTimeMilliseconds();
    if (t0 < 1600000000000LL) return 8;
    printf("db ok\n");
    return 0;
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

// the assertions of the reference's own OHE unit test ("unit-tests/Backend/Machine Learning/ohe-test.cpp":17-45)
static int do_ohe()
{
    OHE ohe;
    if (ohe.size() != 0) return 1;
    ohe.addString("cat");
    ohe.addString("dog");
    ohe.addString("cat");
    if (ohe.size() != 2 || !ohe.contains("cat") || !ohe.contains("dog")) return 2;
    std::vector<float> cat = ohe["cat"], dog = ohe["dog"];
    if (cat.size() != 2 || dog.size() != 2) return 3;
    if (!(cat[0] == 0.99f && cat[1] == 0.01f)) return 4;
    if (!(dog[0] == 0.01f && dog[1] == 0.99f)) return 5;
    if (ohe.indexAt("cat") != 0 || ohe.indexAt("dog") != 1 || ohe.indexAt("bird") != -1) return 6;
    std::vector<float> probe(2); probe[0] = 0.2f; probe[1] = 0.7f;
    if (ohe[probe] != "dog" || ohe.classAt(0) != "cat" || ohe.classAt(5) != "") return 7;
    printf("ohe ok\n");
    return 0;
}

static int do_numberinput(const char* csv, const char* flag, const char* out)
{
    NumberInput di;
    if (!di.standardizeInputTable(csv, !strcmp(flag, "zscore") ? GMath::ZSCORE : GMath::MINMAX)) return 1;
    FILE* fo = fopen(out, "wb");
    if (!fo) return 1;
    float head[3] = {(float)di.getTrainSize(), (float)di.getFeatureCount(), (float)di.getOutputCount()};
    fwrite(head, 4, 3, fo);
    for (unsigned int r = 0; r < di.getTrainSize(); ++r) { std::vector<float> v = di.getTrainRow(r); put(v, fo); }
    for (unsigned int r = 0; r < di.getTrainSize(); ++r) { std::vector<float> v = di.getTrainExpectedRow(r); put(v, fo); }
    fclose(fo);
    for (size_t c = 0; c < di.getOHEMaps().size(); ++c) {
        printf("col %d categorical %d classes", (int)c, (int)di.featureIsCategorical[c]);
        std::vector<std::string> cls = di.getOHEMaps()[c].getStrings();
        for (size_t k = 0; k < cls.size(); ++k) printf(" %s", cls[k].c_str());
        printf("\n");
    }
    return 0;
}

// the flow of the reference's network test ("unit-tests/Backend/Machine Learning/nn-test.cpp":27-75):
// NumberInput::import(csv), NNetwork::load(table), Terminator, glades::train.  Initial weights come
// from srand(seed) + the sampler, or, when a case file is given, from that file (its table is ignored).
struct Case {
    int nl, batch, cost, N;
    std::vector<int32_t> sizes, act;
    std::vector<float> lr, mom, wd1, wd2, par, bias, X, Y;
    std::vector<std::vector<float> > W;
};

static int read_case(const char* in, Case& c)
{
    FILE* f = fopen(in, "rb");
    if (!f) return 1;
    int32_t magic, nl;
    if (fread(&magic, 4, 1, f) != 1 || fread(&nl, 4, 1, f) != 1 || magic != 0x474c4144) return 2;
    c.nl = nl;
    c.sizes.resize(nl + 1);
    if (fread(c.sizes.data(), 4, nl + 1, f) != (size_t)nl + 1) return 2;
    int32_t h4[4];
    if (fread(h4, 4, 4, f) != 4) return 2;
    c.batch = h4[0]; c.cost = h4[1]; c.N = h4[2];
    c.lr.resize(nl); c.mom.resize(nl); c.wd1.resize(nl); c.wd2.resize(nl); c.par.resize(nl); c.act.resize(nl);
    for (int l = 0; l < nl; ++l) {
        float p[4];
        if (fread(p, 4, 4, f) != 4 || fread(&c.act[l], 4, 1, f) != 1 || fread(&c.par[l], 4, 1, f) != 1) return 2;
        c.lr[l] = p[0]; c.mom[l] = p[1]; c.wd1[l] = p[2]; c.wd2[l] = p[3];
    }
    c.W.resize(nl);
    for (int l = 0; l < nl; ++l) {
        c.W[l].resize((size_t)c.sizes[l] * c.sizes[l + 1]);
        if (fread(c.W[l].data(), 4, c.W[l].size(), f) != c.W[l].size()) return 2;
    }
    c.bias.resize(nl);
    if (fread(c.bias.data(), 4, nl, f) != (size_t)nl) return 2;
    c.X.resize((size_t)c.N * c.sizes[0]); c.Y.resize((size_t)c.N * c.sizes[nl]);
    if (fread(c.X.data(), 4, c.X.size(), f) != c.X.size() || fread(c.Y.data(), 4, c.Y.size(), f) != c.Y.size()) return 2;
    fclose(f);
    return 0;
}

// trains `net` on `di`, then runs the RUN_TEST pass, and writes what the tests read
static int train_and_dump(NNetwork& net, DataInput* di, int nl, const char* out)
{
    if (!(net.getAccuracy() < 95.0f)) return 3;  // the reference test's own pre-training assertion
    MetaNetwork* meta = glades::train(&net, di);
    if (!meta || meta->size() != 1) return 4;
    if (!net.getLastError().empty()) { fprintf(stderr, "error: %s\n", net.getLastError().c_str()); return 5; }
    const int trained = net.getEpochs();
    const float acc = net.getAccuracy(), loss = net.getLoss();
    const std::vector<float> curve = net.getLearningCurve();
    if ((int)curve.size() != trained || (trained > 0 && curve.back() != acc)) return 6;  // one accuracy per epoch of the run
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
    glades::test(&net, di);   // RUN_TEST pass: one more epoch counted, parameters untouched
    FILE* fo = fopen(out, "wb");
    if (!fo) return 1;
    float head[6] = {(float)trained, acc, loss, (float)net.getEpochs(), net.getAccuracy(), (float)results.size()};
    fwrite(head, 4, 6, fo);
    put(results, fo);
    for (int l = 0; l < nl; ++l) {
        std::vector<float> w = net.getWeights(l);
        put(w, fo);
    }
    for (int l = 0; l < nl; ++l) {
        std::vector<float> b = net.getBias(l);
        put(b, fo);
    }
    put(tail, fo);
    fclose(fo);
    delete meta;
    return 0;
}

static int do_train(const char* in, const char* out, long stop_epoch, float stop_acc, int mode)
{
    Case c;
    int rc = read_case(in, c);
    if (rc) return rc;
    const int nl = c.nl;
    // skeleton rows: the input row carries weight layer 0's hyper-parameters, hidden row k those of
    // weight layer k (ML/Structure/nninfo.cpp:240-373)
    InputLayerInfo* il = new InputLayerInfo(c.batch, c.lr[0], c.mom[0], c.wd1[0], c.wd2[0], 0.0f, c.act[0], c.par[0]);
    std::vector<HiddenLayerInfo*> hidden;
    for (int k = 1; k < nl; ++k) hidden.push_back(new HiddenLayerInfo(c.sizes[k], c.lr[k], c.mom[k], c.wd1[k], c.wd2[k], 0.0f, c.act[k], c.par[k]));
    OutputLayerInfo* ol = new OutputLayerInfo(c.sizes[nl], c.cost);
    NNInfo info("check", il, hidden, ol);

    glades::init();
    DenseInput di(c.X.data(), c.Y.data(), c.N, c.sizes[0], c.sizes[nl]);
    NNetwork net(&info);
    net.setMode(mode);
    for (int l = 0; l < nl; ++l) {
        net.setWeights(l, c.W[l]);
        if (mode == NNetwork::MODE_EXACT) net.setBias(l, std::vector<float>(1, c.bias[l]));
    }
    net.terminator.setEpoch(stop_epoch);
    net.terminator.setAccuracy(stop_acc);
    return train_and_dump(net, &di, nl, out);
}

static int do_traincsv(const char* csv, const char* table, long stop_epoch, float stop_acc, int seed, const char* out, const char* weights)
{
    glades::init();
    srand(seed);
    NumberInput di;
    di.import(csv);
    NNetwork net;
    if ((net.getEpochs() == 0) && (!net.load(table))) { printf("[NN] Unable to load \"%s\"", table); return 1; }
    const int nl = net.getNNInfo()->numHiddenLayers() + 1;
    if (weights) {
        Case c;
        int rc = read_case(weights, c);
        if (rc) return rc;
        if (c.nl != nl) return 6;
        for (int l = 0; l < nl; ++l) {
            net.setWeights(l, c.W[l]);
            net.setBias(l, std::vector<float>(1, c.bias[l]));
        }
    }
    net.terminator.setEpoch(stop_epoch);
    net.terminator.setAccuracy(stop_acc);
    return train_and_dump(net, &di, nl, out);
}

static NNInfo* case_info(const Case& c)
{
    InputLayerInfo* il = new InputLayerInfo(c.batch, c.lr[0], c.mom[0], c.wd1[0], c.wd2[0], 0.0f, c.act[0], c.par[0]);
    std::vector<HiddenLayerInfo*> hidden;
    for (int k = 1; k < c.nl; ++k) hidden.push_back(new HiddenLayerInfo(c.sizes[k], c.lr[k], c.mom[k], c.wd1[k], c.wd2[k], 0.0f, c.act[k], c.par[k]));
    return new NNInfo("check", il, hidden, new OutputLayerInfo(c.sizes[c.nl], c.cost));
}

// the rows of the table carry the dropout rates: pd[0] on the input row, pd[k] on hidden row k-1
static NNInfo* case_info_dropout(const Case& c, const std::vector<float>& pd)
{
    InputLayerInfo* il = new InputLayerInfo(c.batch, c.lr[0], c.mom[0], c.wd1[0], c.wd2[0], pd[0], c.act[0], c.par[0]);
    std::vector<HiddenLayerInfo*> hidden;
    for (int k = 1; k < c.nl; ++k) hidden.push_back(new HiddenLayerInfo(c.sizes[k], c.lr[k], c.mom[k], c.wd1[k], c.wd2[k], pd[k], c.act[k], c.par[k]));
    return new NNInfo("check", il, hidden, new OutputLayerInfo(c.sizes[c.nl], c.cost));
}

static void seed_net(NNetwork& net, const Case& c, int mode)
{
    net.setMode(mode);
    for (int l = 0; l < c.nl; ++l) {
        net.setWeights(l, c.W[l]);
        if (mode == NNetwork::MODE_EXACT) net.setBias(l, std::vector<float>(1, c.bias[l]));
    }
}

// Dropout through the class API: srand(seed); A trains E1 epochs and saves; B restores and trains on to
// E1 + E2 (the rand() stream runs on); srand(seed) again; C trains E1 + E2 in one go; then C's test pass.
// out: epochs of B and C, their losses, C's test-pass accuracy and rand() % 65536 after it, then
// every layer's weights and bias of B, then of C.
static int do_dropout(const char* in, int seed, int e1, int e2, const char* ckpt, const char* out, const std::vector<float>& pd)
{
    Case c;
    int rc = read_case(in, c);
    if (rc) return rc;
    if ((int)pd.size() != c.nl) return 6;
    glades::init();
    DenseInput di(c.X.data(), c.Y.data(), c.N, c.sizes[0], c.sizes[c.nl]);
    NNInfo* ia = case_info_dropout(c, pd);
    NNInfo* ic = case_info_dropout(c, pd);
    srand(seed);
    {
        NNetwork a(ia);
        seed_net(a, c, NNetwork::MODE_EXACT);
        a.setVerbose(false);
        if (!a.hasDropout()) return 7;
        a.terminator.setEpoch(e1);
        a.train(&di);
        if (a.getEpochs() != e1 || !a.saveCheckpoint(ckpt)) { fprintf(stderr, "save: %s\n", a.getLastError().c_str()); return 3; }
    }
    NNetwork b;
    if (!b.loadCheckpoint(ckpt)) { fprintf(stderr, "load: %s\n", b.getLastError().c_str()); return 4; }
    b.setVerbose(false);
    b.terminator.setEpoch(e1 + e2);
    b.train(&di);
    if (!b.getLastError().empty()) { fprintf(stderr, "b: %s\n", b.getLastError().c_str()); return 5; }
    srand(seed);
    NNetwork cn(ic);
    seed_net(cn, c, NNetwork::MODE_EXACT);
    cn.setVerbose(false);
    cn.terminator.setEpoch(e1 + e2);
    cn.train(&di);
    if (!cn.getLastError().empty()) { fprintf(stderr, "c: %s\n", cn.getLastError().c_str()); return 5; }
    const float train_loss = cn.getLoss();
    const int trained_c = cn.getEpochs();
    std::vector<std::vector<float> > w, bb;
    NNetwork* nets[2] = {&b, &cn};
    for (int k = 0; k < 2; ++k)
        for (int l = 0; l < c.nl; ++l) { w.push_back(nets[k]->getWeights(l)); bb.push_back(nets[k]->getBias(l)); }
    cn.test(&di);  // draws flags as well (network.cpp:407-411)
    FILE* fo = fopen(out, "wb");
    if (!fo) return 1;
    float head[6] = {(float)b.getEpochs(), (float)trained_c, b.getLoss(), train_loss, cn.getAccuracy(), (float)(rand() % 65536)};
    fwrite(head, 4, 6, fo);
    for (size_t k = 0; k < w.size(); ++k) { put(w[k], fo); put(bb[k], fo); }
    fclose(fo);
    return 0;
}

// Canonical mode with dropout rates in the table: trains `epochs` epochs and runs a test pass under srand(seed).
// out: epochs, training loss, test accuracy, the next rand() % 65536, then every layer's weights and bias.
static int do_dropout_canonical(const char* in, int seed, int epochs, const char* out, const std::vector<float>& pd)
{
    Case c;
    int rc = read_case(in, c);
    if (rc) return rc;
    if ((int)pd.size() != c.nl) return 6;
    glades::init();
    DenseInput di(c.X.data(), c.Y.data(), c.N, c.sizes[0], c.sizes[c.nl]);
    NNInfo* info = case_info_dropout(c, pd);
    srand(seed);
    NNetwork net(info);
    seed_net(net, c, NNetwork::MODE_CANONICAL);
    net.setVerbose(false);
    if (!net.hasDropout()) return 7;
    net.terminator.setEpoch(epochs);
    net.train(&di);
    if (!net.getLastError().empty()) { fprintf(stderr, "train: %s\n", net.getLastError().c_str()); return 5; }
    const float train_loss = net.getLoss();
    const int trained = net.getEpochs();
    std::vector<std::vector<float> > w, bb;
    for (int l = 0; l < c.nl; ++l) { w.push_back(net.getWeights(l)); bb.push_back(net.getBias(l)); }
    net.test(&di);  // draws flags as well (network.cpp:407-411)
    if (!net.getLastError().empty()) { fprintf(stderr, "test: %s\n", net.getLastError().c_str()); return 5; }
    FILE* fo = fopen(out, "wb");
    if (!fo) return 1;
    float head[4] = {(float)trained, train_loss, net.getAccuracy(), (float)(rand() % 65536)};
    fwrite(head, 4, 4, fo);
    for (size_t k = 0; k < w.size(); ++k) { put(w[k], fo); put(bb[k], fo); }
    fclose(fo);
    return 0;
}

// A trains E1 epochs and saves; B restores and trains on to E1 + E2; C trains E1 + E2 in one go.
// out: epochs of B and C, then every layer's weights and bias of B, then of C.
static int do_checkpoint(const char* in, int mode, int e1, int e2, const char* ckpt, const char* out)
{
    Case c;
    int rc = read_case(in, c);
    if (rc) return rc;
    glades::init();
    DenseInput di(c.X.data(), c.Y.data(), c.N, c.sizes[0], c.sizes[c.nl]);
    NNInfo* ia = case_info(c);
    NNInfo* ic = case_info(c);
    {
        NNetwork a(ia);
        seed_net(a, c, mode);
        a.terminator.setEpoch(e1);
        a.train(&di);
        if (a.getEpochs() != e1 || !a.saveCheckpoint(ckpt)) { fprintf(stderr, "save: %s\n", a.getLastError().c_str()); return 3; }
    }
    NNetwork b;
    if (!b.loadCheckpoint(ckpt)) { fprintf(stderr, "load: %s\n", b.getLastError().c_str()); return 4; }
    if (b.getEpochs() != e1) return 5;
    b.terminator.setEpoch(e1 + e2);
    b.train(&di);
    NNetwork cn(ic);
    seed_net(cn, c, mode);
    cn.terminator.setEpoch(e1 + e2);
    cn.train(&di);
    FILE* fo = fopen(out, "wb");
    if (!fo) return 1;
    float head[4] = {(float)b.getEpochs(), (float)cn.getEpochs(), b.getLoss(), cn.getLoss()};
    fwrite(head, 4, 4, fo);
    NNetwork* nets[2] = {&b, &cn};
    for (int k = 0; k < 2; ++k)
        for (int l = 0; l < c.nl; ++l) {
            std::vector<float> w = nets[k]->getWeights(l), bb = nets[k]->getBias(l);
            put(w, fo);
            put(bb, fo);
        }
    fclose(fo);
    return 0;
}

// k subnets with the case's weights in one MetaNetwork: trained one after the other, then (fresh
// copies) at the same time.  out: k, seconds in order, seconds concurrent, cross-validation accuracy,
// then per subnet and per run the final loss, and every layer's weights of both runs of subnet 0 and k-1.
static int do_meta(const char* in, int mode, int k, int epochs, const char* out)
{
    Case c;
    int rc = read_case(in, c);
    if (rc) return rc;
    glades::init();
    DenseInput di(c.X.data(), c.Y.data(), c.N, c.sizes[0], c.sizes[c.nl]);
    double secs[2];
    std::vector<float> losses;
    std::vector<std::vector<float> > keep;
    float cv = 0.0f;
    for (int run = 0; run < 2; ++run) {
        MetaNetwork meta("meta");
        meta.setConcurrent(run == 1);
        for (int i = 0; i < k; ++i) {
            meta.addSubnet(case_info(c));
            NNetwork* n = meta.getSubnet(i);
            seed_net(*n, c, mode);
            n->setVerbose(false);
            n->terminator.setEpoch(epochs);
        }
        struct timespec t0, t1;
        clock_gettime(CLOCK_MONOTONIC, &t0);
        if (run == 0) { if (!glades::train(&meta, &di)) return 3; }
        else cv = meta.crossValidate(&di);
        clock_gettime(CLOCK_MONOTONIC, &t1);
        secs[run] = (t1.tv_sec - t0.tv_sec) + 1e-9 * (t1.tv_nsec - t0.tv_nsec);
        for (int i = 0; i < k; ++i) {
            NNetwork* n = meta.getSubnet(i);
            if (!n->getLastError().empty()) { fprintf(stderr, "subnet %d: %s\n", i, n->getLastError().c_str()); return 4; }
            losses.push_back(n->getLoss());
        }
        for (int which = 0; which < 2; ++which) {
            NNetwork* n = meta.getSubnet(which == 0 ? 0 : k - 1);
            std::vector<float> all;
            for (int l = 0; l < c.nl; ++l) { std::vector<float> w = n->getWeights(l); all.insert(all.end(), w.begin(), w.end()); }
            keep.push_back(all);
        }
        for (int i = 0; i < k; ++i) delete meta.getSubnet(i);
    }
    printf("meta: %d subnets x %d epochs x %d rows: in order %.3f s, concurrent (train + test pass) %.3f s\n", k, epochs, c.N, secs[0], secs[1]);
    FILE* fo = fopen(out, "wb");
    if (!fo) return 1;
    float head[4] = {(float)k, (float)secs[0], (float)secs[1], cv};
    fwrite(head, 4, 4, fo);
    put(losses, fo);
    for (size_t i = 0; i < keep.size(); ++i) put(keep[i], fo);
    fclose(fo);
    return 0;
}

// k subnets over one table whose weights are NOT injected, learning rate 0 (so that a trained network
// still holds the weights it was built with), trained `epochs` epochs and tested once each, in the
// reference's order or grouped: writes every subnet's weights and then rand() % 65536
static int do_randpos(const char* in, int seed, int epochs, int k, int concurrent, const char* out)
{
    Case c;
    int rc = read_case(in, c);
    if (rc) return rc;
    glades::init();
    DenseInput di(c.X.data(), c.Y.data(), c.N, c.sizes[0], c.sizes[c.nl]);
    for (int l = 0; l < c.nl; ++l) c.lr[l] = 0.0f;
    srand(seed);
    MetaNetwork meta("meta");
    meta.setConcurrent(concurrent != 0);
    for (int i = 0; i < k; ++i) {
        meta.addSubnet(case_info(c));
        NNetwork* n = meta.getSubnet(i);
        n->setVerbose(false);
        n->terminator.setEpoch(epochs);
    }
    meta.crossValidate(&di);   // every subnet: train, then its test pass
    FILE* fo = fopen(out, "wb");
    if (!fo) return 1;
    for (int i = 0; i < k; ++i) {
        NNetwork* n = meta.getSubnet(i);
        if (!n->getLastError().empty()) { fprintf(stderr, "subnet %d: %s\n", i, n->getLastError().c_str()); return 4; }
        for (int l = 0; l < c.nl; ++l) { std::vector<float> w = n->getWeights(l); put(w, fo); }
    }
    const float next = (float)(rand() % 65536);
    fwrite(&next, 4, 1, fo);
    fclose(fo);
    for (int i = 0; i < k; ++i) delete meta.getSubnet(i);
    return 0;
}

int main(int argc, char** argv)
{
    if (argc >= 8 && !strcmp(argv[1], "initseq")) return do_initseq(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), argv[6], argc - 7, argv + 7);
    if (argc >= 8 && !strcmp(argv[1], "randpos")) return do_randpos(argv[2], atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), atoi(argv[6]), argv[7]);
    if (argc >= 7 && !strcmp(argv[1], "xavier")) return do_xavier(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), argv[6]);
    if (argc >= 4 && !strcmp(argv[1], "nninfo")) return do_nninfo(argv[2], argv[3]);
    if (argc >= 3 && !strcmp(argv[1], "nnedit")) return do_nnedit(argv[2]);
    if (argc >= 3 && !strcmp(argv[1], "db")) return do_db(argv[2]);
    if (argc >= 7 && !strcmp(argv[1], "meta")) return do_meta(argv[2], atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), argv[6]);
    if (argc >= 8 && !strcmp(argv[1], "checkpoint")) return do_checkpoint(argv[2], atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), argv[6], argv[7]);
    if (argc >= 9 && !strcmp(argv[1], "dropout")) {
        std::vector<float> pd;
        for (int k = 8; k < argc; ++k) pd.push_back((float)atof(argv[k]));
        return do_dropout(argv[2], atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), argv[6], argv[7], pd);
    }
    if (argc >= 7 && !strcmp(argv[1], "dropoutcanon")) {
        std::vector<float> pd;
        for (int k = 6; k < argc; ++k) pd.push_back((float)atof(argv[k]));
        return do_dropout_canonical(argv[2], atoi(argv[3]), atoi(argv[4]), argv[5], pd);
    }
    if (argc >= 2 && !strcmp(argv[1], "ohe")) return do_ohe();
    if (argc >= 5 && !strcmp(argv[1], "numberinput")) return do_numberinput(argv[2], argv[3], argv[4]);
    if (argc >= 8 && !strcmp(argv[1], "traincsv")) return do_traincsv(argv[2], argv[3], atol(argv[4]), (float)atof(argv[5]), atoi(argv[6]), argv[7], argc >= 9 ? argv[8] : NULL);
    if (argc >= 5 && !strcmp(argv[1], "cmatrix")) return do_cmatrix(atoi(argv[2]), argv[3], argv[4]);
    if (argc >= 7 && !strcmp(argv[1], "train")) return do_train(argv[2], argv[3], atol(argv[4]), (float)atof(argv[5]), atoi(argv[6]));
    fprintf(stderr, "usage: see the header of host_api_check.cpp\n");
    return 64;
}

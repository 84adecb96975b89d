// Host side of the reference's class API (see glades.h) over the C ABI in include/glades_hip.h.
// Citations are to the reference tree, "ML/" = "Backend/Machine Learning/".
#include "glades.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <sys/time.h>
#include <time.h>
#include <thread>

#include "glades_hip.h"

namespace glades {

// ------------------------------------------------------------------ LayerInfo family

LayerInfo::LayerInfo(int newSize)
    : lSize(newSize), learningRate(0.01f), momentumFactor(0.0f), weightDecay1(0.0f), weightDecay2(0.0f),
      pDropout(0.0f), activationParam(0.0f), activationType(0)
{
}

InputLayerInfo::InputLayerInfo(int newBatchSize, float newLearningRate, float newMomentumFactor,
                               float newWeightDecay1, float newWeightDecay2, float newPDropout,
                               int newActivationType, float newActivationParam)
    : LayerInfo(0), batchSize(newBatchSize)
{
    learningRate = newLearningRate; momentumFactor = newMomentumFactor;
    weightDecay1 = newWeightDecay1; weightDecay2 = newWeightDecay2; pDropout = newPDropout;
    activationType = newActivationType; activationParam = newActivationParam;
}

HiddenLayerInfo::HiddenLayerInfo(int newSize, float newLearningRate, float newMomentumFactor,
                                 float newWeightDecay1, float newWeightDecay2, float newPDropout,
                                 int newActivationType, float newActivationParam)
    : LayerInfo(newSize)
{
    learningRate = newLearningRate; momentumFactor = newMomentumFactor;
    weightDecay1 = newWeightDecay1; weightDecay2 = newWeightDecay2; pDropout = newPDropout;
    activationType = newActivationType; activationParam = newActivationParam;
}

OutputLayerInfo::OutputLayerInfo(int newSize, int newOutputType) : LayerInfo(newSize), outputType(newOutputType) {}

// ------------------------------------------------------------------ NNInfo

NNInfo::NNInfo(const std::string& newName) : name(newName), inputType(0), inputLayer(NULL), outputLayer(NULL) {}

NNInfo::NNInfo(const std::string& newName, const NNTable& table)
    : name(newName), inputType(0), inputLayer(NULL), outputLayer(NULL)
{
    if (!table.empty() && table[0].size() < 10)
        printf("[NNINFO] Bad table size: (%d,%d)\n", (int)table.size(), (int)table[0].size());
    fromTable(newName, table);
}

NNInfo::NNInfo(const std::string& newName, InputLayerInfo* newInputLayer,
               const std::vector<HiddenLayerInfo*>& hidden, OutputLayerInfo* newOutputLayer)
    : name(newName), inputType(0), inputLayer(newInputLayer), outputLayer(newOutputLayer), layers(hidden)
{
}

NNInfo::~NNInfo()
{
    for (size_t i = 0; i < layers.size(); ++i) delete layers[i];
    layers.clear();
    delete inputLayer;
    delete outputLayer;
}

int NNInfo::getOutputType() const { return outputLayer ? outputLayer->getOutputType() : 0; }
float NNInfo::getPInput() const { return inputLayer ? inputLayer->getPDropout() : 0.0f; }
int NNInfo::getBatchSize() const { return inputLayer ? inputLayer->getBatchSize() : 1; }
int NNInfo::getHiddenLayerSize(unsigned int i) const { return (i < layers.size() && layers[i]) ? layers[i]->size() : 0; }
unsigned int NNInfo::getOutputLayerSize() const { return outputLayer ? (unsigned int)outputLayer->size() : 0u; }

// nninfo.cpp:240-373: index 0 = input row, index k = hidden row k-1; defaults when out of range
#define NN_GETTER(NAME, TYPE, DEFAULT, INPUT_EXPR, HIDDEN_EXPR)          \
    TYPE NNInfo::NAME(unsigned int index) const                          \
    {                                                                    \
        if (index > layers.size()) return DEFAULT;                       \
        if (index == 0) return inputLayer ? (INPUT_EXPR) : (DEFAULT);    \
        if (!layers[index - 1]) return DEFAULT;                          \
        return layers[index - 1]->HIDDEN_EXPR;                           \
    }
NN_GETTER(getLearningRate, float, 0.01f, inputLayer->getLearningRate(), getLearningRate())
NN_GETTER(getMomentumFactor, float, 0.0f, inputLayer->getMomentumFactor(), getMomentumFactor())
NN_GETTER(getWeightDecay1, float, 0.0f, inputLayer->getWeightDecay1(), getWeightDecay1())
// the reference returns the input row's weightDecay1 here (nninfo.cpp:305-306)
NN_GETTER(getWeightDecay2, float, 0.0f, inputLayer->getWeightDecay1(), getWeightDecay2())
NN_GETTER(getPDropout, float, 1.0f, inputLayer->getPDropout(), getPDropout())
NN_GETTER(getActivationType, int, 0, inputLayer->getActivationType(), getActivationType())
NN_GETTER(getActivationParam, float, 0.0f, inputLayer->getActivationParam(), getActivationParam())
#undef NN_GETTER

void NNInfo::setOutputType(int v) { if (outputLayer) outputLayer->setOutputType(v); }
void NNInfo::setOutputSize(int v) { if (outputLayer) outputLayer->setSize(v); }
void NNInfo::setBatchSize(int v) { if (inputLayer) inputLayer->setBatchSize(v); }
void NNInfo::setLearningRate(unsigned int index, float v)
{
    if (index > layers.size()) return;
    if (index == 0) { if (inputLayer) inputLayer->setLearningRate(v); }
    else if (layers[index - 1]) layers[index - 1]->setLearningRate(v);
}
void NNInfo::setMomentumFactor(unsigned int index, float v)
{
    if (index > layers.size()) return;
    if (index == 0) { if (inputLayer) inputLayer->setMomentumFactor(v); }
    else if (layers[index - 1]) layers[index - 1]->setMomentumFactor(v);
}
void NNInfo::setActivationType(unsigned int index, int v)
{
    if (index > layers.size()) return;
    if (index == 0) { if (inputLayer) inputLayer->setActivationType(v); }
    else if (layers[index - 1]) layers[index - 1]->setActivationType(v);
}
void NNInfo::setActivationParam(unsigned int index, float v)
{
    if (index > layers.size()) return;
    if (index == 0) { if (inputLayer) inputLayer->setActivationParam(v); }
    else if (layers[index - 1]) layers[index - 1]->setActivationParam(v);
}
void NNInfo::addHiddenLayer(HiddenLayerInfo* l) { if (l) layers.push_back(l); }

void LayerInfo::copyParamsFrom(const LayerInfo* src)
{
    if (!src) return;
    setSize(src->size());
    learningRate = src->getLearningRate(); momentumFactor = src->getMomentumFactor();
    weightDecay1 = src->getWeightDecay1(); weightDecay2 = src->getWeightDecay2();
    pDropout = src->getPDropout(); activationType = src->getActivationType();
}

void NNInfo::setPInput(float v) { if (inputLayer) inputLayer->setPDropout(v); }
void NNInfo::setWeightDecay1(unsigned int index, float v)
{
    if (index > layers.size()) return;
    if (index == 0) { if (inputLayer) inputLayer->setWeightDecay1(v); }
    else if (layers[index - 1]) layers[index - 1]->setWeightDecay1(v);
}
void NNInfo::setWeightDecay2(unsigned int index, float v)
{
    if (index > layers.size()) return;
    if (index == 0) { if (inputLayer) inputLayer->setWeightDecay2(v); }
    else if (index >= 2 && layers[index - 2]) layers[index - 2]->setWeightDecay2(v);
}
void NNInfo::setPDropout(unsigned int index, float v)
{
    if (index > layers.size()) return;
    if (index == 0) { if (inputLayer) inputLayer->setPDropout(v); }
    else if (layers[index - 1]) layers[index - 1]->setPDropout(v);
}
void NNInfo::copyHiddenLayer(unsigned int dst, unsigned int src)
{
    if (dst >= layers.size() || src >= layers.size() || !layers[dst] || !layers[src]) return;
    layers[dst]->copyParamsFrom(layers[src]);
}
void NNInfo::resizeHiddenLayers(unsigned int newCount)
{
    while (layers.size() > newCount) { delete layers.back(); layers.pop_back(); }
    while (layers.size() < newCount) layers.push_back(new HiddenLayerInfo(2, 0.01f, 0.0f, 0.0f, 0.0f, 0.0f, 0, 0.0f));
}
void NNInfo::removeHiddenLayer(unsigned int index)
{
    if (index >= layers.size() || !layers[index]) return;
    layers.erase(layers.begin() + index);
}

void NNInfo::print() const
{
    if (!inputLayer || !outputLayer) return;
    static const char* headers[10] = {"Layer", "Size", "batchSize", "lrnRate", "mFactor", "wDecay", "pDropout", "actvtn", "actParam", "cost"};
    printf("[NNINFO] Current NNInfo Values\n[NNINFO] ");
    for (int i = 0; i < 10; ++i) printf("%s\t", headers[i]);
    printf("\n");
    const NNTable t = toTable();
    for (size_t row = 0; row < t.size(); ++row) {
        printf("[NNINFO] ");
        if (row == 0) printf("Input\t");
        else if (row + 1 < t.size()) printf("H[%d]\t", (int)row);
        else printf("Output\t");
        for (size_t col = 0; col < t[row].size(); ++col) {
            const bool whole = col == COL_SIZE || col == COL_BATCH_SIZE || col == COL_ACTIVATION_TYPE || col == COL_OUTPUT_TYPE;
            if ((int)t[row][col] == -1) printf("\t");
            else if (whole) printf("%d\t", (int)t[row][col]);
            else printf("%f\t", t[row][col]);
        }
        printf("\n");
    }
}

NNTable NNInfo::toTable() const
{
    NNTable t;
    if (!inputLayer || !outputLayer) return t;
    std::vector<float> r(10, -1.0f);
    r[COL_SIZE] = -1.0f; r[COL_BATCH_SIZE] = (float)inputLayer->getBatchSize();
    r[COL_LEARNING_RATE] = inputLayer->getLearningRate(); r[COL_MOMENTUM_FACTOR] = inputLayer->getMomentumFactor();
    r[COL_WEIGHT_DECAY1] = inputLayer->getWeightDecay1(); r[COL_WEIGHT_DECAY2] = inputLayer->getWeightDecay2();
    r[COL_PDROPOUT] = inputLayer->getPDropout(); r[COL_ACTIVATION_TYPE] = (float)inputLayer->getActivationType();
    r[COL_ACTIVATION_PARAM] = inputLayer->getActivationParam(); r[COL_OUTPUT_TYPE] = -1.0f;
    t.push_back(r);
    for (size_t i = 0; i < layers.size(); ++i) {
        const HiddenLayerInfo* h = layers[i];
        r[COL_SIZE] = (float)h->size(); r[COL_BATCH_SIZE] = (float)inputLayer->getBatchSize();
        r[COL_LEARNING_RATE] = h->getLearningRate(); r[COL_MOMENTUM_FACTOR] = h->getMomentumFactor();
        r[COL_WEIGHT_DECAY1] = h->getWeightDecay1(); r[COL_WEIGHT_DECAY2] = h->getWeightDecay2();
        r[COL_PDROPOUT] = h->getPDropout(); r[COL_ACTIVATION_TYPE] = (float)h->getActivationType();
        r[COL_ACTIVATION_PARAM] = h->getActivationParam(); r[COL_OUTPUT_TYPE] = -1.0f;
        t.push_back(r);
    }
    std::vector<float> o(10, -1.0f);
    o[COL_SIZE] = (float)outputLayer->size(); o[COL_BATCH_SIZE] = (float)inputLayer->getBatchSize();
    o[COL_OUTPUT_TYPE] = (float)outputLayer->getOutputType();
    t.push_back(o);
    return t;
}

// nninfo.cpp:738-785: first row = input row (batch size read there), last row = output row
bool NNInfo::fromTable(const std::string& netName, const NNTable& t)
{
    if (t.size() < 2) return false;
    for (size_t i = 0; i < t.size(); ++i)
        if (t[i].size() < 10) return false;
    name = netName;
    for (size_t i = 0; i < layers.size(); ++i) delete layers[i];
    layers.clear();
    delete inputLayer; inputLayer = NULL;
    delete outputLayer; outputLayer = NULL;
    for (size_t i = 0; i < t.size(); ++i) {
        const std::vector<float>& r = t[i];
        if (i == 0)
            inputLayer = new InputLayerInfo((int)r[COL_BATCH_SIZE], r[COL_LEARNING_RATE], r[COL_MOMENTUM_FACTOR],
                                            r[COL_WEIGHT_DECAY1], r[COL_WEIGHT_DECAY2], r[COL_PDROPOUT],
                                            (int)r[COL_ACTIVATION_TYPE], r[COL_ACTIVATION_PARAM]);
        else if (i == t.size() - 1)
            outputLayer = new OutputLayerInfo((int)r[COL_SIZE], (int)r[COL_OUTPUT_TYPE]);
        else
            layers.push_back(new HiddenLayerInfo((int)r[COL_SIZE], r[COL_LEARNING_RATE], r[COL_MOMENTUM_FACTOR],
                                                 r[COL_WEIGHT_DECAY1], r[COL_WEIGHT_DECAY2], r[COL_PDROPOUT],
                                                 (int)r[COL_ACTIVATION_TYPE], r[COL_ACTIVATION_PARAM]));
    }
    return true;
}

bool NNInfo::loadFile(const std::string& path)
{
    FILE* f = fopen(path.c_str(), "r");
    if (!f) return false;
    NNTable t;
    char line[1024];
    bool first = true;
    while (fgets(line, sizeof(line), f)) {
        if (first) { first = false; if (strncmp(line, "Size", 4) == 0) continue; }
        std::vector<float> r;
        for (char* tok = strtok(line, ",\r\n"); tok; tok = strtok(NULL, ",\r\n")) r.push_back((float)atof(tok));
        if (r.size() >= 10) t.push_back(r);
    }
    fclose(f);
    std::string base = path;
    size_t slash = base.find_last_of('/');
    if (slash != std::string::npos) base = base.substr(slash + 1);
    return fromTable(base, t);
}

bool NNInfo::saveFile(const std::string& path) const
{
    NNTable t = toTable();
    if (t.empty()) return false;
    FILE* f = fopen(path.c_str(), "w");
    if (!f) return false;
    fprintf(f, "Size,batchSize,learningRate,momentumFactor,weightDecay1,weightDecay2,pDropout,activationType,activationParam,outputType");
    for (size_t i = 0; i < t.size(); ++i) {
        const std::vector<float>& r = t[i];
        fprintf(f, "\n%d,%d,%f,%f,%f,%f,%f,%d,%f,%d", (int)r[0], (int)r[1], r[2], r[3], r[4], r[5], r[6], (int)r[7], r[8], (int)r[9]);
    }
    fclose(f);
    return true;
}

// ------------------------------------------------------------------ Terminator

Terminator::Terminator() : timestamp(0), epoch(0), accuracy(0.0f) {}

bool Terminator::triggered(int64_t cTimestamp, int64_t cEpoch, float cAccuracy) const
{
    if ((timestamp > 0l) && (cTimestamp % timestamp == 0)) return true;
    if ((epoch > 0l) && (cEpoch % epoch == 0)) return true;
    if ((accuracy > 0.0f) && (cAccuracy >= accuracy)) return true;
    return false;
}

// ------------------------------------------------------------------ DataInput

void DataInput::denseTrain(std::vector<float>& X, std::vector<float>& Y, unsigned int& nOut) const
{
    const unsigned int n = getTrainSize(), f = getFeatureCount();
    nOut = n ? (unsigned int)getTrainExpectedRow(0).size() : 0;
    X.resize((size_t)n * f);
    Y.resize((size_t)n * nOut);
    for (unsigned int r = 0; r < n; ++r) {
        std::vector<float> xr = getTrainRow(r), yr = getTrainExpectedRow(r);
        for (unsigned int c = 0; c < f; ++c) X[(size_t)r * f + c] = c < xr.size() ? xr[c] : 0.0f;
        for (unsigned int c = 0; c < nOut; ++c) Y[(size_t)r * nOut + c] = c < yr.size() ? yr[c] : 0.0f;
    }
}

DenseInput::DenseInput(const float* x, const float* y, unsigned int nRows, unsigned int nFeatures, unsigned int nOutputs)
    : X(x, x + (size_t)nRows * nFeatures), Y(y, y + (size_t)nRows * nOutputs), rows(nRows), feats(nFeatures), outs(nOutputs)
{
    featureIsCategorical.assign(nFeatures, false);
}
std::vector<float> DenseInput::getTrainRow(unsigned int i) const
{
    if (i >= rows) return std::vector<float>();
    return std::vector<float>(X.begin() + (size_t)i * feats, X.begin() + (size_t)(i + 1) * feats);
}
std::vector<float> DenseInput::getTrainExpectedRow(unsigned int i) const
{
    if (i >= rows) return std::vector<float>();
    return std::vector<float>(Y.begin() + (size_t)i * outs, Y.begin() + (size_t)(i + 1) * outs);
}
void DenseInput::denseTrain(std::vector<float>& x, std::vector<float>& y, unsigned int& nOut) const
{
    x = X; y = Y; nOut = outs;
}

// ------------------------------------------------------------------ weight sampler

// ML/GMath/gmath.cpp:355-405 (Acklam's inverse normal CDF; log/sqrt on float arguments are the
// float overloads there, the rational part is evaluated in double)
static float norm_inv_CDF(float x)
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
        return (float)((((((c1 * q + c2) * q + c3) * q + c4) * q + c5) * q + c6) / ((((d1 * q + d2) * q + d3) * q + d4) * q + 1));
    } else if (x < p_high) {
        double q = x - 0.5;
        double r = q * q;
        return (float)(((((((a1 * r + a2) * r + a3) * r + a4) * r + a5) * r + a6) * q) /
                       (((((b1 * r + b2) * r + b3) * r + b4) * r + b5) * r + 1));
    }
    double q = sqrtf(-2 * logf(1 - x));
    return (float)(-(((((c1 * q + c2) * q + c3) * q + c4) * q + c5) * q + c6) / ((((d1 * q + d2) * q + d3) * q + d4) * q + 1));
}

static float normal_pdf(float z) { return (float)((1 / sqrt(6.2831853)) * expf(-(z * z) / 2)); }

void xavierLayer(int fanIn, int nOut, int activationType, float* W)
{
    const unsigned int num_layers = 2048;
    static float zigg[2049];
    float normal_CDF = 1.0;
    for (unsigned int i = 1; i < num_layers; i++) {
        normal_CDF = normal_CDF - (1 / ((float)num_layers * 2));
        zigg[i] = norm_inv_CDF(normal_CDF);
    }
    zigg[0] = zigg[1];
    zigg[num_layers] = 0;
    float std_dev = (activationType != GMath::RELU) ? sqrtf(1 / (float)fanIn) : sqrtf(2 / (float)fanIn);
    for (int o = 0; o < nOut; ++o)
        for (int e = 0; e < fanIn; ++e) {
            bool accepted = false;
            float x = 0.0f;
            while (!accepted) {
                int layer = rand() % 2048;
                x = rand() / (RAND_MAX / zigg[layer]);
                if (layer == 0) continue;
                else if (x < zigg[layer + 1]) accepted = true;
                else if (x > zigg[layer + 1]) {
                    float randU = rand() / RAND_MAX;  // integer division, as the reference writes it
                    float y = normal_pdf(zigg[layer]) + randU * (normal_pdf(zigg[layer - 1] - normal_pdf(zigg[layer])));
                    if (y < normal_pdf(x)) accepted = true;
                }
            }
            W[(size_t)o * fanIn + e] = x * std_dev;
        }
}

bool sampleInitialWeights(const NNInfo* s, int nFeat, int nOut, std::vector<std::vector<float> >& W, std::string* err)
{
    const int H = s->numHiddenLayers();
    const int outputType = s->getOutputType();
    W.assign(H + 1, std::vector<float>());
    bool isPositive = false;
    int prev = nFeat;
    for (int i = 0; i < H; ++i) {
        const int at = s->getActivationType(i);
        const int cur = s->getHiddenLayerSize(i);
        if (!isPositive && (at == GMath::SIGMOID || at == GMath::RELU || at == GMath::LEAKY || outputType == GMath::CLASSIFICATION)) {
            isPositive = true;   // LayerBuilder.cpp:213-222: start over; prev keeps the size of hidden layer i-1
            for (int k = 0; k < H; ++k) W[k].clear();
            i = -1;
            continue;
        }
        const int want = i == 0 ? nFeat : s->getHiddenLayerSize(i - 1);
        if (prev < want) {
            if (err) {
                char buf[256];
                snprintf(buf, sizeof(buf), "the reference would sample the first hidden layer with %d of %d input edges (its hidden-layer "
                         "restart keeps a stale layer size, LayerBuilder.cpp:196-233): that network is not modelled; inject the weights", prev, want);
                *err = buf;
            }
            return false;
        }
        std::vector<float> full((size_t)prev * cur);
        xavierLayer(prev, cur, at, full.data());
        W[i].resize((size_t)want * cur);
        for (int o = 0; o < cur; ++o) memcpy(&W[i][(size_t)o * want], &full[(size_t)o * prev], sizeof(float) * want);
        prev = cur;
    }
    // LayerBuilder.cpp:236-265: fan-in = the last hidden layer, scaled by the last hidden row's activation type
    const int lastSize = H > 0 ? s->getHiddenLayerSize(H - 1) : nFeat;
    W[H].resize((size_t)lastSize * nOut);
    xavierLayer(lastSize, nOut, s->getActivationType(H > 0 ? H - 1 : 0), W[H].data());
    return true;
}

// ------------------------------------------------------------------ NNetwork

static int64_t g_next_id = 1;

NNetwork::NNetwork()
    : di(NULL), skeleton(NULL), dev(NULL), running(false), netType(TYPE_DFF), epochs(0), mode(MODE_EXACT),
      dtype(DTYPE_F32), biasMode(0), verbose(true), overallTotalError(0.0f), overallTotalAccuracy(0.0f), overallClassAccuracy(0.0f), overallClassPrecision(0.0f),
      overallClassRecall(0.0f), overallClassSpecificity(0.0f), overallClassF1(0.0f), overallCorrect(0),
      minibatchSize(1), id(g_next_id++), nRows(0), nFeat(0), nOut(0), dropoutOn(false), prepaidDrawEpochs(0), randFidelity(true)
{
}

NNetwork::NNetwork(NNInfo* newNNInfo)
    : di(NULL), skeleton(newNNInfo), dev(NULL), running(false), netType(TYPE_DFF), epochs(0), mode(MODE_EXACT),
      dtype(DTYPE_F32), biasMode(0), verbose(true), overallTotalError(0.0f), overallTotalAccuracy(0.0f), overallClassAccuracy(0.0f), overallClassPrecision(0.0f),
      overallClassRecall(0.0f), overallClassSpecificity(0.0f), overallClassF1(0.0f), overallCorrect(0),
      minibatchSize(1), id(g_next_id++), nRows(0), nFeat(0), nOut(0), dropoutOn(false), prepaidDrawEpochs(0), randFidelity(true)
{
}

NNetwork::~NNetwork() { clean(); }

void NNetwork::clean()
{
    if (dev) ghip_net_destroy(dev);
    dev = NULL;
    di = NULL;  // borrowed, like the skeleton (network.cpp:745-762)
}

std::string NNetwork::getName() const { return skeleton ? skeleton->getName() : std::string(); }

int64_t NNetwork::getCurrentTimeMilliseconds() const
{
    struct timeval tv;
    gettimeofday(&tv, NULL);
    return (int64_t)((unsigned long long)tv.tv_sec * 1000ULL + (unsigned long long)tv.tv_usec / 1000ULL);
}

void NNetwork::resetGraphs()
{
    learningCurve.clear();
    results.clear();
}

bool NNetwork::save() const
{
    if (!skeleton) return false;
    if (!doesDatabaseExist()) createDatabase();
    mkdir("database/neuralnetworks", 0777);
    return skeleton->saveFile("database/neuralnetworks/" + skeleton->getName());
}

bool NNetwork::load(const std::string& path)
{
    NNInfo* info = new NNInfo("");
    struct stat st;
    const bool as_given = stat(path.c_str(), &st) == 0;
    if (!info->loadFile(as_given ? path : "database/neuralnetworks/" + path)) { delete info; return false; }
    if (!as_given) info->setName(path);
    skeleton = info;  // like the reference, the loaded skeleton is never freed by the network
    return true;
}

bool NNetwork::save(const std::string& path) const { return skeleton ? skeleton->saveFile(path) : false; }

// file: "GLCK" u32 version, i32 mode, i32 dtype, i32 epochs, i32 nLayers, i32 sizes[nLayers+1],
//       u32 tableBytes, table text (the NNInfo CSV), from version 3 on u32 nameBytes, the network's name, then per layer: W, u32 biasLen, bias, u32 aLen, a, u32 bLen, b,
//       and from version 2 on u32 cLen, window lengths (i32), u32 eLen, node error accumulators (exact mode; else 0, 0)
// fwrite / fread of n elements that leave an empty array's (possibly null) pointer alone
static size_t put(const void* p, size_t size, size_t n, FILE* f) { return n ? fwrite(p, size, n, f) : 0; }
static size_t get(void* p, size_t size, size_t n, FILE* f) { return n ? fread(p, size, n, f) : 0; }

bool NNetwork::saveCheckpoint(const std::string& path)
{
    if (!skeleton || !dev) { lastError = "nothing to checkpoint: the network has not run"; return false; }
    const int H = skeleton->numHiddenLayers(), L = H + 1;
    std::vector<int32_t> sizes(L + 1);
    sizes[0] = (int32_t)nFeat;
    for (int i = 0; i < H; ++i) sizes[i + 1] = skeleton->getHiddenLayerSize(i);
    sizes[L] = (int32_t)nOut;
    const std::string tmp = path + ".table";
    if (!skeleton->saveFile(tmp)) { lastError = "cannot write " + tmp; return false; }
    std::string table;
    {
        FILE* t = fopen(tmp.c_str(), "rb");
        if (!t) return false;
        char buf[4096]; size_t got;
        while ((got = fread(buf, 1, sizeof(buf), t)) > 0) table.append(buf, got);
        fclose(t);
        remove(tmp.c_str());
    }
    FILE* f = fopen(path.c_str(), "wb");
    if (!f) { lastError = "cannot write " + path; return false; }
    const std::string netName = skeleton->getName();
    const uint32_t version = 3, tb = (uint32_t)table.size(), nb = (uint32_t)netName.size();
    const int32_t head[4] = {mode, dtype, epochs, L};
    fwrite("GLCK", 1, 4, f); fwrite(&version, 4, 1, f); fwrite(head, 4, 4, f); put(sizes.data(), 4, sizes.size(), f);
    fwrite(&tb, 4, 1, f); put(table.data(), 1, table.size(), f);
    fwrite(&nb, 4, 1, f); put(netName.data(), 1, netName.size(), f);
    bool ok = true;
    for (int l = 0; l < L && ok; ++l) {
        const size_t cnt = (size_t)sizes[l] * sizes[l + 1];
        const uint32_t bl = mode == MODE_EXACT ? 1u : (uint32_t)sizes[l + 1];
        const uint32_t al = (uint32_t)cnt, sl = mode == MODE_EXACT ? (uint32_t)cnt : (uint32_t)sizes[l + 1];
        std::vector<float> W(cnt), b(bl), sa(al), sb(sl);
        ok = ghip_net_get_params(dev, l, W.data(), b.data(), (int)bl) == 0 && ghip_net_get_state(dev, l, sa.data(), sb.data()) == 0;
        if (!ok) { lastError = ghip_last_error(); break; }
        put(W.data(), 4, cnt, f);
        fwrite(&bl, 4, 1, f); put(b.data(), 4, bl, f);
        fwrite(&al, 4, 1, f); put(sa.data(), 4, al, f);
        fwrite(&sl, 4, 1, f); put(sb.data(), 4, sl, f);
        const uint32_t cl = mode == MODE_EXACT ? (uint32_t)cnt : 0u, el = mode == MODE_EXACT ? (uint32_t)sizes[l + 1] : 0u;
        std::vector<int32_t> wc(cl);
        std::vector<float> ed(el);
        if (cl && ghip_net_get_dropout_state(dev, l, wc.data(), ed.data()) != 0) { ok = false; lastError = ghip_last_error(); break; }
        fwrite(&cl, 4, 1, f); put(wc.data(), 4, cl, f);
        fwrite(&el, 4, 1, f); put(ed.data(), 4, el, f);
    }
    fclose(f);
    return ok;
}

bool NNetwork::loadCheckpoint(const std::string& path)
{
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) return false;
    char magic[4];
    uint32_t version = 0, tb = 0;
    int32_t head[4];
    bool ok = fread(magic, 1, 4, f) == 4 && memcmp(magic, "GLCK", 4) == 0 && fread(&version, 4, 1, f) == 1 && version >= 1 && version <= 3 &&
              fread(head, 4, 4, f) == 4 && head[3] >= 1 && head[3] <= 16 &&
              (head[0] == MODE_EXACT || head[0] == MODE_CANONICAL) && (head[1] == DTYPE_F32 || head[1] == DTYPE_BF16) && head[2] >= 0;
    std::vector<int32_t> sizes;
    std::string table, netName;
    bool named = false;
    if (ok) {
        sizes.resize(head[3] + 1);
        ok = get(sizes.data(), 4, sizes.size(), f) == sizes.size() && fread(&tb, 4, 1, f) == 1 && tb < (1u << 20);
        // nothing is allocated from sizes the file does not back up: a layer has 1 .. 2^24 nodes and at most 2^31 edges
        for (size_t l = 0; ok && l < sizes.size(); ++l) ok = sizes[l] >= 1 && sizes[l] <= (1 << 24);
        for (size_t l = 0; ok && l + 1 < sizes.size(); ++l) ok = (int64_t)sizes[l] * sizes[l + 1] <= ((int64_t)1 << 31);
    }
    if (ok) { table.resize(tb); ok = get(tb ? &table[0] : nullptr, 1, tb, f) == tb; }
    if (ok && version >= 3) {
        uint32_t nb = 0;
        ok = fread(&nb, 4, 1, f) == 1 && nb < 4096;
        if (ok) { netName.resize(nb); ok = get(nb ? &netName[0] : nullptr, 1, nb, f) == nb; named = true; }
    }
    std::vector<std::vector<float> > W, B, SA, SB, ED;
    std::vector<std::vector<int32_t> > WC;
    for (int l = 0; ok && l < head[3]; ++l) {
        const size_t cnt = (size_t)sizes[l] * sizes[l + 1];
        std::vector<float> w(cnt), b, sa, sb;
        uint32_t n1 = 0;
        ok = get(w.data(), 4, cnt, f) == cnt;
        ok = ok && fread(&n1, 4, 1, f) == 1 && n1 <= cnt; if (ok) { b.resize(n1); ok = get(b.data(), 4, n1, f) == n1; }
        ok = ok && fread(&n1, 4, 1, f) == 1 && n1 <= cnt; if (ok) { sa.resize(n1); ok = get(sa.data(), 4, n1, f) == n1; }
        ok = ok && fread(&n1, 4, 1, f) == 1 && n1 <= cnt; if (ok) { sb.resize(n1); ok = get(sb.data(), 4, n1, f) == n1; }
        std::vector<int32_t> wc;
        std::vector<float> ed;
        if (version >= 2) {
            ok = ok && fread(&n1, 4, 1, f) == 1 && n1 <= cnt; if (ok) { wc.resize(n1); ok = get(wc.data(), 4, n1, f) == n1; }
            ok = ok && fread(&n1, 4, 1, f) == 1 && n1 <= cnt; if (ok) { ed.resize(n1); ok = get(ed.data(), 4, n1, f) == n1; }
        }
        W.push_back(w); B.push_back(b); SA.push_back(sa); SB.push_back(sb); WC.push_back(wc); ED.push_back(ed);
    }
    fclose(f);
    if (!ok) { lastError = "not a checkpoint of this library: " + path; return false; }
    const std::string tmp = path + ".table";
    {
        FILE* t = fopen(tmp.c_str(), "wb");
        if (!t) return false;
        put(table.data(), 1, table.size(), t);
        fclose(t);
    }
    const bool loaded = load(tmp);
    remove(tmp.c_str());
    if (!loaded) { lastError = "checkpoint holds no valid network table"; return false; }
    // load() names the network after the file it read, here the temporary table: put the saved name back
    // (older files have none: the checkpoint's own file name then)
    skeleton->setName(named ? netName : path.substr(path.find_last_of('/') == std::string::npos ? 0 : path.find_last_of('/') + 1));
    clean();
    mode = head[0]; dtype = head[1]; epochs = head[2];
    initW = W; initB = B; initStateA = SA; initStateB = SB; initCounts = WC; initErrDer = ED;
    return true;
}

void NNetwork::train(DataInput* d) { run(d, RUN_TRAIN); }
void NNetwork::test(DataInput* d) { run(d, RUN_TEST); }

bool NNetwork::setWeights(unsigned int layer, const std::vector<float>& W)
{
    if (!skeleton || layer > (unsigned int)skeleton->numHiddenLayers()) return false;
    if (dev) {
        if (ghip_net_set_params(dev, (int)layer, W.data(), NULL, 0) != 0) { lastError = ghip_last_error(); return false; }
        return true;
    }
    if (initW.size() <= layer) initW.resize(layer + 1);
    initW[layer] = W;
    return true;
}

bool NNetwork::setBias(unsigned int layer, const std::vector<float>& bias)
{
    if (!skeleton || layer > (unsigned int)skeleton->numHiddenLayers()) return false;
    if (initB.size() <= layer) initB.resize(layer + 1);
    initB[layer] = bias;
    return true;
}

std::vector<float> NNetwork::getWeights(unsigned int layer)
{
    std::vector<float> W;
    if (!dev || !skeleton || layer > (unsigned int)skeleton->numHiddenLayers()) return W;
    const int ni = layer == 0 ? (int)nFeat : skeleton->getHiddenLayerSize(layer - 1);
    const int no = layer == (unsigned int)skeleton->numHiddenLayers() ? (int)nOut : skeleton->getHiddenLayerSize(layer);
    W.resize((size_t)ni * no);
    if (ghip_net_get_params(dev, (int)layer, W.data(), NULL, 0) != 0) { lastError = ghip_last_error(); W.clear(); }
    return W;
}

std::vector<float> NNetwork::getBias(unsigned int layer)
{
    std::vector<float> b;
    if (!dev || !skeleton || layer > (unsigned int)skeleton->numHiddenLayers()) return b;
    const int no = layer == (unsigned int)skeleton->numHiddenLayers() ? (int)nOut : skeleton->getHiddenLayerSize(layer);
    b.resize(mode == MODE_EXACT ? 1 : (size_t)no);
    if (ghip_net_get_params(dev, (int)layer, NULL, b.data(), (int)b.size()) != 0) { lastError = ghip_last_error(); b.clear(); }
    return b;
}

// LayerBuilder::build (ML/State/LayerBuilder.cpp:54-267): table to the device, weights sampled
// in the reference's order (hidden layers, then the output layer, node by node) unless injected.
bool NNetwork::hasDropout() const
{
    if (!skeleton) return false;
    const int H = skeleton->numHiddenLayers();
    for (int l = 0; l <= H; ++l) {
        const float p = l == 0 ? skeleton->getPInput() : skeleton->getPDropout(l - 1);
        const int rate = p * 100.0f;  // layer.cpp:107
        if (rate >= 1 && rate < 100) return true;
    }
    return false;
}

// Layer::generateDropout (ML/State/layer.cpp:102-134) for every row in SGDHelper's order
// (network.cpp:407-411): the row's input layer, then the hidden layers; one dart rand()%100+1 per
// node, the layer drawn again while every node came out dropped; a rate outside 0..99 draws nothing.
void NNetwork::drawDropout()
{
    const int H = skeleton->numHiddenLayers();
    std::vector<int> sizes(H + 1);
    sizes[0] = (int)nFeat;
    size_t len = nFeat;
    for (int h = 0; h < H; ++h) { sizes[h + 1] = skeleton->getHiddenLayerSize(h); len += sizes[h + 1]; }
    if (dropFlags.size() != (size_t)nRows * len) dropFlags.assign((size_t)nRows * len, 0);
    std::vector<unsigned char> hidden(len - nFeat, 0);  // the hidden layers are shared by all rows
    if (nRows > 0) memcpy(hidden.data(), &dropFlags[(size_t)(nRows - 1) * len + nFeat], hidden.size());
    for (unsigned int r = 0; r < nRows; ++r) {
        unsigned char* m = &dropFlags[(size_t)r * len];
        memcpy(m + nFeat, hidden.data(), hidden.size());
        size_t off = 0;
        for (int l = 0; l <= H; ++l) {
            const int rate = pNode[l] * 100.0f;
            if (rate >= 0 && rate < 100) {
                bool all;
                do {
                    all = true;
                    for (int i = 0; i < sizes[l]; ++i) {
                        const int dart = (rand() % 100) + 1;
                        const bool dropped = dart <= rate;
                        if (!dropped) all = false;
                        m[off + i] = dropped ? 1 : 0;
                    }
                } while (all);
            }
            off += sizes[l];
        }
        memcpy(hidden.data(), m + nFeat, hidden.size());
    }
}

size_t NNetwork::dropoutDrawsPerEpoch() const
{
    if (!skeleton || mode != MODE_EXACT) return 0;
    const int H = skeleton->numHiddenLayers();
    size_t nodes = 0;
    for (int l = 0; l <= H; ++l) {
        const float p = l == 0 ? skeleton->getPInput() : skeleton->getPDropout(l - 1);
        const int rate = p * 100.0f;  // layer.cpp:107-112: rates below 0 and from 100 up draw nothing
        if (rate >= 0 && rate < 100) nodes += l == 0 ? nFeat : (size_t)skeleton->getHiddenLayerSize(l - 1);
    }
    return nodes * nRows;
}

void NNetwork::skipDropoutDraws(int64_t n)
{
    if (dropoutOn || n <= 0 || !randFidelity) return;  // with dropout the flags themselves are drawn (drawDropout)
    const int64_t paid = prepaidDrawEpochs < n ? prepaidDrawEpochs : n;
    prepaidDrawEpochs -= paid;
    const size_t per = dropoutDrawsPerEpoch();
    for (int64_t e = paid; e < n; ++e)
        for (size_t k = 0; k < per; ++k) (void)rand();
}

void NNetwork::prepayDropoutDraws(int64_t n)
{
    if (dropoutOn || n <= 0 || !randFidelity) return;
    const size_t per = dropoutDrawsPerEpoch();
    for (int64_t e = 0; e < n; ++e)
        for (size_t k = 0; k < per; ++k) (void)rand();
    prepaidDrawEpochs += n;
}

bool NNetwork::samplesOnBuild() const
{
    if (dev || !skeleton) return false;
    const int H = skeleton->numHiddenLayers();
    for (int l = 0; l <= H; ++l)
        if ((size_t)l >= initW.size() || initW[l].empty()) return true;
    return false;
}

bool NNetwork::build()
{
    std::vector<float> X, Y;
    di->denseTrain(X, Y, nOut);
    nRows = di->getTrainSize();
    nFeat = di->getFeatureCount();
    const int H = skeleton->numHiddenLayers();
    if (H + 1 > GHIP_MAX_LAYERS) { lastError = "too many layers"; return false; }
    if (nOut != skeleton->getOutputLayerSize()) { lastError = "expected rows do not match the output layer size"; return false; }
    ghip_net_spec s;
    memset(&s, 0, sizeof(s));
    s.n_layers = H + 1;
    s.sizes[0] = (int)nFeat;
    for (int i = 0; i < H; ++i) s.sizes[i + 1] = skeleton->getHiddenLayerSize(i);
    s.sizes[H + 1] = (int)nOut;
    for (int l = 0; l <= H; ++l) {
        s.lr[l] = skeleton->getLearningRate(l); s.mom[l] = skeleton->getMomentumFactor(l);
        s.wd1[l] = skeleton->getWeightDecay1(l); s.wd2[l] = skeleton->getWeightDecay2(l);
        s.act[l] = skeleton->getActivationType(l); s.act_param[l] = skeleton->getActivationParam(l);
    }
    // network.cpp:407-411: the input layer takes getPInput(), hidden layer h takes getPDropout(h), whose
    // index 0 is the input row again (nninfo.cpp:321-333): the last hidden row's rate is never used
    pNode.assign(H + 1, 0.0f);
    pNode[0] = skeleton->getPInput();
    for (int h = 0; h < H; ++h) pNode[h + 1] = skeleton->getPDropout(h);
    dropoutOn = hasDropout();
    // exact mode follows the reference's per-row algorithm with the flags; canonical mode in fp32 takes the same flags
    // (a dropped node feeds nothing on and gets no delta); the low-precision kernels do not read flags
    if (dropoutOn && mode != MODE_EXACT && dtype != DTYPE_F32) { lastError = "dropout: exact mode, or canonical mode in fp32"; return false; }
    dropFlags.clear();
    s.batch = skeleton->getBatchSize();
    s.cost = skeleton->getOutputType();
    s.mode = mode == MODE_EXACT ? GHIP_MODE_EXACT : GHIP_MODE_CANONICAL;
    s.dtype = dtype == DTYPE_BF16 ? GHIP_BF16 : GHIP_F32;
    s.bias_mode = biasMode;
    // weights: injected ones as they are; if any layer has none, the whole network is sampled in the
    // reference's order (so libc's rand() moves as it does there) and injected layers replace their draw
    std::vector<std::vector<float> > sampled;
    bool allInjected = true;
    for (int l = 0; l <= H; ++l) {
        const size_t want = (size_t)s.sizes[l] * s.sizes[l + 1];
        const size_t have = (size_t)l < initW.size() ? initW[l].size() : 0;
        // a layer either has no injected weights (it is sampled: samplesOnBuild() tells the same story before
        // the sizes are known) or has all of them
        if (have != 0 && have != want) {
            char msg[160];
            snprintf(msg, sizeof(msg), "weight layer %d was given %zu weights, it has %zu", l, have, want);
            lastError = msg;
            return false;
        }
        allInjected = allInjected && have == want;
    }
    if (!allInjected && !sampleInitialWeights(skeleton, (int)nFeat, (int)nOut, sampled, &lastError)) return false;
    if (ghip_net_create(&s, &dev) != 0) { lastError = ghip_last_error(); dev = NULL; return false; }
    for (int l = 0; l <= H; ++l) {
        const int ni = s.sizes[l], no = s.sizes[l + 1];
        std::vector<float> W;
        if ((size_t)l < initW.size() && initW[l].size() == (size_t)ni * no) W = initW[l];
        else W.swap(sampled[l]);
        const float* bp = NULL;
        int bl = 0;
        if ((size_t)l < initB.size() && !initB[l].empty()) { bp = initB[l].data(); bl = (int)initB[l].size(); }
        if (ghip_net_set_params(dev, l, W.data(), bp, bl) != 0) { lastError = ghip_last_error(); return false; }
        if ((size_t)l < initStateA.size() && !initStateA[l].empty() && (size_t)l < initStateB.size() && !initStateB[l].empty())
            if (ghip_net_set_state(dev, l, initStateA[l].data(), initStateB[l].data()) != 0) { lastError = ghip_last_error(); return false; }
        if ((size_t)l < initCounts.size() && initCounts[l].size() == (size_t)ni * no && (size_t)l < initErrDer.size() &&
            initErrDer[l].size() == (size_t)no)
            if (ghip_net_set_dropout_state(dev, l, initCounts[l].data(), initErrDer[l].data()) != 0) { lastError = ghip_last_error(); return false; }
    }
    if (ghip_net_set_dataset(dev, X.data(), Y.data(), (int64_t)nRows) != 0) { lastError = ghip_last_error(); return false; }
    // network.cpp:143-145: classification and KL runs keep a confusion matrix (counted on the device)
    confusionMatrix.clean();
    if ((s.cost == GMath::CLASSIFICATION || s.cost == GMath::KL) && nOut <= 4096) {
        if (ghip_net_confusion_enable(dev, 1) != 0) { lastError = ghip_last_error(); return false; }
        confusionMatrix.build(nOut);
    }
    return true;
}

// ------------------------------------------------------------------ OHE (ML/GMath/OHE.cpp)

void OHE::addString(const std::string& newString)  // OHE.cpp:54-64
{
    const int at = indexAt(newString);
    if (at < 0) { OHEStrings.push_back(newString); classCount.push_back(1); }
    else ++classCount[at];
}
bool OHE::contains(const std::string& s) const { return indexAt(s) >= 0; }
int OHE::indexAt(const std::string& needle) const
{
    for (size_t i = 0; i < OHEStrings.size(); ++i)
        if (OHEStrings[i] == needle) return (int)i;
    return -1;
}
std::string OHE::classAt(unsigned int cid) const { return cid < OHEStrings.size() ? OHEStrings[cid] : std::string(); }
std::vector<float> OHE::operator[](const std::string& needle) const  // OHE.cpp:179-198
{
    std::vector<float> retVal(size(), 0.01f);
    const int at = indexAt(needle);
    if (at >= 0) retVal[at] = 0.99f;
    return retVal;
}
std::string OHE::operator[](const std::vector<float>& needle) const  // OHE.cpp:216-238: >= scan from 0
{
    float max = 0.0f;
    int index = -1;
    for (size_t i = 0; i < needle.size(); ++i)
        if (needle[i] >= max) { max = needle[i]; index = (int)i; }
    return (index >= 0 && (size_t)index < OHEStrings.size()) ? OHEStrings[index] : std::string();
}

// ------------------------------------------------------------------ NumberInput (ML/DataObjects/NumberInput.cpp)

namespace {
std::string trimmed(const std::string& s)
{
    size_t a = 0, b = s.size();
    while (a < b && (s[a] == ' ' || s[a] == '\t' || s[a] == '\r' || s[a] == '\n')) ++a;
    while (b > a && (s[b - 1] == ' ' || s[b - 1] == '\t' || s[b - 1] == '\r' || s[b - 1] == '\n')) --b;
    return s.substr(a, b - a);
}
std::vector<std::string> splitLine(const std::string& line)
{
    std::vector<std::string> out;
    size_t start = 0;
    for (;;) {
        size_t c = line.find(',', start);
        out.push_back(trimmed(line.substr(start, c == std::string::npos ? std::string::npos : c - start)));
        if (c == std::string::npos) break;
        start = c + 1;
    }
    return out;
}
bool parseNumber(const std::string& cell, float* v)
{
    if (cell.empty()) return false;
    char* end = NULL;
    const float f = strtof(cell.c_str(), &end);
    if (end == cell.c_str() || *end != '\0') return false;
    *v = f;
    return true;
}
}  // namespace

void NumberInput::import(std::string fname)
{
    if (loaded) return;
    name = fname;
    standardizeInputTable(fname);
    loaded = true;
}

bool NumberInput::standardizeInputTable(const std::string& fname, int standardizeFlag)
{
    FILE* f = fopen(fname.c_str(), "rb");
    if (!f) return false;
    std::string text;
    char buf[4096];
    size_t got;
    while ((got = fread(buf, 1, sizeof(buf), f)) > 0) text.append(buf, got);
    fclose(f);
    return standardizeText(text, standardizeFlag);
}

bool NumberInput::standardizeText(const std::string& text, int standardizeFlag)
{
    trainTable.clear(); trainExpectedTable.clear(); trainHeaders.clear(); expectedHeaders.clear();
    OHEMaps.clear(); featureIsCategorical.clear(); rows = 0;
    // ---- the table as parsed (stands in for GTable(fname, ',', TYPE_FILE))
    std::vector<std::string> header;
    std::vector<std::vector<std::string> > raw;
    size_t pos = 0;
    bool first = true;
    while (pos <= text.size()) {
        size_t nl = text.find('\n', pos);
        std::string line = text.substr(pos, nl == std::string::npos ? std::string::npos : nl - pos);
        pos = (nl == std::string::npos) ? text.size() + 1 : nl + 1;
        if (trimmed(line).empty()) continue;
        if (first) { header = splitLine(line); first = false; continue; }
        std::vector<std::string> cells = splitLine(line);
        cells.resize(header.size());
        raw.push_back(cells);
    }
    const unsigned int nRows = (unsigned int)raw.size(), nCols = (unsigned int)header.size();
    if (nRows == 0 || nCols == 0) return false;
    std::vector<bool> isOutput(nCols, false);
    if (outputColumns.empty()) isOutput[nCols - 1] = true;
    for (size_t k = 0; k < outputColumns.size(); ++k)
        if (outputColumns[k] >= 0 && (unsigned int)outputColumns[k] < nCols) isOutput[outputColumns[k]] = true;
    std::vector<std::vector<float> > val(nRows, std::vector<float>(nCols, 0.0f));
    std::vector<std::vector<char> > isString(nRows, std::vector<char>(nCols, 0));
    for (unsigned int r = 0; r < nRows; ++r)
        for (unsigned int c = 0; c < nCols; ++c) isString[r][c] = parseNumber(raw[r][c], &val[r][c]) ? 0 : 1;

    std::vector<std::vector<float> > trainCols, expectedCols;  // column major while building
    // ---- NumberInput.cpp:55-73: categorical = first cell is a string; map its feature space
    bool isClassification = false;
    for (unsigned int c = 0; c < nCols; ++c) {
        OHE cOHE;
        featureIsCategorical.push_back(false);
        if (isString[0][c]) {
            for (unsigned int r = 0; r < nRows; ++r)
                if (isString[r][c]) cOHE.addString(raw[r][c]);   // OHE::mapFeatureSpace, OHE.cpp:240-258
            featureIsCategorical[c] = true;
            isClassification = true;
        }
        OHEMaps.push_back(cOHE);
    }
    // ---- NumberInput.cpp:75-283
    for (unsigned int c = 0; c < nCols; ++c) {
        float fMin = 0.0f, fMax = 0.0f, fMean = 0.0f;
        for (unsigned int r = 0; r < nRows; ++r) {
            if (featureIsCategorical[c]) continue;
            if (isString[r][c]) continue;
            const float cell = val[r][c];
            if ((r == 0) && (c == 0)) { fMin = cell; fMax = cell; }
            if (cell < fMin) fMin = cell;
            if (cell > fMax) fMax = cell;
            fMean += cell;
            if (r == (nRows - 1)) fMean /= nRows;
        }
        if (featureIsCategorical[c]) {
            const OHE& vec = OHEMaps[c];
            for (unsigned int cInt = 0; cInt < vec.size(); ++cInt) {
                std::vector<float> newCol(nRows);
                for (unsigned int r = 0; r < nRows; ++r) newCol[r] = vec[raw[r][c]][cInt];
                char num[16];
                snprintf(num, sizeof(num), "%u", cInt);
                if (isOutput[c]) { expectedCols.push_back(newCol); expectedHeaders.push_back(header[c] + num); }
                else { trainCols.push_back(newCol); trainHeaders.push_back(header[c] + num); }
            }
            continue;
        }
        std::vector<float> newCol(nRows);
        if (standardizeFlag == GMath::MINMAX) {
            const float xRange = fMax - fMin;
            if (xRange == 0.0f) {  // a constant: added as it is, to the feature table (:171-176)
                for (unsigned int r = 0; r < nRows; ++r) newCol[r] = val[r][c];
                trainCols.push_back(newCol); trainHeaders.push_back(header[c]);
                continue;
            }
            for (unsigned int r = 0; r < nRows; ++r) {
                if (isString[r][c]) {  // strings MUST be categorical (:186-192)
                    printf("ERROR: String found in non-categorical column.\n");
                    trainTable.clear();
                    return false;
                }
                float cell = val[r][c];
                if (isClassification) cell = ((((cell - fMin) / (xRange)) * 0.98f) + 0.01f);
                else cell = ((cell - fMin) / (xRange));
                newCol[r] = cell;
            }
        } else if (standardizeFlag == GMath::ZSCORE) {
            float fStDev = 0.0f;
            for (unsigned int r = 0; r < nRows; ++r) {
                if (isString[r][c]) { trainTable.clear(); return false; }
                const float cell = val[r][c];
                fStDev += ((cell - fMean) * (cell - fMean));
            }
            fStDev = sqrtf(fStDev / (nRows - 1));
            for (unsigned int r = 0; r < nRows; ++r) newCol[r] = ((val[r][c] - fMean) / fStDev);
        } else {
            continue;
        }
        if (isOutput[c]) { expectedCols.push_back(newCol); expectedHeaders.push_back(header[c]); }
        else { trainCols.push_back(newCol); trainHeaders.push_back(header[c]); }
    }
    rows = nRows;
    trainTable.assign(nRows, std::vector<float>(trainCols.size()));
    trainExpectedTable.assign(nRows, std::vector<float>(expectedCols.size()));
    for (unsigned int r = 0; r < nRows; ++r) {
        for (size_t c = 0; c < trainCols.size(); ++c) trainTable[r][c] = trainCols[c][r];
        for (size_t c = 0; c < expectedCols.size(); ++c) trainExpectedTable[r][c] = expectedCols[c][r];
    }
    return true;
}

std::vector<float> NumberInput::getTrainRow(unsigned int i) const { return i < trainTable.size() ? trainTable[i] : std::vector<float>(); }
std::vector<float> NumberInput::getTrainExpectedRow(unsigned int i) const
{
    return i < trainExpectedTable.size() ? trainExpectedTable[i] : std::vector<float>();
}

// ------------------------------------------------------------------ CMatrix (ML/GMath/cmatrix.cpp)

void CMatrix::build(unsigned int numberOfClasses)
{
    clean();
    n = numberOfClasses;
    matrix.assign((size_t)n * n, 0);
    truePositive.assign(n, 0); trueNegative.assign(n, 0); falsePositive.assign(n, 0); falseNegative.assign(n, 0);
}

static int naiveArgmax(const std::vector<float>& v)  // gmath.cpp:412-433
{
    float mx = 0.0f;
    int index = -1;
    for (size_t i = 0; i < v.size(); ++i)
        if (v[i] > mx) { mx = v[i]; index = (int)i; }
    return index;
}

void CMatrix::addResult(const std::vector<float>& result)  // cmatrix.cpp:57-98
{
    if ((result.size() % 2) != 0) { printf("[CMATRIX] Bad result list size [0]: %d\n", (int)result.size()); return; }
    if ((result.size() / 2) != n) { printf("[CMATRIX] Bad result list size [1]: %d\n", (int)result.size()); return; }
    std::vector<float> expected, predicted;
    for (size_t i = 0; i < result.size(); ++i) ((i % 2) == 0 ? expected : predicted).push_back(result[i]);
    const int e = naiveArgmax(expected), p = naiveArgmax(predicted);
    if (e >= 0 && p >= 0) matrix[(size_t)e * n + p] += 1;
}

void CMatrix::setMatrix(const std::vector<int>& cells)
{
    if (cells.size() == matrix.size()) matrix = cells;
}

void CMatrix::updateResultParams()  // cmatrix.cpp:100-132 (the lists are NOT cleared here, as there)
{
    const int size = (int)n;
    for (int row = 0; row < size; ++row)
        for (int col = 0; col < size; ++col) {
            const int value = matrix[(size_t)row * n + col];
            if (row != col) {
                falsePositive[col] += value;
                falseNegative[row] += value;
            } else {
                for (int itr = 0; itr < size; ++itr) {
                    if (itr == row) truePositive[itr] = value;
                    else trueNegative[itr] += value;
                }
            }
        }
}

std::vector<std::vector<int> > CMatrix::getMatrix() const
{
    std::vector<std::vector<int> > out(n, std::vector<int>(n, 0));
    for (unsigned int r = 0; r < n; ++r)
        for (unsigned int c = 0; c < n; ++c) out[r][c] = matrix[(size_t)r * n + c];
    return out;
}

// the reference's guard is `index > rows` (cmatrix.cpp:141); index == rows is rejected here as well
float CMatrix::getClassAccuracy(unsigned int i) const
{
    if (i >= n) return 0.0f;
    const float truth = (float)(truePositive[i] + trueNegative[i]);
    const float untruth = (float)(falsePositive[i] + falseNegative[i]);
    return truth / (truth + untruth);
}
float CMatrix::getClassPrecision(unsigned int i) const
{
    if (i >= n) return 0.0f;
    return ((float)truePositive[i]) / ((float)(truePositive[i] + falsePositive[i]));
}
float CMatrix::getClassRecall(unsigned int i) const
{
    if (i >= n) return 0.0f;
    return ((float)truePositive[i]) / ((float)(truePositive[i] + falseNegative[i]));
}
float CMatrix::getClassSpecificity(unsigned int i) const
{
    if (i >= n) return 0.0f;
    return ((float)trueNegative[i]) / ((float)(trueNegative[i] + falsePositive[i]));
}
float CMatrix::getClassFalseAlarm(unsigned int i) const
{
    if (i >= n) return 0.0f;
    return ((float)falsePositive[i]) / ((float)(trueNegative[i] + falsePositive[i]));
}
float CMatrix::getClassF1Score(unsigned int i) const
{
    if (i >= n) return 0.0f;
    const float cRecall = getClassRecall(i), cPrecision = getClassPrecision(i);
    return (2.0f * cRecall * cPrecision) / (cRecall + cPrecision);
}
#define GLADES_OVERALL(NAME, CLASSFN)                          \
    float CMatrix::NAME() const                                \
    {                                                          \
        float total = 0.0f;                                    \
        for (unsigned int i = 0; i < n; ++i) total += CLASSFN(i); \
        total /= ((float)n);                                   \
        return total;                                          \
    }
GLADES_OVERALL(getOverallAccuracy, getClassAccuracy)
GLADES_OVERALL(getOverallPrecision, getClassPrecision)
GLADES_OVERALL(getOverallRecall, getClassRecall)
GLADES_OVERALL(getOverallSpecificity, getClassSpecificity)
GLADES_OVERALL(getOverallFalseAlarm, getClassFalseAlarm)
GLADES_OVERALL(getOverallF1Score, getClassF1Score)
#undef GLADES_OVERALL

void CMatrix::print() const
{
    printf("[CMATRIX] Confusion Matrix...\n");
    for (unsigned int r = 0; r < n; ++r) {
        for (unsigned int c = 0; c < n; ++c) printf("%d%s", matrix[(size_t)r * n + c], c + 1 < n ? "," : "\n");
    }
    const char* names[4] = {"True Positives", "True Negatives", "False Positives", "False Negatives"};
    const std::vector<int>* lists[4] = {&truePositive, &trueNegative, &falsePositive, &falseNegative};
    for (int k = 0; k < 4; ++k) {
        printf("[CMATRIX] %s...\n", names[k]);
        for (unsigned int i = 0; i < n; ++i) printf("%d%s", (*lists[k])[i], i + 1 < n ? "," : "\n");
    }
}

void CMatrix::reset()  // cmatrix.cpp:285-298: keeps the shape
{
    matrix.assign((size_t)n * n, 0);
    truePositive.assign(n, 0); trueNegative.assign(n, 0); falsePositive.assign(n, 0); falseNegative.assign(n, 0);
}

void CMatrix::clean()
{
    n = 0;
    matrix.clear(); truePositive.clear(); trueNegative.clear(); falsePositive.clear(); falseNegative.clear();
}

bool NNetwork::prepare(DataInput* newDataInput)
{
    if (!skeleton) return false;
    if (!newDataInput) return false;
    di = newDataInput;
    if ((di->getTrainSize() <= 0) || (di->getFeatureCount() <= 0)) return false;
    if (!dev) {  // network.cpp:127-128 builds when epochs == 0; a restored checkpoint arrives with its epoch count
        if (!build()) {
            if (dev) ghip_net_destroy(dev);
            dev = NULL;
            return false;
        }
    }
    minibatchSize = skeleton->getBatchSize();
    return dev != NULL;
}

// what follows a batch of epochs (network.cpp:193-258): statistics of the last one, class figures, progress line
void NNetwork::afterEpochs(const void* lastMetrics, int ran, int runType)
{
    const ghip_metrics* m = (const ghip_metrics*)lastMetrics;
    epochs += ran;
    overallTotalError = m->loss;
    overallTotalAccuracy = m->accuracy;
    overallCorrect = m->correct;
    const bool classes = confusionMatrix.size() > 0;
    if (classes) {
        // network.cpp:218-224: the device counted the last epoch's cells; the ratios are CMatrix's
        std::vector<int> cells((size_t)nOut * nOut);
        if (ghip_net_confusion_get(dev, cells.data(), (int64_t)cells.size()) == 0) {
            confusionMatrix.reset();
            confusionMatrix.setMatrix(cells);
            confusionMatrix.updateResultParams();
            overallClassAccuracy = confusionMatrix.getOverallAccuracy() * 100.0f;
            overallClassPrecision = confusionMatrix.getOverallPrecision() * 100.0f;
            overallClassRecall = confusionMatrix.getOverallRecall() * 100.0f;
            overallClassSpecificity = confusionMatrix.getOverallSpecificity() * 100.0f;
            overallClassF1 = confusionMatrix.getOverallF1Score() * 100.0f;
        }
    }
    if (verbose && runType == RUN_TRAIN) {
        if (classes)
            printf("\33[2K[NN] %d\t%s%f%%\t%f%%\t%f%%\t%f%%\t%f%%\r", epochs, epochs < 100 ? "\t" : "", overallClassAccuracy,
                   overallClassPrecision, overallClassRecall, overallClassSpecificity, overallClassF1);
        else
            printf("\33[2K[NN] %d\t%f%%\r", epochs, overallTotalAccuracy);
        fflush(stdout);
    }
}

namespace {
// several epochs per launch where the stop conditions allow it: up to the next epoch multiple,
// 1 when a wall-clock condition has to be polled every epoch or for the test pass
int epochChunk(const Terminator& t, int epochs, int runType)
{
    if (runType == NNetwork::RUN_TEST || t.getTimestamp() > 0) return 1;
    if (t.getEpoch() > 0) {
        const int64_t e = t.getEpoch();
        const int64_t left = e - ((int64_t)epochs % e);
        return (int)(left < 4096 ? left : 4096);
    }
    return 16;
}
}  // namespace

// NNetwork::run (ML/Networks/network.cpp:114-397)
void NNetwork::run(DataInput* newDataInput, int runType)
{
    if (!prepare(newDataInput)) return;
    if (verbose && runType == RUN_TRAIN) printf("[NN] Training...\n");
    else if (verbose && runType == RUN_TEST) printf("[NN] Testing...\n");

    const bool want_preds = (size_t)nRows * nOut <= (1u << 20);
    std::vector<float> preds(want_preds ? (size_t)nRows * nOut : 0);
    std::vector<float> Ylast = di->getTrainExpectedRow(nRows - 1);
    resetGraphs();  // network.cpp:167
    running = true;
    while (running) {
        if (mode == MODE_EXACT) {
            // with dropout one epoch per launch: the flags come from libc rand() as the epoch starts
            const int chunk = dropoutOn ? 1 : epochChunk(terminator, epochs, runType);
            std::vector<ghip_metrics> ms(chunk);
            int ran = 0;
            if (dropoutOn) {
                drawDropout();
                if (ghip_net_set_dropout_masks(dev, dropFlags.data(), 1) != 0) { lastError = ghip_last_error(); break; }
            }
            // the darts of a run without dropout: on a second thread while the device runs, where every epoch of the
            // chunk is certain to run (the accuracy condition is the only one looked at inside a launch)
            std::thread payer;
            if (!dropoutOn && randFidelity && terminator.getAccuracy() <= 0.0f && prepaidDrawEpochs == 0)
                payer = std::thread([this, chunk] { prepayDropoutDraws(chunk); });
            const int rc = ghip_net_run_epochs_exact(dev, chunk, runType == RUN_TRAIN ? 1 : 0, terminator.getAccuracy(), ms.data(), &ran,
                                                     want_preds ? preds.data() : NULL);
            if (payer.joinable()) payer.join();
            if (rc != 0) {
                lastError = ghip_last_error();
                break;
            }
            if (ran <= 0) break;
            skipDropoutDraws(ran);  // the darts the reference throws at rate 0 (train and test passes alike)
            for (int e = 0; e < ran; ++e) learningCurve.push_back(ms[e].accuracy);
            afterEpochs(&ms[ran - 1], ran, runType);
        } else {
            // canonical mode: batches [k*mb, (k+1)*mb), the last one averaged over its true size; the confusion
            // counters restart at the head of every epoch (network.cpp:183-185).  Several epochs per call where the
            // stop conditions allow it: a narrow network then runs them as one launch, any other pass by pass with
            // every step of a pass enqueued back to back and the metrics added up on the device.
            const int mb = minibatchSize > 0 ? minibatchSize : (int)nRows;
            // with dropout one epoch per call: the flags come from libc rand() as the epoch starts, as in exact mode
            const int chunk = dropoutOn ? 1 : epochChunk(terminator, epochs, runType);
            std::vector<ghip_metrics> ms(chunk);
            int ran = 0;
            if (dropoutOn) {
                drawDropout();
                if (ghip_net_set_dropout_masks(dev, dropFlags.data(), 1) != 0) { lastError = ghip_last_error(); break; }
            }
            if (ghip_net_run_epochs_canonical(dev, mb, chunk, runType == RUN_TRAIN ? 1 : 0, terminator.getAccuracy(), ms.data(), &ran) != 0) {
                lastError = ghip_last_error();
                break;
            }
            if (ran <= 0) break;
            for (int e = 0; e < ran; ++e) learningCurve.push_back(ms[e].accuracy);
            afterEpochs(&ms[ran - 1], ran, runType);
        }
        if (terminator.triggered(time(NULL), epochs, overallTotalAccuracy)) break;
        if (runType == RUN_TEST) break;
    }
    if (want_preds && mode == MODE_EXACT) {
        results.clear();  // the reference's list holds the last row's (expected, predicted) pairs
        for (unsigned int o = 0; o < nOut; ++o) {
            results.push_back(o < Ylast.size() ? Ylast[o] : 0.0f);
            results.push_back(preds[(size_t)(nRows - 1) * nOut + o]);
        }
    }
    if (verbose && runType == RUN_TRAIN) printf("\n");
    else if (verbose && runType == RUN_TEST) printf("[NN] %s Accuracy: %f%%\n", skeleton->getName().c_str(), overallTotalAccuracy);
    running = false;
}

// Subnets that are the same network in everything but their parameters (exact mode, equal tables,
// equal epoch counters and stop conditions) train in ONE kernel launch per chunk of epochs, a
// workgroup each; a subnet that meets its stop condition leaves the group.
bool MetaNetwork::runGroup(DataInput* d, int runType, bool testsFollow)
{
    std::vector<NNetwork*> act;
    // The reference runs subnet after subnet, so a subnet that samples its weights finds libc's rand()
    // where the runs of the subnets before it left it.  Here all subnets are built first: if a later
    // one samples, the draws of the runs before it are taken ahead of time, which needs their number:
    // known for an epoch-count stop, unknown for an accuracy stop (then the caller runs them in turn).
    bool laterSamples = false;
    for (size_t i = 1; i < subnets.size(); ++i) laterSamples = laterSamples || (subnets[i] && subnets[i]->samplesOnBuild());
    for (size_t i = 0; i < subnets.size(); ++i) {
        NNetwork* n = subnets[i];
        if (!n || !n->skeleton || n->mode != NNetwork::MODE_EXACT) return false;
        if (n->hasDropout()) return false;  // the subnets draw from one rand() stream, in subnet order
        NNetwork* a = subnets[0];
        if (n->epochs != a->epochs || n->biasMode != a->biasMode || n->skeleton->toTable() != a->skeleton->toTable()) return false;
        if (n->terminator.getEpoch() != a->terminator.getEpoch() || n->terminator.getAccuracy() != a->terminator.getAccuracy() ||
            n->terminator.getTimestamp() != 0) return false;
        if (laterSamples && runType == NNetwork::RUN_TRAIN && (n->terminator.getAccuracy() > 0.0f || n->terminator.getEpoch() <= 0)) return false;
    }
    for (size_t i = 0; i < subnets.size(); ++i) {
        if (!subnets[i]->prepare(d)) return false;
        if (laterSamples) {
            NNetwork* n = subnets[i];
            const int64_t e = n->terminator.getEpoch();
            const int64_t ahead = (runType == NNetwork::RUN_TRAIN ? e - ((int64_t)n->epochs % e) : 1) + (testsFollow ? 1 : 0);
            n->prepayDropoutDraws(ahead);
        }
        subnets[i]->resetGraphs();
        subnets[i]->running = true;
        act.push_back(subnets[i]);
    }
    while (!act.empty()) {
        const int chunk = epochChunk(act[0]->terminator, act[0]->epochs, runType);
        std::vector<ghip_net*> handles(act.size());
        for (size_t i = 0; i < act.size(); ++i) handles[i] = act[i]->dev;
        std::vector<ghip_metrics> ms((size_t)chunk * act.size());
        std::vector<int> ran(act.size(), 0);
        if (ghip_net_run_epochs_exact_multi(handles.data(), (int)act.size(), chunk, runType == NNetwork::RUN_TRAIN ? 1 : 0,
                                            act[0]->terminator.getAccuracy(), ms.data(), ran.data()) != 0) {
            for (size_t i = 0; i < act.size(); ++i) { act[i]->lastError = ghip_last_error(); act[i]->running = false; }
            return true;
        }
        std::vector<NNetwork*> next;
        for (size_t i = 0; i < act.size(); ++i) {
            NNetwork* n = act[i];
            if (ran[i] <= 0) { n->running = false; continue; }
            n->skipDropoutDraws(ran[i]);
            for (int e = 0; e < ran[i]; ++e) n->learningCurve.push_back(ms[i * chunk + e].accuracy);
            n->afterEpochs(&ms[i * chunk + ran[i] - 1], ran[i], runType);
            const bool done = !n->running || n->terminator.triggered(time(NULL), n->epochs, n->overallTotalAccuracy) || runType == NNetwork::RUN_TEST;
            if (done) n->running = false;
            else next.push_back(n);
        }
        // the survivors share a launch only while their epoch counters agree
        for (size_t i = 1; i < next.size(); ++i)
            if (next[i]->epochs != next[0]->epochs) {
                for (size_t k = 0; k < next.size(); ++k) { next[k]->running = false; next[k]->run(d, runType); }
                next.clear();
                break;
            }
        act.swap(next);
    }
    return true;
}

// ------------------------------------------------------------------ facade (ML/main.cpp:51-243)

// ML/main.cpp:32-45.  glades::init() of the reference also creates the folder (main.cpp:51-56); here that
// is left to the first NNetwork::save(), so that initialising the device writes nothing to disk.
bool doesDatabaseExist()
{
    struct stat buffer;
    return stat("database", &buffer) == 0 && S_ISDIR(buffer.st_mode);
}
void createDatabase() { mkdir("database", 0777); }

void init() { ghip_init(0); }

bool saveNeuralNetwork(NNetwork* newNet)  // ML/main.cpp:58-73
{
    if (!newNet) return false;
    if (!newNet->save()) {
        printf("Unable to save \"%s\"\n", newNet->getName().c_str());
        return false;
    }
    return true;
}

MetaNetwork* train(NNetwork* net, DataInput* d)
{
    if (!net || !d) return NULL;
    MetaNetwork* m = new MetaNetwork(net->getName());
    m->addSubnet(net);
    return train(m, d);
}

MetaNetwork* train(NNInfo* info, DataInput* d)
{
    if (!info || !d) return NULL;
    return train(new NNetwork(info), d);
}

namespace {
// runs fn(subnet) for every subnet: one host thread each when the MetaNetwork is concurrent (the
// device work of different networks lives on different streams), else in order
template <typename Fn>
void for_each_subnet(MetaNetwork* m, Fn fn)
{
    const std::vector<NNetwork*>& nets = m->getSubnets();
    // libc rand() is one stream and the reference's order is subnet after subnet: subnets that draw
    // dropout flags, or that sample their weights after another subnet's run, take their turn
    bool dropout = false;
    for (size_t i = 0; i < nets.size(); ++i)
        dropout = dropout || (nets[i] && (nets[i]->hasDropout() || (i > 0 && nets[i]->samplesOnBuild())));
    if (!m->getConcurrent() || nets.size() < 2 || dropout) {
        for (size_t i = 0; i < nets.size(); ++i)
            if (nets[i]) fn(nets[i]);
        return;
    }
    std::vector<std::thread> pool;
    for (size_t i = 0; i < nets.size(); ++i)
        if (nets[i]) pool.push_back(std::thread(fn, nets[i]));
    for (size_t i = 0; i < pool.size(); ++i) pool[i].join();
}
}  // namespace

MetaNetwork* train(MetaNetwork* m, DataInput* d)
{
    if (!m || !d) return NULL;
    if (m->getConcurrent() && m->size() > 1 && m->runGroup(d, NNetwork::RUN_TRAIN)) return m;
    for_each_subnet(m, [d](NNetwork* n) { n->train(d); });
    return m;
}

MetaNetwork::MetaNetwork(NNInfo* networkInfo, int subnetCount)
    : name(networkInfo ? networkInfo->getName() : std::string()), collectionType(subnetCount > 1 ? ONE_TO_MANY : ONE_TO_ONE),
      concurrent(true)
{
    for (int i = 0; i < subnetCount; ++i) addSubnet(networkInfo);
}

MetaNetwork::MetaNetwork(const std::string& metaNetName, const std::string& nname, int k)
    : name(metaNetName), collectionType(k > 1 ? ONE_TO_MANY : ONE_TO_ONE), concurrent(true)
{
    for (int i = 0; i < k; ++i) addSubnet(nname);
}

void MetaNetwork::addSubnet(const std::string& nNetName)
{
    if (nNetName.empty()) return;
    NNetwork* n = new NNetwork();
    if (n->load(nNetName)) subnets.push_back(n);
    else delete n;
}

NNetwork* MetaNetwork::getSubnetByName(const std::string& n) const
{
    for (size_t i = 0; i < subnets.size(); ++i)
        if (subnets[i] && subnets[i]->getName() == n) return subnets[i];
    return NULL;
}

float MetaNetwork::crossValidate(DataInput* newDataInput)
{
    if (!newDataInput || subnets.empty()) return 0.0f;
    if (concurrent && subnets.size() > 1 && runGroup(newDataInput, NNetwork::RUN_TRAIN, true)) {
        if (!runGroup(newDataInput, NNetwork::RUN_TEST))
            for_each_subnet(this, [newDataInput](NNetwork* n) { n->test(newDataInput); });
    } else {
        for_each_subnet(this, [newDataInput](NNetwork* n) { n->train(newDataInput); n->test(newDataInput); });
    }
    float cvAccuracy = 0.0f;
    for (size_t i = 0; i < subnets.size(); ++i)
        if (subnets[i]) cvAccuracy += subnets[i]->getAccuracy();
    printf("cvAccuracy: %f \t\n", cvAccuracy / subnets.size());
    return cvAccuracy / subnets.size();
}

MetaNetwork* test(NNetwork* net, DataInput* d)
{
    if (!net || !d) return NULL;
    MetaNetwork* m = new MetaNetwork(net->getName());
    m->addSubnet(net);
    return test(m, d);
}

MetaNetwork* test(NNInfo* info, DataInput* d)
{
    if (!info || !d) return NULL;
    return test(new NNetwork(info), d);
}

MetaNetwork* test(MetaNetwork* m, DataInput* d)
{
    if (!m || !d) return NULL;
    if (m->getConcurrent() && m->size() > 1 && m->runGroup(d, NNetwork::RUN_TEST)) return m;
    for_each_subnet(m, [d](NNetwork* n) { n->test(d); });
    return m;
}

}  // namespace glades

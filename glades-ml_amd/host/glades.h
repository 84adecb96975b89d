// glades.h -- the reference's C++ network/training API for the dense feed-forward path, backed
// by the gfx950 library behind include/glades_hip.h.
//
// Same class names, method names, argument order and error behaviour (silent early returns,
// NULL / false; nothing throws) as the reference, with std types where the reference uses the
// shmea containers (GString -> std::string, GList -> std::vector<float>, GTable -> rows of
// floats).  Citations are to the reference tree, "ML/" = "Backend/Machine Learning/".
//
//   GMath constants        ML/GMath/gmath.h:35-54
//   LayerInfo family       ML/Structure/{layerinfo,inputlayerinfo,hiddenlayerinfo,outputlayerinfo}.h
//   NNInfo                 ML/Structure/nninfo.h:41-127 (index-shifted getters: nninfo.cpp:240-373)
//   Terminator             ML/State/Terminator.h:27-51
//   DataInput              ML/DataObjects/DataInput.h:26-50
//   CMatrix                ML/GMath/cmatrix.h:27-67
//   OHE                    ML/GMath/OHE.h:27-78
//   NumberInput            ML/DataObjects/NumberInput.h:27-84
//   NNetwork               ML/Networks/network.h:59-141
//   MetaNetwork            ML/Networks/metanetwork.h:44-64
//   glades::init/train/test  ML/main.h:44-54
#ifndef GLADES_AMD_HOST_H
#define GLADES_AMD_HOST_H

#include <stdint.h>

#include <string>
#include <vector>

struct ghip_net;

namespace glades {

class GMath
{
public:
    static constexpr float INLIER = 0.954f;
    static constexpr float OUTLIER = 0.046f;
    static const int REGRESSION = 0, CLASSIFICATION = 1, KL = 2;
    static const int TANH = 0, TANHP = 1, SIGMOID = 2, SIGMOIDP = 3, LINEAR = 4, RELU = 5, LEAKY = 6, STEP = 7;
    static const int SOFTMAX = 8;  // extension: canonical mode output layer only
    static const int MINMAX = 0, ZSCORE = 1;
};

class LayerInfo
{
protected:
    int lSize;
    float learningRate, momentumFactor, weightDecay1, weightDecay2, pDropout, activationParam;
    int activationType;

public:
    explicit LayerInfo(int newSize);
    virtual ~LayerInfo() {}
    int size() const { return lSize; }
    float getLearningRate() const { return learningRate; }
    float getMomentumFactor() const { return momentumFactor; }
    float getWeightDecay1() const { return weightDecay1; }
    float getWeightDecay2() const { return weightDecay2; }
    float getPDropout() const { return pDropout; }
    int getActivationType() const { return activationType; }
    float getActivationParam() const { return activationParam; }
    void setSize(int v) { lSize = v; }
    void setLearningRate(float v) { learningRate = v; }
    void setMomentumFactor(float v) { momentumFactor = v; }
    void setWeightDecay1(float v) { weightDecay1 = v; }
    void setWeightDecay2(float v) { weightDecay2 = v; }
    void setPDropout(float v) { pDropout = v; }
    void setActivationType(int v) { activationType = v; }
    void setActivationParam(float v) { activationParam = v; }
    // layerinfo.cpp:57-66: size, rates, decays, dropout and activation type; the activation parameter stays
    void copyParamsFrom(const LayerInfo* src);
};

class InputLayerInfo : public LayerInfo
{
    int batchSize;

public:
    // argument order of inputlayerinfo.cpp:29-32
    InputLayerInfo(int newBatchSize, float newLearningRate, float newMomentumFactor, float newWeightDecay1,
                   float newWeightDecay2, float newPDropout, int newActivationType, float newActivationParam);
    int getBatchSize() const { return batchSize; }
    void setBatchSize(int v) { batchSize = v; }
};

class HiddenLayerInfo : public LayerInfo
{
public:
    // argument order of hiddenlayerinfo.cpp:31-34
    HiddenLayerInfo(int newSize, float newLearningRate, float newMomentumFactor, float newWeightDecay1,
                    float newWeightDecay2, float newPDropout, int newActivationType, float newActivationParam);
};

class OutputLayerInfo : public LayerInfo
{
    int outputType;

public:
    OutputLayerInfo(int newSize, int newOutputType);
    int getOutputType() const { return outputType; }
    void setOutputType(int v) { outputType = v; }
};

// One row of the 10-column table the reference stores a network skeleton in
// (nninfo.h:69-78: Size,batchSize,learningRate,momentumFactor,weightDecay1,weightDecay2,pDropout,
//  activationType,activationParam,outputType).
typedef std::vector<std::vector<float> > NNTable;

class NNInfo
{
    std::string name;
    int inputType;
    InputLayerInfo* inputLayer;
    OutputLayerInfo* outputLayer;
    std::vector<HiddenLayerInfo*> layers;

public:
    static const int BATCH_FULL = 0;
    static const int BATCH_STOCHASTIC = 1;
    static const int COL_SIZE = 0, COL_BATCH_SIZE = 1, COL_LEARNING_RATE = 2, COL_MOMENTUM_FACTOR = 3,
                     COL_WEIGHT_DECAY1 = 4, COL_WEIGHT_DECAY2 = 5, COL_PDROPOUT = 6, COL_ACTIVATION_TYPE = 7,
                     COL_ACTIVATION_PARAM = 8, COL_OUTPUT_TYPE = 9;

    explicit NNInfo(const std::string& newName);
    NNInfo(const std::string& newName, const NNTable& table);  // nninfo.cpp:70-82,738-785
    NNInfo(const std::string& newName, InputLayerInfo*, const std::vector<HiddenLayerInfo*>&, OutputLayerInfo*);
    ~NNInfo();  // owns and deletes its LayerInfos (nninfo.cpp:88-104)

    std::string getName() const { return name; }
    int getInputType() const { return inputType; }
    int getOutputType() const;
    float getPInput() const;
    int getBatchSize() const;
    InputLayerInfo* getInputLayer() const { return inputLayer; }
    std::vector<HiddenLayerInfo*> getLayers() const { return layers; }
    int numHiddenLayers() const { return (int)layers.size(); }
    int getInputLayerSize() const { return inputLayer ? inputLayer->size() : 0; }
    int getHiddenLayerSize(unsigned int) const;
    unsigned int getOutputLayerSize() const;
    // index 0 reads the input row, index k >= 1 the hidden row k-1 (nninfo.cpp:240-373);
    // getWeightDecay2(0) returns the input row's weightDecay1, as the reference does (:305-306)
    float getLearningRate(unsigned int) const;
    float getMomentumFactor(unsigned int) const;
    float getWeightDecay1(unsigned int) const;
    float getWeightDecay2(unsigned int) const;
    float getPDropout(unsigned int) const;
    int getActivationType(unsigned int) const;
    float getActivationParam(unsigned int) const;

    void print() const;  // nninfo.cpp:379-431: "[NNINFO]" lines, one per layer row, -1 cells left blank

    void setName(const std::string& v) { name = v; }
    void setInputType(int v) { inputType = v; }
    void setPInput(float);
    void setLayers(const std::vector<HiddenLayerInfo*>& newLayers) { layers = newLayers; }
    void setOutputType(int);
    void setOutputSize(int);
    void setBatchSize(int);
    void setLearningRate(unsigned int, float);
    void setMomentumFactor(unsigned int, float);
    void setWeightDecay1(unsigned int, float);
    // the reference addresses hidden row index-2 here (nninfo.cpp:586-603), so index 1 reaches no row
    // (there it reads layers[-1]); this does nothing for index 1
    void setWeightDecay2(unsigned int, float);
    void setPDropout(unsigned int, float);
    void setActivationType(unsigned int, int);
    void setActivationParam(unsigned int, float);
    void addHiddenLayer(HiddenLayerInfo*);
    void copyHiddenLayer(unsigned int dst, unsigned int src);
    // new rows are HiddenLayerInfo(2, 0.01, 0, 0, 0, 0, TANH, 0) (nninfo.cpp:683-686), one object per row
    // here (the reference puts ONE object into every new slot and deletes it once per slot); rows cut
    // off are deleted
    void resizeHiddenLayers(unsigned int newCount);
    void removeHiddenLayer(unsigned int index);  // the row leaves the list; like the reference, it is not deleted

    NNTable toTable() const;
    bool fromTable(const std::string& netName, const NNTable& table);
    // CSV form of the table as the reference's fixtures hold it (header line + rows)
    bool loadFile(const std::string& path);
    bool saveFile(const std::string& path) const;
};

class Terminator
{
    int64_t timestamp, epoch;
    float accuracy;

public:
    Terminator();
    int64_t getTimestamp() const { return timestamp; }
    int64_t getEpoch() const { return epoch; }
    float getAccuracy() const { return accuracy; }
    void setTimestamp(int64_t v) { timestamp = v; }
    void setEpoch(int64_t v) { epoch = v; }
    void setAccuracy(float v) { accuracy = v; }
    bool triggered(int64_t cTimestamp, int64_t cEpoch, float cAccuracy) const;  // Terminator.cpp:63-78
};

class DataInput
{
public:
    static const int CSV = 0, IMAGE = 1, TEXT = 2;
    std::vector<bool> featureIsCategorical;
    virtual ~DataInput() {}
    virtual void import(std::string) = 0;
    virtual std::vector<float> getTrainRow(unsigned int) const = 0;
    virtual std::vector<float> getTrainExpectedRow(unsigned int) const = 0;
    virtual std::vector<float> getTestRow(unsigned int) const = 0;
    virtual std::vector<float> getTestExpectedRow(unsigned int) const = 0;
    virtual unsigned int getTrainSize() const = 0;
    virtual unsigned int getTestSize() const = 0;
    virtual unsigned int getFeatureCount() const = 0;
    virtual int getType() const = 0;
    // dense views; the default builds them from the row getters
    virtual void denseTrain(std::vector<float>& X, std::vector<float>& Y, unsigned int& nOut) const;
};

// In-memory table (no counterpart class in the reference; plays the role NumberInput's
// trainTable / trainExpectedTable play after import)
class DenseInput : public DataInput
{
    std::vector<float> X, Y;
    unsigned int rows, feats, outs;

public:
    DenseInput(const float* x, const float* y, unsigned int nRows, unsigned int nFeatures, unsigned int nOutputs);
    void import(std::string) {}
    std::vector<float> getTrainRow(unsigned int) const;
    std::vector<float> getTrainExpectedRow(unsigned int) const;
    std::vector<float> getTestRow(unsigned int i) const { return getTrainRow(i); }
    std::vector<float> getTestExpectedRow(unsigned int i) const { return getTrainExpectedRow(i); }
    unsigned int getTrainSize() const { return rows; }
    unsigned int getTestSize() const { return 0; }
    unsigned int getFeatureCount() const { return feats; }
    int getType() const { return CSV; }
    void denseTrain(std::vector<float>& x, std::vector<float>& y, unsigned int& nOut) const;
};

// One-hot encoder of a string column (ML/GMath/OHE.cpp): classes in order of first appearance,
// a class encodes as 0.99 at its index and 0.01 elsewhere (OHE.cpp:159-198).
class OHE
{
    std::vector<std::string> OHEStrings;
    std::vector<int> classCount;

public:
    void addString(const std::string&);
    unsigned int size() const { return (unsigned int)OHEStrings.size(); }
    std::vector<std::string> getStrings() const { return OHEStrings; }
    bool contains(const std::string&) const;
    int indexAt(const std::string&) const;                     // -1 if absent
    std::string classAt(unsigned int) const;
    std::vector<float> operator[](const std::string&) const;   // 0.99 / 0.01 vector
    std::string operator[](const std::vector<float>&) const;   // class of the largest entry (>= scan, OHE.cpp:216-238)
};

// CSV table -> standardised training table (ML/DataObjects/NumberInput.cpp:43-285).
// The reference reads the file with the shmea GTable parser, which is not part of its tree; this
// class states that boundary itself: first line = header, comma separated, cells trimmed, a cell
// is a string iff it does not parse completely as a number, the LAST column is the output column
// (the convention its fixtures xornet / iris rely on; setOutputColumns overrides it).
// What happens to the parsed table is the reference's: a column whose first cell is a string is
// categorical and one-hot encoded (0.99 / 0.01); any categorical column makes the run a
// classification; numeric columns are min-max scaled to [0.01, 0.99] (classification) or [0, 1]
// (regression), or z-scored; the running minimum / maximum start at the first cell only for
// column 0 and at 0 for every other column (NumberInput.cpp:103-107); a constant column goes to
// the feature table unscaled, output column or not (:171-176).
class NumberInput : public DataInput
{
    std::string name;
    bool loaded;
    std::vector<std::vector<float> > trainTable, trainExpectedTable;  // [row][col]
    std::vector<std::string> trainHeaders, expectedHeaders;
    std::vector<OHE> OHEMaps;
    std::vector<int> outputColumns;  // empty: the last column
    unsigned int rows;

public:
    NumberInput() : loaded(false), rows(0) {}
    void setOutputColumns(const std::vector<int>& cols) { outputColumns = cols; }
    void import(std::string fname);  // NumberInput.cpp:27-41: loads once
    bool standardizeInputTable(const std::string& fname, int standardizeFlag = GMath::MINMAX);
    bool standardizeText(const std::string& csvText, int standardizeFlag = GMath::MINMAX);
    std::vector<float> getTrainRow(unsigned int) const;
    std::vector<float> getTrainExpectedRow(unsigned int) const;
    std::vector<float> getTestRow(unsigned int) const { return std::vector<float>(); }
    std::vector<float> getTestExpectedRow(unsigned int) const { return std::vector<float>(); }
    unsigned int getTrainSize() const { return rows; }
    unsigned int getTestSize() const { return 0; }
    unsigned int getFeatureCount() const { return trainTable.empty() ? 0 : (unsigned int)trainTable[0].size(); }
    unsigned int getOutputCount() const { return trainExpectedTable.empty() ? 0 : (unsigned int)trainExpectedTable[0].size(); }
    int getType() const { return CSV; }
    const std::vector<OHE>& getOHEMaps() const { return OHEMaps; }
    std::vector<std::string> getTrainHeaders() const { return trainHeaders; }
    std::vector<std::string> getExpectedHeaders() const { return expectedHeaders; }
};

// Confusion matrix of a classification run (ML/GMath/cmatrix.cpp).  Row = expected class, column =
// predicted class, both chosen by the strictly-greater-than scan from 0 of GMath::naiveVectorDecomp
// (gmath.cpp:412-455).  The GTable / GLists of the reference are plain int vectors here.  During a
// run the cells are counted on the device and copied in with setMatrix(); addResult() is the
// host-side form for callers that feed (expected, predicted) pairs themselves.
class CMatrix
{
    unsigned int n;
    std::vector<int> matrix;  // n x n, row-major
    std::vector<int> truePositive, trueNegative, falsePositive, falseNegative;

public:
    CMatrix() : n(0) {}
    void build(unsigned int numberOfClasses);
    void addResult(const std::vector<float>& result);  // e0, p0, e1, p1, ... (network.cpp:529-530)
    void setMatrix(const std::vector<int>& cells);     // n x n cells counted elsewhere
    void updateResultParams();
    std::vector<std::vector<int> > getMatrix() const;
    int getCell(unsigned int row, unsigned int col) const { return matrix[(size_t)row * n + col]; }
    unsigned int size() const { return n; }
    float getClassAccuracy(unsigned int) const;
    float getOverallAccuracy() const;
    float getClassPrecision(unsigned int) const;
    float getOverallPrecision() const;
    float getClassRecall(unsigned int) const;
    float getOverallRecall() const;
    float getClassSpecificity(unsigned int) const;
    float getOverallSpecificity() const;
    float getClassFalseAlarm(unsigned int) const;
    float getOverallFalseAlarm() const;
    float getClassF1Score(unsigned int) const;
    float getOverallF1Score() const;
    void print() const;
    void reset();
    void clean();
};

class MetaNetwork;

class NNetwork
{
    friend class MetaNetwork;
    DataInput* di;
    NNInfo* skeleton;
    ghip_net* dev;
    volatile bool running;
    int netType, epochs, mode, dtype, biasMode;
    bool verbose;
    float overallTotalError, overallTotalAccuracy;
    float overallClassAccuracy, overallClassPrecision, overallClassRecall, overallClassSpecificity, overallClassF1;
    CMatrix confusionMatrix;
    int64_t overallCorrect;
    int minibatchSize;
    int64_t id;
    std::vector<float> results;                 // (expected, predicted) pairs of the last row
    std::vector<float> learningCurve;           // accuracy after every epoch of the current run
    std::vector<std::vector<float> > initW;     // weights injected before the first run
    std::vector<std::vector<float> > initB;
    std::vector<std::vector<float> > initStateA, initStateB;  // optimiser state of a restored checkpoint
    std::vector<std::vector<int32_t> > initCounts;            // dropout leftovers of a restored checkpoint:
    std::vector<std::vector<float> > initErrDer;              // window lengths, node error accumulators
    unsigned int nRows, nFeat, nOut;
    std::string lastError;
    // dropout (LayerBuilder::scrambleDropout, ML/State/LayerBuilder.cpp:497-523): probability per node
    // layer (0 = input) as the reference resolves it, and the flags of the last epoch drawn, which the
    // layers whose rate draws nothing keep (Layer::generateDropout returns early, layer.cpp:107-112)
    std::vector<float> pNode;
    std::vector<unsigned char> dropFlags;
    bool dropoutOn;
    void drawDropout();                              // one epoch's flags from libc rand()
    // Layer::generateDropout draws one dart per node and row for every rate in 0..99, also at rate 0,
    // where no dart can drop anything (layer.cpp:102-134): a run without dropout still moves libc's
    // rand() by that many draws per epoch, which the next network's weight sampler then starts from
    int64_t prepaidDrawEpochs;                       // epochs whose draws have been taken ahead of the run
    bool randFidelity;                               // take those draws at all (setRandStreamFidelity)
    size_t dropoutDrawsPerEpoch() const;
    void skipDropoutDraws(int64_t epochs);           // exact mode, no flags: take the draws and throw them away
    void prepayDropoutDraws(int64_t epochs);

    void run(DataInput*, int);
    bool prepare(DataInput*);                        // checks + build on first use
    void afterEpochs(const void* lastMetrics, int ran, int runType);  // statistics, class figures, progress line
    bool build();

public:
    bool hasDropout() const;  // some layer's rate int(p*100) lies in 1..99
    bool samplesOnBuild() const;  // not built yet and not every layer's weights injected: the first run draws weights from rand()
    static const int TYPE_DFF = 0, TYPE_RNN = 1;
    static const int RUN_TRAIN = 0, RUN_TEST = 1, RUN_VALIDATE = 2;
    static const int MODE_EXACT = 0, MODE_CANONICAL = 1;      // extension
    static const int DTYPE_F32 = 0, DTYPE_BF16 = 1;           // extension (canonical mode)

    Terminator terminator;

    NNetwork();
    explicit NNetwork(NNInfo*);
    virtual ~NNetwork();
    int64_t getCurrentTimeMilliseconds() const;  // network.cpp:82-87
    bool getRunning() const { return running; }
    int getEpochs() const { return epochs; }
    void stop() { running = false; }

    // reads an NNInfo table file (network.cpp:701-712).  The reference resolves a network's name inside
    // its database folder (SaveFolder("neuralnetworks"), nninfo.cpp:787-798): a path that does not exist
    // is looked up as database/neuralnetworks/<path>
    bool load(const std::string& path);
    bool save(const std::string& path) const;
    bool save() const;  // network.cpp:714-722 -> NNInfo::save: database/neuralnetworks/<name>

    void train(DataInput*);
    void test(DataInput*);

    int64_t getID() const { return id; }
    std::string getName() const;
    NNInfo* getNNInfo() { return skeleton; }
    float getAccuracy() const { return overallTotalAccuracy; }
    std::vector<float> getResults() const { return results; }
    // The reference declares the list and never fills it (network.cpp:730-733, 764-775); here it holds
    // the accuracy after every epoch since the run started.
    std::vector<float> getLearningCurve() const { return learningCurve; }
    void clean();        // network.cpp:745-762: lets go of the device network and the data
    void resetGraphs();  // network.cpp:764-775

    // ---- absent from the reference (its loss has no getter and its weights are not reachable)
    float getLoss() const { return overallTotalError; }
    int64_t getCorrect() const { return overallCorrect; }
    // the five figures of the reference's progress line (network.cpp:218-224), in percent, and the matrix
    // behind them (private members without getters in the reference)
    float getClassAccuracy() const { return overallClassAccuracy; }
    float getClassPrecision() const { return overallClassPrecision; }
    float getClassRecall() const { return overallClassRecall; }
    float getClassSpecificity() const { return overallClassSpecificity; }
    float getClassF1() const { return overallClassF1; }
    const CMatrix& getConfusionMatrix() const { return confusionMatrix; }
    void setMode(int newMode, int newDtype = DTYPE_F32) { mode = newMode; dtype = newDtype; }
    void setSequentialBias(bool faithful) { biasMode = faithful ? 0 : 1; }
    // A run without dropout still moves libc's rand() by one draw per node and row and epoch, as the reference's
    // does (layer.cpp:102-134), so that whatever draws from rand() next (another network's weight sampler, the
    // caller) finds the stream where the reference leaves it.  That is tens of millions of libc calls per epoch
    // for a table of cfg2's size; they are made on a second host thread while the device runs the epochs where
    // the number of epochs is known ahead (no accuracy condition), after the launch otherwise.  A caller who
    // never reads rand() again may turn them off.
    void setRandStreamFidelity(bool faithful) { randFidelity = faithful; }
    void setVerbose(bool v) { verbose = v; }  // the per-epoch progress line and the [NN] banners
    // layer = weight layer 0..numHiddenLayers(); W is [n_out][n_in] row-major
    bool setWeights(unsigned int layer, const std::vector<float>& W);
    bool setBias(unsigned int layer, const std::vector<float>& bias);  // 1 value (exact) or n_out
    std::vector<float> getWeights(unsigned int layer);
    std::vector<float> getBias(unsigned int layer);
    // Checkpoint = the skeleton's table + epochs run + every layer's weights, bias and optimiser state
    // (exact mode: the pending delta windows; canonical: momentum), so that a restored network
    // continues bit for bit.  The reference saves the table only (network.cpp:714-743: the weight
    // part is a stub); the table text inside the file is its format, the rest is this build's.
    bool saveCheckpoint(const std::string& path);
    bool loadCheckpoint(const std::string& path);  // call train() afterwards with the same DataInput
    std::string getLastError() const { return lastError; }
};

class MetaNetwork
{
    std::string name;
    int collectionType;
    std::vector<NNetwork*> subnets;
    bool concurrent;

public:
    static const int ONE_TO_ONE = 0, ONE_TO_MANY = 1;  // metanetwork.h:36-37
    explicit MetaNetwork(const std::string& newName) : name(newName), collectionType(ONE_TO_ONE), concurrent(true) {}
    // subnetCount networks over the same skeleton (metanetwork.cpp:36-50), e.g. for cross-validation
    MetaNetwork(NNInfo* networkInfo, int subnetCount = 1);
    // k networks loaded from the table `nname` (metanetwork.cpp:52-63)
    MetaNetwork(const std::string& metaNetName, const std::string& nname, int k = 1);
    virtual ~MetaNetwork() { name = ""; clearSubnets(); }  // the list is cleared, the networks are not deleted (metanetwork.cpp:65-69, 129-132)
    // Subnets are independent networks (metanetwork.cpp:86-127): with `concurrent` (the default) train /
    // test / crossValidate run them at the same time, one host thread and one HIP stream each, instead
    // of one after the other as the reference's loop does (ML/main.cpp:137-160).  Results are the same.
    void setConcurrent(bool v) { concurrent = v; }
    bool getConcurrent() const { return concurrent; }
    void addSubnet(NNInfo* info) { if (info) subnets.push_back(new NNetwork(info)); }  // metanetwork.cpp:95-102
    NNetwork* getSubnet(unsigned int i) { return i < subnets.size() ? subnets[i] : NULL; }
    void clearSubnets() { subnets.clear(); }
    // metanetwork.cpp:216-251: every subnet trains on the data, then runs the test pass; prints and
    // returns the mean test accuracy.  (The reference splits the file into k stratified folds with the
    // un-vendored GTable::stratify and then passes the WHOLE DataInput to every subnet all the same;
    // this does what that code does, without the unused split.)
    float crossValidate(DataInput* newDataInput);
    // one kernel launch for all subnets where they allow it (see glades.cpp); false = not applicable.
    // Subnets trained this way keep their metrics, learning curve and weights; getResults() (the last
    // row's predictions) stays empty, since the grouped launch returns no predictions.
    // testsFollow: every subnet's training is followed by its test pass before the next subnet trains
    // (crossValidate), which matters to where libc's rand() stands when a later subnet samples weights.
    bool runGroup(DataInput*, int runType, bool testsFollow = false);
    std::string getName() const { return name; }
    void setName(const std::string& v) { name = v; }
    int getCollectionType() const { return collectionType; }
    void addSubnet(NNetwork* n) { if (n) subnets.push_back(n); }
    void addSubnet(const std::string& nNetName);  // metanetwork.cpp:104-113: a network loaded from that table; nothing on failure
    std::string getSubnetName(unsigned int i) const { return (i < subnets.size() && subnets[i]) ? subnets[i]->getName() : std::string(); }
    NNetwork* getSubnetByName(const std::string& n) const;
    const std::vector<NNetwork*>& getSubnets() const { return subnets; }
    unsigned int size() const { return (unsigned int)subnets.size(); }
};

void init();
bool doesDatabaseExist();                 // ML/main.cpp:32-36: is there a "database" folder in the working directory
void createDatabase();                    // ML/main.cpp:38-45
bool saveNeuralNetwork(NNetwork*);        // ML/main.cpp:58-73
// ML/main.cpp:82-243: wrap in a MetaNetwork the caller owns, run every subnet on the same data
MetaNetwork* train(NNInfo*, DataInput*);
MetaNetwork* train(NNetwork*, DataInput*);
MetaNetwork* train(MetaNetwork*, DataInput*);
MetaNetwork* test(NNInfo*, DataInput*);
MetaNetwork* test(NNetwork*, DataInput*);
MetaNetwork* test(MetaNetwork*, DataInput*);

// The reference's weight sampler (ML/State/layer.cpp:196-217, ML/State/node.cpp:241-276): draws
// from libc rand(), so srand(seed) reproduces the reference's initial weights for a layer.
void xavierLayer(int fanIn, int nOut, int activationType, float* W);
// The initial weights of a whole network in the order LayerBuilder::buildHiddenLayers / buildOutputLayer
// sample them (ML/State/LayerBuilder.cpp:192-265), from libc rand(): W[l] is sizes[l+1] x sizes[l].
// Includes the restart of the hidden layers: the first row whose activation is SIGMOID / RELU / LEAKY
// (any row when the output is CLASSIFICATION) throws the layers built so far away, their draws spent,
// and starts over WITHOUT resetting prevLayerSize (:196,213-222), so after a restart at row i >= 1
// the first hidden layer is sampled with fan-in = size of hidden layer i-1: its scale is that fan-in's
// and, if it is larger than the feature count, the surplus edges exist but are never visited.  A
// stale fan-in SMALLER than the feature count leaves input columns without an edge in the reference;
// that network is not modelled here: false, with a message.
bool sampleInitialWeights(const NNInfo* skeleton, int nFeat, int nOut, std::vector<std::vector<float> >& W, std::string* err);

}  // namespace glades
#endif

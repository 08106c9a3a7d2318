// Stand-in for the reference engine's own headers, for one purpose: to compile the binding headers
// under docs/reference_patch/include/hip/ without the engine (which needs OpenCV, yaml-cpp and more).
// Declarations only -- the class, member and method NAMES the bindings touch, as the reference
// declares them (include/Layer.h:45-148, MaxPoolLayer.h, UpsampleLayer.h, ShortcutLayer.h,
// RouteLayer.h, BatchNormLayer.h, ConvLayer.h, YoloLayer.h, Detection.h, PxTensor.h:440-575), with
// Device::HIP beside Device::CUDA.  Nothing here has a body: a binding that compiles against it
// names only things the engine has, with the argument types the engine has.
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <vector>

namespace cv {
struct Rect2f { float x, y, width, height; };
}

namespace px {

[[noreturn]] void throwError(const char* format, ...);
#define PX_ERROR_THROW(...) ::px::throwError(__VA_ARGS__)

enum class Device { CPU, CUDA, HIP };

template<typename T>
class PxCpuVectorT : public std::vector<T>
{
public:
    using std::vector<T>::vector;
};
using PxCpuVector = PxCpuVectorT<float>;

// PxCudaVectorT with hipMalloc behind it
template<typename T>
class PxHipVectorT
{
public:
    PxHipVectorT();
    explicit PxHipVectorT(std::size_t n, T value = T());
    PxHipVectorT(const T* begin, const T* end);
    T* data() noexcept;
    const T* data() const noexcept;
    std::size_t size() const noexcept;
    bool empty() const noexcept;
    void fill(T value);
    void copy(const PxHipVectorT& rhs);
    void copy(const PxCpuVectorT<T>& rhs);
    void copyHost(const T* host, std::size_t n);
    void copyToHost(T* host, std::size_t n) const;       // the first n elements (cudaMemcpy device to host)
    std::vector<T> asVector() const;
};
using PxHipVector = PxHipVectorT<float>;

enum ActivationType : int { LEAKY = 0, LINEAR, LOGGY, LOGISTIC, MISH, RELU, SOFTPLUS, SWISH, TANH };

template<Device D> class IActivation;
template<Device D> struct Activations { using Ptr = std::shared_ptr<IActivation<D>>; };

struct DarkBox { float x() const; float y() const; float w() const; float h() const; };
struct GroundTruth { DarkBox box; int classId; };
using GroundTruthVec = std::vector<GroundTruth>;

class Detection
{
public:
    Detection(cv::Rect2f box, int batchId, int classIndex, float prob);
};
using Detections = std::vector<Detection>;

template<Device D> class Layer;

// include/Model.h:101-127: per-device state of a model (cuBLAS / cuDNN contexts for Device::CUDA)
template<Device D>
class DeviceExtras
{
};

// The engine keeps the CUDA specialisation right here, under USE_CUDA (include/Model.h:105-127); the lean HIP
// bindings put theirs in the same place.
#ifdef PX_HIP_LEAN_BINDINGS
}   // px
#include "hip_lean/ModelExtras.h"
namespace px {
#endif

template<Device D>
class Model : public DeviceExtras<D>
{
public:
    using V = PxHipVector;
    void update();
    bool gradRescaling() const noexcept;
    float gradThreshold() const noexcept;
    bool gradClipping() const noexcept;
    float gradClipValue() const noexcept;
    int width() const noexcept;
    int height() const noexcept;
    int updateBatch() const noexcept;
    float learningRate() const noexcept;
    float momentum() const noexcept;
    float decay() const noexcept;
    bool adamEnabled() const noexcept;
    float adamBeta1() const noexcept;
    float adamBeta2() const noexcept;
    float adamEpsilon() const noexcept;
    int updateCount() const noexcept;
    std::size_t seen() const noexcept;

private:
    void updateLR();
    std::vector<std::shared_ptr<Layer<D>>> layers_;
    std::size_t optimizerStep_ = 0;
};

template<Device D>
class Layer
{
public:
    using V = typename Model<D>::V;
    using Ptr = std::shared_ptr<Layer<D>>;
    virtual ~Layer() = default;
    virtual void forward(const V& input);
    virtual void backward(const V& input, V* grad);
    virtual void update();
    int batch() const noexcept;
    int channels() const noexcept;
    int height() const noexcept;
    int width() const noexcept;
    int inputs() const noexcept;
    int outChannels() const noexcept;
    int outHeight() const noexcept;
    int outWidth() const noexcept;
    int outputs() const noexcept;
    const V& output() const noexcept;
    V& delta() noexcept;

protected:
    const Model<D>& model() const noexcept;
    bool inferring() const noexcept;
    bool training() const noexcept;
    int classes() const noexcept;
    const GroundTruthVec& groundTruth(std::uint32_t batch) const noexcept;
    virtual void scaleGradients();
    virtual void clipGradients();
    virtual void clipDelta();
    void scaleTensor(V& tensor);
    bool gradientRescaling_ = false;
    float gradientThreshold_ = 0.0f;
    bool gradientClipping_ = false;
    float gradientClipValue_ = 0.0f;
    V output_, delta_;
    float cost_ = 0.0f;
};

template<Device D> class MPExtras;
template<Device D>
class MaxPoolLayer : public Layer<D>, public MPExtras<D>
{
public:
    using V = typename Layer<D>::V;
    void forward(const V& input) override;
    void backward(const V& input, V* grad) override;
private:
    void setup();
    int kernel_ = 0, stride_ = 0, padding_ = 0;
};

template<Device D> class UpsampleExtras;
template<Device D>
class UpsampleLayer : public Layer<D>, public UpsampleExtras<D>
{
public:
    using V = typename Layer<D>::V;
    void forward(const V& input) override;
    void backward(const V& input, V* grad) override;
private:
    void setup();
    int stride_;
    float scale_;
};

template<Device D>
class ShortcutLayer : public Layer<D>
{
public:
    using V = typename Layer<D>::V;
    void forward(const V& input) override;
    void backward(const V& input, V* grad) override;
private:
    typename Activations<D>::Ptr activation_;
    typename Layer<D>::Ptr from_;
    float alpha_, beta_;
    V preActivation_;
};

template<Device D>
class RouteLayer : public Layer<D>
{
public:
    using V = typename Layer<D>::V;
    void forward(const V& input) override;
    void backward(const V& input, V* grad) override;
private:
    std::vector<typename Layer<D>::Ptr> layers_;
};

template<Device D> class BNExtras;
template<Device D>
class BatchNormLayer : public Layer<D>, public BNExtras<D>
{
public:
    using V = typename Layer<D>::V;
    void forward(const V& input) override;
    void backward(const V& input, V* grad) override;
    void update() override;
private:
    void setup();
    void scaleGradients() override;
    void clipGradients() override;
    V biases_, biasUpdates_, scales_, scaleUpdates_, mean_, meanDelta_, var_, varDelta_;
    V rollingMean_, rollingVar_, x_, xNorm_;
};

template<Device D> class CVExtras;
template<Device D>
class ConvLayer : public Layer<D>, public CVExtras<D>
{
public:
    using V = typename Layer<D>::V;
    void forward(const V& input) override;
    void backward(const V& input, V* grad) override;
    void update() override;
private:
    void setup();
    void scaleGradients() override;
    void clipGradients() override;
    typename Activations<D>::Ptr activation_;
    V weights_, weightUpdates_, biases_, biasUpdates_;
    V scales_, scaleUpdates_, mean_, meanDelta_, var_, varDelta_;
    V rollingMean_, rollingVar_, x_, xNorm_;
    V column_, preActivation_;
    int dilation_, filters_, kernel_, padding_, stride_, groups_;
    bool batchNorm_;
};

struct Detector
{
    virtual void addDetects(Detections& detects, float threshold) = 0;
    virtual void addDetects(Detections& detects, int width, int height, float threshold) = 0;
};

template<Device D> class YoloExtras;
template<Device D>
class YoloLayer : public Layer<D>, public Detector, public YoloExtras<D>
{
public:
    using V = typename Layer<D>::V;
    void forward(const V& input) override;
    void backward(const V& input, V* grad) override;
    void addDetects(Detections& detections, float threshold) override;
    void addDetects(Detections& detections, int width, int height, float threshold) override;
private:
    void setup();
    void uploadTruths();        // added by include/hip/YoloLayer.h
    void collectCost();         // added by include/hip/YoloLayer.h
    void resetStats();
    void writeStats();
    std::vector<int> mask_, anchors_;
    int numAnchors_, numMasks_;
    float ignoreThresh_, truthThresh_;
    float coordScale_, objectScale_, noObjectScale_, classScale_;
    float avgIoU_ = 0.0f, recall_ = 0.0f, recall75_ = 0.0f, avgCat_ = 0.0f, avgObj_ = 0.0f, avgAnyObj_ = 0.0f;
    float boxCost_ = 0.0f, objectCost_ = 0.0f, noObjectCost_ = 0.0f, classCost_ = 0.0f;
    int count_ = 0, classCount_ = 0, logInterval_ = 0;
};

template<Device D>
class Adam
{
public:
    using V = typename Model<D>::V;
    Adam(int batch, int t, float lr, float beta1, float beta2, float epsilon, float decay);
    void update(V& w, V& d, V& m, V& v, bool applyDecay);
private:
    int batch_, t_;
    float lr_, beta1_, beta2_, epsilon_, decay_;
};

}   // px

// The layers whose device work is the MI355X non-convolution kernels: conv epilogue (batch norm /
// bias + activation), batch norm, max-pool, upsample, shortcut, route and the YOLO head.
// Each class keeps the reference layer's properties, shape rules and error checks and issues the
// fused C-ABI calls where the reference issues several library calls and copies.
#pragma once

#include <cstring>
#include <functional>

#include "Adam.h"
#include "ParameterSet.h"

namespace px::hip {

// reference: include/ActivationTypes.h:19-30 and the name table in src/Activation.cpp
inline int activationFromName(const std::string& name)
{
    static const std::map<std::string, int> table = {
            { "leaky", PXH_LEAKY }, { "linear", PXH_LINEAR }, { "loggy", PXH_LOGGY },
            { "logistic", PXH_LOGISTIC }, { "mish", PXH_MISH }, { "relu", PXH_RELU },
            { "softplus", PXH_SOFTPLUS }, { "swish", PXH_SWISH }, { "tanh", PXH_TANH } };
    auto it = table.find(name);
    PX_CHECK(it != table.end(), "unknown activation \"" + name + "\"");
    return it->second;
}

// ---------------------------------------------------------------- conv epilogue
// Everything a ConvLayer does after its GEMM and before its weight gradients
// (reference: include/cuda/ConvLayer.h:284-307 forward, 315-338 backward, 388-413 update).
// The convolution itself is delegated: `convolve` writes the raw conv result for an input, and
// `convolveBackward` turns dL/d(conv result) into weight updates and dL/d(input).  Without them
// the layer treats its input as the conv result (the form the kernels are measured in).
class ConvLayer : public Layer
{
public:
    using Convolve = std::function<void(const V& input, V& result)>;
    using ConvolveBackward = std::function<void(const V& input, const V& delta, V* grad)>;

    ConvLayer(Context& context, const Properties& props) : Layer(context, props)
    {
        activation_ = activationFromName(props.get<std::string>("activation", "logistic"));
        batchNorm_ = props.get<bool>("batch_normalize", false);
        filters_ = props.get<int>("filters", channels());
        // shape of the conv RESULT; the delegated convolution owns kernel / stride / pad
        const int oh = props.get<int>("out_height", height());
        const int ow = props.get<int>("out_width", width());
        setOutput(filters_, oh, ow);
        if (training()) {
            context.reserveWorkspace(pxh_bn_workspace_bytes(batch(), filters_, oh * ow));
            context.reserveWorkspace(pxh_bn_clipped_workspace_bytes(batch(), filters_, oh * ow));
        }

        // The weights live here so that update() and the optimizer sidecar cover the whole layer;
        // their values and gradients are the delegated convolution's business ("weights": count).
        const auto nweights = static_cast<std::size_t>(props.get<int>("weights", 0));
        if (nweights) {
            weights_ = V(nweights, 0.0f);
            if (training()) {
                weightUpdates_ = V(nweights, 0.0f);
                weightM_ = V(nweights, 0.0f);
                weightV_ = V(nweights, 0.0f);
            }
        }
        const auto f = static_cast<std::size_t>(filters_);
        biases_ = V(f, 0.0f);
        if (batchNorm_) {
            scales_ = V(f, 1.0f);
            rollingMean_ = V(f, 0.0f);
            rollingVar_ = V(f, 0.0f);
            folded_ = DeviceVector<float>(pxh_bn_folded_bytes(filters_) / sizeof(float));
        }
        if (training()) {
            biasUpdates_ = V(f, 0.0f);
            biasM_ = V(f, 0.0f);
            biasV_ = V(f, 0.0f);
            if (batchNorm_) {
                mean_ = V(f, 0.0f);
                var_ = V(f, 0.0f);
                scaleUpdates_ = V(f, 0.0f);
                scaleM_ = V(f, 0.0f);
                scaleV_ = V(f, 0.0f);
            }
        }
    }

    // The ShortcutLayer behind this layer, when nothing else reads this layer's output and the shortcut
    // is linear over tensors of one shape (every residual block of the shipped YOLOv3 graphs): its sum
    // rides on this layer's epilogue (ShortcutLayer::rideOn).  Forward, this layer writes the SHORTCUT's
    // output (its own is never materialised); backward, it works on the shortcut's delta as its own
    // (alpha = 1: the two hold the same values).
    struct Rider {
        V* output = nullptr;
        V* delta = nullptr;
        const V* from = nullptr;
        float alpha = 1.0f, beta = 1.0f;
    };
    void carry(const Rider& rider)
    {
        PX_CHECK(batchNorm_, "a shortcut rides on a batch-normalised convolution only");
        PX_CHECK(rider.output && rider.from && rider.output->size() == output_.size() &&
                 rider.from->size() == output_.size(), "ConvLayer: the shortcut's tensors do not match the layer's");
        PX_CHECK(!training() || (rider.delta && rider.alpha == 1.0f),
                 "ConvLayer: in training a shortcut rides only with alpha = 1 (the layer takes the shortcut's delta)");
        rider_ = rider;
        setFirstConsumerOverwrites(true);       // this layer's own delta is not used: nothing to clear
    }
    bool carriesShortcut() const noexcept { return rider_.output != nullptr; }

    // The 2 x 2, stride 2 MaxPoolLayer behind this layer, at inference (MaxPoolLayer::rideOn): the epilogue
    // writes the pool's output in its own pass (pxh_bn_folded_act_maxpool_forward).  `keepOutput`: something
    // else reads this layer's output too (a route), so it is written as well; else it is never formed.
    void carryPool(V* pooled, bool keepOutput)
    {
        PX_CHECK(!training() && batchNorm_, "a max-pool rides on a batch-normalised convolution at inference only");
        PX_CHECK(outHeight() % 2 == 0 && outWidth() % 2 == 0, "a max-pool rides only where its windows tile the plane");
        PX_CHECK(pooled && pooled->size() * 4 == output_.size(), "ConvLayer: the pool's output does not match the layer's");
        pooled_ = pooled;
        keepOutput_ = keepOutput;
    }
    bool carriesPool() const noexcept { return pooled_ != nullptr; }

    void setConvolution(Convolve fwd, ConvolveBackward bwd)
    {
        convolve_ = std::move(fwd);
        convolveBackward_ = std::move(bwd);
        result_ = V(output_.size());
    }

    // Parameter loading (reference: ConvLayer<D>::copyBiases etc., include/ConvLayer.h:48-54).
    void copyBiases(const std::vector<float>& b) { load(biases_, b); foldedValid_ = false; }
    void copyScales(const std::vector<float>& s) { load(scales_, s); foldedValid_ = false; }
    void copyRollingMean(const std::vector<float>& m) { load(rollingMean_, m); foldedValid_ = false; }
    void copyRollingVariance(const std::vector<float>& v) { load(rollingVar_, v); foldedValid_ = false; }

    void forward(const V& input) override
    {
        Layer::forward(input);
        const float* x = input.data();
        if (convolve_) {
            convolve_(input, result_);
            x = result_.data();
        } else {
            PX_CHECK(input.size() == output_.size(), "ConvLayer: input is not a conv result of the output shape");
        }
        x_ = x;
        const int spatial = outHeight() * outWidth();
        if (rider_.output) {
            if (training()) {
                PX_HIP_CHECK(pxh_bn_train_act_shortcut_forward(x, rider_.output->data(), nullptr, nullptr, nullptr,
                                                               mean_.data(), var_.data(), rollingMean_.data(),
                                                               rollingVar_.data(), scales_.data(), biases_.data(),
                                                               rider_.from->data(), rider_.alpha, rider_.beta, batch(),
                                                               filters_, spatial, activation_, context().workspace(),
                                                               context().workspaceBytes(), stream()));
                foldedValid_ = false;
            } else {
                fold();
                PX_HIP_CHECK(pxh_bn_folded_act_shortcut_forward(x, rider_.output->data(), nullptr, folded_.data(),
                                                                rider_.from->data(), rider_.alpha, rider_.beta, batch(),
                                                                filters_, spatial, activation_, stream()));
            }
            return;
        }
        if (pooled_) {
            fold();
            PX_HIP_CHECK(pxh_bn_folded_act_maxpool_forward(x, keepOutput_ ? output_.data() : nullptr, pooled_->data(),
                                                           folded_.data(), batch(), filters_, outHeight(), outWidth(),
                                                           activation_, stream()));
            return;
        }
        if (!batchNorm_) {
            PX_HIP_CHECK(pxh_bias_act_forward(x, output_.data(), nullptr, biases_.data(), batch(), filters_, spatial,
                                              activation_, stream()));
        } else if (training()) {
            PX_HIP_CHECK(pxh_bn_train_act_forward(x, output_.data(), nullptr, nullptr, nullptr, mean_.data(),
                                                  var_.data(), rollingMean_.data(), rollingVar_.data(),
                                                  scales_.data(), biases_.data(), batch(), filters_, spatial,
                                                  activation_, context().workspace(), context().workspaceBytes(),
                                                  stream()));
            foldedValid_ = false;       // the rolling statistics moved
        } else {
            fold();
            PX_HIP_CHECK(pxh_bn_folded_act_forward(x, output_.data(), nullptr, folded_.data(), batch(), filters_,
                                                   spatial, activation_, stream()));
        }
    }

    // Needs the conv result of the matching forward to be unchanged (it is re-read instead of
    // keeping saved copies of it, of x_hat and of the pre-activation).
    //
    // Layer::backward's rescale + clip of delta_ rides on the first pass of the epilogue's backward (one
    // call, the delta is not read for its norm alone) -- unless the kernel that wrote delta_ last left its
    // norm behind, in which case the helpers need no read of it anyway and run as in every other layer.
    void backward(const V& input, V* grad) override
    {
        PX_CHECK(training() && x_ != nullptr, "ConvLayer: backward without a training forward");
        const float threshold = rescaleThreshold(), clip = clipValue();
        // with a shortcut riding on the layer, its delta is the shortcut's (already through the shortcut's own
        // helpers, which the layer's repeat without changing a value, as they would on the copy)
        V& d = rider_.delta ? *rider_.delta : delta_;
        const bool fused = (threshold > 0.0f || clip > 0.0f) && (rider_.delta || !context().hasNormGroups(d.data()));
        if (!fused && !rider_.delta) Layer::backward(input, grad);
        const int spatial = outHeight() * outWidth();
        if (batchNorm_) {
            if (fused)
                PX_HIP_CHECK(pxh_bn_act_backward_clipped(d.data(), x_, nullptr, mean_.data(), var_.data(),
                                                         scales_.data(), biases_.data(), scaleUpdates_.data(),
                                                         biasUpdates_.data(), nullptr, nullptr, batch(), filters_,
                                                         spatial, activation_, threshold, clip, nullptr,
                                                         context().workspace(), context().workspaceBytes(), stream()));
            else
                PX_HIP_CHECK(pxh_bn_act_backward(d.data(), x_, nullptr, mean_.data(), var_.data(),
                                                 scales_.data(), biases_.data(), scaleUpdates_.data(),
                                                 biasUpdates_.data(), nullptr, nullptr, batch(), filters_, spatial,
                                                 activation_, context().workspace(), context().workspaceBytes(),
                                                 stream()));
        } else {
            // pre-activation = x + bias is not kept either; the linear head convs need none
            preActivation(spatial);
            const float* pre = pre_.empty() ? nullptr : pre_.data();
            if (fused)
                PX_HIP_CHECK(pxh_bias_act_backward_clipped(d.data(), pre, biasUpdates_.data(), batch(), filters_,
                                                           spatial, activation_, threshold, clip, nullptr,
                                                           context().workspace(), context().workspaceBytes(),
                                                           stream()));
            else
                PX_HIP_CHECK(pxh_bias_act_backward(d.data(), pre, biasUpdates_.data(), batch(), filters_, spatial,
                                                   activation_, context().workspace(), context().workspaceBytes(),
                                                   stream()));
        }
        if (convolveBackward_) {
            convolveBackward_(input, d, grad);
        } else if (grad) {
            PX_HIP_CHECK(pxh_axpy(d.size(), 1.0f, d.data(), grad->data(), stream()));
        }
    }

    // Adam or SGD with momentum on the biases and scales, neither with weight decay (the
    // delegated convolution updates its own weights the same way, with decay: reference
    // include/cuda/ConvLayer.h:362-413).
    void update() override
    {
        const auto& c = context();
        // the reference's scaleGradients / clipGradients hooks (include/ConvLayer.h:323-340)
        Layer::update();
        rescaleAndClip(weightUpdates_);
        rescaleAndClip(biasUpdates_);
        rescaleAndClip(scaleUpdates_);
        if (c.adamEnabled) {
            const Adam adam(c);
            if (!weights_.empty()) adam.update(weights_, weightUpdates_, weightM_, weightV_, true);
            adam.update(biases_, biasUpdates_, biasM_, biasV_, false);
            if (batchNorm_) adam.update(scales_, scaleUpdates_, scaleM_, scaleV_, false);
        } else {
            if (!weights_.empty())
                PX_HIP_CHECK(pxh_sgd_update(weights_.size(), weights_.data(), weightUpdates_.data(), c.updateBatch,
                                            c.learningRate, c.momentum, c.decay, 1, stream()));
            PX_HIP_CHECK(pxh_sgd_update(biases_.size(), biases_.data(), biasUpdates_.data(), c.updateBatch,
                                        c.learningRate, c.momentum, c.decay, 0, stream()));
            if (batchNorm_)
                PX_HIP_CHECK(pxh_sgd_update(scales_.size(), scales_.data(), scaleUpdates_.data(), c.updateBatch,
                                            c.learningRate, c.momentum, c.decay, 0, stream()));
        }
        foldedValid_ = false;
    }

    // the same tensors, hooks and optimiser as update(), for a model that steps all layers together
    void collectParameters(ParameterSet& set) override
    {
        if (!training()) return;
        Layer::collectParameters(set);
        const ParameterSet::Hooks hooks{ rescaleThreshold(), clipValue() };
        if (context().adamEnabled) {
            set.addAdam(weights_, weightUpdates_, weightM_, weightV_, true, hooks);
            set.addAdam(biases_, biasUpdates_, biasM_, biasV_, false, hooks);
            if (batchNorm_) set.addAdam(scales_, scaleUpdates_, scaleM_, scaleV_, false, hooks);
        } else {
            set.addSgd(weights_, weightUpdates_, true, hooks);
            set.addSgd(biases_, biasUpdates_, false, hooks);
            if (batchNorm_) set.addSgd(scales_, scaleUpdates_, false, hooks);
        }
    }

    void parametersUpdated() override { foldedValid_ = false; }

    // biases [, scales, rolling mean, rolling variance], weights as raw fp32 (reference:
    // include/ConvLayer.h:132-171)
    std::streamoff loadWeights(std::istream& is) override
    {
        const auto start = is.tellg();
        for (V* t: weightFileOrder()) {
            std::vector<float> host(t->size());
            is.read(reinterpret_cast<char*>(host.data()), static_cast<std::streamsize>(host.size() * sizeof(float)));
            PX_CHECK(is.good() || host.empty(), "Could not read weights");
            t->copyHost(host, stream());
        }
        foldedValid_ = false;
        return is.tellg() - start;
    }

    std::streamoff saveWeights(std::ostream& os) override
    {
        const auto start = os.tellp();
        for (const V* t: weightFileOrder()) {
            const std::vector<float> host = t->asVector(stream());
            os.write(reinterpret_cast<const char*>(host.data()), static_cast<std::streamsize>(host.size() * sizeof(float)));
        }
        PX_CHECK(os.good(), "Could not write weights");
        return os.tellp() - start;
    }

    // m, v, bias_m, bias_v, scale_m, scale_v as raw fp32 (reference: include/cuda/ConvLayer.h:228-264)
    std::streamoff saveOptimizer(std::ostream& os) override
    {
        const auto start = os.tellp();
        for (const V* t: { &weightM_, &weightV_, &biasM_, &biasV_, &scaleM_, &scaleV_ }) {
            const std::vector<float> host = t->asVector(stream());
            os.write(reinterpret_cast<const char*>(host.data()), static_cast<std::streamsize>(host.size() * sizeof(float)));
        }
        PX_CHECK(os.good(), "Could not write convolution optimizer state");
        return os.tellp() - start;
    }

    std::streamoff loadOptimizer(std::istream& is) override
    {
        const auto start = is.tellg();
        for (V* t: { &weightM_, &weightV_, &biasM_, &biasV_, &scaleM_, &scaleV_ }) {
            std::vector<float> host(t->size());
            is.read(reinterpret_cast<char*>(host.data()), static_cast<std::streamsize>(host.size() * sizeof(float)));
            PX_CHECK(is.good() || host.empty(), "Could not read convolution optimizer state");
            t->copyHost(host, stream());
        }
        return is.tellg() - start;
    }

    // Clears the accumulated parameter updates and the optimizer moments (a fresh start of training).
    void zeroUpdates()
    {
        for (V* t: { &weightUpdates_, &biasUpdates_, &scaleUpdates_, &weightM_, &weightV_, &biasM_, &biasV_, &scaleM_,
                     &scaleV_ })
            if (!t->empty()) t->fill(0.0f, stream());
    }

    V& weights() noexcept { return weights_; }
    V& weightUpdates() noexcept { return weightUpdates_; }
    const V& biases() const noexcept { return biases_; }
    const V& scales() const noexcept { return scales_; }
    const V& rollingMean() const noexcept { return rollingMean_; }
    const V& rollingVariance() const noexcept { return rollingVar_; }
    const V& mean() const noexcept { return mean_; }
    const V& variance() const noexcept { return var_; }
    const V& biasUpdates() const noexcept { return biasUpdates_; }
    const V& scaleUpdates() const noexcept { return scaleUpdates_; }

private:
    std::vector<V*> weightFileOrder()
    {
        if (batchNorm_) return { &biases_, &scales_, &rollingMean_, &rollingVar_, &weights_ };
        return { &biases_, &weights_ };
    }

    void load(V& dst, const std::vector<float>& src)
    {
        PX_CHECK(dst.size() == src.size(), "ConvLayer: parameter vector of the wrong size");
        dst.copyHost(src, stream());
    }

    // x + bias for a non-linear layer without batch norm (the gradient needs it)
    void preActivation(int spatial)
    {
        if (activation_ == PXH_LINEAR) return;
        if (pre_.empty()) pre_ = V(output_.size());
        PX_HIP_CHECK(pxh_bias_act_forward(x_, pre_.data(), nullptr, biases_.data(), batch(), filters_, spatial,
                                          PXH_LINEAR, stream()));
    }

    // the inference constants, folded again only after the parameters changed
    void fold()
    {
        if (foldedValid_) return;
        PX_HIP_CHECK(pxh_bn_fold(rollingMean_.data(), rollingVar_.data(), scales_.data(), biases_.data(), filters_,
                                 folded_.data(), stream()));
        foldedValid_ = true;
    }

    int activation_ = PXH_LOGISTIC, filters_ = 1;
    bool batchNorm_ = false, foldedValid_ = false;
    Rider rider_;
    V* pooled_ = nullptr;           // the riding pool's output
    bool keepOutput_ = false;
    const float* x_ = nullptr;      // conv result of the last forward (borrowed)
    V biases_, scales_, rollingMean_, rollingVar_, mean_, var_, folded_;
    V biasUpdates_, scaleUpdates_, biasM_, biasV_, scaleM_, scaleV_;
    V weights_, weightUpdates_, weightM_, weightV_;
    V result_, pre_;
    Convolve convolve_;
    ConvolveBackward convolveBackward_;
};

// ---------------------------------------------------------------- stand-alone batch norm
// reference: include/BatchNormLayer.h:39-183, include/cuda/BatchNormLayer.h:59-137.  The layer's
// input is read again in backward (the reference keeps copies x_ and xNorm_ of it instead), so it
// must be unchanged between the two calls, as it is when a model drives the layers in order.
class BatchNormLayer : public Layer
{
public:
    BatchNormLayer(Context& context, const Properties& props) : Layer(context, props)
    {
        setOutput(channels(), height(), width());
        if (training()) context.reserveWorkspace(pxh_bn_workspace_bytes(batch(), channels(), height() * width()));
        const auto c = static_cast<std::size_t>(channels());
        biases_ = V(c, 0.0f);
        scales_ = V(c, 1.0f);
        rollingMean_ = V(c, 0.0f);
        rollingVar_ = V(c, 0.0f);
        folded_ = V(pxh_bn_folded_bytes(channels()) / sizeof(float));
        if (training()) {
            mean_ = V(c, 0.0f);
            var_ = V(c, 0.0f);
            biasUpdates_ = V(c, 0.0f);
            scaleUpdates_ = V(c, 0.0f);
        }
    }

    void forward(const V& input) override
    {
        Layer::forward(input);
        checkInput(input, "BatchNormLayer");
        const int spatial = outHeight() * outWidth();
        if (training()) {
            PX_HIP_CHECK(pxh_bn_train_act_forward(input.data(), output_.data(), nullptr, nullptr, nullptr, mean_.data(),
                                                  var_.data(), rollingMean_.data(), rollingVar_.data(),
                                                  scales_.data(), biases_.data(), batch(), channels(), spatial,
                                                  PXH_LINEAR, context().workspace(), context().workspaceBytes(),
                                                  stream()));
            foldedValid_ = false;
            return;
        }
        if (!foldedValid_) {
            PX_HIP_CHECK(pxh_bn_fold(rollingMean_.data(), rollingVar_.data(), scales_.data(), biases_.data(),
                                     channels(), folded_.data(), stream()));
            foldedValid_ = true;
        }
        PX_HIP_CHECK(pxh_bn_folded_act_forward(input.data(), output_.data(), nullptr, folded_.data(), batch(),
                                               channels(), spatial, PXH_LINEAR, stream()));
    }

    void backward(const V& input, V* grad) override
    {
        Layer::backward(input, grad);
        PX_CHECK(training(), "BatchNormLayer: backward needs a training context");
        checkInput(input, "BatchNormLayer");
        PX_HIP_CHECK(pxh_bn_act_backward(delta_.data(), input.data(), nullptr, mean_.data(), var_.data(),
                                         scales_.data(), biases_.data(), scaleUpdates_.data(), biasUpdates_.data(),
                                         nullptr, nullptr, batch(), channels(), outHeight() * outWidth(), PXH_LINEAR,
                                         context().workspace(), context().workspaceBytes(), stream()));
        if (grad) PX_HIP_CHECK(pxh_axpy(delta_.size(), 1.0f, delta_.data(), grad->data(), stream()));
    }

    // plain momentum steps on biases and scales, no weight decay (include/BatchNormLayer.h:166-181)
    void update() override
    {
        const auto& c = context();
        // scaleGradients / clipGradients (include/BatchNormLayer.h:160-176)
        Layer::update();
        rescaleAndClip(biasUpdates_);
        rescaleAndClip(scaleUpdates_);
        PX_HIP_CHECK(pxh_sgd_update(biases_.size(), biases_.data(), biasUpdates_.data(), c.updateBatch, c.learningRate,
                                    c.momentum, 0.0f, 0, stream()));
        PX_HIP_CHECK(pxh_sgd_update(scales_.size(), scales_.data(), scaleUpdates_.data(), c.updateBatch,
                                    c.learningRate, c.momentum, 0.0f, 0, stream()));
        foldedValid_ = false;
    }

    void collectParameters(ParameterSet& set) override
    {
        if (!training()) return;
        Layer::collectParameters(set);
        const ParameterSet::Hooks hooks{ rescaleThreshold(), clipValue() };
        set.addSgd(biases_, biasUpdates_, false, hooks);
        set.addSgd(scales_, scaleUpdates_, false, hooks);
    }

    void parametersUpdated() override { foldedValid_ = false; }

    // biases, scales, rolling mean, rolling variance as raw fp32 (include/BatchNormLayer.h:72-113)
    std::streamoff loadWeights(std::istream& is) override
    {
        const auto start = is.tellg();
        for (V* t: { &biases_, &scales_, &rollingMean_, &rollingVar_ }) {
            std::vector<float> host(t->size());
            is.read(reinterpret_cast<char*>(host.data()), static_cast<std::streamsize>(host.size() * sizeof(float)));
            PX_CHECK(is.good(), "Could not read batch normalize parameters");
            t->copyHost(host, stream());
        }
        foldedValid_ = false;
        return is.tellg() - start;
    }

    std::streamoff saveWeights(std::ostream& os) override
    {
        const auto start = os.tellp();
        for (const V* t: { &biases_, &scales_, &rollingMean_, &rollingVar_ }) {
            const std::vector<float> host = t->asVector(stream());
            os.write(reinterpret_cast<const char*>(host.data()), static_cast<std::streamsize>(host.size() * sizeof(float)));
        }
        PX_CHECK(os.good(), "Could not write batch normalize parameters");
        return os.tellp() - start;
    }

    const V& biases() const noexcept { return biases_; }
    const V& scales() const noexcept { return scales_; }
    const V& rollingMean() const noexcept { return rollingMean_; }
    const V& rollingVariance() const noexcept { return rollingVar_; }
    const V& mean() const noexcept { return mean_; }
    const V& variance() const noexcept { return var_; }
    const V& biasUpdates() const noexcept { return biasUpdates_; }
    const V& scaleUpdates() const noexcept { return scaleUpdates_; }

private:
    bool foldedValid_ = false;
    V biases_, scales_, rollingMean_, rollingVar_, mean_, var_, folded_, biasUpdates_, scaleUpdates_;
};

// ---------------------------------------------------------------- max-pool
// reference: include/MaxPoolLayer.h:50-158, include/cuda/MaxPoolLayer.h
class MaxPoolLayer : public Layer
{
public:
    MaxPoolLayer(Context& context, const Properties& props) : Layer(context, props)
    {
        kernel_ = props.get<int>("kernel", 1);
        stride_ = props.get<int>("stride", 1);
        padding_ = props.get<int>("padding", std::max(0, kernel_ - 1));
        PX_CHECK(kernel_ > 0, "maxpool kernel must be positive");
        PX_CHECK(stride_ > 0, "maxpool stride must be positive");
        PX_CHECK(padding_ >= 0, "maxpool padding cannot be negative");
        const int oh = (height() + padding_ - kernel_) / stride_ + 1;
        const int ow = (width() + padding_ - kernel_) / stride_ + 1;
        PX_CHECK(oh > 0 && ow > 0, "maxpool output dimensions must be positive");
        setOutput(channels(), oh, ow);
        if (training()) indexes_ = IntVector(output_.size());
    }

    // At inference this pool rides on the epilogue of the convolution in front of it
    // (pxh_bn_folded_act_maxpool_forward): for whoever builds the network, for the 2 x 2 window at stride 2
    // over planes of even size.  `convOutputIsRead`: something else reads the convolution's output as well.
    // forward() then finds its output written (and keeps no indexes: nothing reads them at inference).
    void rideOn(ConvLayer& conv, bool convOutputIsRead)
    {
        PX_CHECK(kernel_ == 2 && stride_ == 2 && padding_ <= 1, "only the 2 x 2 pool at stride 2 rides");
        PX_CHECK(conv.batch() == batch() && conv.outChannels() == channels() && conv.outHeight() == height() &&
                 conv.outWidth() == width(), "maxpool: the convolution in front has another shape");
        conv.carryPool(&output_, convOutputIsRead);
        riding_ = true;
    }

    void forward(const V& input) override
    {
        Layer::forward(input);
        if (riding_) return;        // the convolution in front has written output_
        checkInput(input, "MaxPoolLayer");
        if (indexes_.empty()) indexes_ = IntVector(output_.size());
        PX_HIP_CHECK(pxh_maxpool_forward(input.data(), output_.data(), indexes_.data(), batch(), channels(),
                                         height(), width(), outHeight(), outWidth(), kernel_, stride_, padding_,
                                         stream()));
    }

    void backward(const V& input, V* grad) override
    {
        Layer::backward(input, grad);
        if (grad == nullptr) return;
        PX_HIP_CHECK(pxh_maxpool_backward(delta_.data(), indexes_.data(), grad->data(), batch(), channels(),
                                          height(), width(), outHeight(), outWidth(), kernel_, stride_, padding_,
                                          stream()));
    }

    const IntVector& indexes() const noexcept { return indexes_; }

private:
    int kernel_ = 1, stride_ = 1, padding_ = 0;
    bool riding_ = false;
    IntVector indexes_;
};

// ---------------------------------------------------------------- upsample
// reference: include/UpsampleLayer.h:48-121, include/cuda/UpsampleLayer.h
class UpsampleLayer : public Layer
{
public:
    UpsampleLayer(Context& context, const Properties& props) : Layer(context, props)
    {
        stride_ = props.get<int>("stride", 2);
        scale_ = props.get<float>("scale", 1.0f);
        PX_CHECK(stride_ > 0, "upsample stride must be positive");
        setOutput(channels(), height() * stride_, width() * stride_);
    }

    void forward(const V& input) override
    {
        Layer::forward(input);
        checkInput(input, "UpsampleLayer");
        if (outSlice_) {
            PX_HIP_CHECK(pxh_upsample_strided(input.data(), width(), height(), channels(), batch(), stride_, 1, scale_,
                                              nullptr, outSlice_, imageStride_, stream()));
            return;
        }
        PX_HIP_CHECK(pxh_upsample(input.data(), width(), height(), channels(), batch(), stride_, 1, scale_, nullptr,
                                  output_.data(), stream()));
    }

    void backward(const V& input, V* grad) override
    {
        Layer::backward(input, grad);
        if (grad == nullptr) return;
        if (outSlice_) {
            PX_HIP_CHECK(pxh_upsample_strided(nullptr, width(), height(), channels(), batch(), stride_, 0, scale_,
                                              grad->data(), deltaSlice_, imageStride_, stream()));
            return;
        }
        PX_HIP_CHECK(pxh_upsample(nullptr, width(), height(), channels(), batch(), stride_, 0, scale_, grad->data(),
                                  delta_.data(), stream()));
    }

    // The route layer that is this layer's only consumer hands over the channel slice of its own
    // buffers where the upsampled tensor belongs (image n at slice + n * imageStride): forward
    // writes there, backward reads the delta there, and this layer's own tensors are released.
    void writeInto(float* outSlice, float* deltaSlice, long long imageStride)
    {
        PX_CHECK(outSlice != nullptr && imageStride >= outputs(), "upsample: bad slice to write into");
        PX_CHECK(!training() || deltaSlice != nullptr, "upsample: a training layer needs the delta slice too");
        outSlice_ = outSlice;
        deltaSlice_ = deltaSlice;
        imageStride_ = imageStride;
        output_ = V();
        delta_ = V();
    }

    bool writesIntoConsumer() const noexcept { return outSlice_ != nullptr; }

private:
    int stride_ = 2;
    float scale_ = 1.0f;
    float* outSlice_ = nullptr;
    float* deltaSlice_ = nullptr;
    long long imageStride_ = 0;
};

// ---------------------------------------------------------------- shortcut
// reference: include/ShortcutLayer.h:45-141, include/cuda/ShortcutLayer.h:23-55
class ShortcutLayer : public Layer
{
public:
    ShortcutLayer(Context& context, const Properties& props, Layer::Ptr from) : Layer(context, props),
                                                                                 from_(std::move(from))
    {
        PX_CHECK(from_ != nullptr, "shortcut needs its \"from\" layer");
        activation_ = activationFromName(props.get<std::string>("activation", "linear"));
        alpha_ = props.get<float>("alpha", 1.0f);
        beta_ = props.get<float>("beta", 1.0f);
        PX_CHECK(from_->batch() == batch(), "shortcut: batch sizes differ");
        setOutput(channels(), height(), width());
        sameShape_ = from_->outChannels() == outChannels() && from_->outHeight() == outHeight() &&
                     from_->outWidth() == outWidth();
        if (training() && (activation_ != PXH_LINEAR || !sameShape_)) preActivation_ = V(output_.size());
        // "first_writer": in the backward pass this shortcut runs before every other reader of the
        // layer in front of it and of its `from` layer (true of a residual block: the block's first
        // conv reads `from` too, but comes earlier in the network).  It then overwrites both deltas
        // instead of adding to them, and neither needs clearing: the `from` layer is told here, the
        // layer in front by whoever builds the network (setFirstConsumerOverwrites).
        firstWriter_ = training() && sameShape_ && props.get<bool>("first_writer", false);
        if (firstWriter_) from_->setFirstConsumerOverwrites(true);
        // "leaves_norm": this shortcut is the LAST to write the delta of the layer in front of it before
        // that layer's backward (true when nothing else reads that layer's output, as in a residual
        // block).  Its backward then leaves the norm and peak of that delta behind, and the gradient
        // rescale + clip that opens that layer's backward does not read the tensor for them.
        leavesNorm_ = training() && sameShape_ && props.get<bool>("leaves_norm", false);
        if (leavesNorm_) normGroups_ = normGroupsFor(output_.size());
    }

    // This shortcut's sum rides on the epilogue of the convolution in front of it
    // (pxh_bn_train_act_shortcut_forward): for whoever builds the network, when nothing but this shortcut
    // reads that convolution's output.  forward() then finds its output written, and backward() leaves the
    // convolution's delta alone: the convolution works on this layer's.
    void rideOn(ConvLayer& conv)
    {
        PX_CHECK(sameShape_ && activation_ == PXH_LINEAR, "a shortcut rides only with a linear activation over one shape");
        PX_CHECK(!leavesNorm_, "a riding shortcut writes no delta of the layer in front: nothing to leave a norm of");
        PX_CHECK(conv.batch() == batch() && conv.outChannels() == outChannels() && conv.outHeight() == outHeight() &&
                 conv.outWidth() == outWidth(), "shortcut: the convolution in front has another shape");
        conv.carry(ConvLayer::Rider{ &output_, training() ? &delta_ : nullptr, &from_->output(), alpha_, beta_ });
        riding_ = true;
    }

    void forward(const V& input) override
    {
        Layer::forward(input);
        if (riding_) return;        // the convolution in front has written output_
        checkInput(input, "ShortcutLayer");
        float* pre = preActivation_.empty() ? nullptr : preActivation_.data();
        if (sameShape_) {
            PX_HIP_CHECK(pxh_shortcut_forward(input.data(), from_->output().data(), output_.data(), pre,
                                              output_.size(), alpha_, beta_, activation_, stream()));
            return;
        }
        // differing shapes: the index-mapped blend of the reference, then the activation
        output_.copy(input, stream());
        PX_HIP_CHECK(pxh_shortcut(batch(), outWidth(), outHeight(), outChannels(), from_->output().data(),
                                  from_->outWidth(), from_->outHeight(), from_->outChannels(), alpha_, beta_,
                                  output_.data(), stream()));
        if (pre) preActivation_.copy(output_, stream());
        PX_HIP_CHECK(pxh_activate(activation_, output_.data(), output_.size(), stream()));
    }

    void backward(const V& input, V* grad) override
    {
        const float* pre = preActivation_.empty() ? nullptr : preActivation_.data();
        // A first writer's targets are plain functions of its delta: Layer::backward's rescale + clip and the
        // layer's own backward run as one call that reads the delta once when nothing has to change
        // (pxh_shortcut_backward_clipped; the values of the two calls to the bit).  Not where the norm of the
        // delta is already known from its writer, nor where this layer has to leave one behind.
        const float threshold = rescaleThreshold(), clip = clipValue();
        const bool fused = firstWriter_ && sameShape_ && (threshold > 0.0f || clip > 0.0f) && !leavesNorm_ &&
                           (riding_ || grad != nullptr) && !context().hasNormGroups(delta_.data());
        if (fused) {
            context().reserveWorkspace(pxh_rescale_workspace_bytes());
            PX_HIP_CHECK(pxh_shortcut_backward_clipped(delta_.data(), pre, from_->delta().data(),
                                                       riding_ ? nullptr : grad->data(), delta_.size(), alpha_, beta_,
                                                       activation_, 1, threshold, clip, nullptr, context().workspace(),
                                                       context().workspaceBytes(), stream()));
            return;
        }
        Layer::backward(input, grad);
        if (riding_) {
            // the `from` layer's share only; the convolution in front takes delta_ itself
            if (firstWriter_)
                PX_HIP_CHECK(pxh_shortcut_backward_first(delta_.data(), nullptr, from_->delta().data(), nullptr,
                                                         delta_.size(), alpha_, beta_, activation_, stream()));
            else
                PX_HIP_CHECK(pxh_shortcut_backward(delta_.data(), nullptr, from_->delta().data(), nullptr, delta_.size(),
                                                   alpha_, beta_, activation_, stream()));
            return;
        }
        if (leavesNorm_ && grad) {
            PX_HIP_CHECK(pxh_shortcut_backward_norm(delta_.data(), pre, from_->delta().data(), grad->data(),
                                                    delta_.size(), alpha_, beta_, activation_, firstWriter_ ? 1 : 0,
                                                    normGroups_.data(), stream()));
            context().noteNormGroups(grad->data(), normGroups_.data());
            return;
        }
        if (firstWriter_) {
            PX_CHECK(grad != nullptr, "a first-writer shortcut needs the delta of the layer in front of it");
            PX_HIP_CHECK(pxh_shortcut_backward_first(delta_.data(), pre, from_->delta().data(), grad->data(),
                                                     delta_.size(), alpha_, beta_, activation_, stream()));
            return;
        }
        if (sameShape_) {
            PX_HIP_CHECK(pxh_shortcut_backward(delta_.data(), pre, from_->delta().data(),
                                               grad ? grad->data() : nullptr, delta_.size(), alpha_, beta_,
                                               activation_, stream()));
            return;
        }
        if (activation_ != PXH_LINEAR)
            PX_HIP_CHECK(pxh_gradient(activation_, pre, delta_.size(), delta_.data(), stream()));
        PX_HIP_CHECK(pxh_shortcut(batch(), from_->outWidth(), from_->outHeight(), from_->outChannels(),
                                  delta_.data(), outWidth(), outHeight(), outChannels(), 1.0f, beta_,
                                  from_->delta().data(), stream()));
        if (grad) PX_HIP_CHECK(pxh_axpy(delta_.size(), alpha_, delta_.data(), grad->data(), stream()));
    }

private:
    Layer::Ptr from_;
    int activation_ = PXH_LINEAR;
    float alpha_ = 1.0f, beta_ = 1.0f;
    bool sameShape_ = true, firstWriter_ = false, leavesNorm_ = false, riding_ = false;
    V preActivation_, normGroups_;
};

// ---------------------------------------------------------------- route
// reference: include/RouteLayer.h:39-137, include/cuda/RouteLayer.h:23-71
class RouteLayer : public Layer
{
public:
    RouteLayer(Context& context, const Properties& props, std::vector<Layer::Ptr> layers)
            : Layer(context, props), layers_(std::move(layers))
    {
        PX_CHECK(!layers_.empty(), "route needs at least one source layer");
        int outChannels = 0;
        const int oh = layers_[0]->outHeight(), ow = layers_[0]->outWidth();
        for (const auto& layer: layers_) {
            PX_CHECK(layer->outHeight() == oh && layer->outWidth() == ow, "route: source layers differ in size");
            PX_CHECK(layer->batch() == batch(), "route: batch sizes differ");
            outChannels += layer->outChannels();
        }
        setOutput(outChannels, oh, ow);
        // "absorb_upsample": an upsample layer among the sources, read by no other layer, writes
        // straight into its channel slice here, which saves its copy in both directions.  The
        // caller vouches for "no other reader"; the reference's graphs (yolov3.yml, yolov3-tiny.yml)
        // meet it: every upsample is followed by the route that reads it.
        absorbed_.assign(layers_.size(), false);
        if (props.get<bool>("absorb_upsample", false)) {
            int offset = 0;
            for (std::size_t i = 0; i < layers_.size(); ++i) {
                if (auto* up = dynamic_cast<UpsampleLayer*>(layers_[i].get())) {
                    up->writeInto(output_.data() + offset, training() ? delta_.data() + offset : nullptr, outputs());
                    absorbed_[i] = true;
                }
                offset += layers_[i]->outputs();
            }
        }
    }

    void forward(const V& input) override
    {
        Layer::forward(input);
        int offset = 0;
        for (std::size_t i = 0; i < layers_.size(); ++i) {
            const auto& layer = layers_[i];
            if (!absorbed_[i])
                PX_HIP_CHECK(pxh_route_forward(layer->output().data(), output_.data(), batch(), layer->outputs(),
                                               outputs(), offset, stream()));
            offset += layer->outputs();
        }
    }

    void backward(const V& input, V* grad) override
    {
        Layer::backward(input, grad);
        int offset = 0;
        for (std::size_t i = 0; i < layers_.size(); ++i) {
            const auto& layer = layers_[i];
            if (!absorbed_[i])
                PX_HIP_CHECK(pxh_route_backward(delta_.data(), layer->delta().data(), batch(), layer->outputs(),
                                                outputs(), offset, stream()));
            offset += layer->outputs();
        }
    }

private:
    std::vector<Layer::Ptr> layers_;
    std::vector<bool> absorbed_;
};

// ---------------------------------------------------------------- detections
// reference: Detection, include/Detection.h:23-40 (the box is left, top, width, height)
struct Detection
{
    float x, y, w, h;
    int batchId;
    int classIndex;
    float prob;
};

using Detections = std::vector<Detection>;

// Detections that stay on the device: the YOLO layers of a pass append their records to one list
// (Model::detections walks the layers the same way, include/Model.h:1078-1109), nms() runs on it in
// place, and only the survivors cross to the host.  A list of at most 512 records (an inference
// pass) is suppressed in a single launch.
class DeviceDetections
{
public:
    explicit DeviceDetections(int capacity) : capacity_(capacity)
    {
        PX_CHECK(capacity > 0, "a detection list needs a positive capacity");
        static_assert(sizeof(pxh_detection) == 8 * sizeof(int), "record layout");
        records_ = IntVector(static_cast<std::size_t>(capacity) * 8);
        spare_ = IntVector(static_cast<std::size_t>(capacity) * 8);
        count_ = IntVector(1, 0);
        spareCount_ = IntVector(1, 0);
        nmsWorkspace_ = FloatVector((pxh_nms_workspace_bytes(capacity) + sizeof(float) - 1) / sizeof(float));
    }

    int capacity() const noexcept { return capacity_; }
    pxh_detection* records() noexcept { return reinterpret_cast<pxh_detection*>(records_.data()); }
    int* count() noexcept { return count_.data(); }

    // Empties the list (ordered on `stream`).
    void clear(hipStream_t stream = nullptr)
    {
        count_.fill(0, stream);
        nextOrder_ = 0;
    }

    // The emission order of the next head's first record, and its advance by that head's pairs of
    // (slot, class).
    unsigned nextOrder() const noexcept { return nextOrder_; }
    void advanceOrder(unsigned pairs) noexcept { nextOrder_ += pairs; }

    // nms, src/Box.cpp:56-147, on the device; the list then holds the survivors by descending
    // probability.  `batch` and `classes` bound the image and class numbers of the records.
    void nms(int batch, int classes, float threshold, hipStream_t stream = nullptr)
    {
        PX_HIP_CHECK(pxh_nms(records(), count_.data(), capacity_, batch, classes, threshold,
                             reinterpret_cast<pxh_detection*>(spare_.data()), spareCount_.data(),
                             nmsWorkspace_.empty() ? nullptr : nmsWorkspace_.data(),
                             nmsWorkspace_.size() * sizeof(float), stream));
        std::swap(records_, spare_);
        std::swap(count_, spareCount_);
    }

    // Blocking: how many records the YOLO layers found.  More than capacity() means the list overflowed
    // and holds whichever records arrived first; the caller then repeats the pass with a larger list.
    int found(hipStream_t stream = nullptr)
    {
        PX_HIP_RUNTIME_CHECK(hipStreamSynchronize(stream));
        return count_.asVector()[0];
    }

    // Blocking copy to the host, in the list's order.  A list that overflowed holds `capacity` records.
    Detections toHost(hipStream_t stream = nullptr)
    {
        PX_HIP_RUNTIME_CHECK(hipStreamSynchronize(stream));
        const int found = std::min(std::max(count_.asVector()[0], 0), capacity_);
        const std::vector<int> raw = records_.asVector();
        Detections out;
        out.reserve(static_cast<std::size_t>(found));
        for (int i = 0; i < found; ++i) {
            pxh_detection r;
            std::memcpy(&r, raw.data() + static_cast<std::size_t>(i) * 8, sizeof(r));
            out.push_back(Detection{ r.x, r.y, r.w, r.h, r.batch, r.class_index, r.prob });
        }
        return out;
    }

private:
    int capacity_;
    IntVector records_, spare_, count_, spareCount_;
    FloatVector nmsWorkspace_;      // the list's own: nms of two lists on two streams may overlap
    unsigned nextOrder_ = 0;
};

// ---------------------------------------------------------------- YOLO head
// reference: include/YoloLayer.h:115-239, 390-547, include/cuda/YoloLayer.h:70-166.
// The reference assigns the positive slots on the host and uploads them on every training
// forward; here the assignment happens inside the same device pass as the decode.
class YoloLayer : public Layer
{
public:
    static constexpr int kStats = 12;

    YoloLayer(Context& context, const Properties& props) : Layer(context, props)
    {
        anchors_ = props.get<std::vector<int>>("anchors");
        mask_ = props.get<std::vector<int>>("mask");
        numAnchors_ = props.get<int>("num", 1);
        ignoreThresh_ = props.get<float>("ignore_thresh", 0.5f);
        truthThresh_ = props.get<float>("truth_thresh", 1.0f);
        coordScale_ = props.get<float>("coord_scale", 1.0f);
        objectScale_ = props.get<float>("object_scale", 1.0f);
        noObjectScale_ = props.get<float>("noobject_scale", 1.0f);
        classScale_ = props.get<float>("class_scale", 1.0f);
        PX_CHECK(static_cast<int>(anchors_.size()) == 2 * numAnchors_, "yolo: anchors must hold 2 * num values");
        PX_CHECK(!mask_.empty(), "yolo: empty mask");
        for (int m: mask_) PX_CHECK(m >= 0 && m < numAnchors_, "yolo: mask entry outside the anchors");
        const int expect = static_cast<int>(mask_.size()) * (context.classes + 5);
        PX_CHECK(channels() == expect, "yolo: channels must equal masks * (classes + 5)");
        setOutput(channels(), height(), width());
        if (training()) {
            stats_ = V(kStats, 0.0f);
            costDevice_ = V(1, 0.0f);
            context.reserveWorkspace(pxh_yolo_workspace_bytes(batch(), static_cast<int>(mask_.size()), context.classes,
                                                              width(), height(), 0));
            // "leaves_norm": nothing but this head reads the layer in front of it (true of every head of
            // the shipped networks), so `grad += delta` below is the last write of that layer's delta
            // and leaves its norm and peak behind for the rescale + clip that opens its backward.
            if (props.get<bool>("leaves_norm", false)) normGroups_ = normGroupsFor(output_.size());
            // "deferred": the training forward of this head waits for forwardDeferred(), which the model
            // calls once after its last layer's forward and which runs all waiting heads as one pass
            deferred_ = props.get<bool>("deferred", false);
            if (deferred_) {
                context.deferredHeadsWorkspace += pxh_yolo_workspace_bytes(batch(), static_cast<int>(mask_.size()),
                                                                           context.classes, width(), height(), 0);
                context.reserveWorkspace(context.deferredHeadsWorkspace);
            }
        }
    }

    bool hasCost() const noexcept override { return true; }

    // Runs the training forward of every head of `context` that is waiting for it (reference: each
    // YoloLayer's own forward, include/YoloLayer.h:164-239, in one device pass).  To be called after the
    // forward of the model's last layer, before anything reads a head's delta, cost or statistics.
    static void forwardDeferred(Context& context)
    {
        auto& waiting = context.deferredHeads;
        if (waiting.empty()) return;
        constexpr std::size_t kPerCall = 4;      // heads per call of the library
        for (std::size_t first = 0; first < waiting.size(); first += kPerCall) {
            const std::size_t count = std::min(kPerCall, waiting.size() - first);
            pxh_yolo_head heads[kPerCall];
            const YoloLayer* lead = static_cast<const YoloLayer*>(waiting[first]);
            for (std::size_t h = 0; h < count; ++h) {
                auto* y = static_cast<YoloLayer*>(waiting[first + h]);
                PX_CHECK(y->batch() == lead->batch() && y->anchors_ == lead->anchors_,
                         "yolo: deferred heads must share the batch and the anchor list");
                heads[h] = pxh_yolo_head{ y->pendingInput_, y->output_.data(), y->delta_.data(), y->mask_.data(),
                                          static_cast<int>(y->mask_.size()), y->width(), y->height(), y->ignoreThresh_,
                                          y->truthThresh_, y->coordScale_, y->objectScale_, y->noObjectScale_,
                                          y->classScale_, y->stats_.data(), y->costDevice_.data() };
            }
            PX_HIP_CHECK(pxh_yolo_forward_train_heads(static_cast<int>(count), heads, context.truths().data(),
                                                      context.truthCounts().data(), context.maxTruth(),
                                                      lead->anchors_.data(), lead->numAnchors_, lead->batch(),
                                                      context.classes, context.width, context.height,
                                                      context.workspace(), context.workspaceBytes(), context.stream));
        }
        waiting.clear();
    }

    void forward(const V& input) override
    {
        // no zero-fill of delta_ (Layer::forward): the training pass writes every element of it
        cost_ = 0.0f;
        checkInput(input, "YoloLayer");
        const auto& c = context();
        const int masks = static_cast<int>(mask_.size());
        if (inferring()) {
            PX_HIP_CHECK(pxh_yolo_activate(input.data(), output_.data(), batch(), masks, c.classes,
                                           width() * height(), stream()));
            return;
        }
        PX_CHECK(static_cast<int>(c.truthCounts().size()) == batch(), "yolo: ground truth of another batch size");
        costReady_ = false;
        if (deferred_) {
            pendingInput_ = input.data();
            context().deferredHeads.push_back(this);
            return;
        }
        PX_HIP_CHECK(pxh_yolo_forward_train(input.data(), output_.data(), delta_.data(), c.truths().data(),
                                            c.truthCounts().data(), c.maxTruth(), mask_.data(), anchors_.data(),
                                            stats_.data(), costDevice_.data(), batch(), masks, numAnchors_,
                                            c.classes, width(), height(), c.width, c.height, ignoreThresh_,
                                            truthThresh_, coordScale_, objectScale_, noObjectScale_, classScale_,
                                            context().workspace(), context().workspaceBytes(), stream()));
        costReady_ = false;
    }

    void backward(const V& input, V* grad) override
    {
        Layer::backward(input, grad);
        if (grad == nullptr) return;
        if (!normGroups_.empty()) {
            PX_HIP_CHECK(pxh_axpy_norm(delta_.size(), 1.0f, delta_.data(), grad->data(), normGroups_.data(), stream()));
            context().noteNormGroups(grad->data(), normGroups_.data());
            return;
        }
        PX_HIP_CHECK(pxh_axpy(delta_.size(), 1.0f, delta_.data(), grad->data(), stream()));
    }

    // Appends the detections of the last forward, in the reference's order (image, cell, mask,
    // class), relative boxes (reference: include/YoloLayer.h:713-720).  Blocking; only the
    // detections cross to the host, not the head.
    void addDetects(Detections& detections, float threshold) { addDetects(detections, 0, 0, threshold); }

    // The same with boxes in pixels of a width x height image that was letterboxed into the
    // network input (reference: include/YoloLayer.h:700-711).
    void addDetects(Detections& detections, int width, int height, float threshold)
    {
        const auto& c = context();
        if (detectCount_.empty()) detectCount_ = IntVector(1, 0);
        if (detectCapacity_ == 0) growDetections(4096);
        for (;;) {
            PX_HIP_CHECK(pxh_yolo_detections(output_.data(), batch(), mask_.data(), static_cast<int>(mask_.size()),
                                             anchors_.data(), numAnchors_, c.classes, this->width(), this->height(),
                                             c.width, c.height, width, height, threshold,
                                             reinterpret_cast<pxh_detection*>(detectRecords_.data()),
                                             detectCapacity_, detectCount_.data(), stream()));
            PX_HIP_RUNTIME_CHECK(hipStreamSynchronize(stream()));
            const int found = detectCount_.asVector()[0];
            if (found <= detectCapacity_) {
                appendSorted(detections, found);
                return;
            }
            growDetections(found);
        }
    }

    // The same onto a device-resident list, without synchronising: the records go behind those of
    // the YOLO layers asked before, with emission orders that continue theirs.
    void addDetects(DeviceDetections& list, int width, int height, float threshold)
    {
        const auto& c = context();
        PX_HIP_CHECK(pxh_yolo_detections_append(output_.data(), batch(), mask_.data(), static_cast<int>(mask_.size()),
                                                anchors_.data(), numAnchors_, c.classes, this->width(),
                                                this->height(), c.width, c.height, width, height, threshold,
                                                list.nextOrder(), list.records(), list.capacity(), list.count(),
                                                stream()));
        list.advanceOrder(static_cast<unsigned>(batch()) * static_cast<unsigned>(mask_.size()) *
                          static_cast<unsigned>(this->width() * this->height()) * static_cast<unsigned>(c.classes));
    }

    // Blocking: cost = sum(delta^2) / max(1, batch) (reference: include/cuda/YoloLayer.h:132).
    float fetchCost()
    {
        if (!costReady_ && !costDevice_.empty()) {
            PX_HIP_RUNTIME_CHECK(hipStreamSynchronize(stream()));
            cost_ = costDevice_.asVector()[0] / static_cast<float>(std::max(1, batch()));
            costReady_ = true;
        }
        return cost_;
    }

    // Blocking: the 12 counters of the last training forward.
    std::vector<float> fetchStats() const
    {
        PX_HIP_RUNTIME_CHECK(hipStreamSynchronize(stream()));
        return stats_.asVector();
    }

private:
    void growDetections(int capacity)
    {
        detectCapacity_ = capacity;
        detectRecords_ = IntVector(static_cast<std::size_t>(capacity) * (sizeof(pxh_detection) / sizeof(int)));
    }

    void appendSorted(Detections& detections, int found)
    {
        static_assert(sizeof(pxh_detection) == 8 * sizeof(int), "record layout");
        const std::vector<int> raw = detectRecords_.asVector();
        std::vector<pxh_detection> records(static_cast<std::size_t>(found));
        if (found) std::memcpy(records.data(), raw.data(), records.size() * sizeof(pxh_detection));
        std::sort(records.begin(), records.end(),
                  [](const pxh_detection& a, const pxh_detection& b) { return a.order < b.order; });
        for (const auto& r: records) detections.push_back(Detection{ r.x, r.y, r.w, r.h, r.batch, r.class_index, r.prob });
    }

    std::vector<int> anchors_, mask_;
    int numAnchors_ = 1;
    float ignoreThresh_, truthThresh_, coordScale_, objectScale_, noObjectScale_, classScale_;
    V stats_, costDevice_;
    bool costReady_ = false;
    bool deferred_ = false;
    const float* pendingInput_ = nullptr;
    V normGroups_;
    IntVector detectRecords_, detectCount_;
    int detectCapacity_ = 0;
};

}   // px::hip

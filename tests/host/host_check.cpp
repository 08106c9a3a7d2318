// Drives the C++ layer interface (pixienn_amd/host) on the GPU and checks every layer against the
// CPU checker on the inputs the GPU layer actually saw.  Test code: it links the checker, the
// product headers do not.
//
//   host_check          all checks (needs a GPU)
//   host_check --cpu    only the checks that touch no device (argument and property errors)
//
// Exit status 0 when every check passes.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include <sstream>

#include "pixienn/Layers.h"
#include "pixienn/CapturedSequence.h"
#include "pixienn/OptimizerState.h"
#include "pixienn/WeightsFile.h"
#include "px_oracle.h"

using namespace px::hip;
using Host = std::vector<float>;

namespace {

int failures = 0;
int checks = 0;

void report(const std::string& what, bool ok, const std::string& detail = "")
{
    ++checks;
    if (!ok) ++failures;
    std::printf("%-58s %s %s\n", what.c_str(), ok ? "ok" : "FAILED", detail.c_str());
    std::fflush(stdout);
}

// counter-based generator: the same values on every host
struct Rng {
    uint64_t state;
    explicit Rng(uint64_t seed) : state(seed * 0x9E3779B97F4A7C15ull + 0x1234567ull) {}
    uint32_t next()
    {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        return static_cast<uint32_t>(state >> 33);
    }
    float uniform() { return (next() & 0xFFFFFF) / 16777216.0f; }
    float normal()      // sum of 12 uniforms - 6
    {
        float s = 0;
        for (int i = 0; i < 12; ++i) s += uniform();
        return s - 6.0f;
    }
};

Host normals(uint64_t seed, size_t n, float scale = 1.0f, float shift = 0.0f)
{
    Rng r(seed);
    Host v(n);
    for (auto& x: v) x = shift + scale * r.normal();
    return v;
}

Host uniforms(uint64_t seed, size_t n, float lo, float hi)
{
    Rng r(seed);
    Host v(n);
    for (auto& x: v) x = lo + (hi - lo) * r.uniform();
    return v;
}

void expectExact(const std::string& what, const Host& got, const Host& want)
{
    bool ok = got.size() == want.size();
    size_t bad = 0;
    for (size_t i = 0; ok && i < got.size(); ++i)
        if (std::memcmp(&got[i], &want[i], 4) != 0 && !(std::isnan(got[i]) && std::isnan(want[i]))) ++bad;
    report(what, ok && bad == 0, bad ? std::to_string(bad) + " elements differ" : "");
}

void expectExact(const std::string& what, const std::vector<int>& got, const std::vector<int>& want)
{
    report(what, got == want);
}

// |got - want| <= rtol * max(|want|, floor)
void expectClose(const std::string& what, const Host& got, const Host& want, double rtol, double floor)
{
    bool ok = got.size() == want.size();
    double worst = 0;
    for (size_t i = 0; ok && i < got.size(); ++i) {
        const double err = std::fabs(double(got[i]) - double(want[i]));
        const double bound = rtol * std::max(std::fabs(double(want[i])), floor);
        worst = std::max(worst, err / std::max(std::fabs(double(want[i])), floor));
        if (!(err <= bound)) ok = false;
    }
    char buf[64];
    std::snprintf(buf, sizeof buf, "max rel %.2e", worst);
    report(what, ok, buf);
}

Host readFloats(const std::string& bytes, size_t offset, size_t count)
{
    Host v(count);
    std::memcpy(v.data(), bytes.data() + offset, count * sizeof(float));
    return v;
}

template<typename F>
void expectThrows(const std::string& what, F&& f, const std::string& needle)
{
    try {
        f();
        report(what, false, "no exception");
    } catch (const px::Error& e) {
        const bool ok = std::string(e.what()).find(needle) != std::string::npos;
        report(what, ok, ok ? "" : e.what());
    }
}

// ---------------------------------------------------------------- checks without a device
void hostOnlyChecks()
{
    Context ctx;
    expectThrows("maxpool rejects kernel 0", [&] {
        MaxPoolLayer l(ctx, { { "batch", 1 }, { "channels", 1 }, { "height", 4 }, { "width", 4 }, { "kernel", 0 } });
    }, "kernel must be positive");
    expectThrows("maxpool rejects negative padding", [&] {
        MaxPoolLayer l(ctx, { { "batch", 1 }, { "channels", 1 }, { "height", 4 }, { "width", 4 }, { "kernel", 2 },
                              { "stride", 2 }, { "padding", -1 } });
    }, "padding cannot be negative");
    expectThrows("yolo needs its anchors", [&] {
        YoloLayer l(ctx, { { "batch", 1 }, { "channels", 8 }, { "height", 2 }, { "width", 2 } });
    }, "no property named \"anchors\"");
    expectThrows("unknown activation name", [&] { activationFromName("gelu"); }, "unknown activation");
    expectThrows("C-ABI status becomes px::Error", [&] {
        PX_HIP_CHECK(pxh_activate(99, reinterpret_cast<float*>(256), 4, nullptr));
    }, "unknown activation");
    Properties p{ { "stride", 3 }, { "scale", 2 } };
    report("property int -> float conversion", p.get<float>("scale") == 2.0f && p.get<int>("stride", 1) == 3 &&
                                                p.get<int>("absent", 7) == 7);
}

// ---------------------------------------------------------------- the mini network
constexpr int N = 2, C = 8, S = 16, CLASSES = 3;

struct Net {
    Context ctx;
    std::shared_ptr<ConvLayer> conv0, conv2, conv6;
    std::shared_ptr<MaxPoolLayer> pool1;
    std::shared_ptr<ShortcutLayer> short3;
    std::shared_ptr<UpsampleLayer> up4;
    std::shared_ptr<RouteLayer> route5;
    std::shared_ptr<YoloLayer> yolo7;
    std::vector<int> mask{ 0, 2 }, anchors{ 10, 14, 23, 27, 37, 58 };
    Host scale0, bias0, scale2, bias2, bias6;

    std::vector<Layer*> all() const
    {
        return { conv0.get(), pool1.get(), conv2.get(), short3.get(), up4.get(), route5.get(), conv6.get(), yolo7.get() };
    }

    explicit Net(bool training, bool leavesNorm = false)
    {
        ctx.training = training;
        ctx.width = ctx.height = 128;
        ctx.classes = CLASSES;
        ctx.updateBatch = N;
        ctx.timeStep = 3;
        conv0 = std::make_shared<ConvLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S },
                                                             { "width", S }, { "filters", C },
                                                             { "batch_normalize", true },
                                                             { "activation", std::string("leaky") } });
        pool1 = std::make_shared<MaxPoolLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S },
                                                                { "width", S }, { "kernel", 2 }, { "stride", 2 } });
        conv2 = std::make_shared<ConvLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S / 2 },
                                                             { "width", S / 2 }, { "filters", C },
                                                             { "batch_normalize", true },
                                                             { "activation", std::string("mish") } });
        short3 = std::make_shared<ShortcutLayer>(ctx, Properties{ { "batch", N }, { "channels", C },
                                                                  { "height", S / 2 }, { "width", S / 2 },
                                                                  { "alpha", 1.0f }, { "beta", 0.5f },
                                                                  { "leaves_norm", leavesNorm } }, pool1);
        up4 = std::make_shared<UpsampleLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S / 2 },
                                                               { "width", S / 2 }, { "stride", 2 } });
        route5 = std::make_shared<RouteLayer>(ctx, Properties{ { "batch", N }, { "channels", 2 * C },
                                                               { "height", S }, { "width", S } },
                                              std::vector<Layer::Ptr>{ up4, conv0 });
        conv6 = std::make_shared<ConvLayer>(ctx, Properties{ { "batch", N }, { "channels", 2 * C }, { "height", S },
                                                             { "width", S }, { "filters", 2 * C },
                                                             { "activation", std::string("linear") } });
        yolo7 = std::make_shared<YoloLayer>(ctx, Properties{ { "batch", N }, { "channels", 2 * C }, { "height", S },
                                                             { "width", S }, { "num", 3 }, { "mask", mask },
                                                             { "anchors", anchors }, { "ignore_thresh", 0.5f },
                                                             { "object_scale", 2.0f }, { "noobject_scale", 0.5f },
                                                             { "leaves_norm", leavesNorm } });
        scale0 = uniforms(11, C, 0.5f, 1.5f); bias0 = normals(12, C, 0.1f);
        scale2 = uniforms(13, C, 0.5f, 1.5f); bias2 = normals(14, C, 0.1f);
        bias6 = normals(15, 2 * C, 0.1f);
        conv0->copyScales(scale0); conv0->copyBiases(bias0);
        conv0->copyRollingMean(normals(16, C, 0.1f)); conv0->copyRollingVariance(uniforms(17, C, 0.5f, 1.5f));
        conv2->copyScales(scale2); conv2->copyBiases(bias2);
        conv2->copyRollingMean(normals(18, C, 0.1f)); conv2->copyRollingVariance(uniforms(19, C, 0.5f, 1.5f));
        conv6->copyBiases(bias6);
    }
};

void convForwardCheck(const std::string& name, ConvLayer& layer, const Host& input, bool bn, bool training, int act,
                      int channels, int size, Host* meanOut = nullptr, Host* varOut = nullptr)
{
    Host want = input;
    Host mean(channels, 0.0f), var(channels, 0.0f);
    Host rmean = layer.rollingMean().asVector(), rvar = layer.rollingVariance().asVector();
    // the layer has already run: undo nothing, the inference path does not move the rolling values and
    // the training check compares mean / var, which do not depend on them
    Host scales = bn ? layer.scales().asVector() : Host(channels, 1.0f);
    Host biases = layer.biases().asVector();
    if (!bn) { rmean.assign(channels, 0.0f); rvar.assign(channels, 1.0f); }
    Host x(training && bn ? input.size() : 0), xnorm(training && bn ? input.size() : 0);
    pxo_conv_epilogue_forward(bn, training, act, N, channels, size, size, want.data(), nullptr, mean.data(),
                              var.data(), rmean.data(), rvar.data(), scales.data(), biases.data(),
                              x.empty() ? nullptr : x.data(), xnorm.empty() ? nullptr : xnorm.data(), 0);
    expectClose(name + " forward", layer.output().asVector(), want, 1e-5, training ? 4.0 : 1.0);
    if (training && bn) {
        expectClose(name + " batch mean", layer.mean().asVector(), mean, 1e-5, 0.05);
        expectClose(name + " batch variance", layer.variance().asVector(), var, 1e-5, 1.0);
    }
    if (meanOut) *meanOut = mean;
    if (varOut) *varOut = var;
}

// the device vector's contract (reference: tests/src/vector.cpp -- fill, initializer list, copies)
void deviceVectorChecks()
{
    FloatVector filled(7, 7.0f);
    report("vector(count, value) fills", filled.asVector() == Host(7, 7.0f));
    const FloatVector listed{ 1.0f, 2.0f, 3.0f, 4.0f };
    report("vector from an initializer list", listed.size() == 4 && listed.asVector() == Host{ 1, 2, 3, 4 });
    IntVector ints{ 1, 2, 3 };
    report("int vector", ints.asVector() == std::vector<int>{ 1, 2, 3 });
    FloatVector copy(4);
    copy.copy(listed);
    report("device to device copy", copy.asVector() == Host{ 1, 2, 3, 4 });
    FloatVector part(6, 0.0f);
    part.copyDevice(listed.data() + 1, 3);
    report("copy from a raw device pointer", part.asVector() == Host{ 2, 3, 4, 0, 0, 0 });
    part.copyHost(Host{ 9, 8 });
    report("copy from the host", part.asVector() == Host{ 9, 8, 4, 0, 0, 0 });
    FloatVector moved(std::move(part));
    report("move leaves the source empty", part.empty() && moved.size() == 6);
    moved.release();
    report("release frees", moved.empty() && moved.data() == nullptr);
    expectThrows("copy between different sizes is refused", [&] { copy.copy(filled); }, "different sizes");
}

void inferenceChecks()
{
    Net net(false);
    FloatVector input(normals(100, size_t(N) * C * S * S));
    net.conv0->forward(input);
    convForwardCheck("conv0 (bn, leaky, inference)", *net.conv0, input.asVector(), true, false, PXO_LEAKY, C, S);
    net.conv0->forward(input);      // second call reuses the folded constants
    convForwardCheck("conv0 again (folded constants reused)", *net.conv0, input.asVector(), true, false, PXO_LEAKY,
                     C, S);
    net.pool1->forward(net.conv0->output());
    {
        const Host in = net.conv0->output().asVector();
        Host out(net.pool1->output().size());
        std::vector<int> idx(out.size());
        pxo_maxpool_forward(in.data(), out.data(), idx.data(), N, C, S, S, S / 2, S / 2, 2, 2, 1);
        expectExact("pool1 forward values", net.pool1->output().asVector(), out);
        expectExact("pool1 forward indexes", net.pool1->indexes().asVector(), idx);
    }
    net.conv2->forward(net.pool1->output());
    convForwardCheck("conv2 (bn, mish, inference)", *net.conv2, net.pool1->output().asVector(), true, false,
                     PXO_MISH, C, S / 2);
    net.short3->forward(net.conv2->output());
    {
        const Host a = net.conv2->output().asVector(), b = net.pool1->output().asVector();
        Host out(a.size()), pre(a.size());
        pxo_shortcut_forward(PXO_LINEAR, N, S / 2, S / 2, C, a.data(), b.data(), 1.0f, 0.5f, out.data(), pre.data());
        expectExact("short3 forward", net.short3->output().asVector(), out);
    }
    net.up4->forward(net.short3->output());
    {
        const Host in = net.short3->output().asVector();
        Host out(net.up4->output().size(), 0.0f);
        pxo_upsample(in.data(), S / 2, S / 2, C, N, 2, 1, 1.0f, nullptr, out.data());
        expectExact("up4 forward", net.up4->output().asVector(), out);
    }
    net.route5->forward(net.up4->output());
    {
        const Host a = net.up4->output().asVector(), b = net.conv0->output().asVector();
        Host out(net.route5->output().size(), -1.0f);
        pxo_route_forward(a.data(), out.data(), N, C * S * S, 2 * C * S * S, 0);
        pxo_route_forward(b.data(), out.data(), N, C * S * S, 2 * C * S * S, C * S * S);
        expectExact("route5 forward", net.route5->output().asVector(), out);
    }
    net.conv6->forward(net.route5->output());
    convForwardCheck("conv6 (bias, linear)", *net.conv6, net.route5->output().asVector(), false, false, PXO_LINEAR,
                     2 * C, S);
    net.yolo7->forward(net.conv6->output());
    {
        pxo_yolo_cfg cfg{ N, S, S, CLASSES, 2, 3, net.mask.data(), net.anchors.data(), 128, 128, 0.5f, 1.0f, 1.0f,
                          2.0f, 0.5f, 1.0f };
        const Host in = net.conv6->output().asVector();
        Host out(in.size());
        pxo_yolo_decode(&cfg, in.data(), out.data());
        expectClose("yolo7 decode (inference)", net.yolo7->output().asVector(), out, 1e-5, 1e-3);

        // detections of that head, from the decoded values the layer holds
        const Host decoded = net.yolo7->output().asVector();
        for (int scaled = 0; scaled < 2; ++scaled) {
            const int iw = scaled ? 320 : 0, ih = scaled ? 200 : 0;
            std::vector<pxo_detection> want(4096);
            const int found = pxo_yolo_detections(&cfg, decoded.data(), 0.3f, iw, ih, want.data(), 4096);
            Detections got;
            if (scaled) net.yolo7->addDetects(got, iw, ih, 0.3f); else net.yolo7->addDetects(got, 0.3f);
            bool same = found > 0 && found <= 4096 && static_cast<int>(got.size()) == found;
            Host gb, wb;
            for (int k = 0; same && k < found; ++k) {
                same = got[k].batchId == want[k].batch && got[k].classIndex == want[k].class_index &&
                       got[k].prob == want[k].prob;
                gb.insert(gb.end(), { got[k].x, got[k].y, got[k].w, got[k].h });
                wb.insert(wb.end(), { want[k].x, want[k].y, want[k].w, want[k].h });
            }
            report(std::string("yolo7 detections, order and scores") + (scaled ? " (pixel boxes)" : ""), same,
                   std::to_string(found) + " found");
            // integer pixel boxes may differ by one where a last-place difference in exp moves a truncation
            expectClose(std::string("yolo7 detection boxes") + (scaled ? " (pixel boxes)" : ""), gb, wb,
                        scaled ? 1.0 / 320.0 : 1e-5, scaled ? 320.0 : 4.0);
            // the same records kept on the device, the head asked twice (as two YOLO layers would be),
            // then nms there; the checker's nms runs on the host copies of the device's own records
            for (int capacity: { 512, 16384 }) {         // one-launch form and sorting form
                // the short list needs a confidence that leaves at most 256 records per head
                float confidence = 0.3f;
                Detections once;
                for (float c: { 0.3f, 0.8f, 0.9f, 0.95f, 0.98f }) {
                    confidence = c;
                    once.clear();
                    net.yolo7->addDetects(once, iw, ih, confidence);
                    if (2 * static_cast<int>(once.size()) <= capacity) break;
                }
                const int each = static_cast<int>(once.size());
                DeviceDetections list(capacity);
                list.clear();
                net.yolo7->addDetects(list, iw, ih, confidence);
                net.yolo7->addDetects(list, iw, ih, confidence);
                const Detections both = list.toHost();
                std::vector<pxo_detection> input;
                for (int pass = 0; pass < 2; ++pass)
                    for (const auto& d: once)
                        input.push_back(pxo_detection{ d.x, d.y, d.w, d.h, d.prob, d.batchId, d.classIndex,
                                                       static_cast<unsigned>(input.size()) });
                const bool fits = each > 0 && 2 * each <= capacity;
                report("two heads append " + std::to_string(both.size()) + " records into a list of " +
                       std::to_string(capacity), fits && static_cast<int>(both.size()) == 2 * each);
                if (!fits) continue;
                std::vector<pxo_detection> kept(input.size());
                const int keptCount = pxo_nms(input.data(), static_cast<int>(input.size()), 0.45f, kept.data());
                list.nms(N, CLASSES, 0.45f);
                const Detections survivors = list.toHost();
                bool equal = static_cast<int>(survivors.size()) == keptCount && keptCount > 0 && keptCount <= each;
                for (int k = 0; equal && k < keptCount; ++k)
                    equal = survivors[k].x == kept[k].x && survivors[k].y == kept[k].y && survivors[k].w == kept[k].w &&
                            survivors[k].h == kept[k].h && survivors[k].prob == kept[k].prob &&
                            survivors[k].batchId == kept[k].batch && survivors[k].classIndex == kept[k].class_index;
                report(std::string("nms on the device list") + (scaled ? " (pixel boxes)" : "") + ", capacity " +
                       std::to_string(capacity), equal, std::to_string(keptCount) + " of " +
                       std::to_string(input.size()) + " kept");
            }
        }
    }
}

std::vector<GroundTruthVec> makeTruth()
{
    Rng r(77);
    std::vector<GroundTruthVec> truth(N);
    for (int b = 0; b < N; ++b) {
        const int count = 3 + b * 2;
        for (int t = 0; t < count; ++t) {
            GroundTruth g;
            g.x = r.uniform(); g.y = r.uniform();
            g.w = 0.05f + 0.5f * r.uniform(); g.h = 0.05f + 0.5f * r.uniform();
            g.classId = static_cast<int>(r.next() % CLASSES);
            truth[b].push_back(g);
        }
    }
    return truth;
}

void trainingChecks()
{
    Net net(true);
    const auto truth = makeTruth();
    net.ctx.setGroundTruth(truth);
    FloatVector input(normals(200, size_t(N) * C * S * S));
    const Host rmeanBefore = net.conv0->rollingMean().asVector();

    // ---- forward
    net.conv0->forward(input);
    Host mean0, var0;
    convForwardCheck("conv0 (bn, leaky, training)", *net.conv0, input.asVector(), true, true, PXO_LEAKY, C, S, &mean0,
                     &var0);
    {
        Host want(C);
        for (int c = 0; c < C; ++c) want[c] = 0.99f * rmeanBefore[c] + 0.01f * mean0[c];
        expectClose("conv0 rolling mean moved", net.conv0->rollingMean().asVector(), want, 1e-5, 0.05);
    }
    net.pool1->forward(net.conv0->output());
    net.conv2->forward(net.pool1->output());
    Host mean2, var2;
    convForwardCheck("conv2 (bn, mish, training)", *net.conv2, net.pool1->output().asVector(), true, true, PXO_MISH,
                     C, S / 2, &mean2, &var2);
    net.short3->forward(net.conv2->output());
    net.up4->forward(net.short3->output());
    net.route5->forward(net.up4->output());
    net.conv6->forward(net.route5->output());
    net.yolo7->forward(net.conv6->output());

    // ---- YOLO head against the checker
    const int maxTruth = net.ctx.maxTruth();
    Host yoloDelta;
    {
        pxo_yolo_cfg cfg{ N, S, S, CLASSES, 2, 3, net.mask.data(), net.anchors.data(), 128, 128, 0.5f, 1.0f, 1.0f,
                          2.0f, 0.5f, 1.0f };
        const Host in = net.conv6->output().asVector();
        const Host truths = net.ctx.truths().asVector();
        const std::vector<int> counts = net.ctx.truthCounts().asVector();
        Host out(in.size()), delta(in.size(), 0.0f), stats(12, 0.0f);
        float cost = 0;
        pxo_yolo_forward(&cfg, in.data(), truths.data(), counts.data(), maxTruth, out.data(), delta.data(), &cost,
                         stats.data());
        expectClose("yolo7 output (training)", net.yolo7->output().asVector(), out, 1e-5, 1e-3);
        yoloDelta = net.yolo7->delta().asVector();
        expectClose("yolo7 delta", yoloDelta, delta, 1e-5, 2.0);
        expectClose("yolo7 cost", Host{ net.yolo7->fetchCost() }, Host{ cost }, 1e-5, 1e-3);
        const Host gs = net.yolo7->fetchStats();
        expectClose("yolo7 positives counted", Host{ gs[6] }, Host{ stats[6] }, 0.0, 1.0);
    }

    // ---- backward, last layer first; every layer accumulates into its predecessor's delta.
    // The head rescales its delta to a norm threshold and clamps it first.
    {
        Host want = yoloDelta;
        const float norm = pxo_rescale_clip(want.data(), want.size(), 0.0f, 0.0f);
        want = yoloDelta;
        pxo_rescale_clip(want.data(), want.size(), 0.5f * norm, 0.05f);
        net.yolo7->setGradientRescaling(true, 0.5f * norm);
        net.yolo7->setGradientClipping(true, 0.05f);
        net.yolo7->backward(net.conv6->output(), &net.conv6->delta());
        yoloDelta = net.yolo7->delta().asVector();
        expectClose("yolo7 delta rescaled and clamped", yoloDelta, want, 1e-6, 1e-6);
    }
    expectExact("yolo7 backward: grad += delta", net.conv6->delta().asVector(), yoloDelta);

    {   // conv6: bias backward, then (identity convolution) grad += delta
        Host d = net.conv6->delta().asVector();
        Host biasUpd(2 * C, 0.0f);
        const Host pre = net.conv6->output().asVector();      // linear: the output is the pre-activation
        // Layer::backward's helpers ride on the bias backward: the rescale bites, the clamp is far away
        Host probe = d;
        const float norm = pxo_rescale_clip(probe.data(), probe.size(), 0.0f, 0.0f);
        pxo_rescale_clip(d.data(), d.size(), 0.5f * norm, 1e3f);
        net.conv6->setGradientRescaling(true, 0.5f * norm);
        net.conv6->setGradientClipping(true, 1e3f);
        pxo_conv_epilogue_backward(0, PXO_LINEAR, N, 2 * C, S, S, d.data(), pre.data(), nullptr, nullptr, nullptr,
                                   nullptr, nullptr, nullptr, biasUpd.data(), nullptr, nullptr, 0);
        net.conv6->backward(net.route5->output(), &net.route5->delta());
        expectClose("conv6 bias updates (delta rescaled)", net.conv6->biasUpdates().asVector(), biasUpd, 1e-5, 1.0);
        expectExact("conv6 backward into route5 delta (rescaled)", net.route5->delta().asVector(), d);
    }
    {   // route5 -> up4.delta and conv0.delta
        const Host rd = net.route5->delta().asVector();
        Host a(net.up4->delta().size(), 0.0f), b(net.conv0->delta().size(), 0.0f);
        pxo_route_backward(rd.data(), a.data(), N, C * S * S, 2 * C * S * S, 0);
        pxo_route_backward(rd.data(), b.data(), N, C * S * S, 2 * C * S * S, C * S * S);
        net.route5->backward(net.up4->output(), &net.up4->delta());
        expectExact("route5 backward into up4 delta", net.up4->delta().asVector(), a);
        expectExact("route5 backward into conv0 delta", net.conv0->delta().asVector(), b);
    }
    {   // up4 -> short3.delta
        const Host d = net.up4->delta().asVector();
        Host acc(net.short3->delta().size(), 0.0f), dcopy = d;
        pxo_upsample(nullptr, S / 2, S / 2, C, N, 2, 0, 1.0f, acc.data(), dcopy.data());
        net.up4->backward(net.short3->output(), &net.short3->delta());
        expectExact("up4 backward into short3 delta", net.short3->delta().asVector(), acc);
    }
    {   // short3 -> pool1.delta (from) and conv2.delta (grad)
        Host d = net.short3->delta().asVector();
        Host from(net.pool1->delta().size(), 0.0f), grad(net.conv2->delta().size(), 0.0f);
        const Host pre = net.short3->output().asVector();     // linear: the output is the pre-activation
        pxo_shortcut_backward(PXO_LINEAR, N, S / 2, S / 2, C, d.data(), pre.data(), from.data(), grad.data(), 1.0f,
                              0.5f);
        net.short3->backward(net.conv2->output(), &net.conv2->delta());
        expectExact("short3 backward into pool1 delta", net.pool1->delta().asVector(), from);
        expectExact("short3 backward into conv2 delta", net.conv2->delta().asVector(), grad);
    }
    {   // conv2: activation gradient + batch norm backward, accumulated into pool1.delta
        Host d = net.conv2->delta().asVector();
        const Host x = net.pool1->output().asVector();
        const Host mean = net.conv2->mean().asVector(), var = net.conv2->variance().asVector();
        // the checker wants x_hat and the pre-activation of the forward
        Host xn = x, pre(x.size());
        pxo_normalize(xn.data(), mean.data(), var.data(), N, C, (S / 2) * (S / 2));
        for (size_t i = 0; i < x.size(); ++i) {
            const int c = static_cast<int>(i / ((S / 2) * (S / 2))) % C;
            const float scaled = xn[i] * net.scale2[c];
            pre[i] = scaled + net.bias2[c];
        }
        // Layer::backward's helpers ride on the epilogue's backward: rescale and clamp both bite here
        Host probe = d;
        const float norm = pxo_rescale_clip(probe.data(), probe.size(), 0.0f, 0.0f);
        const float rms = norm / std::sqrt(static_cast<float>(d.size()));
        pxo_rescale_clip(d.data(), d.size(), 0.6f * norm, 0.9f * rms);
        net.conv2->setGradientRescaling(true, 0.6f * norm);
        net.conv2->setGradientClipping(true, 0.9f * rms);
        Host md(C), vd(C), su(C, 0.0f), bu(C, 0.0f);
        pxo_conv_epilogue_backward(1, PXO_MISH, N, C, S / 2, S / 2, d.data(), pre.data(), mean.data(), var.data(),
                                   md.data(), vd.data(), net.scale2.data(), su.data(), bu.data(), x.data(), xn.data(),
                                   0);
        Host want = net.pool1->delta().asVector();
        for (size_t i = 0; i < want.size(); ++i) want[i] += d[i];
        net.conv2->backward(net.pool1->output(), &net.pool1->delta());
        expectClose("conv2 scale updates (delta rescaled, clamped)", net.conv2->scaleUpdates().asVector(), su, 1e-5, 1.0);
        expectClose("conv2 bias updates (delta rescaled, clamped)", net.conv2->biasUpdates().asVector(), bu, 1e-5, 1.0);
        expectClose("conv2 backward into pool1 delta (rescaled, clamped)", net.pool1->delta().asVector(), want, 1e-5, 1.0);
    }
    {   // pool1 -> conv0.delta
        const Host d = net.pool1->delta().asVector();
        const std::vector<int> idx = net.pool1->indexes().asVector();
        Host grad = net.conv0->delta().asVector();
        pxo_maxpool_backward(d.data(), idx.data(), grad.data(), d.size());
        net.pool1->backward(net.conv0->output(), &net.conv0->delta());
        expectExact("pool1 backward into conv0 delta", net.conv0->delta().asVector(), grad);
    }
    net.conv0->backward(input, nullptr);

    // ---- update: SGD with momentum on conv0's biases, then Adam on conv2's scales
    {
        Host w = net.conv0->biases().asVector(), d = net.conv0->biasUpdates().asVector();
        pxo_sgd_update(C, w.data(), d.data(), net.ctx.updateBatch, net.ctx.learningRate, net.ctx.momentum,
                       net.ctx.decay, 0);
        net.ctx.adamEnabled = false;
        net.conv0->update();
        expectClose("conv0 SGD update of the biases", net.conv0->biases().asVector(), w, 1e-6, 1e-3);
        expectClose("conv0 bias updates keep the momentum term", net.conv0->biasUpdates().asVector(), d, 1e-6, 1e-3);
    }
    net.ctx.adamEnabled = true;
    {
        Host w = net.conv2->scales().asVector(), d = net.conv2->scaleUpdates().asVector();
        Host m(C, 0.0f), v(C, 0.0f);
        pxo_adam_update(C, w.data(), d.data(), m.data(), v.data(), net.ctx.updateBatch, net.ctx.timeStep,
                        net.ctx.learningRate, net.ctx.adamBeta1, net.ctx.adamBeta2, net.ctx.adamEpsilon,
                        net.ctx.decay, 0);
        net.conv2->update();
        expectClose("conv2 Adam update of the scales", net.conv2->scales().asVector(), w, 1e-6, 1e-3);
        expectExact("conv2 scale updates consumed", net.conv2->scaleUpdates().asVector(), Host(C, 0.0f));
    }

    // ---- optimizer sidecar: layout, round trip, stale file
    {
        const std::vector<Layer::Ptr> layers{ net.conv0, net.pool1, net.conv2, net.short3, net.conv6 };
        std::stringstream file(std::ios::in | std::ios::out | std::ios::binary);
        saveOptimizerState(file, OptimizerHeader{ 6400, 400, true }, layers);
        const std::string bytes = file.str();
        // header 4 + 8 + 8, conv0 and conv2: (bias m,v + scale m,v) * C floats, conv6: bias m,v * 2C floats
        const size_t expect = 20 + 2 * (4 * C) * 4 + (2 * 2 * C) * 4;
        report("optimizer sidecar size", bytes.size() == expect, std::to_string(bytes.size()) + " bytes");
        std::uint32_t magic = 0;
        std::memcpy(&magic, bytes.data(), 4);
        report("optimizer sidecar magic", magic == 0x50584f32);
        // conv2's scale moments sit after conv0's block and conv2's bias moments
        const Host scaleM = readFloats(bytes, 20 + (4 * C) * 4 + (2 * C) * 4, C);
        Host w = net.scale2, d = net.conv2->scaleUpdates().asVector();
        (void) w; (void) d;
        bool moved = false;
        for (float v: scaleM) moved = moved || v != 0.0f;
        report("conv2 scale moments are in their place", moved);

        Net fresh(true);
        const std::vector<Layer::Ptr> freshLayers{ fresh.conv0, fresh.pool1, fresh.conv2, fresh.short3, fresh.conv6 };
        OptimizerHeader h;
        std::stringstream again(bytes, std::ios::in | std::ios::binary);
        report("sidecar of other weights is refused", !loadOptimizerState(again, 1234, h, freshLayers));
        std::stringstream third(bytes, std::ios::in | std::ios::binary);
        const bool loaded = loadOptimizerState(third, 6400, h, freshLayers);
        report("sidecar header round trip", loaded && h.seen == 6400 && h.step == 400);
        std::stringstream out(std::ios::in | std::ios::out | std::ios::binary);
        saveOptimizerState(out, h, freshLayers);
        report("sidecar round trip is byte identical", out.str() == bytes);
    }
}

// The stand-alone batch-norm layer: inference, training forward/backward/update and the weight file
// section, against the checker's batchNormForward / batchNormBackward.
void batchNormLayerChecks()
{
    const int BC = 6, BS = 12;
    const size_t total = size_t(N) * BC * BS * BS;
    const Host x = normals(401, total, 1.5f, 0.3f);
    const Host biases = normals(402, BC, 0.2f), scales = uniforms(403, BC, 0.5f, 1.5f);
    const Host rmean = normals(404, BC, 0.1f), rvar = uniforms(405, BC, 0.5f, 1.5f);
    std::stringstream file(std::ios::in | std::ios::out | std::ios::binary);
    for (const Host* t: { &biases, &scales, &rmean, &rvar })
        file.write(reinterpret_cast<const char*>(t->data()), std::streamsize(t->size() * sizeof(float)));
    const Properties props{ { "batch", N }, { "channels", BC }, { "height", BS }, { "width", BS } };
    const FloatVector input(x);
    {
        Context ctx;
        ctx.training = false;
        BatchNormLayer layer(ctx, props);
        file.seekg(0);
        const auto bytes = layer.loadWeights(file);
        report("batchnorm weight section is 4 x channels floats", bytes == std::streamoff(4 * BC * sizeof(float)));
        layer.forward(input);
        Host want(total), m(BC), v(BC), rm = rmean, rv = rvar;
        pxo_batchnorm_forward(0, N, BC, BS, BS, x.data(), want.data(), m.data(), v.data(), rm.data(), rv.data(),
                              scales.data(), biases.data(), nullptr, nullptr, 0);
        expectClose("batchnorm layer, inference", layer.output().asVector(), want, 1e-5, 1.0);
        std::stringstream out(std::ios::in | std::ios::out | std::ios::binary);
        layer.saveWeights(out);
        report("batchnorm weights round trip", out.str() == file.str());
    }
    {   // a conv layer's section: biases, scales, rolling mean, rolling variance, then the weights
        Context ctx;
        ctx.training = false;
        const int weights = BC * BC * 9;
        ConvLayer conv(ctx, Properties{ { "batch", N }, { "channels", BC }, { "height", BS }, { "width", BS },
                                         { "filters", BC }, { "batch_normalize", true }, { "weights", weights },
                                         { "activation", std::string("leaky") } });
        const Host w = normals(408, weights, 0.02f);
        std::stringstream section(std::ios::in | std::ios::out | std::ios::binary);
        for (const Host* t: { &biases, &scales, &rmean, &rvar, &w })
            section.write(reinterpret_cast<const char*>(t->data()), std::streamsize(t->size() * sizeof(float)));
        const auto bytes = conv.loadWeights(section);
        report("conv weight section: 4 x filters + weights floats",
               bytes == std::streamoff((4 * BC + weights) * sizeof(float)) && conv.weights().asVector() == w &&
               conv.scales().asVector() == scales && conv.rollingVariance().asVector() == rvar);
        std::stringstream out(std::ios::in | std::ios::out | std::ios::binary);
        conv.saveWeights(out);
        report("conv weights round trip", out.str() == section.str());
        ConvLayer plain(ctx, Properties{ { "batch", N }, { "channels", BC }, { "height", BS }, { "width", BS },
                                          { "filters", BC }, { "weights", weights } });
        std::stringstream two(std::ios::in | std::ios::out | std::ios::binary);
        for (const Host* t: { &biases, &w })
            two.write(reinterpret_cast<const char*>(t->data()), std::streamsize(t->size() * sizeof(float)));
        report("conv without batch norm: biases, then weights",
               plain.loadWeights(two) == std::streamoff((BC + weights) * sizeof(float)) &&
               plain.biases().asVector() == biases && plain.weights().asVector() == w);
        std::stringstream shortFile(std::string(10, 'x'), std::ios::in | std::ios::binary);
        expectThrows("a truncated weight section is refused", [&] { plain.loadWeights(shortFile); },
                     "Could not read weights");
    }
    Context ctx;
    ctx.training = true;
    ctx.updateBatch = N;
    ctx.learningRate = 0.01f;
    ctx.momentum = 0.9f;
    BatchNormLayer layer(ctx, props);
    file.clear();
    file.seekg(0);
    layer.loadWeights(file);
    layer.forward(input);
    Host want(total), mean(BC), var(BC), rm = rmean, rv = rvar, xs(total), xn(total);
    pxo_batchnorm_forward(1, N, BC, BS, BS, x.data(), want.data(), mean.data(), var.data(), rm.data(), rv.data(),
                          scales.data(), biases.data(), xs.data(), xn.data(), 0);
    expectClose("batchnorm layer, training forward", layer.output().asVector(), want, 1e-5, 4.0);
    expectClose("batchnorm layer, rolling mean", layer.rollingMean().asVector(), rm, 1e-5, 0.05);
    expectClose("batchnorm layer, rolling variance", layer.rollingVariance().asVector(), rv, 1e-5, 1.0);
    Host delta = normals(406, total);
    const Host grad0 = normals(407, total);
    layer.delta().copyHost(delta);
    FloatVector grad(grad0);
    layer.backward(input, &grad);
    Host md(BC), vd(BC), su(BC, 0.0f), bu(BC, 0.0f);
    pxo_batchnorm_backward(N, BC, BS, BS, delta.data(), mean.data(), var.data(), md.data(), vd.data(), scales.data(),
                           su.data(), bu.data(), xs.data(), xn.data(), 0);
    Host wantGrad = grad0;
    for (size_t i = 0; i < total; ++i) wantGrad[i] = wantGrad[i] + delta[i];
    expectClose("batchnorm layer, backward delta", layer.delta().asVector(), delta, 1e-5, 2.0);
    expectClose("batchnorm layer, backward into grad", grad.asVector(), wantGrad, 1e-5, 2.0);
    expectClose("batchnorm layer, scale updates", layer.scaleUpdates().asVector(), su, 1e-5, 30.0);
    expectClose("batchnorm layer, bias updates", layer.biasUpdates().asVector(), bu, 1e-5, 30.0);
    layer.update();
    Host wb = biases, ws = scales, dsu = layer.scaleUpdates().asVector(), dbu = layer.biasUpdates().asVector();
    // the layer's own updates before the step were su / bu up to rounding; use the checker's
    pxo_sgd_update(BC, wb.data(), bu.data(), N, 0.01f, 0.9f, 0.0f, 0);
    pxo_sgd_update(BC, ws.data(), su.data(), N, 0.01f, 0.9f, 0.0f, 0);
    expectClose("batchnorm layer, biases after update", layer.biases().asVector(), wb, 1e-5, 1.0);
    expectClose("batchnorm layer, scales after update", layer.scales().asVector(), ws, 1e-5, 1.0);
    expectClose("batchnorm layer, momentum kept in the updates", dbu, bu, 1e-5, 30.0);

    // the same step with the gradient helpers switched on: update() rescales and clamps the update
    // buffers before it applies them (include/BatchNormLayer.h:160-176)
    BatchNormLayer guarded(ctx, props);
    file.clear();
    file.seekg(0);
    guarded.loadWeights(file);
    guarded.forward(input);
    guarded.delta().copyHost(normals(406, total));
    guarded.backward(input, nullptr);
    Host gsu = guarded.scaleUpdates().asVector(), gbu = guarded.biasUpdates().asVector();
    const float thr = 0.5f * pxo_rescale_clip(gsu.data(), gsu.size(), 0.0f, 0.0f);
    guarded.setGradientRescaling(true, thr);
    guarded.setGradientClipping(true, 0.4f * thr);
    guarded.update();
    pxo_rescale_clip(gsu.data(), gsu.size(), thr, 0.4f * thr);
    pxo_rescale_clip(gbu.data(), gbu.size(), thr, 0.4f * thr);
    Host gb = biases, gs = scales;
    pxo_sgd_update(BC, gb.data(), gbu.data(), N, 0.01f, 0.9f, 0.0f, 0);
    pxo_sgd_update(BC, gs.data(), gsu.data(), N, 0.01f, 0.9f, 0.0f, 0);
    expectClose("guarded update: scales", guarded.scales().asVector(), gs, 1e-5, 1.0);
    expectClose("guarded update: biases", guarded.biases().asVector(), gb, 1e-5, 1.0);
    expectClose("guarded update: clamped scale updates", guarded.scaleUpdates().asVector(), gsu, 1e-5, 1.0);
}

// The whole training step of the mini network (forward, backward, update) recorded as one HIP graph
// and replayed on new inputs: every tensor must be what the same calls give when issued one by one.
void capturedSequenceChecks()
{
    hipStream_t stream = nullptr;
    PX_HIP_RUNTIME_CHECK(hipStreamCreate(&stream));
    {
        Net eager(true), captured(true);
        eager.ctx.stream = stream;
        captured.ctx.stream = stream;
        const auto truth = makeTruth();
        eager.ctx.setGroundTruth(truth);
        captured.ctx.setGroundTruth(truth);
        FloatVector inputEager(size_t(N) * C * S * S), inputCaptured(size_t(N) * C * S * S);
        auto step = [](Net& net, const FloatVector& input) {
            net.conv0->forward(input);
            net.pool1->forward(net.conv0->output());
            net.conv2->forward(net.pool1->output());
            net.short3->forward(net.conv2->output());
            net.up4->forward(net.short3->output());
            net.route5->forward(net.up4->output());
            net.conv6->forward(net.route5->output());
            net.yolo7->forward(net.conv6->output());
            net.yolo7->backward(net.conv6->output(), &net.conv6->delta());
            net.conv6->backward(net.route5->output(), &net.route5->delta());
            net.route5->backward(net.up4->output(), &net.up4->delta());
            net.up4->backward(net.short3->output(), &net.short3->delta());
            net.short3->backward(net.conv2->output(), &net.conv2->delta());
            net.conv2->backward(net.pool1->output(), &net.pool1->delta());
            net.pool1->backward(net.conv0->output(), &net.conv0->delta());
            net.conv0->backward(input, nullptr);
            for (Layer* l: std::initializer_list<Layer*>{ net.conv0.get(), net.conv2.get(), net.conv6.get() }) l->update();
        };
        inputCaptured.copyHost(normals(500, inputCaptured.size()));
        step(captured, inputCaptured);                 // eager once: the library sizes its workspace
        PX_HIP_RUNTIME_CHECK(hipStreamSynchronize(stream));
        CapturedSequence graph;
        graph.capture(stream, [&] { step(captured, inputCaptured); });
        report("a training step is captured as one graph", graph.captured());
        // bring both networks to the same state: the capture run and the warm-up moved `captured` only
        Net* nets[2] = { &eager, &captured };
        bool same = true;
        for (int round = 1; round <= 3; ++round) {
            const Host in = normals(500 + round, inputEager.size());
            inputEager.copyHost(in);
            inputCaptured.copyHost(in);
            if (round == 1) {
                // parameters and rolling statistics back to the initial ones on both sides
                for (Net* n: nets) {
                    n->conv0->copyScales(n->scale0); n->conv0->copyBiases(n->bias0);
                    n->conv0->copyRollingMean(normals(16, C, 0.1f));
                    n->conv0->copyRollingVariance(uniforms(17, C, 0.5f, 1.5f));
                    n->conv2->copyScales(n->scale2); n->conv2->copyBiases(n->bias2);
                    n->conv2->copyRollingMean(normals(18, C, 0.1f));
                    n->conv2->copyRollingVariance(uniforms(19, C, 0.5f, 1.5f));
                    n->conv6->copyBiases(n->bias6);
                    n->conv0->zeroUpdates(); n->conv2->zeroUpdates(); n->conv6->zeroUpdates();
                }
            }
            graph.replay(stream);
            step(eager, inputEager);
            PX_HIP_RUNTIME_CHECK(hipStreamSynchronize(stream));
            same = same && captured.yolo7->delta().asVector() == eager.yolo7->delta().asVector() &&
                   captured.conv0->delta().asVector() == eager.conv0->delta().asVector() &&
                   captured.conv0->scales().asVector() == eager.conv0->scales().asVector() &&
                   captured.conv2->biases().asVector() == eager.conv2->biases().asVector() &&
                   captured.conv0->rollingVariance().asVector() == eager.conv0->rollingVariance().asVector() &&
                   captured.yolo7->fetchStats() == eager.yolo7->fetchStats();
            report("replay " + std::to_string(round) + " equals the eager step", same);
        }
        expectThrows("capture on the null stream is refused", [&] {
            CapturedSequence g;
            g.capture(nullptr, [] {});
        }, "null stream");
    }
    PX_HIP_RUNTIME_CHECK(hipStreamDestroy(stream));
}

// A model that steps all its parameter tensors together (ParameterSet) against the layer-by-layer
// update(): the same values in every tensor, with Adam and with SGD, with the hooks on.
void parameterSetChecks()
{
    for (const bool adam: { true, false }) {
        Net byLayer(true), together(true);
        const auto truth = makeTruth();
        FloatVector input(size_t(N) * C * S * S);
        input.copyHost(normals(900, input.size()));
        Net* nets[2] = { &byLayer, &together };
        for (Net* n: nets) {
            n->ctx.adamEnabled = adam;
            n->ctx.setGroundTruth(truth);
            for (Layer* l: n->all()) {
                l->setGradientRescaling(true, 0.05f);      // small enough to bite on these update buffers
                l->setGradientClipping(true, 0.01f);
            }
        }
        ParameterSet params;
        for (Layer* l: together.all()) l->collectParameters(params);
        report(std::string("parameter set: ") + (adam ? "Adam" : "SGD") + ": 5 tensors of three convolutions",
               params.tensors() == 5);
        bool same = true;
        for (int step = 1; step <= 2; ++step) {
            for (Net* n: nets) {
                n->ctx.timeStep = step;
                n->conv0->forward(input);
                n->pool1->forward(n->conv0->output());
                n->conv2->forward(n->pool1->output());
                n->short3->forward(n->conv2->output());
                n->up4->forward(n->short3->output());
                n->route5->forward(n->up4->output());
                n->conv6->forward(n->route5->output());
                n->yolo7->forward(n->conv6->output());
                n->yolo7->backward(n->conv6->output(), &n->conv6->delta());
                n->conv6->backward(n->route5->output(), &n->route5->delta());
                n->route5->backward(n->up4->output(), &n->up4->delta());
                n->up4->backward(n->short3->output(), &n->short3->delta());
                n->short3->backward(n->conv2->output(), &n->conv2->delta());
                n->conv2->backward(n->pool1->output(), &n->pool1->delta());
                n->pool1->backward(n->conv0->output(), &n->conv0->delta());
                n->conv0->backward(input, nullptr);
            }
            for (Layer* l: byLayer.all()) l->update();
            params.update(together.ctx);
            for (Layer* l: together.all()) l->parametersUpdated();
            // the deltas went through the helpers once more on both sides
            same = same && together.conv0->delta().asVector() == byLayer.conv0->delta().asVector() &&
                   together.short3->delta().asVector() == byLayer.short3->delta().asVector() &&
                   together.yolo7->delta().asVector() == byLayer.yolo7->delta().asVector() &&
                   together.conv0->scales().asVector() == byLayer.conv0->scales().asVector() &&
                   together.conv0->biases().asVector() == byLayer.conv0->biases().asVector() &&
                   together.conv2->scales().asVector() == byLayer.conv2->scales().asVector() &&
                   together.conv2->biases().asVector() == byLayer.conv2->biases().asVector() &&
                   together.conv6->biases().asVector() == byLayer.conv6->biases().asVector();
            report(std::string("parameter set: ") + (adam ? "Adam" : "SGD") + " step " + std::to_string(step) +
                   " leaves every tensor as the layers' own update does", same);
        }
        const Host moved = together.conv0->scales().asVector();
        report(std::string("parameter set: ") + (adam ? "Adam" : "SGD") + ": the parameters moved", moved != together.scale0);
    }
}

// A residual block whose shortcut overwrites the two deltas it is the first to write: the same
// gradients as the clearing-and-accumulating form, with the two zero-fills gone.
void firstWriterShortcutChecks()
{
    struct Block {
        Context ctx;
        std::shared_ptr<ConvLayer> a, b, c;
        std::shared_ptr<ShortcutLayer> add;
        Block(bool firstWriter, float threshold, float clip)
        {
            ctx.training = true;
            const Properties conv{ { "batch", N }, { "channels", C }, { "height", S }, { "width", S }, { "filters", C },
                                   { "batch_normalize", true }, { "activation", std::string("leaky") } };
            a = std::make_shared<ConvLayer>(ctx, conv);
            b = std::make_shared<ConvLayer>(ctx, conv);
            c = std::make_shared<ConvLayer>(ctx, conv);
            add = std::make_shared<ShortcutLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S },
                                                                   { "width", S }, { "first_writer", firstWriter } }, a);
            if (firstWriter) c->setFirstConsumerOverwrites(true);
            for (Layer* l: { static_cast<Layer*>(a.get()), static_cast<Layer*>(b.get()), static_cast<Layer*>(c.get()),
                             static_cast<Layer*>(add.get()) }) {
                l->setGradientRescaling(threshold > 0.0f, threshold);
                l->setGradientClipping(clip > 0.0f, clip);
            }
        }
        void step(const FloatVector& input, const Host& outDelta)
        {
            a->forward(input);
            b->forward(a->output());
            c->forward(b->output());
            add->forward(c->output());
            add->delta().copyHost(outDelta);
            add->backward(c->output(), &c->delta());
            c->backward(b->output(), &b->delta());
            b->backward(a->output(), &a->delta());
            a->backward(input, nullptr);
        }
    };
    const FloatVector input(normals(701, size_t(N) * C * S * S));
    double norm = 0.0;
    for (float v: normals(702, size_t(N) * C * S * S)) norm += double(v) * v;
    norm = std::sqrt(norm);
    // with the layers' gradient helpers on, the first writer's rescale + clip and its backward are one call
    // that reads the delta once (pxh_shortcut_backward_clipped): the same values again
    struct Case { const char* name; float threshold, clip; };
    const Case cases[] = { { "helpers off", 0.0f, 0.0f }, { "below the threshold", float(4.0 * norm), 0.0f },
                           { "rescaled", float(0.5 * norm), 0.0f }, { "rescaled and clamped", float(0.5 * norm), 0.25f } };
    for (const Case& k: cases) {
        Block plain(false, k.threshold, k.clip), first(true, k.threshold, k.clip);
        report("the shortcut marks its from layer", first.a->firstConsumerOverwrites() &&
                                                    !plain.a->firstConsumerOverwrites() && !first.b->firstConsumerOverwrites());
        for (int round = 0; round < 2; ++round) {
            const Host outDelta = normals(702 + round, size_t(N) * C * S * S);
            // stale values where the fill used to be: they must not survive
            first.a->delta().fill(std::nanf(""));
            first.c->delta().fill(std::nanf(""));
            plain.step(input, outDelta);
            first.step(input, outDelta);
            const std::string tag = std::string(" (") + k.name + ", step " + std::to_string(round + 1) + ")";
            expectClose("first-writer block: delta of the layer in front" + tag, first.c->delta().asVector(),
                        plain.c->delta().asVector(), 0.0, 1.0);
            expectClose("first-writer block: delta of the from layer" + tag, first.a->delta().asVector(),
                        plain.a->delta().asVector(), 0.0, 1.0);
            expectClose("first-writer block: the shortcut's own delta" + tag, first.add->delta().asVector(),
                        plain.add->delta().asVector(), 0.0, 1.0);
            expectClose("first-writer block: scale updates of the from layer" + tag, first.a->scaleUpdates().asVector(),
                        plain.a->scaleUpdates().asVector(), 0.0, 1.0);
        }
    }
}

// A residual block whose shortcut leaves the norm and peak of the delta it writes last: the rescale +
// clip that opens the backward of the layer in front starts from them instead of reading the tensor,
// and every gradient behind it is the same to the bit -- below the threshold, above it, and clamped.
void leavesNormShortcutChecks()
{
    struct Block {
        Context ctx;
        std::shared_ptr<ConvLayer> a, b, c;
        std::shared_ptr<ShortcutLayer> add;
        Block(bool leavesNorm, bool firstWriter, float threshold, float clip)
        {
            ctx.training = true;
            const Properties conv{ { "batch", N }, { "channels", C }, { "height", S }, { "width", S }, { "filters", C },
                                   { "batch_normalize", true }, { "activation", std::string("leaky") } };
            a = std::make_shared<ConvLayer>(ctx, conv);
            b = std::make_shared<ConvLayer>(ctx, conv);
            c = std::make_shared<ConvLayer>(ctx, conv);
            add = std::make_shared<ShortcutLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S },
                                                                   { "width", S }, { "first_writer", firstWriter },
                                                                   { "leaves_norm", leavesNorm } }, a);
            if (firstWriter) c->setFirstConsumerOverwrites(true);
            for (auto* l: { a.get(), b.get(), c.get() }) {
                l->setGradientRescaling(threshold > 0.0f, threshold);
                l->setGradientClipping(clip > 0.0f, clip);
            }
        }
        void step(const FloatVector& input, const Host& outDelta)
        {
            a->forward(input);
            b->forward(a->output());
            c->forward(b->output());
            add->forward(c->output());
            add->delta().copyHost(outDelta);
            add->backward(c->output(), &c->delta());
            c->backward(b->output(), &b->delta());
            b->backward(a->output(), &a->delta());
            a->backward(input, nullptr);
        }
    };
    const FloatVector input(normals(711, size_t(N) * C * S * S));
    const Host outDelta = normals(712, size_t(N) * C * S * S);
    double norm = 0.0;
    for (float v: outDelta) norm += double(v) * v;
    norm = std::sqrt(norm);
    struct Case { const char* name; float threshold, clip; };
    const Case cases[] = { { "below the threshold", float(4.0 * norm), 0.0f }, { "rescaled", float(0.5 * norm), 0.0f },
                           { "rescaled and clamped", float(0.5 * norm), 0.25f }, { "helpers off", 0.0f, 0.0f } };
    for (const bool firstWriter: { false, true }) {
        for (const Case& k: cases) {
            Block plain(false, firstWriter, k.threshold, k.clip), fused(true, firstWriter, k.threshold, k.clip);
            for (int round = 0; round < 2; ++round) {
                plain.step(input, outDelta);
                fused.step(input, outDelta);
                const std::string tag = std::string(" (") + k.name + (firstWriter ? ", first writer" : "") + ", step " +
                                        std::to_string(round + 1) + ")";
                report("norm from the shortcut: delta behind the layer in front" + tag,
                       fused.b->delta().asVector() == plain.b->delta().asVector());
                report("norm from the shortcut: scale updates of the layer in front" + tag,
                       fused.c->scaleUpdates().asVector() == plain.c->scaleUpdates().asVector());
                report("norm from the shortcut: delta of the from layer" + tag,
                       fused.a->delta().asVector() == plain.a->delta().asVector());
            }
            report(std::string("norm from the shortcut: the note is taken (") + k.name + ")",
                   fused.ctx.takeNormGroups(fused.c->delta().data()) == nullptr);
        }
    }
}

// A residual block whose shortcut rides on the epilogue of the convolution in front of it: that
// convolution writes the shortcut's output (its own is never formed) and takes the shortcut's delta as its
// own.  Output, every gradient behind it and every update buffer are those of the two layers one after the
// other, bit for bit -- helpers off, below the threshold, rescaled, clamped; training and inference.
void ridingShortcutChecks()
{
    struct Block {
        Context ctx;
        std::shared_ptr<ConvLayer> a, b, c;
        std::shared_ptr<ShortcutLayer> add;
        Block(bool riding, bool firstWriter, bool training, float threshold, float clip)
        {
            ctx.training = training;
            const Properties conv{ { "batch", N }, { "channels", C }, { "height", S }, { "width", S }, { "filters", C },
                                   { "batch_normalize", true }, { "activation", std::string("leaky") } };
            a = std::make_shared<ConvLayer>(ctx, conv);
            b = std::make_shared<ConvLayer>(ctx, conv);
            c = std::make_shared<ConvLayer>(ctx, conv);
            add = std::make_shared<ShortcutLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S },
                                                                   { "width", S }, { "first_writer", firstWriter },
                                                                   { "beta", 0.75f } }, a);
            if (firstWriter) c->setFirstConsumerOverwrites(true);
            if (riding) add->rideOn(*c);
            int seed = 730;
            for (auto* l: { a.get(), b.get(), c.get() }) {
                l->copyScales(normals(seed++, C));
                l->copyBiases(normals(seed++, C));
                l->copyRollingMean(normals(seed++, C));
                Host var = normals(seed++, C);
                for (float& v: var) v = 0.5f + v * v;
                l->copyRollingVariance(var);
            }
            for (Layer* l: { static_cast<Layer*>(a.get()), static_cast<Layer*>(b.get()), static_cast<Layer*>(c.get()),
                             static_cast<Layer*>(add.get()) }) {
                l->setGradientRescaling(threshold > 0.0f, threshold);
                l->setGradientClipping(clip > 0.0f, clip);
            }
        }
        void forward(const FloatVector& input)
        {
            a->forward(input);
            b->forward(a->output());
            c->forward(b->output());
            add->forward(c->output());
        }
        void step(const FloatVector& input, const Host& outDelta)
        {
            forward(input);
            add->delta().copyHost(outDelta);
            add->backward(c->output(), &c->delta());
            c->backward(b->output(), &b->delta());
            b->backward(a->output(), &a->delta());
            a->backward(input, nullptr);
        }
    };
    const FloatVector input(normals(721, size_t(N) * C * S * S));
    const Host outDelta = normals(722, size_t(N) * C * S * S);
    double norm = 0.0;
    for (float v: outDelta) norm += double(v) * v;
    norm = std::sqrt(norm);
    {
        Block plain(false, false, false, 0.0f, 0.0f), riding(true, false, false, 0.0f, 0.0f);
        plain.forward(input);
        riding.forward(input);
        report("riding shortcut: output at inference", riding.add->output().asVector() == plain.add->output().asVector());
        report("riding shortcut: the convolution says so", riding.c->carriesShortcut() && !plain.c->carriesShortcut());
    }
    struct Case { const char* name; float threshold, clip; };
    const Case cases[] = { { "helpers off", 0.0f, 0.0f }, { "below the threshold", float(4.0 * norm), 0.0f },
                           { "rescaled", float(0.5 * norm), 0.0f }, { "rescaled and clamped", float(0.5 * norm), 0.25f } };
    for (const bool firstWriter: { false, true }) {
        for (const Case& k: cases) {
            Block plain(false, firstWriter, true, k.threshold, k.clip), riding(true, firstWriter, true, k.threshold, k.clip);
            for (int round = 0; round < 2; ++round) {
                plain.step(input, outDelta);
                riding.step(input, outDelta);
                const std::string tag = std::string(" (") + k.name + (firstWriter ? ", first writer" : "") + ", step " +
                                        std::to_string(round + 1) + ")";
                report("riding shortcut: output" + tag, riding.add->output().asVector() == plain.add->output().asVector());
                report("riding shortcut: delta behind the convolution" + tag,
                       riding.b->delta().asVector() == plain.b->delta().asVector());
                report("riding shortcut: the convolution's updates" + tag,
                       riding.c->scaleUpdates().asVector() == plain.c->scaleUpdates().asVector() &&
                       riding.c->biasUpdates().asVector() == plain.c->biasUpdates().asVector());
                report("riding shortcut: delta and updates of the from layer" + tag,
                       riding.a->delta().asVector() == plain.a->delta().asVector() &&
                       riding.a->scaleUpdates().asVector() == plain.a->scaleUpdates().asVector());
            }
        }
    }
    expectThrows("a shortcut with an activation of its own does not ride", [] {
        Context ctx;
        const Properties conv{ { "batch", N }, { "channels", C }, { "height", S }, { "width", S }, { "filters", C },
                               { "batch_normalize", true } };
        auto a = std::make_shared<ConvLayer>(ctx, conv);
        ShortcutLayer add(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S }, { "width", S },
                                           { "activation", std::string("leaky") } }, a);
        add.rideOn(*a);
    }, "linear");
}

// At inference a 2 x 2 / 2 max-pool rides on the epilogue of the convolution in front of it: the pool's output
// is that of the two layers one after the other, bit for bit; the convolution's own output is written only
// when something else reads it.
void ridingPoolChecks()
{
    struct Pair {
        Context ctx;
        std::shared_ptr<ConvLayer> conv;
        std::shared_ptr<MaxPoolLayer> pool;
        Pair(bool riding, bool keep)
        {
            ctx.training = false;
            conv = std::make_shared<ConvLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S },
                                                                { "width", S }, { "filters", C },
                                                                { "batch_normalize", true },
                                                                { "activation", std::string("leaky") } });
            pool = std::make_shared<MaxPoolLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S },
                                                                   { "width", S }, { "kernel", 2 }, { "stride", 2 } });
            conv->copyScales(normals(741, C));
            conv->copyBiases(normals(742, C));
            conv->copyRollingMean(normals(743, C));
            Host var = normals(744, C);
            for (float& v: var) v = 0.5f + v * v;
            conv->copyRollingVariance(var);
            if (riding) pool->rideOn(*conv, keep);
        }
        void forward(const FloatVector& input)
        {
            conv->forward(input);
            pool->forward(conv->output());
        }
    };
    const FloatVector input(normals(745, size_t(N) * C * S * S));
    Pair plain(false, false), riding(true, false), keeping(true, true);
    plain.forward(input);
    riding.forward(input);
    keeping.forward(input);
    report("riding pool: the convolution says so", riding.conv->carriesPool() && !plain.conv->carriesPool());
    report("riding pool: the pool's output", riding.pool->output().asVector() == plain.pool->output().asVector());
    report("riding pool: the pool's output, the convolution's kept",
           keeping.pool->output().asVector() == plain.pool->output().asVector());
    report("riding pool: the convolution's output when kept",
           keeping.conv->output().asVector() == plain.conv->output().asVector());
    expectThrows("a pool does not ride in training", [] {
        Context ctx;
        ctx.training = true;
        ConvLayer conv(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S }, { "width", S }, { "filters", C },
                                        { "batch_normalize", true } });
        MaxPoolLayer pool(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S }, { "width", S },
                                           { "kernel", 2 }, { "stride", 2 } });
        pool.rideOn(conv, false);
    }, "inference");
}

// The small network with the shortcut and the head leaving the norms of the deltas they write last
// (conv2's and conv6's): every delta and every update buffer as without, bit for bit.
void leavesNormNetChecks()
{
    Net plain(true), fused(true, true);
    const auto truth = makeTruth();
    FloatVector input(size_t(N) * C * S * S);
    input.copyHost(normals(910, input.size()));
    Net* nets[2] = { &plain, &fused };
    for (int step = 1; step <= 2; ++step) {
        for (Net* n: nets) {
            n->ctx.setGroundTruth(truth);
            for (Layer* l: n->all()) {
                l->setGradientRescaling(true, step == 1 ? 0.05f : 1e6f);      // bites on the first step only
                l->setGradientClipping(true, 0.01f);
            }
            n->conv0->forward(input);
            n->pool1->forward(n->conv0->output());
            n->conv2->forward(n->pool1->output());
            n->short3->forward(n->conv2->output());
            n->up4->forward(n->short3->output());
            n->route5->forward(n->up4->output());
            n->conv6->forward(n->route5->output());
            n->yolo7->forward(n->conv6->output());
            n->yolo7->backward(n->conv6->output(), &n->conv6->delta());
            n->conv6->backward(n->route5->output(), &n->route5->delta());
            n->route5->backward(n->up4->output(), &n->up4->delta());
            n->up4->backward(n->short3->output(), &n->short3->delta());
            n->short3->backward(n->conv2->output(), &n->conv2->delta());
            n->conv2->backward(n->pool1->output(), &n->pool1->delta());
            n->pool1->backward(n->conv0->output(), &n->conv0->delta());
            n->conv0->backward(input, nullptr);
        }
        const bool same = fused.conv6->delta().asVector() == plain.conv6->delta().asVector() &&
                          fused.conv6->biasUpdates().asVector() == plain.conv6->biasUpdates().asVector() &&
                          fused.conv2->delta().asVector() == plain.conv2->delta().asVector() &&
                          fused.conv2->scaleUpdates().asVector() == plain.conv2->scaleUpdates().asVector() &&
                          fused.pool1->delta().asVector() == plain.pool1->delta().asVector() &&
                          fused.conv0->delta().asVector() == plain.conv0->delta().asVector() &&
                          fused.conv0->scaleUpdates().asVector() == plain.conv0->scaleUpdates().asVector();
        report("norms from the shortcut and the head: every gradient as without, step " + std::to_string(step), same);
    }
    const Host moved = fused.conv0->scaleUpdates().asVector();
    bool any = false;
    for (float v: moved) any = any || v != 0.0f;
    report("norms from the shortcut and the head: gradients reached the first layer", any);
}

// A model's weights file: header of either seen-width, every layer's section in network order, exact length.
// Two heads that wait for the end of the forward pass and run as one pass give what each gives alone.
void deferredHeadsChecks()
{
    const std::vector<int> anchors{ 10, 14, 23, 27, 37, 58, 81, 82 };
    struct Pair {
        Context ctx;
        std::shared_ptr<YoloLayer> small, large;
    };
    const auto build = [&](Pair& p, bool deferred) {
        p.ctx.training = true;
        p.ctx.width = p.ctx.height = 128;
        p.ctx.classes = CLASSES;
        p.small = std::make_shared<YoloLayer>(p.ctx, Properties{ { "batch", N }, { "channels", 2 * (CLASSES + 5) },
                                                                 { "height", 5 }, { "width", 5 }, { "num", 4 },
                                                                 { "mask", std::vector<int>{ 2, 3 } },
                                                                 { "anchors", anchors }, { "ignore_thresh", 0.5f },
                                                                 { "object_scale", 2.0f }, { "deferred", deferred } });
        p.large = std::make_shared<YoloLayer>(p.ctx, Properties{ { "batch", N }, { "channels", 2 * (CLASSES + 5) },
                                                                 { "height", 12 }, { "width", 12 }, { "num", 4 },
                                                                 { "mask", std::vector<int>{ 0, 1 } },
                                                                 { "anchors", anchors }, { "ignore_thresh", 0.7f },
                                                                 { "noobject_scale", 0.5f }, { "deferred", deferred } });
        std::vector<GroundTruthVec> truth(N);
        Rng r(77);
        for (int b = 0; b < N; ++b)
            for (int t = 0; t < 1 + b % 3; ++t)
                truth[b].push_back(GroundTruth{ r.uniform(), r.uniform(), 0.05f + 0.5f * r.uniform(),
                                                0.05f + 0.5f * r.uniform(), static_cast<int>(r.next() % CLASSES) });
        p.ctx.setGroundTruth(truth);
    };
    Pair apart, together;
    build(apart, false);
    build(together, true);
    Layer::V inSmall(static_cast<size_t>(N) * 2 * (CLASSES + 5) * 25), inLarge(static_cast<size_t>(N) * 2 * (CLASSES + 5) * 144);
    inSmall.copyHost(normals(78, inSmall.size(), 1.5f));
    inLarge.copyHost(normals(79, inLarge.size(), 1.5f));
    apart.small->forward(inSmall);
    apart.large->forward(inLarge);
    together.small->forward(inSmall);
    together.large->forward(inLarge);
    report("deferred heads wait for the end of the pass", together.ctx.deferredHeads.size() == 2);
    YoloLayer::forwardDeferred(together.ctx);
    report("... and are gone from the list once run", together.ctx.deferredHeads.empty());
    expectExact("deferred small head: output", together.small->output().asVector(), apart.small->output().asVector());
    expectExact("deferred small head: delta", together.small->delta().asVector(), apart.small->delta().asVector());
    expectExact("deferred large head: output", together.large->output().asVector(), apart.large->output().asVector());
    expectExact("deferred large head: delta", together.large->delta().asVector(), apart.large->delta().asVector());
    expectClose("deferred small head: cost", Host{ together.small->fetchCost() }, Host{ apart.small->fetchCost() }, 1e-6, 1e-3);
    expectClose("deferred large head: cost", Host{ together.large->fetchCost() }, Host{ apart.large->fetchCost() }, 1e-6, 1e-3);
    expectClose("deferred large head: statistics", together.large->fetchStats(), apart.large->fetchStats(), 1e-5, 1.0);
}

void weightsFileChecks()
{
    auto build = [](Context& ctx) {
        std::vector<Layer::Ptr> layers;
        layers.push_back(std::make_shared<ConvLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S },
                                                                      { "width", S }, { "filters", C }, { "weights", 27 * C },
                                                                      { "batch_normalize", true } }));
        layers.push_back(std::make_shared<MaxPoolLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S },
                                                                         { "width", S }, { "kernel", 2 }, { "stride", 2 } }));
        layers.push_back(std::make_shared<BatchNormLayer>(ctx, Properties{ { "batch", N }, { "channels", C },
                                                                           { "height", S / 2 }, { "width", S / 2 } }));
        layers.push_back(std::make_shared<ConvLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S / 2 },
                                                                      { "width", S / 2 }, { "filters", 5 },
                                                                      { "weights", 5 * C } }));
        return layers;
    };
    Context ctx;
    auto source = build(ctx);
    auto* conv = static_cast<ConvLayer*>(source[0].get());
    conv->copyBiases(normals(601, C, 0.1f)); conv->copyScales(uniforms(602, C, 0.5f, 1.5f));
    conv->copyRollingMean(normals(603, C, 0.1f)); conv->copyRollingVariance(uniforms(604, C, 0.5f, 1.5f));
    conv->weights().copyHost(normals(605, 27 * C, 0.02f));
    auto* last = static_cast<ConvLayer*>(source[3].get());
    last->copyBiases(normals(606, 5, 0.1f));
    last->weights().copyHost(normals(607, 5 * C, 0.02f));
    for (const bool wide: { false, true }) {
        WeightsHeader h;
        if (wide) { h.major = 0; h.minor = 2; }
        h.seen = wide ? 0x123456789aull : 64000u;
        std::stringstream file(std::ios::in | std::ios::out | std::ios::binary);
        saveWeightsFile(file, h, source);
        const size_t floats = (4 * C + 27 * C) + 4 * C + (5 + 5 * C);
        report(std::string("weights file length, ") + (wide ? "64-bit" : "32-bit") + " seen",
               file.str().size() == 12 + (wide ? 8 : 4) + floats * sizeof(float));
        auto target = build(ctx);
        const WeightsHeader back = loadWeightsFile(file, target);
        report("weights file header round trip", back.major == h.major && back.minor == h.minor && back.seen == h.seen);
        report("weights file restores every layer",
               static_cast<ConvLayer*>(target[0].get())->weights().asVector() == conv->weights().asVector() &&
               static_cast<ConvLayer*>(target[0].get())->rollingVariance().asVector() == conv->rollingVariance().asVector() &&
               static_cast<ConvLayer*>(target[3].get())->biases().asVector() == last->biases().asVector() &&
               static_cast<ConvLayer*>(target[3].get())->weights().asVector() == last->weights().asVector());
        std::stringstream longer(file.str() + "tail", std::ios::in | std::ios::binary);
        expectThrows("trailing bytes are refused", [&] { loadWeightsFile(longer, target); }, "Did not fully read");
        std::stringstream shorter(file.str().substr(0, file.str().size() - 8), std::ios::in | std::ios::binary);
        expectThrows("a truncated file is refused", [&] { loadWeightsFile(shorter, target); }, "Could not read");
    }
}

// An upsample layer absorbed by the route that reads it gives the same tensors as the two-step form.
void absorbedUpsampleChecks()
{
    struct Pair {
        Context ctx;
        std::shared_ptr<UpsampleLayer> up;
        std::shared_ptr<MaxPoolLayer> pool;
        std::shared_ptr<RouteLayer> route;
        explicit Pair(bool absorb)
        {
            ctx.training = true;
            up = std::make_shared<UpsampleLayer>(ctx, Properties{ { "batch", N }, { "channels", C }, { "height", S / 2 },
                                                                  { "width", S / 2 }, { "stride", 2 },
                                                                  { "scale", 0.5f } });
            pool = std::make_shared<MaxPoolLayer>(ctx, Properties{ { "batch", N }, { "channels", 3 }, { "height", 2 * S },
                                                                   { "width", 2 * S }, { "kernel", 2 }, { "stride", 2 } });
            route = std::make_shared<RouteLayer>(ctx, Properties{ { "batch", N }, { "channels", C + 3 }, { "height", S },
                                                                  { "width", S }, { "absorb_upsample", absorb } },
                                                 std::vector<Layer::Ptr>{ pool, up });
        }
    };
    Pair plain(false), fused(true);
    report("absorbed upsample releases its own tensors",
           fused.up->writesIntoConsumer() && fused.up->output().empty() && !plain.up->writesIntoConsumer());
    const FloatVector small(normals(301, size_t(N) * C * (S / 2) * (S / 2)));
    const FloatVector large(normals(302, size_t(N) * 3 * 2 * S * 2 * S));
    const Host routeDelta = normals(303, size_t(N) * (C + 3) * S * S);
    const Host grad0 = normals(304, small.size());
    Host out[2], upGrad[2], poolDelta[2];
    int k = 0;
    for (Pair* net: { &plain, &fused }) {
        net->pool->forward(large);
        net->up->forward(small);
        net->route->forward(net->up->output());
        out[k] = net->route->output().asVector();
        net->route->delta().copyHost(routeDelta);
        FloatVector grad(grad0);
        net->route->backward(net->up->output(), nullptr);
        net->up->backward(small, &grad);
        upGrad[k] = grad.asVector();
        poolDelta[k] = net->pool->delta().asVector();
        ++k;
    }
    expectExact("route output with an absorbed upsample", out[1], out[0]);
    expectExact("upsample backward from the route's delta slice", upGrad[1], upGrad[0]);
    expectExact("other route source's delta unchanged", poolDelta[1], poolDelta[0]);
}

}   // namespace

int main(int argc, char** argv)
{
    const bool cpuOnly = argc > 1 && std::strcmp(argv[1], "--cpu") == 0;
    try {
        hostOnlyChecks();
        if (!cpuOnly) {
            int devices = 0;
            if (hipGetDeviceCount(&devices) != hipSuccess || devices == 0) {
                std::printf("no GPU visible\n");
                return 2;
            }
            deviceVectorChecks();
            inferenceChecks();
            trainingChecks();
            absorbedUpsampleChecks();
            batchNormLayerChecks();
            weightsFileChecks();
            firstWriterShortcutChecks();
            leavesNormShortcutChecks();
            ridingShortcutChecks();
            ridingPoolChecks();
            leavesNormNetChecks();
            deferredHeadsChecks();
            capturedSequenceChecks();
            parameterSetChecks();
        }
    } catch (const std::exception& e) {
        std::printf("unexpected exception: %s\n", e.what());
        return 3;
    }
    std::printf("%d checks, %d failed\n", checks, failures);
    return failures ? 1 : 0;
}

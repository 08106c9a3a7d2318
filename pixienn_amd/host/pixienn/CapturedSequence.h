// A sequence of layer calls recorded once as a HIP graph and replayed with one launch.
//
// The reference issues every kernel from the host, layer by layer (Model<D>::forward / backward,
// include/Model.h:1740-1792); at batch 16 most of the small layers of a YOLO network run for less
// time than their launch takes.  Every entry point of the kernel library only enqueues work on the
// caller's stream -- no allocation once the library's workspace exists, no memset, no host
// synchronisation -- so a model's whole forward, backward or update over fixed buffers can be
// captured and replayed.  What changes between replays has to live in device memory (inputs,
// ground truth): host scalars such as Adam's step count are baked in at capture time.
#pragma once

#include <utility>

#include "Error.h"

namespace px::hip {

class CapturedSequence
{
public:
    CapturedSequence() = default;
    CapturedSequence(const CapturedSequence&) = delete;
    CapturedSequence& operator=(const CapturedSequence&) = delete;
    ~CapturedSequence() { reset(); }

    // Records what `body` enqueues on `stream` (not the null stream).  Run the sequence once eagerly
    // before capturing it: the first call of some entry points sizes the library's workspace.
    template<typename Body>
    void capture(hipStream_t stream, Body&& body)
    {
        PX_CHECK(stream != nullptr, "a sequence is captured on a stream of its own, not on the null stream");
        reset();
        PX_HIP_RUNTIME_CHECK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
        try {
            std::forward<Body>(body)();
        } catch (...) {
            hipGraph_t abandoned = nullptr;
            (void) hipStreamEndCapture(stream, &abandoned);
            if (abandoned) (void) hipGraphDestroy(abandoned);
            throw;
        }
        PX_HIP_RUNTIME_CHECK(hipStreamEndCapture(stream, &graph_));
        PX_HIP_RUNTIME_CHECK(hipGraphInstantiate(&exec_, graph_, nullptr, nullptr, 0));
    }

    bool captured() const noexcept { return exec_ != nullptr; }

    // Enqueues the whole recorded sequence on `stream`.
    void replay(hipStream_t stream)
    {
        PX_CHECK(exec_ != nullptr, "nothing has been captured");
        PX_HIP_RUNTIME_CHECK(hipGraphLaunch(exec_, stream));
    }

    void reset() noexcept
    {
        if (exec_) (void) hipGraphExecDestroy(exec_);
        if (graph_) (void) hipGraphDestroy(graph_);
        exec_ = nullptr;
        graph_ = nullptr;
    }

private:
    hipGraph_t graph_ = nullptr;
    hipGraphExec_t exec_ = nullptr;
};

}   // px::hip

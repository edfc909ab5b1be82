#include "DeviceGraph.h"

#include <string>

#include "AutoDiff.h"
#include "Ctorch_Error.h"
#include "ctorch_amd.h"
#include "kernels.h"

using namespace ctorch_amd_host;

namespace {
[[noreturn]] void graph_error(const char* what) {
    Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::PLATFORM_API, std::string(what) + ": " + ctamd_last_error());
}

// One stream for every graph of the process: graphs are recorded on it and replayed on it, so the
// replays of different graphs run in the order they were issued (they share the device scratch
// and, often, tensors).  It is an ordinary blocking stream of default priority: work on the null
// stream - everything the front-end launches outside a recording - waits for it and it waits for
// that work, which orders replays against eager launches as well.  Kept until the process ends.
void* graph_stream() {
    static void* stream = nullptr;
    if (!stream && ctamd_stream_create(&stream) != CTAMD_OK) graph_error("ctamd_stream_create");
    return stream;
}
}  // namespace

DeviceGraph::~DeviceGraph() {
    if (stream_) ctamd_sync(stream_);
    if (graph_) ctamd_graph_destroy(graph_);
    reservation_destroy(reservation_);
}

void DeviceGraph::record(const std::function<void()>& body) {
    if (graph_) Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::TENSOR_STATE, "DeviceGraph: already recorded");
    init_device();
    stream_ = graph_stream();
    prepare_backward_seed();                        // made and filled now, not as a recorded launch in this graph's memory
    device_sync();                                  // earlier work on the null stream is done
    if (ctamd_sync(stream_) != CTAMD_OK) graph_error("ctamd_sync");   // and so are earlier replays
    void* outer = current_stream();
    reservation_destroy(reservation_);              // of a recording that failed earlier
    reservation_ = reservation_begin();
    set_current_stream(stream_);
    if (ctamd_graph_begin(stream_) != CTAMD_OK) {
        set_current_stream(outer);
        reservation_stop();
        graph_error("ctamd_graph_begin");
    }
    set_recording(true);
    bool failed = false;
    std::string why;
    try {
        body();
    } catch (const std::exception& e) {
        failed = true;
        why = e.what();
    }
    set_recording(false);
    int rc = ctamd_graph_end(stream_, &graph_);     // always ends the recording, also after a failure
    set_current_stream(outer);
    reservation_stop();
    if (failed || rc != CTAMD_OK) {
        if (graph_) ctamd_graph_destroy(graph_);
        graph_ = nullptr;
        reservation_destroy(reservation_);          // nothing will replay into this memory
        reservation_ = nullptr;
    }
    if (failed) {
        Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::TENSOR_STATE, "DeviceGraph: the recorded body failed: " + why);
    }
    if (rc != CTAMD_OK) graph_error("ctamd_graph_end");
}

void DeviceGraph::replay() {
    if (!graph_) Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::TENSOR_STATE, "DeviceGraph: nothing recorded");
    if (ctamd_graph_launch(graph_, stream_) != CTAMD_OK) graph_error("ctamd_graph_launch");
}

void DeviceGraph::wait() {
    if (stream_ && ctamd_sync(stream_) != CTAMD_OK) graph_error("ctamd_sync");
}

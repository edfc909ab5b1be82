#include "DeviceGraph.h"

#include <string>

#include "Ctorch_Error.h"
#include "ctorch_amd.h"
#include "kernels.h"

using namespace ctorch_amd_host;

namespace {
[[noreturn]] void graph_error(const char* what) {
    Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::PLATFORM_API, std::string(what) + ": " + ctamd_last_error());
}
}  // namespace

DeviceGraph::~DeviceGraph() {
    if (graph_ || stream_) ctamd_sync(stream_);
    if (graph_) ctamd_graph_destroy(graph_);
    if (stream_) ctamd_stream_destroy(stream_);
    reservation_destroy(reservation_);
}

void DeviceGraph::record(const std::function<void()>& body) {
    if (graph_) Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::TENSOR_STATE, "DeviceGraph: already recorded");
    init_device();
    if (!stream_ && ctamd_stream_create(&stream_) != CTAMD_OK) graph_error("ctamd_stream_create");
    device_sync();                                  // earlier work on the null stream is done
    void* outer = current_stream();
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
    if (failed) {
        if (graph_) ctamd_graph_destroy(graph_);
        graph_ = nullptr;
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

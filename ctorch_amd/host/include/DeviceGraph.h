// A fixed sequence of device launches recorded once and replayed with a single launch (a HIP
// graph).  For steps that are launch-bound: a training step of a small model is tens of launches
// of a few microseconds of GPU work each, and issuing them costs about 3 us apiece; replayed as a
// graph the step costs one launch.  The reference has no counterpart (it is synchronous CPU code).
//
//   DeviceGraph g;
//   g.record([&] { loss = model.train_step_on_device(x, y); });   // runs the front-end once, recording
//   for (...) { /* refresh the contents of x and y in place */ g.replay(); }
//   float v = loss.item<float>();                                  // waits for the replays
//
// What is recorded are launches with the device addresses they had: tensors that the body reads
// must keep their storage (update them in place), and tensors it creates that are read afterwards
// must be kept alive by the caller.  All memory the body allocates stays reserved for the graph
// until it is destroyed.  While recording, anything that makes the host wait for the device
// (item(), to_vector(), transfers) throws.  The host-side work of the body - tape bookkeeping,
// shape checks - runs once, at recording time, not at replay.
#ifndef CTORCH_AMD_HOST_DEVICE_GRAPH_H
#define CTORCH_AMD_HOST_DEVICE_GRAPH_H

#include <functional>

#include "Storage.h"

class DeviceGraph {
   public:
    DeviceGraph() = default;
    ~DeviceGraph();
    DeviceGraph(const DeviceGraph&) = delete;
    DeviceGraph& operator=(const DeviceGraph&) = delete;

    void record(const std::function<void()>& body);
    void replay();             // asynchronous; ordered after everything issued before it: all graphs replay on one
                               // stream, which the launches outside recordings (null stream) wait for and which waits for them
    void wait();               // until the replays issued so far have finished
    bool recorded() const { return graph_ != nullptr; }

   private:
    void* stream_ = nullptr;
    void* graph_ = nullptr;
    ctorch_amd_host::BlockReservation* reservation_ = nullptr;
};

#endif

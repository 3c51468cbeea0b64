// Records the work enqueued inside a scope into a HIP graph and launches it when the scope ends. Mirrors
// include/common/SyclGraph.h:20-35 and source/common/SyclGraph.cpp:44-86 of the reference (capture_guard returns a
// scope guard; a null or already-recording stream records nothing) and its ScopeGuard (include/common/ScopeGuard.h).
// Every scope is recorded anew; an executable graph that exists already is updated in place when the new recording has the
// same shape (same kernels, other arguments), otherwise it is rebuilt.
#pragma once

#include <functional>
#include <utility>

#include "common.h"

namespace tinydpcppnn {

class ScopeGuard {
  public:
    ScopeGuard() = default;
    explicit ScopeGuard(std::function<void()> &&callback) : m_callback(std::move(callback)) {}
    ScopeGuard(ScopeGuard &&other) : m_callback(std::move(other.m_callback)) { other.m_callback = {}; }
    ScopeGuard &operator=(ScopeGuard &&other) {
        std::swap(m_callback, other.m_callback);
        return *this;
    }
    ScopeGuard(const ScopeGuard &) = delete;
    ScopeGuard &operator=(const ScopeGuard &) = delete;
    ~ScopeGuard() noexcept(false) {
        if (m_callback) m_callback();
    }

  private:
    std::function<void()> m_callback;
};

class HipGraph {
  public:
    HipGraph() = default;
    HipGraph(const HipGraph &) = delete;
    HipGraph &operator=(const HipGraph &) = delete;
    ~HipGraph() { reset(); }

    void reset() {
        if (m_exec) (void)hipGraphExecDestroy(m_exec);
        if (m_graph) (void)hipGraphDestroy(m_graph);
        m_exec = nullptr;
        m_graph = nullptr;
    }

    /// Starts recording `stream`; the returned guard stops the recording and launches the graph on the same stream.
    /// The legacy default stream cannot be recorded: work then runs as it is enqueued, as for a null pointer.
    ScopeGuard capture_guard(tnn::queue *stream) {
        if (stream == nullptr || stream->get() == nullptr) return ScopeGuard{};
        hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
        tnn::hip_check(hipStreamIsCapturing(stream->get(), &status), "hipStreamIsCapturing");
        if (status != hipStreamCaptureStatusNone) return ScopeGuard{}; // the caller is being recorded already
        tnn::hip_check(hipStreamBeginCapture(stream->get(), hipStreamCaptureModeRelaxed), "hipStreamBeginCapture");
        hipStream_t s = stream->get();
        return ScopeGuard{[this, s]() {
            if (m_graph) {
                (void)hipGraphDestroy(m_graph);
                m_graph = nullptr;
            }
            tnn::hip_check(hipStreamEndCapture(s, &m_graph), "hipStreamEndCapture");
            if (m_exec) {
                hipGraphExecUpdateResult result;
                hipGraphNode_t error_node = nullptr;
                if (hipGraphExecUpdate(m_exec, m_graph, &error_node, &result) != hipSuccess) {
                    (void)hipGetLastError();
                    (void)hipGraphExecDestroy(m_exec);
                    m_exec = nullptr;
                }
            }
            if (!m_exec) tnn::hip_check(hipGraphInstantiate(&m_exec, m_graph, nullptr, nullptr, 0), "hipGraphInstantiate");
            ++m_launches;
            tnn::hip_check(hipGraphLaunch(m_exec, s), "hipGraphLaunch");
            if (m_synchronize_when_capture_done) {
                tnn::hip_check(hipStreamSynchronize(s), "hipStreamSynchronize");
                m_synchronize_when_capture_done = false;
            }
        }};
    }

    void schedule_synchronize() { m_synchronize_when_capture_done = true; }
    size_t launches() const { return m_launches; }

  private:
    hipGraph_t m_graph = nullptr;
    hipGraphExec_t m_exec = nullptr;
    bool m_synchronize_when_capture_done = false;
    size_t m_launches = 0;
};

} // namespace tinydpcppnn

/*
 * The stream the library works on, and capture of its launches into a HIP
 * graph.
 *
 * Every kernel launch, asynchronous copy and memset of the library goes to the
 * calling thread's current stream: the null stream unless blt_hip_set_stream
 * chose another one (the reference's device backend runs everything on stream
 * 0, csrc/ops/memory.cu:37-77; that stays the default).
 *
 * blt_hip_capture_begin / _end record the launches issued in between on a
 * library-owned stream into an executable graph: a decode step of several
 * small kernels is then replayed with one graph launch instead of one
 * dispatch per kernel.  Entry points that would have to allocate or stage
 * through host memory while a capture is open end with a message instead of
 * recording something that cannot be replayed: warm the call up once, eagerly,
 * before capturing it.
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "launch.h"

namespace {

thread_local hipStream_t t_stream = nullptr;
thread_local hipStream_t t_saved = nullptr;
thread_local bool t_capturing = false;
thread_local bool t_captured_device_length_step = false; /* the open capture recorded a KV step that reads self_len on the device */
hipStream_t g_capture_stream = nullptr; /* default priority, non-blocking; lives until the process ends */

} // namespace

struct blt_hip_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    /* The graph holds a KV step with device-resident lengths: a replay can outgrow what the
     * captured launch was sized for, which its kernels report through the sticky device error
     * word; every replay therefore arms the host's look at that word. */
    bool device_length_step = false;
};

hipStream_t blt_stream() { return t_stream; }
hipStream_t blt_stream_key() { return t_capturing ? t_saved : t_stream; }
bool blt_stream_capturing() { return t_capturing; }
void blt_stream_note_device_length_step() {
    if (t_capturing) t_captured_device_length_step = true;
}

extern "C" void blt_hip_set_stream(void *stream) {
    BLT_REQUIRE(!t_capturing, "blt_hip_set_stream: a capture is open on this thread");
    t_stream = static_cast<hipStream_t>(stream);
}

extern "C" void *blt_hip_get_stream(void) { return t_stream; }

extern "C" void blt_hip_capture_begin(void) {
    BLT_REQUIRE(!t_capturing, "blt_hip_capture_begin: a capture is already open on this thread");
    BLT_REQUIRE(!blt_profile_is_open(), "blt_hip_capture_begin: close the kernel-time profile first");
    if (!g_capture_stream) HIP_CHECK(hipStreamCreateWithFlags(&g_capture_stream, hipStreamNonBlocking));
    HIP_CHECK(hipStreamSynchronize(t_stream)); /* work issued so far is not part of the graph and must be done */
    t_saved = t_stream;
    t_stream = g_capture_stream;
    HIP_CHECK(hipStreamBeginCapture(g_capture_stream, hipStreamCaptureModeThreadLocal));
    t_capturing = true;
    t_captured_device_length_step = false;
}

extern "C" blt_hip_graph *blt_hip_capture_end(void) {
    BLT_REQUIRE(t_capturing, "blt_hip_capture_end: no capture is open on this thread");
    blt_hip_graph *g = new blt_hip_graph();
    const hipError_t e = hipStreamEndCapture(g_capture_stream, &g->graph);
    t_capturing = false;
    t_stream = t_saved;
    if (e != hipSuccess || g->graph == nullptr) BLT_FATAL("blt_hip_capture_end: capture failed: %s", hipGetErrorString(e));
    HIP_CHECK(hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0));
    g->device_length_step = t_captured_device_length_step;
    return g;
}

extern "C" void blt_hip_graph_launch(const blt_hip_graph *g) {
    BLT_REQUIRE(g != NULL && g->exec != nullptr, "blt_hip_graph_launch: graph must not be NULL");
    BLT_REQUIRE(!t_capturing, "blt_hip_graph_launch: a capture is open on this thread");
    HIP_CHECK(hipGraphLaunch(g->exec, t_stream));
    if (g->device_length_step) blt_kv_arm_device_error_check();
}

extern "C" void blt_hip_graph_destroy(blt_hip_graph *g) {
    if (!g) return;
    HIP_CHECK(hipDeviceSynchronize());
    if (g->exec) HIP_CHECK(hipGraphExecDestroy(g->exec));
    if (g->graph) HIP_CHECK(hipGraphDestroy(g->graph));
    delete g;
}

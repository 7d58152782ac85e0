// Stream capture into an executable HIP graph, for callers that replay a fixed launch sequence
// (one micro-batch forward or backward of a stage: about a hundred kernels on static buffers).
// Capture records the launches without running them; the caller launches the graph afterwards.
// Every kernel of the sequence must have run once eagerly before it is captured: first launches
// configure kernel attributes, which a capturing stream does not accept.
#include "common.h"

extern "C" int bb_graph_begin(void* stream) {
    BB_REQUIRE(stream != nullptr, "bb_graph_begin: the default stream cannot be captured; pass a created stream");
    BB_HIP_CHECK(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
    return BB_OK;
}

extern "C" int bb_graph_end(void* stream, void** exec_out) {
    BB_REQUIRE(stream != nullptr && exec_out != nullptr, "bb_graph_end: null argument");
    *exec_out = nullptr;
    hipGraph_t graph = nullptr;
    BB_HIP_CHECK(hipStreamEndCapture((hipStream_t)stream, &graph));
    BB_REQUIRE(graph != nullptr, "bb_graph_end: the capture was invalidated");
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    BB_HIP_CHECK(e);
    *exec_out = (void*)exec;
    return BB_OK;
}

extern "C" int bb_graph_launch(void* exec, void* stream) {
    BB_REQUIRE(exec != nullptr, "bb_graph_launch: null graph");
    BB_HIP_CHECK(hipGraphLaunch((hipGraphExec_t)exec, (hipStream_t)stream));
    return BB_OK;
}

extern "C" int bb_graph_destroy(void* exec) {
    if (exec) BB_HIP_CHECK(hipGraphExecDestroy((hipGraphExec_t)exec));
    return BB_OK;
}

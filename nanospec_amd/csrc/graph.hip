// Capture of a stream's launches into a HIP graph and its replay: the decode step is launch-bound,
// so its kernels are recorded once per batch-size bucket and replayed as one submission.
// (reference: engine/graphs.py:171-210, which does the same with torch.cuda.CUDAGraph)
//
// Nothing captured here may be a memset node: buffers are cleared with ns_fill_u32.
#include "common.h"

extern "C" int ns_graph_begin(hipStream_t stream) {
  return (int)hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed);
}

extern "C" int ns_graph_end(hipStream_t stream, void** exec_out) {
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture(stream, &graph);
  if (e != hipSuccess) return (int)e;
  hipGraphExec_t exec = nullptr;
  e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) return (int)e;
  *exec_out = (void*)exec;
  return NS_OK;
}

extern "C" int ns_graph_launch(void* exec, hipStream_t stream) { return (int)hipGraphLaunch((hipGraphExec_t)exec, stream); }

extern "C" int ns_graph_destroy(void* exec) { return (int)hipGraphExecDestroy((hipGraphExec_t)exec); }

extern "C" const char* ns_error_string(int code) {
  if (code == NS_ERR_BAD_ARG) return "bad argument (a size the kernel does not take)";
  if (code == NS_ERR_UNSUPPORTED) return "unsupported dtype or option";
  if (code == NS_ERR_SCRATCH_TOO_SMALL) return "the product needs more partial sums than the library's own array holds";
  return hipGetErrorString((hipError_t)code);
}

// Diagnostic build only (make DIAG=-DBPSX_QUERY_TRACE OUT=../libbpsx_trace.so): a device buffer
// with start/end time (100 MHz wall clock), nodes expanded and cost class of every path search,
// and the one extra export that reads it.  Included twice by kernels.hip, never by the default
// build: first for the device buffer, then (BPSX_DIAG_TRACE_HOST) for the host reader.
#ifndef BPSX_DIAG_TRACE_HOST
__device__ unsigned long long g_trace[1 << 17][4];
__device__ unsigned int g_trace_n;
#else
// Copies up to max_rows rows of the trace to out ([row][4] u64) and clears it; returns the row count.
extern "C" __attribute__((visibility("default"))) int bpsx_debug_trace(unsigned long long* out, unsigned int max_rows) {
  unsigned int n = 0;
  (void)hipDeviceSynchronize();
  (void)hipMemcpyFromSymbol(&n, HIP_SYMBOL(g_trace_n), 4);
  if (n > (1u << 17)) n = 1u << 17;
  if (n > max_rows) n = max_rows;
  if (out && n) (void)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_trace), (size_t)n * 32);
  const unsigned int zero = 0;
  (void)hipMemcpyToSymbol(HIP_SYMBOL(g_trace_n), &zero, 4);
  return (int)n;
}
#endif

// libpkh3attn_bench.so: the measurement hook of include/pkh3_attn_bench.h, kept out of the product library because
// it synchronises with the device.  Links against libpkh3attn.so and launches its attention kernel.
#include "../../include/pkh3_attn_bench.h"

#include "pkh3_internal.h"

namespace pkh3 {
int prepare_call(const pkh3_attn_args* a, hipStream_t st, FwdParams* out);  // pkh3_api.hip
int report_error(int code, const char* text);                                // sets pkh3_last_error()
}  // namespace pkh3

using namespace pkh3;

extern "C" int pkh3_attn_time_kernel(const pkh3_attn_args* a, void* stream, int iters, float* ms_out) {
  if (!ms_out) return report_error(PKH3_ENULL, "ms_out is NULL");
  if (iters < 1) return report_error(PKH3_EARG, "iters must be >= 1");
  hipStream_t st = (hipStream_t)stream;
  FwdParams f;
  int rc = prepare_call(a, st, &f);
  if (rc) return rc;
  hipError_t e;
  if ((e = launch_attn_fwd(f, st)) != hipSuccess) return report_error(PKH3_EHIP, hipGetErrorString(e));  // warm
  hipEvent_t e0, e1;
  if ((e = hipEventCreate(&e0)) != hipSuccess) return report_error(PKH3_EHIP, hipGetErrorString(e));
  if ((e = hipEventCreate(&e1)) != hipSuccess) {
    hipEventDestroy(e0);
    return report_error(PKH3_EHIP, hipGetErrorString(e));
  }
  hipEventRecord(e0, st);
  for (int i = 0; i < iters; ++i)
    if ((e = launch_attn_fwd(f, st)) != hipSuccess) break;
  hipEventRecord(e1, st);
  const hipError_t es = hipEventSynchronize(e1);
  float ms = 0.f;
  if (e == hipSuccess && es == hipSuccess) hipEventElapsedTime(&ms, e0, e1);
  hipEventDestroy(e0);
  hipEventDestroy(e1);
  if (e != hipSuccess) return report_error(PKH3_EHIP, hipGetErrorString(e));
  if (es != hipSuccess) return report_error(PKH3_EHIP, hipGetErrorString(es));
  *ms_out = ms / iters;
  return PKH3_OK;
}

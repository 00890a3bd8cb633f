// Status strings and the last-HIP-error slot of libquik_hip.so.
#include "common.h"

#include <atomic>
#include <cstring>

namespace quik {
namespace {
thread_local char g_last_error[256] = "";
}

void set_last_hip_error(hipError_t e) {
  std::strncpy(g_last_error, hipGetErrorString(e), sizeof(g_last_error) - 1);
  g_last_error[sizeof(g_last_error) - 1] = '\0';
}

// Compute units of the GPU (all GPUs of a box are the same part: asked once per process; 256 when no device answers,
// e.g. for the size queries on a machine without a GPU).
int num_cus() {
  static const int n = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
      (void)hipGetLastError();
      return 256;
    }
    return cus;
  }();
  return n;
}

int check_launch() {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return QUIK_OK;
  set_last_hip_error(e);
  return QUIK_ERR_LAUNCH;
}
}  // namespace quik

extern "C" const char *quik_status_string(int status) {
  switch (status) {
    case QUIK_OK: return "ok";
    case QUIK_ERR_BITS: return "bits argument must be either 4 or 8";
    case QUIK_ERR_SHAPE: return "inconsistent tensor sizes";
    case QUIK_ERR_DTYPE: return "unsupported dtype (expected float16 or bfloat16)";
    case QUIK_ERR_ALIGN: return "operand violates the alignment this op needs";
    case QUIK_ERR_NULL: return "required pointer is null";
    case QUIK_ERR_RANGE: return "size beyond what the kernel supports";
    case QUIK_ERR_LAUNCH: return "HIP launch failed";
    default: return "unknown status";
  }
}

extern "C" const char *quik_last_hip_error(void) { return quik::g_last_error; }

extern "C" int quik_abi_version(void) { return 1; }

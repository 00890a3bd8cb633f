// Status strings and the last-HIP-error slot of libquik_hip.so.
#include "colmap.h"
#include "common.h"

#include <atomic>
#include <cstring>
#include <mutex>
#include <unordered_map>

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

// ---- flags of the column maps this process has used -----------------------------------------------------------
// The flags word of a column map (colmap.h) lives on the device.  Entry points that have no kernel path for a map
// without the streaming flag (or without the in-place order) must refuse such a map instead of launching a kernel
// that writes nothing, so they need the word on the host: it is copied once per (address, shape), with one stream
// synchronisation, and remembered.  quik_colmap_build forgets the address it writes to, so an address that is
// reused for another map is read again; a map must therefore be used at the address it was built at (a copy to
// another address is simply read once more; overwriting a known map by other means than quik_colmap_build is not
// supported).  A stream that is being captured cannot be synchronised: a map whose flags are not known yet is
// refused there (QUIK_ERR_COLMAP); call quik_colmap_streaming once per map outside the capture.
namespace {
struct ColmapFlags {
  int64_t cols, num_int, num_fp;
  uint32_t words[4];  // the map's four flag words (colmap.h): flags, dirty groups, holes, reserved
};
std::mutex g_colmap_mutex;
std::unordered_map<const void *, ColmapFlags> g_colmap_flags;
constexpr size_t kMaxKnownColmaps = 1 << 16;
}  // namespace

void colmap_forget(const void *colmap) {
  std::lock_guard<std::mutex> lock(g_colmap_mutex);
  g_colmap_flags.erase(colmap);
}

int colmap_flags(const void *colmap, int64_t cols, int64_t num_int, int64_t num_fp, hipStream_t st, uint32_t *flags) {
  uint32_t words[4];
  if (int rc = colmap_words(colmap, cols, num_int, num_fp, st, words)) return rc;
  *flags = words[0];
  return QUIK_OK;
}

int colmap_words(const void *colmap, int64_t cols, int64_t num_int, int64_t num_fp, hipStream_t st, uint32_t (&out)[4]) {
  {
    std::lock_guard<std::mutex> lock(g_colmap_mutex);
    auto it = g_colmap_flags.find(colmap);
    if (it != g_colmap_flags.end() && it->second.cols == cols && it->second.num_int == num_int &&
        it->second.num_fp == num_fp) {
      for (int i = 0; i < 4; ++i) out[i] = it->second.words[i];
      return QUIK_OK;
    }
  }
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &capture) != hipSuccess) {
    set_last_hip_error(hipGetLastError());
    return QUIK_ERR_LAUNCH;
  }
  if (capture != hipStreamCaptureStatusNone) return QUIK_ERR_COLMAP;
  const ColmapLayout l = colmap_layout(cols, num_int, num_fp);
  uint32_t word[4] = {0, 0, 0, 0};
  if (hipMemcpyAsync(word, static_cast<const uint8_t *>(colmap) + l.off_flags, sizeof(word), hipMemcpyDeviceToHost,
                     st) != hipSuccess ||
      hipStreamSynchronize(st) != hipSuccess) {
    set_last_hip_error(hipGetLastError());
    return QUIK_ERR_LAUNCH;
  }
  {
    std::lock_guard<std::mutex> lock(g_colmap_mutex);
    if (g_colmap_flags.size() >= kMaxKnownColmaps) g_colmap_flags.clear();
    g_colmap_flags[colmap] = ColmapFlags{cols, num_int, num_fp, {word[0], word[1], word[2], word[3]}};
  }
  for (int i = 0; i < 4; ++i) out[i] = word[i];
  return QUIK_OK;
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
    case QUIK_ERR_COLMAP:
      return "the column map does not select the streaming quantize kernel (ascending int_indices that partition "
             "the columns with fp_indices), or its flags are not known yet inside a stream capture";
    default: return "unknown status";
  }
}

extern "C" const char *quik_last_hip_error(void) { return quik::g_last_error; }

extern "C" int quik_abi_version(void) { return 1; }

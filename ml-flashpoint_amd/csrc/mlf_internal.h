// Internal to the translation units behind include/mlf_hip.h: error reporting, small host helpers, and the
// interface between the checksum code (mlf_crc.hip) and the copy engine (mlf_engine.hip).
#ifndef MLF_INTERNAL_H_
#define MLF_INTERNAL_H_

#include "mlf_hip.h"

#include <hip/hip_runtime.h>
#include <errno.h>
#include <stdint.h>
#include <string.h>
#include <unistd.h>

#include <chrono>
#include <string>

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_u __attribute__((aligned(1)));  // dwordx4 access at any byte address

namespace mlf {

enum { MLF_HIP_OK = 0, MLF_HIP_BAD_ARG = 1, MLF_HIP_RUNTIME = 2 };

// Message of the calling thread's last failure (what mlf_hip_last_error returns).
std::string& last_error();
// Records `msg` for the calling thread and returns `code`.
int fail(int code, const std::string& msg);

#define HIP_TRY(expr)                                                                                   \
  do {                                                                                                  \
    hipError_t e__ = (expr);                                                                            \
    if (e__ != hipSuccess)                                                                              \
      return ::mlf::fail(::mlf::MLF_HIP_RUNTIME, std::string(#expr) + " failed: " + hipGetErrorString(e__)); \
  } while (0)

inline double now_s() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

// pread / pwrite of a whole range; return 0 or an errno value
inline int full_pwrite(int fd, const char* buf, size_t len, uint64_t off) {
  while (len) {
    ssize_t w = pwrite(fd, buf, len, (off_t)off);
    if (w < 0) {
      if (errno == EINTR) continue;
      return errno;
    }
    buf += w;
    off += (uint64_t)w;
    len -= (size_t)w;
  }
  return 0;
}

inline int full_pread(int fd, char* buf, size_t len, uint64_t off) {
  while (len) {
    ssize_t r = pread(fd, buf, len, (off_t)off);
    if (r < 0) {
      if (errno == EINTR) continue;
      return errno;
    }
    if (r == 0) return ENODATA;  // file shorter than the requested range
    buf += r;
    off += (uint64_t)r;
    len -= (size_t)r;
  }
  return 0;
}

// ---- CRC-32C arithmetic shared by the checksum code and the copy kernels that fold remainders as they copy ----
constexpr uint32_t kCrcPolyReflected = 0x82F63B78u;

// a(x) * b(x) mod P in the reflected representation (bit 31 is x^0).
__host__ __device__ inline uint32_t gf_mul(uint32_t a, uint32_t b) {
  uint32_t p = 0;
  for (int i = 31; i >= 0; --i) {
    p ^= ((a >> i) & 1u) ? b : 0u;
    b = (b >> 1) ^ ((b & 1u) ? kCrcPolyReflected : 0u);
  }
  return p;
}

// x^(8*nbytes) mod P.
uint32_t x_pow_bytes(uint64_t nbytes);

// Checksum state of a plan whose copy kernels fold remainders (plan option crc_chunk_kib).  The image is cut into
// cells of 4 KiB, entries of 16 cells (64 KiB) and groups of rows * wgs_per_group cells; a chunk is a whole number
// of groups.  `fast_val` holds one remainder per workgroup of the fused copy kernel (groups [0, fused_groups)),
// `ent_val` one per entry that the copy kernels do not cover (listed in `slow_list`, taken from the finished image).
struct CrcConsts;
struct FusedCrc {
  uint64_t image_bytes = 0, chunk_bytes = 0;
  uint32_t rows = 16;           // cells per workgroup of the fused copy kernel
  uint32_t wgs_per_group = 0;   // G: a workgroup's cells are G cells apart
  uint64_t fused_groups = 0;
  uint64_t n_ent = 0, n_groups = 0, n_chunks = 0, n_slow = 0;
  uint64_t* d_ent = nullptr;      // per entry: tensor-side address of its first byte, 0 = not served by the fused kernel
  uint32_t* d_slow_list = nullptr;
  uint32_t* d_ent_val = nullptr;  // zero except at listed entries
  uint32_t* d_fast_val = nullptr;
  uint32_t* d_group_val = nullptr;
  uint32_t* d_row_tab = nullptr;  // [4][256]: state advanced by wgs_per_group cells, sliced by state byte
  u32x4* d_lane_w = nullptr;      // [256]: weight of each lane's four dwords within a cell
  char* d_sink = nullptr;         // 4 KiB that the fused kernel writes instead of cells that are not its own
  CrcConsts* d_consts = nullptr;  // lookup constants of the segment kernel
  uint32_t* d_out = nullptr;
  uint32_t* h_out = nullptr;      // pinned
  hipEvent_t done = nullptr;
  bool launched = false;
};

// Allocates and fills everything in `f` but d_ent / d_slow_list (the plan builds those); image_bytes, chunk_bytes,
// wgs_per_group, fused_groups, n_ent must be set.  crc_fused_destroy frees all of it (d_ent and d_slow_list too).
int crc_fused_setup(FusedCrc* f);
void crc_fused_destroy(FusedCrc* f);
// After the copy kernels of a launch are enqueued on `stream`: remainders of the listed entries from the image, the
// chain over groups and chunks, the copy of the chunk values to the pinned array, and the event behind it.
int crc_fused_finish(FusedCrc* f, const void* image, hipStream_t stream);

// Scratch of the stand-alone checksum pass: lookup constants, one value per segment, one per chunk on the device and
// a pinned copy of the latter.  Owned by whoever runs the passes (the copy engine, or the library per device) and
// kept from pass to pass: allocating and releasing device memory per pass would synchronise the whole device.
struct CrcScratch {
  CrcConsts* d_consts = nullptr;
  uint32_t* d_seg = nullptr;
  uint64_t seg_cap = 0;
  uint32_t* d_out = nullptr;
  uint32_t* h_out = nullptr;  // pinned
  uint64_t out_cap = 0;
};

// Enqueues the two CRC kernels and the copy of the per-chunk values on `stream`; does not wait.  Grows `scratch`
// first if this pass needs more than it holds (its previous user must have finished).  `background`: the pass runs
// beside other work on the device (a save's checksum beside the training step) and takes the variant that leaves the
// CUs' LDS to that work, at 85 % of the speed of the one that fills it with table copies.
int crc_enqueue(const void* dev_ptr, uint64_t nbytes, uint64_t chunk_bytes, uint64_t n_out, hipStream_t stream,
                CrcScratch* scratch, bool background);
// Waits for `stream` and hands out the values of the pass enqueued last (`n_chunks` of them).
int crc_finish(CrcScratch* scratch, hipStream_t stream, uint64_t n_chunks, uint32_t* out_host);
// Frees the scratch (its stream must be idle).
void crc_scratch_free(CrcScratch* scratch);
// Looks up, once, where the fixed scratch array of mlf_crc32c_device_noalloc lies on `device` (the current device), so
// that the entry point's first call there has nothing left to resolve - it may be made while a stream is captured.
int crc_noalloc_prime(int device);

}  // namespace mlf

#endif  // MLF_INTERNAL_H_

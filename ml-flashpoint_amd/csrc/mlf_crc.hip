// CRC-32C (Castagnoli) of a checkpoint image: per-chunk values computed on the GPU, the same function on host
// memory and on a byte range of a file, and the combine law.  Part of the library behind include/mlf_hip.h.
//
// Device side: per wavefront a segment (64 KiB to 512 KiB, by the size of the buffer) is read as coalesced 1 KiB
// rows; every lane keeps four Horner accumulators advanced by x^8192 through LDS tables, then lanes are folded with
// GF(2) multiplies; a second, tiny kernel chains the segment values of every chunk.
#include "mlf_internal.h"

#include <nmmintrin.h>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

namespace mlf {

struct CrcConsts {
  uint32_t row_tab[4][256];  // state advanced by one 1 KiB row, sliced by state byte
  uint32_t x4, x16, x32, x64, x128, x256, x512;  // x^(8*n) for the fold steps
};

}  // namespace mlf

namespace mlf {

uint32_t x_pow_bytes(uint64_t nbytes) {
  uint32_t result = 0x80000000u;      // x^0
  uint32_t sq = gf_mul(0x40000000u, 0x40000000u);  // x^2
  sq = gf_mul(sq, sq);                // x^4
  sq = gf_mul(sq, sq);                // x^8 : one byte
  while (nbytes) {
    if (nbytes & 1) result = gf_mul(result, sq);
    sq = gf_mul(sq, sq);
    nbytes >>= 1;
  }
  return result;
}

}  // namespace mlf

using namespace mlf;

namespace {

// ---------------------------------------------------------------------------------------------------------
// CRC-32C
// ---------------------------------------------------------------------------------------------------------
constexpr uint32_t kPolyReflected = kCrcPolyReflected;
constexpr uint32_t kCrcSegBytes = 64 * 1024;  // smallest segment (bytes per wavefront); chunks are multiples of it
constexpr uint32_t kCrcMaxSegBytes = 512 * 1024;
constexpr int kCrcTableCopies = 16;           // copies of the lookup tables in LDS, interleaved over the banks
constexpr int kCrcThreads = 512;
constexpr uint32_t kCrcRowBytes = 1024;       // one coalesced wavefront row: 64 lanes x 16 bytes

__device__ __forceinline__ uint32_t crc_byte_step(uint32_t s, uint8_t b) {
  s ^= b;
  for (int k = 0; k < 8; ++k) s = (s >> 1) ^ ((s & 1u) ? kPolyReflected : 0u);
  return s;
}

// One wavefront per segment: raw remainder (zero initial state, no final xor) of the segment's bytes.
//
// The four 256-entry tables are kept R times in LDS, entry v of copy c at word v * R + c, and lane l reads copy
// l % R: lookups with random v then spread over R times as many banks as a single copy would let them (measured on
// random bytes: 4.2 conflict cycles per lookup with one copy, 2.0 with sixteen).  Folding the lanes costs about
// 1 800 vector instructions per segment, as much as 50 rows of lookups: hence segments as long as the buffer allows.
template <int R>
__global__ void __launch_bounds__(kCrcThreads) mlf_crc_segments_kernel(const char* __restrict__ data, uint64_t nbytes,
                                                                       const CrcConsts* __restrict__ consts,
                                                                       uint32_t* __restrict__ seg_crc, uint32_t n_segs,
                                                                       uint32_t seg_bytes,
                                                                       const uint32_t* __restrict__ seg_list) {
  __shared__ uint32_t tab[4 * 256 * R];
  for (uint32_t i = threadIdx.x; i < 1024; i += blockDim.x) {
    const uint32_t v = consts->row_tab[i >> 8][i & 255];
#pragma unroll
    for (int c = 0; c < R; ++c) tab[i * R + c] = v;
  }
  __syncthreads();
  // wavefront k takes segment k, or, with a list, segment seg_list[k] (and reports under that number)
  const uint32_t slot = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (slot >= n_segs) return;
  const uint32_t seg = seg_list ? seg_list[slot] : slot;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t* my = tab + (lane & (R - 1));
  const uint64_t seg_off = (uint64_t)seg * seg_bytes;
  const uint64_t remaining = nbytes - seg_off;
  const uint32_t seg_len = remaining < seg_bytes ? (uint32_t)remaining : seg_bytes;
  const uint32_t rows = seg_len / kCrcRowBytes;
  const u32x4* p = reinterpret_cast<const u32x4*>(data + seg_off) + lane;
  uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0;
#define MLF_ROW_ADV(a)                                                                                   \
  (my[((a) & 255u) * R] ^ my[(256u + (((a) >> 8) & 255u)) * R] ^ my[(512u + (((a) >> 16) & 255u)) * R] ^ \
   my[(768u + ((a) >> 24)) * R])
  uint32_t r = 0;
  // four rows are requested before the first of them is used: bytes in flight per wavefront that cover the memory
  // latency at the occupancy the tables leave
  for (; r + 4 <= rows; r += 4) {
    u32x4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = __builtin_nontemporal_load(p + (size_t)(r + k) * 64);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      a0 = MLF_ROW_ADV(a0) ^ v[k].x;
      a1 = MLF_ROW_ADV(a1) ^ v[k].y;
      a2 = MLF_ROW_ADV(a2) ^ v[k].z;
      a3 = MLF_ROW_ADV(a3) ^ v[k].w;
    }
  }
  for (; r < rows; ++r) {
    const u32x4 v = __builtin_nontemporal_load(p + (size_t)r * 64);
    a0 = MLF_ROW_ADV(a0) ^ v.x;
    a1 = MLF_ROW_ADV(a1) ^ v.y;
    a2 = MLF_ROW_ADV(a2) ^ v.z;
    a3 = MLF_ROW_ADV(a3) ^ v.w;
  }
#undef MLF_ROW_ADV
  // fold the four columns of this lane: x^128*a0 + x^96*a1 + x^64*a2 + x^32*a3
  const uint32_t x4 = consts->x4;
  uint32_t acc = gf_mul(x4, a0) ^ a1;
  acc = gf_mul(x4, acc) ^ a2;
  acc = gf_mul(x4, acc) ^ a3;
  acc = gf_mul(x4, acc);
  // fold lanes pairwise: lower lane is earlier in the message, so it is the one that gets shifted
  const uint32_t xs[6] = {consts->x16, consts->x32, consts->x64, consts->x128, consts->x256, consts->x512};
#pragma unroll
  for (int s = 0; s < 6; ++s) {
    const uint32_t other = __shfl_down(acc, 1u << s, 64);
    acc = gf_mul(xs[s], acc) ^ other;
  }
  if (lane == 0) {
    // bytes of a short last segment that do not fill a row
    uint32_t state = rows ? acc : 0u;
    const char* tailp = data + seg_off + (uint64_t)rows * kCrcRowBytes;
    for (uint32_t i = 0, n = seg_len - rows * kCrcRowBytes; i < n; ++i) state = crc_byte_step(state, (uint8_t)tailp[i]);
    seg_crc[seg] = state;
  }
}

// One thread per chunk: chain the segment remainders, apply init and final xor.
__global__ void mlf_crc_chunks_kernel(const uint32_t* __restrict__ seg_crc, uint32_t segs_per_chunk, uint32_t n_segs,
                                      uint32_t xseg, uint32_t x_last_seg, uint32_t* __restrict__ out,
                                      uint32_t n_chunks) {
  const uint32_t c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= n_chunks) return;
  uint32_t s = 0xFFFFFFFFu;
  const uint32_t first = c * segs_per_chunk;
  const uint32_t last = first + segs_per_chunk < n_segs ? first + segs_per_chunk : n_segs;
  for (uint32_t i = first; i < last; ++i) s = gf_mul(i == n_segs - 1 ? x_last_seg : xseg, s) ^ seg_crc[i];
  out[c] = s ^ 0xFFFFFFFFu;
}

// ---------------------------------------------------------------------------------------------------------
// chaining the remainders of a plan whose copy kernels fold them as they copy (struct FusedCrc)
// ---------------------------------------------------------------------------------------------------------
constexpr uint32_t kCellBytes = 4096;
constexpr uint32_t kEntryBytes = 65536;

// One thread per group: the remainder of the group's bytes from (a) the values of its fused-copy workgroups -
// workgroup w holds cells w, w + G, ..., so consecutive values are one cell apart - and (b) the values of its entries
// that were checksummed from the image.  Both are taken relative to the group's end (the image's end for the last,
// possibly partial, group).
__global__ void mlf_crc_groups_kernel(const uint64_t* __restrict__ ent, const uint32_t* __restrict__ ent_val,
                                      const uint32_t* __restrict__ fast_val, uint32_t G, uint32_t ents_per_group,
                                      uint64_t fused_groups, uint64_t n_ent, uint64_t n_groups, uint32_t x_cell,
                                      uint32_t x_entry, uint32_t x_last_entry, uint32_t* __restrict__ group_val) {
  const uint64_t g = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= n_groups) return;
  uint32_t fast = 0;
  if (g < fused_groups)
    for (uint32_t w = 0; w < G; ++w) fast = gf_mul(x_cell, fast) ^ fast_val[g * G + w];
  uint32_t slow = 0;
  const uint64_t e0 = g * ents_per_group;
  const uint64_t e1 = e0 + ents_per_group < n_ent ? e0 + ents_per_group : n_ent;
  for (uint64_t e = e0; e < e1; ++e)
    slow = gf_mul(e == n_ent - 1 ? x_last_entry : x_entry, slow) ^ (ent[e] ? 0u : ent_val[e]);
  group_val[g] = fast ^ slow;
}

// One thread per chunk: chain the group remainders, apply init and final xor.
__global__ void mlf_crc_group_chunks_kernel(const uint32_t* __restrict__ group_val, uint32_t groups_per_chunk,
                                            uint64_t n_groups, uint32_t x_group, uint32_t x_last_group,
                                            uint32_t* __restrict__ out, uint32_t n_chunks) {
  const uint32_t c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= n_chunks) return;
  uint32_t s = 0xFFFFFFFFu;
  const uint64_t first = (uint64_t)c * groups_per_chunk;
  const uint64_t last = first + groups_per_chunk < n_groups ? first + groups_per_chunk : n_groups;
  for (uint64_t g = first; g < last; ++g) s = gf_mul(g == n_groups - 1 ? x_last_group : x_group, s) ^ group_val[g];
  out[c] = s ^ 0xFFFFFFFFu;
}

// ---------------------------------------------------------------------------------------------------------
// scratch of the allocation-free entry point (mlf_crc32c_device_noalloc)
// ---------------------------------------------------------------------------------------------------------
// A fixed array in every device's copy of this code object: the lookup constants, then one value per segment.
// 256 Ki segment values cover 128 GiB at 512 KiB segments.  The array's name is a host-side stand-in, not a device
// address: host code uses the per-device address that hipGetSymbolAddress returned, never the name.
constexpr uint32_t kNoAllocMaxSegs = 256 * 1024;
constexpr size_t kNoAllocConstsBytes = 8192;  // sizeof(CrcConsts) rounded up; the segment values follow
constexpr size_t kNoAllocScratchBytes = kNoAllocConstsBytes + (size_t)kNoAllocMaxSegs * sizeof(uint32_t);
static_assert(sizeof(CrcConsts) <= kNoAllocConstsBytes, "the constants must fit in front of the segment values");
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

constexpr int kNoAllocMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kNoAllocMaxDevices];  // device address of `scratch` on each device, looked up on first use there

// The device address of `scratch` on `device`, which must be the current device.  Looked up once per device (the
// lookup may load the code object there: not something to do while a stream is being captured) and kept.
int noalloc_scratch_of(int device, void** out) {
  if (device < 0 || device >= kNoAllocMaxDevices) return fail(MLF_HIP_BAD_ARG, "device index beyond the per-device table");
  std::lock_guard<std::mutex> g(g_scratch_mu);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(MLF_HIP_RUNTIME, "hipGetSymbolAddress returned a null address for the scratch array");
    g_scratch_ptr[device] = p;
  }
  *out = g_scratch_ptr[device];
  return MLF_HIP_OK;
}

struct CrcFoldConsts {
  uint32_t xrow, x4, x16, x32, x64, x128, x256, x512;
};

// Writes the lookup constants where a later kernel on the same stream reads them: 1024 threads, one table entry each.
__global__ void __launch_bounds__(1024) mlf_crc_fill_consts_kernel(CrcConsts* __restrict__ consts, CrcFoldConsts k) {
  const uint32_t i = threadIdx.x;
  consts->row_tab[i >> 8][i & 255u] = gf_mul(k.xrow, (i & 255u) << (8u * (i >> 8)));
  if (i == 0) {
    consts->x4 = k.x4;
    consts->x16 = k.x16;
    consts->x32 = k.x32;
    consts->x64 = k.x64;
    consts->x128 = k.x128;
    consts->x256 = k.x256;
    consts->x512 = k.x512;
  }
}

std::once_flag g_crc_once;
CrcConsts g_crc_host;

// The longest segment that divides the chunks and still leaves every CU several blocks of wavefronts.
uint64_t pick_seg_bytes(uint64_t nbytes, uint64_t chunk_bytes) {
  uint64_t seg_bytes = kCrcSegBytes;
  while (seg_bytes < kCrcMaxSegBytes && chunk_bytes % (2 * seg_bytes) == 0 && nbytes / (2 * seg_bytes) >= 8192) seg_bytes *= 2;
  return seg_bytes;
}

void crc_init_host() {
  const uint32_t xrow = x_pow_bytes(kCrcRowBytes);
  for (int b = 0; b < 4; ++b)
    for (uint32_t v = 0; v < 256; ++v) g_crc_host.row_tab[b][v] = gf_mul(xrow, v << (8 * b));
  g_crc_host.x4 = x_pow_bytes(4);
  g_crc_host.x16 = x_pow_bytes(16);
  g_crc_host.x32 = x_pow_bytes(32);
  g_crc_host.x64 = x_pow_bytes(64);
  g_crc_host.x128 = x_pow_bytes(128);
  g_crc_host.x256 = x_pow_bytes(256);
  g_crc_host.x512 = x_pow_bytes(512);
}

}  // namespace

namespace mlf {

int crc_noalloc_prime(int device) {
  void* unused = nullptr;
  return noalloc_scratch_of(device, &unused);
}



void crc_fused_destroy(FusedCrc* f) {
  (void)hipFree(f->d_ent);
  (void)hipFree(f->d_slow_list);
  (void)hipFree(f->d_ent_val);
  (void)hipFree(f->d_fast_val);
  (void)hipFree(f->d_group_val);
  (void)hipFree(f->d_row_tab);
  (void)hipFree(f->d_lane_w);
  (void)hipFree(f->d_sink);
  (void)hipFree(f->d_consts);
  (void)hipFree(f->d_out);
  if (f->h_out) (void)hipHostFree(f->h_out);
  if (f->done) (void)hipEventDestroy(f->done);
  *f = FusedCrc();
}

int crc_fused_setup(FusedCrc* f) {
  std::call_once(g_crc_once, crc_init_host);
  const uint64_t group_bytes = (uint64_t)f->rows * f->wgs_per_group * kCellBytes;
  f->n_groups = (f->image_bytes + group_bytes - 1) / group_bytes;
  f->n_chunks = (f->image_bytes + f->chunk_bytes - 1) / f->chunk_bytes;
  // state advanced by one row of the fused kernel's walk (its cells are wgs_per_group cells apart), sliced by byte
  // and, behind it, advanced by four bytes: joins the remainders of a lane's four neighbouring dwords
  std::vector<uint32_t> row_tab(2048);
  const uint32_t x_row = x_pow_bytes((uint64_t)kCellBytes * f->wgs_per_group), x_dword = x_pow_bytes(4);
  for (int b = 0; b < 4; ++b)
    for (uint32_t v = 0; v < 256; ++v) {
      row_tab[b * 256 + v] = gf_mul(x_row, v << (8 * b));
      row_tab[1024 + b * 256 + v] = gf_mul(x_dword, v << (8 * b));
    }
  // dword j of lane t's vector lies 4096 - 16 t - 4 j bytes in front of its cell's end (its own four bytes included)
  std::vector<uint32_t> lane_w(1024);
  for (uint32_t t = 0; t < 256; ++t)
    for (uint32_t j = 0; j < 4; ++j) lane_w[t * 4 + j] = x_pow_bytes(kCellBytes - 16 * t - 4 * j);
  const uint64_t n_fast = f->fused_groups * f->wgs_per_group;
  HIP_TRY(hipMalloc(reinterpret_cast<void**>(&f->d_ent_val), std::max<uint64_t>(f->n_ent, 1) * sizeof(uint32_t)));
  HIP_TRY(hipMemset(f->d_ent_val, 0, std::max<uint64_t>(f->n_ent, 1) * sizeof(uint32_t)));
  HIP_TRY(hipMalloc(reinterpret_cast<void**>(&f->d_fast_val), std::max<uint64_t>(n_fast, 1) * sizeof(uint32_t)));
  HIP_TRY(hipMalloc(reinterpret_cast<void**>(&f->d_group_val), std::max<uint64_t>(f->n_groups, 1) * sizeof(uint32_t)));
  HIP_TRY(hipMalloc(reinterpret_cast<void**>(&f->d_row_tab), 8192));
  HIP_TRY(hipMemcpy(f->d_row_tab, row_tab.data(), 8192, hipMemcpyHostToDevice));
  HIP_TRY(hipMalloc(reinterpret_cast<void**>(&f->d_lane_w), 4096));
  HIP_TRY(hipMemcpy(f->d_lane_w, lane_w.data(), 4096, hipMemcpyHostToDevice));
  HIP_TRY(hipMalloc(reinterpret_cast<void**>(&f->d_sink), 4096));
  HIP_TRY(hipMalloc(reinterpret_cast<void**>(&f->d_consts), sizeof(CrcConsts)));
  HIP_TRY(hipMemcpy(f->d_consts, &g_crc_host, sizeof(CrcConsts), hipMemcpyHostToDevice));
  HIP_TRY(hipMalloc(reinterpret_cast<void**>(&f->d_out), std::max<uint64_t>(f->n_chunks, 1) * sizeof(uint32_t)));
  HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&f->h_out), std::max<uint64_t>(f->n_chunks, 1) * sizeof(uint32_t), hipHostMallocDefault));
  HIP_TRY(hipEventCreateWithFlags(&f->done, hipEventDisableTiming));
  return MLF_HIP_OK;
}

int crc_fused_finish(FusedCrc* f, const void* image, hipStream_t stream) {
  if (f->n_slow) {
    // entries the copy kernels did not fold: one wavefront each, from the image that is complete at this point of
    // the stream; values land in ent_val under the entry's number
    const uint32_t waves_per_block = kCrcThreads / 64;
    const uint32_t grid = (uint32_t)((f->n_slow + waves_per_block - 1) / waves_per_block);
    hipLaunchKernelGGL(mlf_crc_segments_kernel<kCrcTableCopies>, dim3(grid), dim3(kCrcThreads), 0, stream,
                       static_cast<const char*>(image), f->image_bytes, f->d_consts, f->d_ent_val, (uint32_t)f->n_slow,
                       kEntryBytes, f->d_slow_list);
    HIP_TRY(hipGetLastError());
  }
  const uint64_t group_bytes = (uint64_t)f->rows * f->wgs_per_group * kCellBytes;
  const uint32_t ents_per_group = (uint32_t)(group_bytes / kEntryBytes);
  const uint64_t last_entry_len = f->image_bytes - (f->n_ent - 1) * kEntryBytes;
  hipLaunchKernelGGL(mlf_crc_groups_kernel, dim3((uint32_t)((f->n_groups + 63) / 64)), dim3(64), 0, stream, f->d_ent,
                     f->d_ent_val, f->d_fast_val, f->wgs_per_group, ents_per_group, f->fused_groups, f->n_ent, f->n_groups,
                     x_pow_bytes(kCellBytes), x_pow_bytes(kEntryBytes), x_pow_bytes(last_entry_len), f->d_group_val);
  HIP_TRY(hipGetLastError());
  const uint64_t last_group_len = f->image_bytes - (f->n_groups - 1) * group_bytes;
  hipLaunchKernelGGL(mlf_crc_group_chunks_kernel, dim3((uint32_t)((f->n_chunks + 63) / 64)), dim3(64), 0, stream,
                     f->d_group_val, (uint32_t)(f->chunk_bytes / group_bytes), f->n_groups, x_pow_bytes(group_bytes),
                     x_pow_bytes(last_group_len), f->d_out, (uint32_t)f->n_chunks);
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipMemcpyAsync(f->h_out, f->d_out, f->n_chunks * sizeof(uint32_t), hipMemcpyDeviceToHost, stream));
  HIP_TRY(hipEventRecord(f->done, stream));
  f->launched = true;
  return MLF_HIP_OK;
}

void crc_scratch_free(CrcScratch* sc) {
  (void)hipFree(sc->d_consts);
  (void)hipFree(sc->d_seg);
  (void)hipFree(sc->d_out);
  if (sc->h_out) (void)hipHostFree(sc->h_out);
  *sc = CrcScratch();
}

namespace {

int crc_scratch_ensure(CrcScratch* sc, uint64_t n_segs, uint64_t n_chunks) {
  if (!sc->d_consts) {
    std::call_once(g_crc_once, crc_init_host);
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&sc->d_consts), sizeof(CrcConsts)));
    HIP_TRY(hipMemcpy(sc->d_consts, &g_crc_host, sizeof(CrcConsts), hipMemcpyHostToDevice));
  }
  if (n_segs > sc->seg_cap) {
    (void)hipFree(sc->d_seg);
    sc->d_seg = nullptr;
    sc->seg_cap = 0;
    const uint64_t cap = std::max<uint64_t>(n_segs + n_segs / 4, 4096);  // some headroom: objects of one job differ little
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&sc->d_seg), cap * sizeof(uint32_t)));
    sc->seg_cap = cap;
  }
  if (n_chunks > sc->out_cap) {
    (void)hipFree(sc->d_out);
    if (sc->h_out) (void)hipHostFree(sc->h_out);
    sc->d_out = sc->h_out = nullptr;
    sc->out_cap = 0;
    const uint64_t cap = std::max<uint64_t>(n_chunks + n_chunks / 4, 1024);
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&sc->d_out), cap * sizeof(uint32_t)));
    HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&sc->h_out), cap * sizeof(uint32_t), hipHostMallocDefault));
    sc->out_cap = cap;
  }
  return MLF_HIP_OK;
}

}  // namespace

// Enqueues the two CRC kernels and the copy of the per-chunk values on `stream`; does not wait.
int crc_enqueue(const void* dev_ptr, uint64_t nbytes, uint64_t chunk_bytes, uint64_t n_out, hipStream_t stream,
                CrcScratch* sc, bool background) {
  if (!dev_ptr) return fail(MLF_HIP_BAD_ARG, "null pointer");
  if (reinterpret_cast<uintptr_t>(dev_ptr) & 15) return fail(MLF_HIP_BAD_ARG, "device buffer must be 16-byte aligned");
  if (chunk_bytes == 0 || chunk_bytes % kCrcSegBytes)
    return fail(MLF_HIP_BAD_ARG, "chunk_bytes must be a positive multiple of 65536");
  const uint64_t n_chunks = (nbytes + chunk_bytes - 1) / chunk_bytes;
  if (n_out < n_chunks) return fail(MLF_HIP_BAD_ARG, "output array too small");
  const uint64_t seg_bytes = pick_seg_bytes(nbytes, chunk_bytes);
  const uint64_t n_segs = (nbytes + seg_bytes - 1) / seg_bytes;
  if (n_segs > 0xFFFFFFF0ull) return fail(MLF_HIP_BAD_ARG, "buffer too large for one CRC call");
  if (int rc = crc_scratch_ensure(sc, n_segs, n_chunks)) return rc;
  if (background) {
    // one copy of the tables (4 KiB of LDS per workgroup instead of 64 KiB): the CUs' LDS stays available to the
    // kernels this pass runs beside
    const uint32_t grid = (uint32_t)((n_segs + 3) / 4);
    hipLaunchKernelGGL(mlf_crc_segments_kernel<1>, dim3(grid), dim3(256), 0, stream, static_cast<const char*>(dev_ptr),
                       nbytes, sc->d_consts, sc->d_seg, (uint32_t)n_segs, (uint32_t)seg_bytes, nullptr);
  } else {
    const uint32_t waves_per_block = kCrcThreads / 64;
    const uint32_t grid = (uint32_t)((n_segs + waves_per_block - 1) / waves_per_block);
    hipLaunchKernelGGL(mlf_crc_segments_kernel<kCrcTableCopies>, dim3(grid), dim3(kCrcThreads), 0, stream,
                       static_cast<const char*>(dev_ptr), nbytes, sc->d_consts, sc->d_seg, (uint32_t)n_segs,
                       (uint32_t)seg_bytes, nullptr);
  }
  HIP_TRY(hipGetLastError());
  const uint64_t last_seg_len = nbytes - (n_segs - 1) * seg_bytes;
  hipLaunchKernelGGL(mlf_crc_chunks_kernel, dim3((uint32_t)((n_chunks + 63) / 64)), dim3(64), 0, stream, sc->d_seg,
                     (uint32_t)(chunk_bytes / seg_bytes), (uint32_t)n_segs, x_pow_bytes(seg_bytes),
                     x_pow_bytes(last_seg_len), sc->d_out, (uint32_t)n_chunks);
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipMemcpyAsync(sc->h_out, sc->d_out, n_chunks * sizeof(uint32_t), hipMemcpyDeviceToHost, stream));
  return MLF_HIP_OK;
}

int crc_finish(CrcScratch* sc, hipStream_t stream, uint64_t n_chunks, uint32_t* out_host) {
  HIP_TRY(hipStreamSynchronize(stream));
  if (!out_host) return fail(MLF_HIP_BAD_ARG, "null pointer");
  memcpy(out_host, sc->h_out, n_chunks * sizeof(uint32_t));
  return MLF_HIP_OK;
}

}  // namespace mlf

extern "C" {

// ---------------------------------------------------------------------------------------------------------
// CRC entry points
// ---------------------------------------------------------------------------------------------------------
uint32_t mlf_crc32c_host(const void* data, uint64_t nbytes) {
  const unsigned char* p = static_cast<const unsigned char*>(data);
  uint64_t s = 0xFFFFFFFFu;
  while (nbytes && (reinterpret_cast<uintptr_t>(p) & 7)) {
    s = _mm_crc32_u8((uint32_t)s, *p++);
    --nbytes;
  }
  for (; nbytes >= 8; nbytes -= 8, p += 8) {
    uint64_t w;
    memcpy(&w, p, 8);
    s = _mm_crc32_u64(s, w);
  }
  while (nbytes--) s = _mm_crc32_u8((uint32_t)s, *p++);
  return (uint32_t)s ^ 0xFFFFFFFFu;
}

uint32_t mlf_crc32c_combine(uint32_t crc_a, uint32_t crc_b, uint64_t len_b) {
  return gf_mul(x_pow_bytes(len_b), crc_a) ^ crc_b;
}

int mlf_crc32c_file(int fd, uint64_t file_offset, uint64_t nbytes, uint64_t chunk_bytes, uint32_t* out_host,
                    uint64_t n_out, uint32_t threads) {
  if (fd < 0) return fail(MLF_HIP_BAD_ARG, "bad file descriptor");
  if (nbytes == 0) return MLF_HIP_OK;
  if (chunk_bytes == 0 || !out_host) return fail(MLF_HIP_BAD_ARG, "chunk_bytes must be positive and out_host non-null");
  const uint64_t n_chunks = (nbytes + chunk_bytes - 1) / chunk_bytes;
  if (n_out < n_chunks) return fail(MLF_HIP_BAD_ARG, "checksum output too small");
  if (threads < 1 || threads > 256) return fail(MLF_HIP_BAD_ARG, "threads must be in [1, 256]");
  const size_t piece = (size_t)std::min<uint64_t>(chunk_bytes, (uint64_t)4 << 20);  // read granularity per thread
  std::atomic<uint64_t> next{0};
  std::atomic<int> err{0};
  auto work = [&] {
    std::vector<char> buf(piece);
    for (;;) {
      const uint64_t c = next.fetch_add(1);
      if (c >= n_chunks || err.load()) return;
      const uint64_t begin = c * chunk_bytes, len = std::min(chunk_bytes, nbytes - begin);
      uint32_t crc = 0;
      for (uint64_t done = 0; done < len; done += piece) {
        const size_t n = (size_t)std::min<uint64_t>(piece, len - done);
        if (int e = full_pread(fd, buf.data(), n, file_offset + begin + done)) {
          err.store(e);
          return;
        }
        const uint32_t part = mlf_crc32c_host(buf.data(), n);
        crc = done == 0 ? part : mlf_crc32c_combine(crc, part, n);
      }
      out_host[c] = crc;
    }
  };
  std::vector<std::thread> pool;
  const unsigned width = (unsigned)std::min<uint64_t>(threads, n_chunks);
  for (unsigned i = 1; i < width; ++i) pool.emplace_back(work);
  work();
  for (auto& t : pool) t.join();
  if (int e = err.load()) return fail(MLF_HIP_RUNTIME, std::string("pread() failed: ") + strerror(e));
  return MLF_HIP_OK;
}

int mlf_crc32c_device(const void* dev_ptr, uint64_t nbytes, uint64_t chunk_bytes, uint32_t* out_host,
                      uint64_t n_out, void* stream_) {
  if (nbytes == 0) return MLF_HIP_OK;
  // one scratch per device, kept for the life of the library; calls on one device take turns
  static std::mutex mu[kNoAllocMaxDevices];
  static CrcScratch scratch[kNoAllocMaxDevices];
  int device = 0;
  HIP_TRY(hipGetDevice(&device));
  if (device < 0 || device >= kNoAllocMaxDevices) return fail(MLF_HIP_BAD_ARG, "device index beyond the per-device table");
  std::lock_guard<std::mutex> g(mu[device]);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = crc_enqueue(dev_ptr, nbytes, chunk_bytes, n_out, stream, &scratch[device], false)) return rc;
  return crc_finish(&scratch[device], stream, (nbytes + chunk_bytes - 1) / chunk_bytes, out_host);
}

int mlf_crc32c_device_noalloc(const void* dev_ptr, uint64_t nbytes, uint64_t chunk_bytes, uint32_t* out_dev,
                              uint64_t n_out, void* stream_) {
  if (nbytes == 0) return MLF_HIP_OK;
  if (!dev_ptr || !out_dev) return fail(MLF_HIP_BAD_ARG, "null pointer");
  if (reinterpret_cast<uintptr_t>(dev_ptr) & 15) return fail(MLF_HIP_BAD_ARG, "device buffer must be 16-byte aligned");
  if (reinterpret_cast<uintptr_t>(out_dev) & 3) return fail(MLF_HIP_BAD_ARG, "output array must be 4-byte aligned");
  if (chunk_bytes == 0 || chunk_bytes % kCrcSegBytes)
    return fail(MLF_HIP_BAD_ARG, "chunk_bytes must be a positive multiple of 65536");
  const uint64_t n_chunks = (nbytes + chunk_bytes - 1) / chunk_bytes;
  if (n_out < n_chunks) return fail(MLF_HIP_BAD_ARG, "output array too small");
  if (n_chunks > 0xFFFFFFF0ull) return fail(MLF_HIP_BAD_ARG, "buffer too large for one CRC call");
  // segments as the allocating entry point cuts them, doubled while their values would not fit in the fixed array
  // (a segment must still divide the chunk size)
  uint64_t seg_bytes = pick_seg_bytes(nbytes, chunk_bytes);
  while ((nbytes + seg_bytes - 1) / seg_bytes > kNoAllocMaxSegs && chunk_bytes % (2 * seg_bytes) == 0 &&
         2 * seg_bytes <= (1ull << 30))
    seg_bytes *= 2;
  const uint64_t n_segs = (nbytes + seg_bytes - 1) / seg_bytes;
  if (n_segs > kNoAllocMaxSegs)
    return fail(MLF_HIP_BAD_ARG,
                "mlf_crc32c_device_noalloc: " + std::to_string(nbytes) + " bytes in chunks of " + std::to_string(chunk_bytes) +
                    " need " + std::to_string(n_segs) + " segment values, the fixed scratch array holds " +
                    std::to_string(kNoAllocMaxSegs) + " (use larger chunks, several calls, or mlf_crc32c_device)");
  int device = 0;
  HIP_TRY(hipGetDevice(&device));
  void* base = nullptr;
  if (int rc = noalloc_scratch_of(device, &base)) return rc;  // looked up on the first call on a device, kept since
  CrcConsts* consts = static_cast<CrcConsts*>(base);
  uint32_t* seg = reinterpret_cast<uint32_t*>(static_cast<char*>(base) + kNoAllocConstsBytes);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  // Every call writes all it later reads (the constants, then one value per segment of this call), in stream order:
  // nothing has to start at zero and what an earlier call left behind is never looked at.
  CrcFoldConsts k;
  k.xrow = x_pow_bytes(kCrcRowBytes);
  k.x4 = x_pow_bytes(4);
  k.x16 = x_pow_bytes(16);
  k.x32 = x_pow_bytes(32);
  k.x64 = x_pow_bytes(64);
  k.x128 = x_pow_bytes(128);
  k.x256 = x_pow_bytes(256);
  k.x512 = x_pow_bytes(512);
  hipLaunchKernelGGL(mlf_crc_fill_consts_kernel, dim3(1), dim3(1024), 0, stream, consts, k);
  HIP_TRY(hipGetLastError());
  const uint32_t waves_per_block = kCrcThreads / 64;
  const uint32_t grid = (uint32_t)((n_segs + waves_per_block - 1) / waves_per_block);
  hipLaunchKernelGGL(mlf_crc_segments_kernel<kCrcTableCopies>, dim3(grid), dim3(kCrcThreads), 0, stream,
                     static_cast<const char*>(dev_ptr), nbytes, consts, seg, (uint32_t)n_segs, (uint32_t)seg_bytes,
                     nullptr);
  HIP_TRY(hipGetLastError());
  const uint64_t last_seg_len = nbytes - (n_segs - 1) * seg_bytes;
  hipLaunchKernelGGL(mlf_crc_chunks_kernel, dim3((uint32_t)((n_chunks + 63) / 64)), dim3(64), 0, stream, seg,
                     (uint32_t)(chunk_bytes / seg_bytes), (uint32_t)n_segs, x_pow_bytes(seg_bytes),
                     x_pow_bytes(last_seg_len), out_dev, (uint32_t)n_chunks);
  HIP_TRY(hipGetLastError());
  return MLF_HIP_OK;
}

}  // extern "C"

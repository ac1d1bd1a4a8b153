// MI355X (gfx950) save/restore data path behind the C-ABI in include/mlf_hip.h.  This file: plans and the pack /
// unpack kernels.  mlf_crc.hip holds the checksum, mlf_engine.hip the copy engine between HBM and host memory.
//
//   pack    live tensors (+ host blob of headers)  -> byte-exact image of a checkpoint object, in HBM
//   unpack  image in HBM                           -> live tensors
//
// Everything here is integer byte movement, so the bound is HBM bandwidth.  Kernels are written for 64-wide
// wavefronts, 16-byte accesses and the eight XCDs (each with its own L2) that workgroups reach round-robin:
//   * flat kernel: one small workgroup per tile (default 256 threads x one 16-byte vector = 4 KiB).  Tiles are cut
//     on a 4 KiB grid of the destination, so full tiles write whole lines with non-temporal dwordx4 stores; the
//     source is read with dwordx4 loads, or, where it is byte-misaligned relative to the destination, as aligned
//     granules that are realigned across lanes.  No LDS, no barriers.  Workgroups are short-lived and follow the
//     tiles in address order, so the set of tiles in flight is a compact, sequential window of HBM (worth ~25 %
//     over long-running workgroups that each stream a private region); within groups of 512 the tiles are dealt
//     out so that every XCD gets 64 consecutive ones and lines that straddle a cut stay in one L2.
//     Tiles are not listed one by one: a table entry ("span") describes up to 128 (or 16, or 1) consecutive
//     tiles of one contiguous item and the workgroups that share it derive their tile from their number.
//   * small kernel: pieces of at most 1 KiB (record headers, scalars, tails), one per wavefront.
//   * transpose kernel: views whose contiguous dimension differs between tensor and image (e.g. `.t()`) go
//     through an LDS tile so that both sides move whole 16-byte vectors along their contiguous dimension.
//   * strided kernel: generic, division-free N-d index walk for every other non-contiguous source/target and
//     for sub-box restores, plus a vector gather for packing `[..., ::k]` out of long rows.
#include "mlf_internal.h"

#include <algorithm>
#include <memory>
#include <string>
#include <vector>

using namespace mlf;

namespace mlf {

std::string& last_error() {
  thread_local std::string message;
  return message;
}

int fail(int code, const std::string& msg) {
  last_error() = msg;
  return code;
}

}  // namespace mlf

namespace {

// ---------------------------------------------------------------------------------------------------------
// device-side tables
// ---------------------------------------------------------------------------------------------------------

// Tensor addresses arrive as integers, which the compiler can only treat as generic ("flat") pointers: flat accesses
// count against both memory counters and are kept in order with LDS traffic.  Everything this library touches is
// global memory, so the hot accesses say so.
#define MLF_GLOBAL __attribute__((address_space(1)))
template <typename T>
__device__ __forceinline__ const MLF_GLOBAL T* gload(const void* p) {
  return (const MLF_GLOBAL T*)p;
}
template <typename T>
__device__ __forceinline__ MLF_GLOBAL T* gstore(void* p) {
  return (MLF_GLOBAL T*)p;
}

struct Span {       // n bytes of one contiguous item, copied by the (1 << shift) workgroups that share the entry
  uint64_t tensor;  // absolute device address on the tensor (or blob) side
  uint64_t image;   // byte offset in the image
  uint32_t n;
  uint32_t pad;
};

struct StridedDesc {
  uint64_t tensor;  // device address of element 0
  uint64_t image;   // byte offset of element 0 in the image
  uint32_t esz;
  uint32_t ndim;
  int64_t shape[MLF_MAX_DIMS];
  int64_t tstride[MLF_MAX_DIMS];  // bytes
  int64_t istride[MLF_MAX_DIMS];  // bytes
  int64_t step[MLF_MAX_DIMS];     // 256 written in the mixed radix of `shape`: what one loop trip adds to the index
};

struct StridedWork {  // one workgroup's work: elements [start, start+count) of descriptor `desc`
  uint64_t start;
  uint32_t count;
  uint32_t desc;
};

// A piece of one row of an item whose image side is contiguous along the last dimension while the tensor side takes
// every k-th element (k = 2..4) of long rows: `count` elements, consecutive in the image, k * esz bytes apart in the
// tensor.  Packing reads whole vectors and keeps what it needs; unpacking hands image vectors out through LDS.
struct GatherWork {
  uint64_t tensor;  // device address of the piece's first element
  uint64_t image;   // its byte offset in the image
  uint32_t count;
  uint16_t k, esz;
};

constexpr int kMaxBatchDims = MLF_MAX_DIMS - 2;

// A 2-D transposition (plus outer "batch" dims): dim a is contiguous on the tensor side, dim b on the image side.
// The tile grid starts a_lead elements before element 0 along a and b_lead before it along b, so that tile cuts fall
// on 128-byte lines of the tensor side (a) and of the image side (b) in every row whose pitch is a multiple of 128.
struct TransDesc {
  uint64_t tensor;  // device address of element 0
  uint64_t image;   // byte offset of element 0 in the image
  uint32_t esz;
  uint32_t nbatch;
  int64_t na, nb;   // extents of a and b
  int64_t ld_t;     // tensor-side byte stride of dim b (dim a has byte stride esz there)
  int64_t ld_i;     // image-side byte stride of dim a  (dim b has byte stride esz there)
  uint32_t a_lead, b_lead;
  int64_t bshape[kMaxBatchDims];
  int64_t bts[kMaxBatchDims];  // bytes
  int64_t bis[kMaxBatchDims];  // bytes
};

struct TransTile {  // one workgroup's tile: (ta, tb) of batch `batch` of descriptor `desc`; desc == kNoTile: none
  uint32_t desc;
  uint32_t ta, tb;
  uint32_t batch;
};
constexpr uint32_t kNoTile = 0xFFFFFFFFu;
constexpr int kTransClasses = 5;  // element sizes 1, 2, 4, 8, 16


// ---------------------------------------------------------------------------------------------------------
// flat kernel
// ---------------------------------------------------------------------------------------------------------
// Workgroup b of a class serves tile (b & mask) of span (b >> shift).  Tile boundaries inside a span sit on a grid
// of the destination (image offsets when packing, tensor addresses when unpacking; up to 4 KiB, so that full tiles
// write whole, aligned lines): tile 0 is [0, head + T), tile j is [head + j*T, head + (j+1)*T), the last one
// is cut at the span's end, where head = bytes from the span's first destination byte to the next grid line.
// Threads interleave at 16-byte granularity, so a wavefront moves 1 KiB of consecutive bytes per access.
constexpr int kFlatClasses = 3;  // span tables whose entries are shared by 128, 16 and 1 workgroups
constexpr uint32_t kXcdRun = 64;  // consecutive tiles handed to one XCD (see mlf_flat_kernel)

__host__ __device__ constexpr uint32_t flat_shift(int cls) { return cls == 0 ? 7u : cls == 1 ? 4u : 0u; }

// One launch serves every class: workgroups are numbered x-fastest over a (possibly) 2-D grid of 2^grid_x_log2
// columns, because a grid dimension may not exceed 2^32 - 1 threads while a 100 GB image needs 2^32.7 of them.
// Classes follow one another: class c owns workgroups [first_c, first_{c+1}), first_0 = 0.
//
// A workgroup lives for a few microseconds (one 4 KiB tile by default), so the scalar loads in front of its first
// vector load are a visible part of its life.  Everything it needs to find its span comes in as plain scalar
// arguments, and the span entry is read unconditionally in one go; a workgroup with nothing to do (padding of the
// last grid row, unused slot of a partly filled span) simply ends up with zero bytes.
template <bool PACK, int U>
__global__ void __launch_bounds__(1024) mlf_flat_kernel(const Span* __restrict__ spans0, const Span* __restrict__ spans1,
                                                        const Span* __restrict__ spans2, uint32_t first1,
                                                        uint32_t first2, uint32_t total, uint32_t grid_x_log2,
                                                        uint32_t tile_bytes, uint32_t block_threads,
                                                        uint32_t cut_mask, uint32_t cut_on_tensor,
                                                        char* __restrict__ image) {
  uint32_t wg = (blockIdx.y << grid_x_log2) + blockIdx.x;
  const bool live = wg < total;
  wg = live ? wg : 0u;
  const Span* __restrict__ table = wg >= first2 ? spans2 : wg >= first1 ? spans1 : spans0;
  const uint32_t shift = wg >= first2 ? flat_shift(2) : wg >= first1 ? flat_shift(1) : flat_shift(0);
  const uint32_t cls_first = wg >= first2 ? first2 : wg >= first1 ? first1 : 0u;
  const uint32_t cls_end = wg >= first2 ? total : wg >= first1 ? first2 : first1;
  uint32_t local = wg - cls_first;
  {
    // Workgroups go to the eight XCDs round-robin, so neighbouring tiles would land in eight different L2s and a
    // source line that straddles a tile cut would be fetched from HBM by both.  Within every full group of
    // 8 * kXcdRun workgroups the tiles are dealt out so that each XCD gets kXcdRun consecutive ones (256 KiB).
    // Measured on the 112 GB shard: runs of 1 / 16 / 64 / 256 tiles -> 35.7 / 34.8 / 34.2 / 37.5 ms per pack.
    constexpr uint32_t G = 8u * kXcdRun;
    const uint32_t g0 = local / G * G;
    if (cls_first + g0 + G <= cls_end) {
      const uint32_t c0 = cls_first & 7u;        // XCD of the class's first workgroup
      const uint32_t rp = (local - g0) + c0;     // position in the group, counted from XCD 0's slot
      const uint32_t xcd = rp & 7u;
      local = g0 + xcd * kXcdRun + (rp >> 3) - (xcd < c0 ? 1u : 0u);
    }
  }
  const Span sp = table[local >> shift];
  const uint32_t sub = local & ((1u << shift) - 1u);
  const uint32_t span_n = live ? sp.n : 0u;
  const char* src0 = PACK ? reinterpret_cast<const char*>(sp.tensor) : image + sp.image;
  char* dst0 = PACK ? image + sp.image : reinterpret_cast<char*>(sp.tensor);
  // tile cuts sit on the plan's grid: multiples of (cut_mask + 1) bytes of the image offset or of the tensor address
  const uint32_t cut_pos = (uint32_t)(cut_on_tensor ? sp.tensor : sp.image);
  uint32_t head0 = (0u - cut_pos) & cut_mask;
  head0 = head0 < span_n ? head0 : span_n;
  uint32_t start = sub ? head0 + sub * tile_bytes : 0u;
  start = start < span_n ? start : span_n;  // unused slot of a partly filled span: nothing left
  uint32_t end = head0 + (sub + 1u) * tile_bytes;
  end = end < span_n ? end : span_n;

  const char* src = src0 + start;
  char* dst = dst0 + start;
  uint32_t n = end - start;
  const uint32_t tid = threadIdx.x;
  const uint32_t bd = block_threads;
  // bytes up to the destination's next 16-byte boundary (none when the cuts are on the destination's side, except
  // in a span's first tile)
  uint32_t head = (0u - (uint32_t)reinterpret_cast<uintptr_t>(dst)) & 15u;
  head = head < n ? head : n;
  if (tid < head) dst[tid] = src[tid];
  src += head;
  dst += head;
  n -= head;

  const uint32_t nvec = n >> 4;
  u32x4* __restrict__ d = reinterpret_cast<u32x4*>(dst);
  uint32_t i = tid;
  if (U > 1) {
    for (; i + (U - 1) * bd < nvec; i += U * bd) {
      u32x4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        v[u] = __builtin_nontemporal_load(gload<u32x4_u>(src + (size_t)(i + u * bd) * 16));
#pragma unroll
      for (int u = 0; u < U; ++u) __builtin_nontemporal_store(v[u], gstore<u32x4>(&d[i + u * bd]));
    }
  }
  const uint32_t delta = (uint32_t)(reinterpret_cast<uintptr_t>(src) & 15u);  // uniform over the workgroup
  if ((delta & 3u) == 0u) {
    // dwordx4 loads need dword alignment only: a source that is off the 16-byte grid by 4, 8 or 12 bytes is read
    // directly (measured faster than the exchange below: 6.44 vs 6.29 TB/s at delta = 8)
    for (; i < nvec; i += bd) {
      u32x4 v = __builtin_nontemporal_load(gload<u32x4_u>(src + (size_t)i * 16));
      __builtin_nontemporal_store(v, gstore<u32x4>(&d[i]));
    }
  } else {
    // The source is off the destination's grid by a number of bytes that is not a multiple of 4.  Instead of
    // byte-misaligned dwordx4 loads, every lane loads one aligned 16-byte granule, takes the next one from its
    // neighbour lane and funnel-shifts the pair (measured 6.29 vs 6.07 TB/s at delta = 5).  Granule i holds source bytes [16 i - delta, 16 i - delta + 16): it always
    // contains at least one byte of the tile, also for i == nvec, so no access leaves the pages the tile is on.
    const u32x4* __restrict__ a = reinterpret_cast<const u32x4*>(src - delta);
    const uint32_t lane = tid & 63u;
    const uint32_t q = delta >> 2, r = delta & 3u;
    for (; (i & ~63u) < nvec; i += bd) {  // whole wavefronts stay in the loop: the lane exchange needs them
      u32x4 lo = {0u, 0u, 0u, 0u}, far = {0u, 0u, 0u, 0u}, hi;
      const bool edge = lane == 63u && i < nvec;  // this lane's neighbour is in another wavefront
      if (i <= nvec) lo = __builtin_nontemporal_load(gload<u32x4>(a + i));
      if (edge) far = __builtin_nontemporal_load(gload<u32x4>(a + i + 1));  // issued with the load above, not after the exchange
      hi.x = (uint32_t)__shfl_down((int)lo.x, 1);
      hi.y = (uint32_t)__shfl_down((int)lo.y, 1);
      hi.z = (uint32_t)__shfl_down((int)lo.z, 1);
      hi.w = (uint32_t)__shfl_down((int)lo.w, 1);
      if (edge) hi = far;
      if (i < nvec) {
        uint32_t w0, w1, w2, w3, w4;
        switch (q) {
          case 0: w0 = lo.x; w1 = lo.y; w2 = lo.z; w3 = lo.w; w4 = hi.x; break;
          case 1: w0 = lo.y; w1 = lo.z; w2 = lo.w; w3 = hi.x; w4 = hi.y; break;
          case 2: w0 = lo.z; w1 = lo.w; w2 = hi.x; w3 = hi.y; w4 = hi.z; break;
          default: w0 = lo.w; w1 = hi.x; w2 = hi.y; w3 = hi.z; w4 = hi.w; break;
        }
        u32x4 v;
        v.x = __builtin_amdgcn_alignbyte(w1, w0, r);
        v.y = __builtin_amdgcn_alignbyte(w2, w1, r);
        v.z = __builtin_amdgcn_alignbyte(w3, w2, r);
        v.w = __builtin_amdgcn_alignbyte(w4, w3, r);
        __builtin_nontemporal_store(v, gstore<u32x4>(&d[i]));
      }
    }
  }
  const uint32_t tail = n & 15u;
  if (tid < tail) {
    const uint32_t o = (nvec << 4) + tid;
    dst[o] = src[o];
  }
}

// Items of at most 1 KiB (record headers, scalars, step counters, the tails of small tensors): one wavefront per
// item, four items per workgroup, so that thousands of tiny items do not each occupy a workgroup of their own.
constexpr uint32_t kSmallItemBytes = 1024;

template <bool PACK>
__global__ void __launch_bounds__(256) mlf_small_kernel(const Span* __restrict__ spans, uint32_t n_spans,
                                                        char* __restrict__ image) {
  const uint32_t item = blockIdx.x * 4u + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (item >= n_spans) return;
  const uint32_t lane = threadIdx.x & 63u;
  const Span sp = spans[item];
  const char* src = PACK ? reinterpret_cast<const char*>(sp.tensor) : image + sp.image;
  char* dst = PACK ? image + sp.image : reinterpret_cast<char*>(sp.tensor);
  uint32_t n = sp.n;
  uint32_t head = (16u - (uint32_t)(reinterpret_cast<uintptr_t>(dst) & 15u)) & 15u;
  head = head < n ? head : n;
  if (lane < head) dst[lane] = src[lane];
  src += head;
  dst += head;
  n -= head;
  const uint32_t nvec = n >> 4;  // <= 64: one vector per lane
  if (lane < nvec)
    reinterpret_cast<u32x4*>(dst)[lane] = *reinterpret_cast<const u32x4_u*>(src + (size_t)lane * 16);
  const uint32_t tail = n & 15u;
  if (lane < tail) {
    const uint32_t o = (nvec << 4) + lane;
    dst[o] = src[o];
  }
}

// ---------------------------------------------------------------------------------------------------------
// strided kernel (generic)
// ---------------------------------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ void copy_elem(char* dst, const char* src) {
  typedef T unaligned_t __attribute__((aligned(1)));
  *gstore<unaligned_t>(dst) = *gload<unaligned_t>(src);
}

// Generic N-d walk.  A thread decomposes its first element index once (divisions), then advances the multi-index
// by the block size with one add-and-carry per dimension per trip: no division in the loop.
template <bool PACK, typename T>
__device__ __forceinline__ void strided_walk(const StridedDesc* __restrict__ d, const StridedWork& w,
                                             char* __restrict__ image) {
  const int ndim = (int)d->ndim;
  char* tbase = reinterpret_cast<char*>(d->tensor);
  char* ibase = image + d->image;
  int64_t idx[MLF_MAX_DIMS];
  {
    uint64_t e = w.start + threadIdx.x;
#pragma unroll
    for (int dim = MLF_MAX_DIMS - 1; dim >= 0; --dim) {
      idx[dim] = 0;
      if (dim < ndim) {
        const uint64_t extent = (uint64_t)d->shape[dim];
        const uint64_t q = e / extent;
        idx[dim] = (int64_t)(e - q * extent);
        e = q;
      }
    }
  }
  for (uint32_t k = threadIdx.x; k < w.count; k += 256) {
    int64_t toff = 0, ioff = 0;
#pragma unroll
    for (int dim = 0; dim < MLF_MAX_DIMS; ++dim) {
      if (dim < ndim) {
        toff += idx[dim] * d->tstride[dim];
        ioff += idx[dim] * d->istride[dim];
      }
    }
    copy_elem<T>(PACK ? ibase + ioff : tbase + toff, PACK ? tbase + toff : ibase + ioff);
    int64_t carry = 0;
#pragma unroll
    for (int dim = MLF_MAX_DIMS - 1; dim >= 0; --dim) {
      if (dim < ndim) {
        int64_t v = idx[dim] + d->step[dim] + carry;
        carry = 0;
        if (v >= d->shape[dim]) {
          v -= d->shape[dim];
          carry = 1;
        }
        idx[dim] = v;
      }
    }
  }
}

// Packing `x[..., ::k]` (k = 2, 3, 4) out of long rows.  Element-sized accesses top out near 0.45 T elements/s on
// this part whatever the loop around them looks like, so the kept elements are cut out of whole 16-byte vectors with
// compile-time shuffles and written as whole vectors.  A work item (a piece of one row, at most kGatherUnitsPerBlock
// output vectors) is shared by kGatherSplit workgroups that make one trip each: short-lived workgroups that follow
// each other through the rows keep the traffic a compact window on both sides, as in the flat kernel.
constexpr uint32_t kGatherSplit = 4;

template <int K, typename T>
__device__ __forceinline__ void gather_units(const char* __restrict__ sp, char* __restrict__ dp, uint32_t u0,
                                             uint32_t u1) {
  constexpr int EPV = 16 / (int)sizeof(T);
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t w0 = u0 + (threadIdx.x & ~63u);  // this wavefront's 64 units
  if (K == 2 && w0 + 64u <= u1) {
    // k = 2, a whole block of 64 units: 2 KiB in, 1 KiB out.  Every lane loads one vector of the block's first KiB
    // and one of its second (two loads that each cover a KiB of consecutive bytes, instead of 64 pieces of 16 bytes
    // 32 apart), keeps the even elements of both - 8 bytes for output position 8 * lane, 8 bytes for 512 + 8 * lane -
    // and trades one half with its neighbour, so that the even lane stores the pair's 16 bytes of the first half of
    // the output block and the odd lane those of the second.
    const char* s = sp + (size_t)w0 * 32;
    union {
      u32x4 v;
      T e[EPV];
    } a, b;
    a.v = __builtin_nontemporal_load(gload<u32x4_u>(s + lane * 16u));
    b.v = __builtin_nontemporal_load(gload<u32x4_u>(s + 1024u + lane * 16u));
    union {
      uint32_t w[2];
      T e[EPV / 2];
    } ca, cb;
#pragma unroll
    for (int j = 0; j < EPV / 2; ++j) {
      ca.e[j] = a.e[2 * j];
      cb.e[j] = b.e[2 * j];
    }
    const bool odd = lane & 1u;
    const uint32_t give0 = odd ? ca.w[0] : cb.w[0], give1 = odd ? ca.w[1] : cb.w[1];
    // quad_perm [1, 0, 3, 2]: every lane reads its neighbour in the pair
    const uint32_t take0 = (uint32_t)__builtin_amdgcn_mov_dpp((int)give0, 0xB1, 0xF, 0xF, true);
    const uint32_t take1 = (uint32_t)__builtin_amdgcn_mov_dpp((int)give1, 0xB1, 0xF, 0xF, true);
    u32x4 out;
    out.x = odd ? take0 : ca.w[0];
    out.y = odd ? take1 : ca.w[1];
    out.z = odd ? cb.w[0] : take0;
    out.w = odd ? cb.w[1] : take1;
    char* o = dp + (size_t)w0 * 16 + (odd ? 512u + (lane - 1u) * 8u : lane * 8u);
    __builtin_nontemporal_store(out, gstore<u32x4_u>(o));
    return;
  }
  const uint32_t u = w0 + lane;
  if (u >= u1) return;
  union {
    u32x4 v[K];
    T e[K * EPV];
  } in;
  union {
    u32x4 v;
    T e[EPV];
  } out;
  const char* s = sp + (size_t)u * (16 * K);
#pragma unroll
  for (int j = 0; j < K; ++j) in.v[j] = __builtin_nontemporal_load(gload<u32x4_u>(s + 16 * j));
#pragma unroll
  for (int j = 0; j < EPV; ++j) out.e[j] = in.e[j * K];
  __builtin_nontemporal_store(out.v, gstore<u32x4_u>(dp + (size_t)u * 16));
}

template <typename T>
__device__ __forceinline__ void gather_piece(const GatherWork& w, uint32_t sub, char* __restrict__ image) {
  typedef T elem_u __attribute__((aligned(1)));
  constexpr uint32_t EPV = 16 / (uint32_t)sizeof(T);
  const uint32_t K = w.k;
  const char* sp = reinterpret_cast<const char*>(w.tensor);
  char* dp = image + w.image;
  // whole units only where all 16 K source bytes lie at or before the piece's last element: a vector load must not
  // run past the end of the row (the storage may end there)
  const uint32_t n_units = (uint32_t)((((uint64_t)w.count - 1) * K + 1) / (uint64_t)(EPV * K));
  const uint32_t u0 = sub * 256u, u1 = n_units < u0 + 256u ? n_units : u0 + 256u;
  if (u0 < u1) {
    switch (K) {
      case 2: gather_units<2, T>(sp, dp, u0, u1); break;
      case 3: gather_units<3, T>(sp, dp, u0, u1); break;
      default: gather_units<4, T>(sp, dp, u0, u1); break;
    }
  }
  // the elements after the last whole unit (fewer than 2 EPV): one each for the first threads of the last workgroup
  const uint32_t j = n_units * EPV + threadIdx.x;
  if (sub == kGatherSplit - 1u && j < w.count)
    *gstore<elem_u>(dp + (size_t)j * sizeof(T)) = *gload<elem_u>(sp + (size_t)j * (K * sizeof(T)));
}

__global__ void __launch_bounds__(256) mlf_gather_kernel(const GatherWork* __restrict__ work, uint32_t n_wgs,
                                                         char* __restrict__ image) {
  // Workgroups reach the eight XCDs round-robin; the image side of neighbouring workgroups meets in partly written
  // lines (image offsets are arbitrary), which should meet in one L2: of every 8 * kRun workgroups each XCD takes
  // kRun consecutive ones.  Measured on 667 `[r0:r1, ::2]` bands of 2-16 MB (TB/s of 2 x payload; 4.3 is the ceiling
  // of a kernel that must fetch the skipped elements too): runs of 1 / 4 / 16 / 64 / 256 workgroups 3.88 / 3.92 /
  // 4.09 / 4.23 / 4.25; one workgroup per work item making four trips, lanes reading 16 bytes 32 apart: 3.37.
  constexpr uint32_t kRun = 64, G = 8u * kRun;
  uint32_t wg = blockIdx.x;
  const uint32_t g0 = wg / G * G;
  if (g0 + G <= n_wgs) wg = g0 + (wg & 7u) * kRun + ((wg - g0) >> 3);
  const GatherWork w = work[wg / kGatherSplit];
  const uint32_t sub = wg % kGatherSplit;
  switch (w.esz) {
    case 1: gather_piece<uint8_t>(w, sub, image); break;
    case 2: gather_piece<uint16_t>(w, sub, image); break;
    case 4: gather_piece<uint32_t>(w, sub, image); break;
    default: gather_piece<uint64_t>(w, sub, image); break;
  }
}

// The way back, unpacking into `x[..., ::k]`: the gaps must not be written, so the stores stay element-sized, but
// the image side is read as whole vectors and handed out through LDS so that neighbouring lanes store neighbouring
// elements.  That removes almost half of the element-sized accesses (all the loads).
template <typename T>
__device__ __forceinline__ void scatter_piece(const GatherWork& w, char* __restrict__ image, u32x4* __restrict__ lds) {
  typedef T elem_u __attribute__((aligned(1)));
  constexpr uint32_t EPV = 16 / (uint32_t)sizeof(T);
  const int64_t ts = (int64_t)w.k * (int64_t)sizeof(T);
  const char* sp = image + w.image;
  char* dp = reinterpret_cast<char*>(w.tensor);
  const uint32_t n_units = w.count / EPV;
  const T* __restrict__ lds_elems = reinterpret_cast<const T*>(lds);
  for (uint32_t base = 0; base < n_units; base += 256) {  // uniform trip count: every thread reaches the barriers
    const uint32_t u = base + threadIdx.x;
    if (u < n_units) lds[threadIdx.x] = __builtin_nontemporal_load(gload<u32x4_u>(sp + (size_t)u * 16));
    __syncthreads();
    const uint32_t here = (n_units - base < 256u ? n_units - base : 256u) * EPV;
#pragma unroll 4
    for (uint32_t e = threadIdx.x; e < here; e += 256)
      *gstore<elem_u>(dp + (int64_t)(base * EPV + e) * ts) = lds_elems[e];
    __syncthreads();
  }
  const uint32_t j = n_units * EPV + threadIdx.x;  // fewer than EPV elements are left
  if (j < w.count) *gstore<elem_u>(dp + (int64_t)j * ts) = *gload<elem_u>(sp + (size_t)j * sizeof(T));
}

__global__ void __launch_bounds__(256) mlf_scatter_kernel(const GatherWork* __restrict__ work, char* __restrict__ image) {
  __shared__ u32x4 lds[256];
  const GatherWork w = work[blockIdx.x];
  switch (w.esz) {
    case 1: scatter_piece<uint8_t>(w, image, lds); break;
    case 2: scatter_piece<uint16_t>(w, image, lds); break;
    case 4: scatter_piece<uint32_t>(w, image, lds); break;
    default: scatter_piece<uint64_t>(w, image, lds); break;
  }
}

template <bool PACK>
__global__ void __launch_bounds__(256) mlf_strided_kernel(const StridedDesc* __restrict__ descs,
                                                          const StridedWork* __restrict__ work,
                                                          char* __restrict__ image) {
  const StridedWork w = work[blockIdx.x];
  const StridedDesc* __restrict__ d = descs + w.desc;
  switch (d->esz) {
    case 1: strided_walk<PACK, uint8_t>(d, w, image); break;
    case 2: strided_walk<PACK, uint16_t>(d, w, image); break;
    case 4: strided_walk<PACK, uint32_t>(d, w, image); break;
    case 8: strided_walk<PACK, uint64_t>(d, w, image); break;
    default: strided_walk<PACK, u32x4>(d, w, image); break;  // 16
  }
}

// ---------------------------------------------------------------------------------------------------------
// transpose kernel (LDS-tiled)
// ---------------------------------------------------------------------------------------------------------
// One workgroup moves one tile of A x B elements of a 2-D transposition through LDS so that both the read (along
// the source's contiguous dimension) and the write (along the destination's) are made of whole 16-byte vectors in
// runs of at least 128 consecutive bytes (narrower accesses are bound by the number of lane accesses, not by
// bytes).  The tile lies in LDS as it is read, rows along the source's contiguous dimension, and the 16-byte columns
// of row y are permuted by xor with (y / elements-per-vector): vector writes stay aligned and conflict-free, and
// the column walk that assembles a destination vector from EPV rows meets a different bank group in every lane.
constexpr uint32_t kTransThreads = 256;

// Tile extents in elements along the side that is read (x) and the side that is written (y): 128 bytes by 256 for
// elements of up to 8 bytes (the tile then holds 32 / 16 / 8 / 4 KiB for 1 / 2 / 4 / 8-byte elements), 16 x 16
// elements of 16 bytes.  Measured on 667 transposed blocks of 2-16 MB with pitches off the 128-byte lines (TB/s of
// 2 x payload, pack / unpack): 128 x 128 bytes 4.20 / 4.41, 128 x 256 4.47 / 4.50, 256 x 256 4.02 / 3.89,
// 64 x 256 4.30 / 4.32, 128 x 512 3.83 / 4.10: longer runs on the written side pay (partly written lines cost more
// than partly used fetched ones) until the tile's LDS footprint cuts the number of resident workgroups.
__host__ __device__ constexpr uint32_t trans_tile_x(uint32_t esz) { return esz == 16 ? 16u : 128u / esz; }
__host__ __device__ constexpr uint32_t trans_tile_y(uint32_t esz) { return esz == 16 ? 16u : 256u / esz; }
// tile extents in elements along a (contiguous on the tensor side) and b (contiguous on the image side)
__host__ __device__ constexpr uint32_t trans_tile_a(uint32_t esz, bool pack) {
  return pack ? trans_tile_x(esz) : trans_tile_y(esz);
}
__host__ __device__ constexpr uint32_t trans_tile_b(uint32_t esz, bool pack) {
  return pack ? trans_tile_y(esz) : trans_tile_x(esz);
}
template <bool PACK, typename E, uint32_t A, uint32_t B>
__device__ __forceinline__ void trans_tile(const TransDesc* __restrict__ d, uint64_t batch, uint32_t ta, uint32_t tb,
                                           char* __restrict__ image, char* __restrict__ lds) {
  typedef u32x4 V;
  constexpr uint32_t ESZ = sizeof(E), EPV = 16 / ESZ;
  // x: the source's contiguous dimension, y: the destination's
  constexpr uint32_t TX = PACK ? A : B, TY = PACK ? B : A;
  constexpr uint32_t VX = TX / EPV, VY = TY / EPV;  // vectors per source row / per destination row
  constexpr uint32_t pitch = TX * ESZ;
  static_assert((VX & (VX - 1)) == 0 && (VY & (VY - 1)) == 0, "tile extents are powers of two");
  static_assert((TY * VX) % kTransThreads == 0 && (TX * VY) % kTransThreads == 0, "whole trips over a tile");
  typedef V vec_u __attribute__((aligned(1)));
  typedef E elem_u __attribute__((aligned(1)));

  int64_t toff = 0, ioff = 0;
  for (int k = (int)d->nbatch - 1; k >= 0; --k) {
    const uint64_t extent = (uint64_t)d->bshape[k];
    const uint64_t q = batch / extent;
    const int64_t i = (int64_t)(batch - q * extent);
    batch = q;
    toff += i * d->bts[k];
    ioff += i * d->bis[k];
  }
  // the tile's first element; negative in the first tile row / column when the grid starts before element 0
  const int64_t a0 = (int64_t)ta * A - (int64_t)d->a_lead, b0 = (int64_t)tb * B - (int64_t)d->b_lead;
  const int64_t nx = PACK ? d->na : d->nb, ny = PACK ? d->nb : d->na;
  const int64_t x0 = PACK ? a0 : b0, y0 = PACK ? b0 : a0;
  const int64_t ld_src = PACK ? d->ld_t : d->ld_i, ld_dst = PACK ? d->ld_i : d->ld_t;
  const char* src = (PACK ? reinterpret_cast<const char*>(d->tensor) + toff : image + d->image + ioff) + x0 * ESZ + y0 * ld_src;
  char* dst = (PACK ? image + d->image + ioff : reinterpret_cast<char*>(d->tensor) + toff) + x0 * ld_dst + y0 * ESZ;
  // the part of the tile that belongs to the item: [xlo, xhi) x [ylo, yhi)
  const uint32_t xlo = x0 < 0 ? (uint32_t)(-x0) : 0u, ylo = y0 < 0 ? (uint32_t)(-y0) : 0u;
  const uint32_t xhi = (uint32_t)(nx - x0 < (int64_t)TX ? nx - x0 : TX);
  const uint32_t yhi = (uint32_t)(ny - y0 < (int64_t)TY ? ny - y0 : TY);
  const uint32_t tid = threadIdx.x;

  if (xlo == 0u && ylo == 0u && xhi == TX && yhi == TY) {
    // a whole tile: every load is issued before the first LDS access
    constexpr uint32_t N1 = TY * VX / kTransThreads, N2 = TX * VY / kTransThreads;
    V in[N1];
#pragma unroll
    for (uint32_t i = 0; i < N1; ++i) {
      const uint32_t v = tid + i * kTransThreads, y = v / VX, xv = v % VX;
      in[i] = *gload<vec_u>(src + (int64_t)y * ld_src + xv * 16u);
    }
#pragma unroll
    for (uint32_t i = 0; i < N1; ++i) {
      const uint32_t v = tid + i * kTransThreads, y = v / VX, xv = v % VX;
      *reinterpret_cast<V*>(lds + y * pitch + ((xv ^ ((y / EPV) & (VX - 1u))) << 4)) = in[i];
    }
    __syncthreads();
#pragma unroll
    for (uint32_t i = 0; i < N2; ++i) {
      const uint32_t v = tid + i * kTransThreads, x = v / VY, yv = v % VY;
      const char* l = lds + yv * EPV * pitch + (((x / EPV) ^ (yv & (VX - 1u))) << 4) + (x % EPV) * ESZ;
      V out;
      E* parts = reinterpret_cast<E*>(&out);
#pragma unroll
      for (uint32_t k = 0; k < EPV; ++k) parts[k] = *reinterpret_cast<const E*>(l + k * pitch);
      *gstore<vec_u>(dst + (int64_t)x * ld_dst + yv * 16u) = out;
    }
    return;
  }
  // a tile on the item's edge: the same walk, element by element where a vector is not wholly inside
  for (uint32_t v = tid; v < TY * VX; v += kTransThreads) {
    const uint32_t y = v / VX, xv = v % VX, x = xv * EPV;
    if (y < ylo || y >= yhi || x + EPV <= xlo || x >= xhi) continue;
    const char* g = src + (int64_t)y * ld_src + xv * 16u;
    char* l = lds + y * pitch + ((xv ^ ((y / EPV) & (VX - 1u))) << 4);
    if (x >= xlo && x + EPV <= xhi) {
      *reinterpret_cast<V*>(l) = *gload<vec_u>(g);
    } else {
      for (uint32_t k = 0; k < EPV; ++k)
        if (x + k >= xlo && x + k < xhi) reinterpret_cast<E*>(l)[k] = *gload<elem_u>(g + k * ESZ);
    }
  }
  __syncthreads();
  for (uint32_t v = tid; v < TX * VY; v += kTransThreads) {
    const uint32_t x = v / VY, yv = v % VY, y = yv * EPV;
    if (x < xlo || x >= xhi || y + EPV <= ylo || y >= yhi) continue;
    char* g = dst + (int64_t)x * ld_dst + yv * 16u;
    const char* l = lds + y * pitch + (((x / EPV) ^ (yv & (VX - 1u))) << 4) + (x % EPV) * ESZ;
    if (y >= ylo && y + EPV <= yhi) {
      V out;
      E* parts = reinterpret_cast<E*>(&out);
#pragma unroll
      for (uint32_t k = 0; k < EPV; ++k) parts[k] = *reinterpret_cast<const E*>(l + k * pitch);
      *gstore<vec_u>(g) = out;
    } else {
      for (uint32_t k = 0; k < EPV; ++k)
        if (y + k >= ylo && y + k < yhi) *gstore<elem_u>(g + k * ESZ) = *reinterpret_cast<const E*>(l + k * pitch);
    }
  }
}

// Which tile a workgroup takes comes from a table the plan builds on the host, one entry per workgroup, because the
// order matters.  Workgroups reach the eight XCDs round-robin, and every XCD has its own L2: tiles next to each other
// along a share lines of the tensor side, tiles next to each other along b lines of the image side, wherever a tile
// row does not start on a line.  The table gives XCD x (entries x, x + 8, x + 16 ...) compact patches of
// neighbouring tiles, one after the other: lines that two of its tiles share are fetched from HBM once and merged in
// that L2 before they are written; only the patches' rims meet another L2.
template <bool PACK, typename E>
__global__ void __launch_bounds__(kTransThreads) mlf_transpose_kernel(const TransDesc* __restrict__ descs,
                                                            const TransTile* __restrict__ tiles,
                                                            char* __restrict__ image) {
  constexpr uint32_t A = trans_tile_a(sizeof(E), PACK), B = trans_tile_b(sizeof(E), PACK);
  __shared__ __attribute__((aligned(16))) char lds[A * B * sizeof(E)];
  const TransTile t = tiles[blockIdx.x];
  if (t.desc == kNoTile) return;  // uniform: nobody reaches the barrier
  trans_tile<PACK, E, A, B>(descs + t.desc, t.batch, t.ta, t.tb, image, lds);
}

// ---------------------------------------------------------------------------------------------------------
// fused copy + CRC-32C kernel
// ---------------------------------------------------------------------------------------------------------
// For plans that also checksum the image (plan option crc_chunk_kib).  The image is seen as cells of 4 KiB; an
// "entry" is 16 cells (64 KiB), and the plan's entry table gives, for every entry that lies inside one contiguous
// item, the tensor-side address of its first byte.  A workgroup moves kFusedRows cells that are G cells apart (G
// workgroups form a group of kFusedRows * G consecutive cells, a chunk is a whole number of groups): at any moment
// the workgroups of a group are working on G consecutive cells, which keeps the traffic as sequential as with one
// tile per workgroup, while every lane sees kFusedRows vectors at a fixed distance and can carry four Horner
// accumulators from one to the next through a byte-sliced table in LDS (advance by G cells, then add the new
// vector).  At the end the accumulators are weighted by the lane's position in the cell and summed over the
// workgroup: the remainder, relative to the end of the workgroup's last cell, of its cells laid G apart - one
// value per workgroup, chained by mlf_crc_groups_kernel.  Cells of entries without an address (record headers, item
// edges, strided items ...) are skipped here; the other kernels move them and their remainders are taken from the
// finished image.  The checksum arithmetic hides behind the memory traffic completely: with the table lookups and
// the closing multiplications taken out (values then wrong, timing only) a 51.5 GB pack takes 17.9 ms against 17.8
// with them, where the flat kernel takes 15.8; without the LDS tables and the barrier as well: 18.1; 4 / 8 / 16 / 32
// rows per workgroup with the arithmetic: 17.7 / 17.8 / 17.8 / 18.7; 2 / 3 / 4 / 6 / 8 rows requested ahead: 17.9 /
// 17.8 / 17.8 / 18.0 / 17.7; aligned granules realigned across lanes instead of byte-misaligned loads: 18.5.  What
// the kernel gives up against the flat kernel (about 11 %) is in how its workgroups walk the image, not in what
// they compute.  The closing joins a lane's four accumulators with three four-byte advances (table lookups) and
// multiplies once by the lane's weight; four general products there made 40 % of the kernel's vector instructions.
constexpr uint32_t kFusedRows = 16;   // cells per workgroup; FusedCrc::rows
constexpr uint32_t kFusedAhead = 4;   // rows requested before the first is used
constexpr uint32_t kFusedGridLog2 = 16;  // workgroups per grid row, as in the flat kernel's launch (one long row: 3 % slower)
// workgroups per group: 64 (groups of 4 MiB) and 512 (32 MiB) move the 112 GB shard equally fast when packing; unpacking
// into byte-misaligned tensors is faster with 64 (5.5 against 4.7 TB/s), and chaining 64 values per group takes 0.05 ms
// where 512 take 0.6
constexpr uint32_t kFusedMaxGroupWgs = 64;
// copies of the Horner table in LDS (4 KiB each): four copies changed nothing (11.07 against 10.84 ms on a 28 GB
// shard), the lookups are not what bounds this kernel
constexpr uint32_t kFusedTabCopies = 1;
constexpr uint32_t kCellBytes = 4096;
constexpr uint32_t kEntryBytes = 65536;
constexpr uint32_t kCellsPerEntryLog2 = 4;

template <bool PACK>
__global__ void __launch_bounds__(256) mlf_fused_crc_kernel(const uint64_t* __restrict__ ent, char* __restrict__ image,
                                                            uint32_t G, uint32_t xcd_sets, uint32_t n_wgs,
                                                            const uint32_t* __restrict__ row_tab,
                                                            const u32x4* __restrict__ lane_w,
                                                            uint32_t* __restrict__ fast_val, char* __restrict__ sink) {
  // kFusedTabCopies copies of the table, entry v of copy c at word v * copies + c, lane l reads copy l % copies:
  // lookups with random v then spread over that many times more banks
  __shared__ uint32_t tab[1024 * kFusedTabCopies];
  __shared__ uint32_t tab4[1024];  // state advanced by four bytes, sliced by state byte
  __shared__ uint32_t part[4];
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  const uint32_t wg = (blockIdx.y << kFusedGridLog2) + blockIdx.x;
  if (wg >= n_wgs) return;  // padding of the last grid row
  uint32_t group = wg / G;
  uint32_t w = wg - group * G;
  // Workgroups reach the eight XCDs round-robin, and a source line that straddles a cell cut should be served by one
  // L2, not fetched from HBM by two: neighbouring cells go to the same XCD.
  if ((G & 511u) == 0) {
    // within every 512 workgroups XCD x takes 64 consecutive cells of a row
    const uint32_t lo = w & 511u;
    w = (w & ~511u) + (lo & 7u) * 64u + (lo >> 3);
  } else if (wg < xcd_sets * 8u * G) {
    // smaller groups: of every eight consecutive groups XCD x takes group x whole (measured on the 112 GB shard with
    // groups of 64: fetched bytes 1.047 -> 1.030 x the payload, same time; what is left is one extra 128-byte line
    // per misaligned cell, fetched again because the neighbour's row passed through that L2 some microseconds earlier)
    const uint32_t set = wg / (8u * G), lo = wg - set * 8u * G;
    group = set * 8u + (lo & 7u);
    w = lo >> 3;
  }
  const uint64_t cell0 = (uint64_t)group * kFusedRows * G + w;
  uint32_t* out = fast_val + (uint64_t)group * G + w;
  // tensor-side address of each of this workgroup's cells, 0 = not ours (uniform over the workgroup: scalar loads)
  uint64_t base[kFusedRows];
  bool any = false;
#pragma unroll
  for (uint32_t k = 0; k < kFusedRows; ++k) {
    const uint64_t cell = cell0 + (uint64_t)k * G;
    const uint64_t e = ent[cell >> kCellsPerEntryLog2];
    base[k] = e ? e + ((cell & ((1u << kCellsPerEntryLog2) - 1u)) << 12) : 0;
    any |= e != 0;
  }
  if (!any) {
    if (tid == 0) *out = 0u;
    return;
  }
  u32x4 raw[kFusedAhead];
  // PACK reads the tensor side where it lies (dwordx4 loads at any byte address: the realignment across lanes that
  // the flat kernel uses for such sources costs registers here and gains nothing), UNPACK the image cell.  There is
  // no branch around a row that is not ours: it reads a 4 KiB table instead, writes to a 4 KiB sink nobody reads,
  // and is masked out of the sums.  (Uniform branches here cost a quarter of the throughput: the compiler ends the
  // waits for outstanding loads at every block boundary, and the rows no longer overlap.)
  const char* const spare_src = reinterpret_cast<const char*>(lane_w);
#define MLF_FUSED_SRC(k)                                                                          \
  ((base[k] ? (PACK ? reinterpret_cast<const char*>(base[k])                                      \
                    : const_cast<const char*>(image) + ((cell0 + (uint64_t)(k) * G) << 12))       \
            : spare_src) + tid * 16u)
#define MLF_FUSED_DST(k)                                                                          \
  ((base[k] ? (PACK ? image + ((cell0 + (uint64_t)(k) * G) << 12) : reinterpret_cast<char*>(base[k])) : sink) + tid * 16u)
#define MLF_FUSED_LOAD(slot, k) raw[slot] = __builtin_nontemporal_load(gload<u32x4_u>(MLF_FUSED_SRC(k)))
#pragma unroll
  for (uint32_t k = 0; k < kFusedAhead; ++k) MLF_FUSED_LOAD(k, k);
#pragma unroll
  for (uint32_t k = 0; k < 4; ++k) {
    const uint32_t t = row_tab[tid + 256u * k];
#pragma unroll
    for (uint32_t c = 0; c < kFusedTabCopies; ++c) tab[(tid + 256u * k) * kFusedTabCopies + c] = t;
    tab4[tid + 256u * k] = row_tab[1024u + tid + 256u * k];
  }
  __syncthreads();
  const uint32_t* my = tab + (lane & (kFusedTabCopies - 1u));
#define MLF_FUSED_ADV(a)                                                                          \
  (my[((a) & 255u) * kFusedTabCopies] ^ my[(256u + (((a) >> 8) & 255u)) * kFusedTabCopies] ^      \
   my[(512u + (((a) >> 16) & 255u)) * kFusedTabCopies] ^ my[(768u + ((a) >> 24)) * kFusedTabCopies])
  uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0;
#pragma unroll
  for (uint32_t k = 0; k < kFusedRows; ++k) {
    const u32x4 v = raw[k % kFusedAhead];  // the cell's vector as it lies in the image
    if (k + kFusedAhead < kFusedRows)      // the slot just read is free again
      MLF_FUSED_LOAD(k % kFusedAhead, k + kFusedAhead);
    __builtin_nontemporal_store(v, gstore<u32x4_u>(MLF_FUSED_DST(k)));
    const uint32_t ours = base[k] ? 0xFFFFFFFFu : 0u;
    a0 = MLF_FUSED_ADV(a0) ^ (v.x & ours);
    a1 = MLF_FUSED_ADV(a1) ^ (v.y & ours);
    a2 = MLF_FUSED_ADV(a2) ^ (v.z & ours);
    a3 = MLF_FUSED_ADV(a3) ^ (v.w & ours);
    // rows stay in this order (without the fence the compiler may hoist all sixteen loads to the top)
    __asm__ volatile("" ::: "memory");
  }
#undef MLF_FUSED_SRC
#undef MLF_FUSED_DST
#undef MLF_FUSED_ADV
#undef MLF_FUSED_LOAD
  // The lane's four dwords lie next to each other, so their remainders are joined by three advances of four bytes
  // (table lookups), and only the joined value needs a general multiplication by the lane's weight: one bitwise
  // product per lane and workgroup instead of four.
#define MLF_FUSED_ADV4(a) \
  (tab4[(a) & 255u] ^ tab4[256u + (((a) >> 8) & 255u)] ^ tab4[512u + (((a) >> 16) & 255u)] ^ tab4[768u + ((a) >> 24)])
  uint32_t joined = MLF_FUSED_ADV4(a0) ^ a1;
  joined = MLF_FUSED_ADV4(joined) ^ a2;
  joined = MLF_FUSED_ADV4(joined) ^ a3;
#undef MLF_FUSED_ADV4
  uint32_t acc = gf_mul(joined, lane_w[tid].w);
#pragma unroll
  for (int s = 1; s < 64; s <<= 1) acc ^= (uint32_t)__shfl_xor((int)acc, s, 64);
  if (lane == 0u) part[tid >> 6] = acc;
  __syncthreads();
  if (tid == 0) *out = part[0] ^ part[1] ^ part[2] ^ part[3];
}

}  // namespace

// ---------------------------------------------------------------------------------------------------------
// plan
// ---------------------------------------------------------------------------------------------------------
constexpr int kSpanClasses = 4;
constexpr int kSmallClass = 3;  // items <= kSmallItemBytes: served per wavefront by mlf_small_kernel
constexpr uint32_t kSpanShift[kSpanClasses] = {flat_shift(0), flat_shift(1), flat_shift(2), 0};  // 128, 16 or 1 tiles per entry
static_assert(kSmallClass == kFlatClasses, "the small-item class follows the flat classes");

struct mlf_plan {
  int device = 0;
  Span* d_spans[kSpanClasses] = {nullptr, nullptr, nullptr, nullptr};
  uint64_t n_spans[kSpanClasses] = {0, 0, 0, 0};
  uint32_t tile_bytes = 4096;
  StridedDesc* d_descs = nullptr;
  StridedWork* d_work = nullptr;   // work of the generic walk
  GatherWork* d_gwork = nullptr;  // row pieces of the `[..., ::k]` items: vector gather when packing, LDS scatter when unpacking
  uint64_t n_work = 0, n_gwork = 0;
  TransDesc* d_tdescs = nullptr;
  // the transpose kernel's tile table when packing [0] and unpacking [1]: one range per element size 1, 2, 4, 8, 16
  TransTile* d_ttiles[2] = {nullptr, nullptr};
  uint64_t ttiles_first[2][kTransClasses + 1] = {{0}, {0}};
  char* d_blob = nullptr;
  uint64_t blob_size = 0;
  char* h_blob = nullptr;            // pinned staging of mlf_plan_update_blob, allocated on first use
  hipEvent_t blob_copied = nullptr;  // recorded behind the last upload out of h_blob
  mutable hipEvent_t launched = nullptr;  // recorded behind the last launch (plans with a blob): an upload of new
                                          // blob bytes on another stream waits for the kernels that read the old ones
  uint32_t block_threads = 256;
  uint32_t unroll = 1;
  uint32_t cut_mask = 15;     // tile cuts sit on multiples of cut_mask + 1 bytes ...
  uint32_t cut_on_tensor = 0;  // ... of the tensor address (1) or of the image offset (0)
  uint32_t grid_x_log2 = 20;  // log2 of the workgroups per grid row of the flat kernel's launch
  uint32_t flat_first[kFlatClasses] = {0, 0, 0};  // first workgroup of each span class in that launch
  uint32_t flat_total = 0;
  mlf_plan_info info{};
  bool has_crc = false;      // launches also fold the image's CRC-32C (plan option crc_chunk_kib)
  mutable FusedCrc crc;      // its tables and values; the values are rewritten by every launch
  mlf_plan() = default;
  mlf_plan(const mlf_plan&) = delete;
  mlf_plan& operator=(const mlf_plan&) = delete;
  ~mlf_plan() {  // every exit path of mlf_plan_create, and mlf_plan_destroy
    for (Span* t : d_spans) (void)hipFree(t);
    (void)hipFree(d_descs);
    (void)hipFree(d_work);
    (void)hipFree(d_gwork);
    (void)hipFree(d_tdescs);
    (void)hipFree(d_ttiles[0]);
    (void)hipFree(d_ttiles[1]);
    (void)hipFree(d_blob);
    if (h_blob) (void)hipHostFree(h_blob);
    if (blob_copied) (void)hipEventDestroy(blob_copied);
    if (launched) (void)hipEventDestroy(launched);
    crc_fused_destroy(&crc);
  }
};

namespace {

constexpr uint32_t kDefaultTileBytes = 4096;
constexpr uint32_t kStridedElemsPerBlock = 32 * 1024;
constexpr uint32_t kGatherMinRow = 256;         // `[..., ::k]` rows at least this long take the vector gather
constexpr uint32_t kGatherUnitsPerBlock = 256 * kGatherSplit;  // 16-byte output vectors per work item: one per thread of each of its workgroups

struct SpanTables {
  std::vector<Span> cls[kSpanClasses];
};

// Covers [0, n) of one contiguous item with spans: as many 128-tile entries as fit, then 16-tile entries, then
// single tiles; a rest of at most 1 KiB goes to the per-wavefront table.  Every entry is self-contained (the kernel derives tile cuts from the entry's own first
// destination address), so pieces may start anywhere.
void cut_spans(SpanTables& out, uint64_t tensor_addr, uint64_t image_off, uint64_t n, uint32_t tile,
               bool align_to_tensor, uint32_t cut_mask) {
  uint64_t done = 0;
  while (done < n) {
    const uint64_t cut_pos = (align_to_tensor ? tensor_addr : image_off) + done;
    const uint64_t head = (0 - cut_pos) & cut_mask;  // bytes to the next grid line; 0 after an item's first span
    const uint64_t left = n - done;
    if (left <= kSmallItemBytes) {
      out.cls[kSmallClass].push_back(Span{tensor_addr + done, image_off + done, (uint32_t)left, 0});
      break;
    }
    // an entry of class c holds head + (tile << shift) bytes: its first tile carries the head on top, so every
    // later tile, and every later span of the item, starts on the grid; the single-tile class also takes a short rest
    int c = kSmallClass - 1;
    for (int k = 0; k < kSmallClass; ++k) {
      if (left >= head + ((uint64_t)tile << kSpanShift[k])) {
        c = k;
        break;
      }
    }
    const uint64_t len = std::min<uint64_t>(left, head + ((uint64_t)tile << kSpanShift[c]));
    out.cls[c].push_back(Span{tensor_addr + done, image_off + done, (uint32_t)len, 0});
    done += len;
  }
}

// One contiguous run of an item.  With checksums, the whole 64 KiB entries of the image that the run covers (below
// `fused_entries`) go to the fused copy + CRC kernel - the entry table gets their tensor-side addresses - and only
// the edges go to the span tables.
struct FlatSink {
  SpanTables* tables;
  std::vector<uint64_t>* ent;  // null: no checksums
  uint64_t fused_entries;
  uint64_t fused_bytes;
  uint32_t tile;
  bool align_to_tensor;
  uint32_t cut_mask;
  void add(uint64_t tensor_addr, uint64_t image_off, uint64_t n) {
    if (ent) {
      const uint64_t e0 = (image_off + kEntryBytes - 1) / kEntryBytes;
      const uint64_t e1 = std::min<uint64_t>((image_off + n) / kEntryBytes, fused_entries);
      if (e1 > e0) {
        // An entry has one address: when two runs cover the same image range (an unpack that restores one record
        // into two targets), the first keeps the entry and the later run's share of it goes to the span tables
        // like any edge, so both targets are written and every byte of the image is checksummed once.
        uint64_t at = 0;  // bytes of the run handed out so far
        for (uint64_t e = e0; e < e1; ++e) {
          if ((*ent)[e]) continue;
          const uint64_t from = e * kEntryBytes - image_off;
          if (from > at) cut_spans(*tables, tensor_addr + at, image_off + at, from - at, tile, align_to_tensor, cut_mask);
          (*ent)[e] = tensor_addr + from;
          fused_bytes += kEntryBytes;
          at = from + kEntryBytes;
        }
        if (at < n) cut_spans(*tables, tensor_addr + at, image_off + at, n - at, tile, align_to_tensor, cut_mask);
        return;
      }
    }
    cut_spans(*tables, tensor_addr, image_off, n, tile, align_to_tensor, cut_mask);
  }
};

struct Collapsed {
  int ndim;
  int64_t shape[MLF_MAX_DIMS], ts[MLF_MAX_DIMS], is[MLF_MAX_DIMS];
};

// Drops size-1 dims and merges neighbours that are jointly contiguous on both sides (strides in elements).
Collapsed collapse_dims(const mlf_item& it) {
  Collapsed c{};
  int n = 0;
  for (uint32_t d = 0; d < it.ndim; ++d) {
    if (it.shape[d] == 1) continue;
    if (n > 0 && c.ts[n - 1] == it.stride[d] * it.shape[d] && c.is[n - 1] == it.image_stride[d] * it.shape[d]) {
      c.shape[n - 1] *= it.shape[d];
      c.ts[n - 1] = it.stride[d];
      c.is[n - 1] = it.image_stride[d];
    } else {
      c.shape[n] = it.shape[d];
      c.ts[n] = it.stride[d];
      c.is[n] = it.image_stride[d];
      ++n;
    }
  }
  c.ndim = n;
  return c;
}

// The transpose kernel's tile table.  Every transposed item's tile grid is cut into patches of patch_a x patch_b
// neighbouring tiles (the grid's rim: what is left); a patch goes, whole, to the XCD whose list is shortest so far,
// which keeps the eight lists level and neighbouring patches in flight at about the same time.  The table interleaves
// the lists - entry 8 s + x is the s-th tile of XCD x - and pads the shorter ones with empty entries.
// Patches are long along the side that is written - partly written lines then meet in one L2, which matters more
// than partly used fetched lines meeting there.  Same 667 blocks, patches of (tiles along the read side) x (along
// the written side): 1 x 64 4.17 / 3.93 with 128 x 128-byte tiles, 64 x 1 3.13 / 4.39 (the written side is a for an
// unpack), 8 x 8 4.10 / 4.41; with 128 x 256-byte tiles 2 x 16 4.34 / 4.49, 4 x 16 4.47 / 4.50, 8 x 8 4.36 / 4.44;
// larger patches change nothing (8 x 16 4.43 / 4.45, 4 x 32 4.47 / 4.46, 4 x 64 4.49 / 4.43, 16 x 32 4.37 / 4.33).
constexpr uint32_t kTransPatchRead = 4, kTransPatchWritten = 16;
struct TransOrder {
  uint32_t patch_a = 1, patch_b = 1;
  std::vector<TransTile> list[8];
  uint32_t next = 0;  // where the search for the shortest list starts: ties go round
  void add(uint32_t desc, uint32_t tiles_a, uint32_t tiles_b, uint32_t batches) {
    for (uint32_t batch = 0; batch < batches; ++batch)
      for (uint32_t a0 = 0; a0 < tiles_a; a0 += patch_a)
        for (uint32_t b0 = 0; b0 < tiles_b; b0 += patch_b) {
          uint32_t x = next;
          for (uint32_t k = 1; k < 8; ++k)
            if (list[(next + k) & 7].size() < list[x].size()) x = (next + k) & 7;
          next = (x + 1) & 7;
          const uint32_t a1 = std::min(tiles_a, a0 + patch_a), b1 = std::min(tiles_b, b0 + patch_b);
          for (uint32_t tb = b0; tb < b1; ++tb)
            for (uint32_t ta = a0; ta < a1; ++ta) list[x].push_back(TransTile{desc, ta, tb, batch});
        }
  }
  std::vector<TransTile> interleaved() const {
    size_t longest = 0;
    for (const auto& l : list) longest = std::max(longest, l.size());
    std::vector<TransTile> out(longest * 8, TransTile{kNoTile, 0, 0, 0});
    for (uint32_t x = 0; x < 8; ++x)
      for (size_t s = 0; s < list[x].size(); ++s) out[s * 8 + x] = list[x][s];
    return out;
  }
};

template <typename T>
int upload(const std::vector<T>& host, T** dev) {
  *dev = nullptr;
  if (host.empty()) return MLF_HIP_OK;
  HIP_TRY(hipMalloc(reinterpret_cast<void**>(dev), host.size() * sizeof(T)));
  HIP_TRY(hipMemcpy(*dev, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice));
  return MLF_HIP_OK;
}

}  // namespace

extern "C" {

const char* mlf_hip_last_error(void) { return last_error().c_str(); }

int mlf_hip_device_count(int* out) {
  if (!out) return fail(MLF_HIP_BAD_ARG, "null out");
  HIP_TRY(hipGetDeviceCount(out));
  return MLF_HIP_OK;
}

int mlf_hip_set_device(int device) {
  HIP_TRY(hipSetDevice(device));
  // set-up of the library on this device: the address of mlf_crc32c_device_noalloc's scratch array is resolved here,
  // so that the entry point itself may be called while a stream is being captured
  return crc_noalloc_prime(device);
}

int mlf_hip_mem_info(uint64_t* free_bytes, uint64_t* total_bytes) {
  size_t f = 0, t = 0;
  HIP_TRY(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = f;
  if (total_bytes) *total_bytes = t;
  return MLF_HIP_OK;
}

int mlf_plan_create(const mlf_item* items, uint64_t n_items, const void* host_blob, uint64_t blob_bytes,
                    uint64_t image_bytes, const mlf_plan_opts* opts, mlf_plan** out) {
  if (!out) return fail(MLF_HIP_BAD_ARG, "null out");
  *out = nullptr;
  if (n_items && !items) return fail(MLF_HIP_BAD_ARG, "null items");
  if (blob_bytes && !host_blob) return fail(MLF_HIP_BAD_ARG, "null host_blob with blob_bytes > 0");
  if (image_bytes >> 60) return fail(MLF_HIP_BAD_ARG, "image_bytes is not a plausible size");  // keeps the checks below from wrapping
  uint32_t tile = opts && opts->tile_bytes ? opts->tile_bytes : kDefaultTileBytes;
  uint32_t threads = opts && opts->block_threads ? opts->block_threads : 256;
  const bool align_to_tensor = opts && opts->align_to_tensor;
  if (tile % 1024 || tile > (1u << 20)) return fail(MLF_HIP_BAD_ARG, "tile_bytes must be a multiple of 1024, at most 1 MiB");
  if (threads % 64 || threads > 1024) return fail(MLF_HIP_BAD_ARG, "block_threads must be a multiple of 64, at most 1024");

  std::unique_ptr<mlf_plan> plan(new mlf_plan());
  HIP_TRY(hipGetDevice(&plan->device));
  plan->block_threads = threads;
  plan->tile_bytes = tile;
  plan->unroll = opts && opts->unroll ? opts->unroll : 1;
  // cuts on the largest power of two that divides the tile size, at most 4 KiB: full tiles then write whole lines
  plan->cut_mask = std::min<uint32_t>(tile & (0u - tile), 4096u) - 1u;
  plan->cut_on_tensor = align_to_tensor ? 1u : 0u;
  // gridDim.x * blockDim.x must stay below 2^32.  Rows of 2^16 workgroups measured fastest on the 112 GB shard
  // (36.5 ms per pack; rows of 2^20: 36.9 ms, of 2^23: 39.2 ms)
  uint32_t widest = 0;
  while (((uint64_t)2 << widest) * threads < ((uint64_t)1 << 32)) ++widest;
  plan->grid_x_log2 = opts && opts->grid_x_log2 ? opts->grid_x_log2 - 1 : 16;
  if (plan->grid_x_log2 > widest) return fail(MLF_HIP_BAD_ARG, "grid_x_log2: a grid row of that many workgroups exceeds 2^32 threads");
  if (plan->unroll != 1 && plan->unroll != 2 && plan->unroll != 4 && plan->unroll != 8)
    return fail(MLF_HIP_BAD_ARG, "unroll must be 1, 2, 4 or 8");
  std::vector<uint64_t> ent;
  uint64_t fused_entries = 0;
  if (opts && opts->crc_chunk_kib && image_bytes) {
    if (opts->crc_chunk_kib % 64) return fail(MLF_HIP_BAD_ARG, "crc_chunk_kib must be a multiple of 64");
    FusedCrc& f = plan->crc;
    f.image_bytes = image_bytes;
    f.chunk_bytes = (uint64_t)opts->crc_chunk_kib << 10;
    f.rows = kFusedRows;
    // a chunk is a whole number of groups of rows * G cells: G = the largest divisor of chunk cells / rows up to 512
    const uint64_t m = f.chunk_bytes / kCellBytes / kFusedRows;
    uint32_t G = 1;
    for (uint32_t d = 1; d <= kFusedMaxGroupWgs && d <= m; ++d)
      if (m % d == 0) G = d;
    f.wgs_per_group = G;
    // whole groups only, and no more workgroups than one grid row holds
    f.fused_groups = std::min<uint64_t>(image_bytes / kCellBytes / ((uint64_t)kFusedRows * G), ((1u << 24) - 1) / G);
    f.n_ent = (image_bytes + kEntryBytes - 1) / kEntryBytes;
    if (f.n_ent >= 0xFFFFFFF0ull) return fail(MLF_HIP_BAD_ARG, "image too large for per-chunk checksums");
    fused_entries = f.fused_groups * kFusedRows * G / (kEntryBytes / kCellBytes);
    ent.assign(f.n_ent, 0);
    plan->has_crc = true;
  }
  plan->blob_size = blob_bytes;
  if (blob_bytes) {
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&plan->d_blob), blob_bytes));
    HIP_TRY(hipMemcpy(plan->d_blob, host_blob, blob_bytes, hipMemcpyHostToDevice));
  }
  const uint64_t blob_base = reinterpret_cast<uint64_t>(plan->d_blob);

  SpanTables tiles;
  FlatSink flat{&tiles, plan->has_crc ? &ent : nullptr, fused_entries, 0, tile, align_to_tensor, plan->cut_mask};
  std::vector<StridedDesc> descs;
  std::vector<StridedWork> work;
  std::vector<GatherWork> gwork;
  std::vector<TransDesc> tdescs;
  TransOrder torder[2][kTransClasses];
  for (auto& o : torder[0]) o.patch_a = kTransPatchRead, o.patch_b = kTransPatchWritten;
  for (auto& o : torder[1]) o.patch_a = kTransPatchWritten, o.patch_b = kTransPatchRead;
  mlf_plan_info& info = plan->info;
  info.n_items = n_items;
  info.image_bytes = image_bytes;
  int rc = MLF_HIP_OK;
  for (uint64_t k = 0; k < n_items && rc == MLF_HIP_OK; ++k) {
    const mlf_item& it = items[k];
    if (it.nbytes == 0) continue;
    if (it.image_off > image_bytes || it.nbytes > image_bytes - it.image_off) {
      rc = fail(MLF_HIP_BAD_ARG, "item " + std::to_string(k) + " does not fit in the image");
      break;
    }
    if (it.kind == MLF_ITEM_BLOB) {
      if (it.ptr > blob_bytes || it.nbytes > blob_bytes - it.ptr) {
        rc = fail(MLF_HIP_BAD_ARG, "blob item " + std::to_string(k) + " lies outside the host blob");
        break;
      }
      flat.add(blob_base + it.ptr, it.image_off, it.nbytes);
      info.blob_bytes += it.nbytes;
      continue;
    }
    if (it.kind != MLF_ITEM_DEVICE) {
      rc = fail(MLF_HIP_BAD_ARG, "item " + std::to_string(k) + " has an unknown kind");
      break;
    }
    const uint32_t esz = it.elem_size;
    if (!(esz == 1 || esz == 2 || esz == 4 || esz == 8 || esz == 16) || it.ndim > MLF_MAX_DIMS || it.ptr == 0) {
      rc = fail(MLF_HIP_BAD_ARG, "item " + std::to_string(k) + " has a bad element size, rank or null pointer");
      break;
    }
    uint64_t numel = 1;
    bool bad = false;
    for (uint32_t d = 0; d < it.ndim && !bad; ++d)
      bad = it.shape[d] <= 0 || __builtin_mul_overflow(numel, (uint64_t)it.shape[d], &numel);
    if (bad || numel > it.nbytes || numel * esz != it.nbytes) {
      rc = fail(MLF_HIP_BAD_ARG, "item " + std::to_string(k) + ": shape does not match nbytes");
      break;
    }
    // the image side must stay inside the item's declared span of the image
    {
      int64_t lo = 0, hi = 0;
      bool wraps = false;
      for (uint32_t d = 0; d < it.ndim; ++d) {
        int64_t reach = 0;
        wraps |= __builtin_mul_overflow(it.shape[d] - 1, it.image_stride[d], &reach);
        wraps |= __builtin_add_overflow(reach < 0 ? lo : hi, reach, reach < 0 ? &lo : &hi);
      }
      wraps |= lo < -((int64_t)1 << 56) || hi > ((int64_t)1 << 56);  // times at most 16 bytes per element below
      const int64_t first = wraps ? -1 : (int64_t)it.image_off + lo * (int64_t)esz;
      const uint64_t last = wraps ? 0 : it.image_off + (uint64_t)hi * esz + esz;
      if (wraps || first < 0 || last > image_bytes) {
        rc = fail(MLF_HIP_BAD_ARG, "item " + std::to_string(k) + ": image-side strides reach outside the image");
        break;
      }
    }
    info.device_bytes += it.nbytes;
    const Collapsed c = collapse_dims(it);
    if (c.ndim == 0 || (c.ndim == 1 && c.ts[0] == 1 && c.is[0] == 1)) {
      flat.add(it.ptr, it.image_off, it.nbytes);
      continue;
    }
    // rows that are contiguous on both sides and long enough go through the flat kernel, one row at a time
    const int last = c.ndim - 1;
    const uint64_t row_bytes = (uint64_t)c.shape[last] * esz;
    const uint64_t n_rows = numel / (uint64_t)c.shape[last];
    if (c.ts[last] == 1 && c.is[last] == 1 && row_bytes >= 2048 && n_rows <= (1u << 22)) {
      int64_t idx[MLF_MAX_DIMS] = {0};
      for (uint64_t r = 0; r < n_rows; ++r) {
        int64_t toff = 0, ioff = 0;
        for (int d = 0; d < last; ++d) {
          toff += idx[d] * c.ts[d];
          ioff += idx[d] * c.is[d];
        }
        flat.add(it.ptr + (uint64_t)(toff * (int64_t)esz), it.image_off + (uint64_t)(ioff * (int64_t)esz), row_bytes);
        for (int d = last - 1; d >= 0; --d) {
          if (++idx[d] < c.shape[d]) break;
          idx[d] = 0;
        }
      }
      continue;
    }
    // a dimension other than the last that is contiguous on the tensor side while the last one is contiguous on
    // the image side: a transposition.  Both extents must be worth a tile.
    if (c.is[last] == 1 && c.ts[last] != 1 && c.shape[last] >= 16) {
      int a = -1;
      for (int d = 0; d < last; ++d)
        if (c.ts[d] == 1 && c.shape[d] >= 16) a = d;
      if (a >= 0) {
        TransDesc td{};
        td.tensor = it.ptr;
        td.image = it.image_off;
        td.esz = esz;
        td.na = c.shape[a];
        td.nb = c.shape[last];
        td.ld_t = c.ts[last] * (int64_t)esz;
        td.ld_i = c.is[a] * (int64_t)esz;
        // tile cuts on the 128-byte lines of both sides (where the addresses are multiples of the element size)
        if (it.ptr % esz == 0) td.a_lead = (uint32_t)(it.ptr % 128u) / esz;
        if (it.image_off % esz == 0) td.b_lead = (uint32_t)(it.image_off % 128u) / esz;
        uint64_t batches = 1;
        for (int d = 0; d < last; ++d) {
          if (d == a) continue;
          td.bshape[td.nbatch] = c.shape[d];
          td.bts[td.nbatch] = c.ts[d] * (int64_t)esz;
          td.bis[td.nbatch] = c.is[d] * (int64_t)esz;
          ++td.nbatch;
          batches *= (uint64_t)c.shape[d];
        }
        if (batches >> 32 || td.na >> 35 || td.nb >> 35 || tdescs.size() >= kNoTile) {
          rc = fail(MLF_HIP_BAD_ARG, "item " + std::to_string(k) + ": too many tiles in a transposed view");
          break;
        }
        for (int dir = 0; dir < 2; ++dir) {
          const uint32_t A = trans_tile_a(esz, dir == 0), B = trans_tile_b(esz, dir == 0);
          torder[dir][__builtin_ctz(esz)].add((uint32_t)tdescs.size(), (uint32_t)((td.na + td.a_lead + A - 1) / A),
                          (uint32_t)((td.nb + td.b_lead + B - 1) / B), (uint32_t)batches);
        }
        tdescs.push_back(td);
        ++info.n_transposed_items;
        continue;
      }
    }
    const int lastd = c.ndim - 1;
    // `[..., ::k]` of long rows.  Measured on `[:, ::k]` of 8192 x 16384 parents (TB/s of 2 x payload, element walk ->
    // vector gather): k = 2: 1.0 -> 3.2 (1-byte), 1.7 -> 3.5 (2), 3.2 -> 3.6 (4), 3.3 -> 3.6 (8); k = 3: 1.0 -> 2.1 (1),
    // 1.6 -> 2.2 (2), but 2.3 -> 1.7 (4): wider elements keep the element walk unless k = 2
    if (esz <= 8 && c.is[lastd] == 1 && c.ts[lastd] >= 2 && c.ts[lastd] <= 4 && (esz <= 2 || c.ts[lastd] == 2) &&
        c.shape[lastd] >= (int64_t)kGatherMinRow && numel / (uint64_t)c.shape[lastd] <= (1u << 24)) {
      // row by row: a work item never crosses a row, so its elements are evenly spaced on both sides
      const uint64_t row_len = (uint64_t)c.shape[lastd], rows = numel / row_len;
      const uint64_t piece = (uint64_t)kGatherUnitsPerBlock * (16 / esz);
      const uint64_t k = (uint64_t)c.ts[lastd];
      int64_t idx[MLF_MAX_DIMS] = {0};
      for (uint64_t r = 0; r < rows; ++r) {
        int64_t toff = 0, ioff = 0;
        for (int d = 0; d < lastd; ++d) {
          toff += idx[d] * c.ts[d];
          ioff += idx[d] * c.is[d];
        }
        const uint64_t trow = it.ptr + (uint64_t)(toff * (int64_t)esz), irow = it.image_off + (uint64_t)(ioff * (int64_t)esz);
        for (uint64_t j = 0; j < row_len; j += piece)
          gwork.push_back(GatherWork{trow + j * k * esz, irow + j * esz, (uint32_t)std::min<uint64_t>(piece, row_len - j),
                                     (uint16_t)k, (uint16_t)esz});
        for (int d = lastd - 1; d >= 0; --d) {
          if (++idx[d] < c.shape[d]) break;
          idx[d] = 0;
        }
      }
      ++info.n_strided_items;
      continue;
    }
    StridedDesc sd{};
    sd.tensor = it.ptr;
    sd.image = it.image_off;
    sd.esz = esz;
    sd.ndim = (uint32_t)c.ndim;
    for (int d = 0; d < c.ndim; ++d) {
      sd.shape[d] = c.shape[d];
      sd.tstride[d] = c.ts[d] * (int64_t)esz;
      sd.istride[d] = c.is[d] * (int64_t)esz;
    }
    {  // 256 in the mixed radix of the collapsed shape (least significant digit = last dimension)
      uint64_t rest = 256;
      for (int d = c.ndim - 1; d >= 0; --d) {
        sd.step[d] = (int64_t)(rest % (uint64_t)c.shape[d]);
        rest /= (uint64_t)c.shape[d];
      }
    }
    const uint32_t desc_idx = (uint32_t)descs.size();
    descs.push_back(sd);
    for (uint64_t s0 = 0; s0 < numel; s0 += kStridedElemsPerBlock)
      work.push_back(StridedWork{s0, (uint32_t)std::min<uint64_t>(kStridedElemsPerBlock, numel - s0), desc_idx});
    ++info.n_strided_items;
  }
  for (int c = 0; c < kSpanClasses && rc == MLF_HIP_OK; ++c) {
    if (rc == MLF_HIP_OK) rc = upload(tiles.cls[c], &plan->d_spans[c]);
    plan->n_spans[c] = tiles.cls[c].size();
  }
  if (rc == MLF_HIP_OK) rc = upload(descs, &plan->d_descs);
  if (rc == MLF_HIP_OK) rc = upload(work, &plan->d_work);
  if (rc == MLF_HIP_OK) rc = upload(gwork, &plan->d_gwork);
  plan->n_work = work.size();
  plan->n_gwork = gwork.size();
  if (rc == MLF_HIP_OK) rc = upload(tdescs, &plan->d_tdescs);
  for (int dir = 0; dir < 2; ++dir) {
    std::vector<TransTile> ttiles;
    for (int cls = 0; cls < kTransClasses; ++cls) {
      const std::vector<TransTile> part = torder[dir][cls].interleaved();
      ttiles.insert(ttiles.end(), part.begin(), part.end());
      plan->ttiles_first[dir][cls + 1] = ttiles.size();
    }
    if (rc == MLF_HIP_OK) rc = upload(ttiles, &plan->d_ttiles[dir]);
  }
  if (rc == MLF_HIP_OK && plan->has_crc) {
    // entries the fused kernel does not serve are checksummed from the finished image
    std::vector<uint32_t> slow;
    for (uint64_t e = 0; e < ent.size(); ++e)
      if (!ent[e]) slow.push_back((uint32_t)e);
    plan->crc.n_slow = slow.size();
    rc = upload(ent, &plan->crc.d_ent);
    if (rc == MLF_HIP_OK) rc = upload(slow, &plan->crc.d_slow_list);
    if (rc == MLF_HIP_OK) rc = crc_fused_setup(&plan->crc);
    info.fused_crc_bytes = flat.fused_bytes;
    info.crc_chunks = plan->crc.n_chunks;
  }
  if (rc != MLF_HIP_OK) {
    const std::string keep = last_error();
    mlf_plan_destroy(plan.release());
    last_error() = keep;
    return rc;
  }
  info.n_flat_tiles = 0;
  info.table_bytes = descs.size() * sizeof(StridedDesc) + work.size() * sizeof(StridedWork) + gwork.size() * sizeof(GatherWork) +
                     tdescs.size() * sizeof(TransDesc) + (plan->ttiles_first[0][kTransClasses] + plan->ttiles_first[1][kTransClasses]) * sizeof(TransTile) + blob_bytes;
  info.n_transposed_work = std::max(plan->ttiles_first[0][kTransClasses], plan->ttiles_first[1][kTransClasses]);
  for (int c = 0; c < kSpanClasses; ++c) {
    if (c != kSmallClass) info.n_flat_tiles += plan->n_spans[c] << kSpanShift[c];
    info.table_bytes += plan->n_spans[c] * sizeof(Span);
  }
  info.n_small_items = plan->n_spans[kSmallClass];
  {
    uint64_t wgs = 0;
    for (int c = 0; c < kFlatClasses; ++c) {
      plan->flat_first[c] = (uint32_t)wgs;
      wgs += plan->n_spans[c] << kSpanShift[c];
    }
    if (wgs >= 0xFFFFFFFFull || ((wgs + (1ull << plan->grid_x_log2) - 1) >> plan->grid_x_log2) > 65535) {
      mlf_plan_destroy(plan.release());
      return fail(MLF_HIP_BAD_ARG, "too many tiles for one launch: use a larger tile_bytes");
    }
    plan->flat_total = (uint32_t)wgs;
  }
  info.n_strided_work = work.size() + gwork.size();
  *out = plan.release();
  return MLF_HIP_OK;
}

int mlf_plan_destroy(mlf_plan* plan) {
  delete plan;  // the destructor frees the device tables
  return MLF_HIP_OK;
}

int mlf_plan_update_blob(mlf_plan* plan, const void* host_blob, uint64_t blob_bytes, void* stream) {
  if (!plan) return fail(MLF_HIP_BAD_ARG, "null plan");
  if (blob_bytes != plan->blob_size)
    return fail(MLF_HIP_BAD_ARG, "blob of " + std::to_string(blob_bytes) + " bytes for a plan built with " +
                                     std::to_string(plan->blob_size));
  if (blob_bytes == 0) return MLF_HIP_OK;
  if (!host_blob) return fail(MLF_HIP_BAD_ARG, "null host_blob");
  HIP_TRY(hipSetDevice(plan->device));
  if (!plan->h_blob) {
    if (!plan->blob_copied) HIP_TRY(hipEventCreateWithFlags(&plan->blob_copied, hipEventDisableTiming));
    HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&plan->h_blob), blob_bytes, hipHostMallocDefault));
  } else {
    HIP_TRY(hipEventSynchronize(plan->blob_copied));  // the previous upload has left the staging buffer
  }
  memcpy(plan->h_blob, host_blob, blob_bytes);
  // behind the launches that still read the old bytes - also when they ran on another stream than this one -
  // and, ordered on the caller's stream, ahead of those to come
  if (plan->launched) HIP_TRY(hipStreamWaitEvent(static_cast<hipStream_t>(stream), plan->launched, 0));
  HIP_TRY(hipMemcpyAsync(plan->d_blob, plan->h_blob, blob_bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
  HIP_TRY(hipEventRecord(plan->blob_copied, static_cast<hipStream_t>(stream)));
  return MLF_HIP_OK;
}

int mlf_plan_get_info(const mlf_plan* plan, mlf_plan_info* out) {
  if (!plan || !out) return fail(MLF_HIP_BAD_ARG, "null argument");
  *out = plan->info;
  return MLF_HIP_OK;
}

}  // extern "C"

namespace {

template <bool PACK>
int launch_plan(const mlf_plan* plan, char* image, hipStream_t stream) {
  if (!plan) return fail(MLF_HIP_BAD_ARG, "null plan");
  if (!image && plan->info.image_bytes) return fail(MLF_HIP_BAD_ARG, "null image");
  if (reinterpret_cast<uintptr_t>(image) & 255) return fail(MLF_HIP_BAD_ARG, "image must be 256-byte aligned");
  if (plan->has_crc) {
    const FusedCrc& f = plan->crc;
    const uint64_t n_wg = f.fused_groups * f.wgs_per_group;
    if (n_wg) {
      const dim3 grid(std::min<uint32_t>((uint32_t)n_wg, 1u << kFusedGridLog2),
                      (uint32_t)((n_wg + (1u << kFusedGridLog2) - 1) >> kFusedGridLog2));
      hipLaunchKernelGGL((mlf_fused_crc_kernel<PACK>), grid, dim3(256), 0, stream, f.d_ent, image,
                         f.wgs_per_group, (uint32_t)(f.fused_groups / 8), (uint32_t)n_wg, f.d_row_tab, f.d_lane_w,
                         f.d_fast_val, f.d_sink);
      HIP_TRY(hipGetLastError());
    }
  }
  if (plan->flat_total) {
    // gridDim.x * blockDim.x must stay below 2^32; what does not fit in one row of workgroups goes to gridDim.y
    const uint32_t row_log2 = plan->grid_x_log2, total = plan->flat_total;
    const dim3 grid(std::min(total, 1u << row_log2), (total + (1u << row_log2) - 1) >> row_log2), block(plan->block_threads);
#define MLF_FLAT_LAUNCH(U)                                                                                     \
  hipLaunchKernelGGL((mlf_flat_kernel<PACK, U>), grid, block, 0, stream, plan->d_spans[0], plan->d_spans[1],     \
                     plan->d_spans[2], plan->flat_first[1], plan->flat_first[2], total, row_log2,              \
                     plan->tile_bytes, plan->block_threads, plan->cut_mask, plan->cut_on_tensor, image)
    switch (plan->unroll) {
      case 2: MLF_FLAT_LAUNCH(2); break;
      case 4: MLF_FLAT_LAUNCH(4); break;
      case 8: MLF_FLAT_LAUNCH(8); break;
      default: MLF_FLAT_LAUNCH(1); break;
    }
#undef MLF_FLAT_LAUNCH
    HIP_TRY(hipGetLastError());
  }
  for (uint64_t first = 0; first < plan->n_spans[kSmallClass]; first += (1u << 24)) {
    const uint32_t count = (uint32_t)std::min<uint64_t>(1u << 24, plan->n_spans[kSmallClass] - first);
    hipLaunchKernelGGL((mlf_small_kernel<PACK>), dim3((count + 3) / 4), dim3(256), 0, stream,
                       plan->d_spans[kSmallClass] + first, count, image);
    HIP_TRY(hipGetLastError());
  }
  for (int cls = 0; cls < kTransClasses; ++cls) {
    const uint64_t* range = plan->ttiles_first[PACK ? 0 : 1] + cls;
    for (uint64_t first = range[0]; first < range[1]; first += (1u << 23)) {  // whole sets of eight
      const dim3 grid((uint32_t)std::min<uint64_t>(1u << 23, range[1] - first)), block(kTransThreads);
      const TransTile* tiles = plan->d_ttiles[PACK ? 0 : 1] + first;
      switch (cls) {
        case 0: hipLaunchKernelGGL((mlf_transpose_kernel<PACK, uint8_t>), grid, block, 0, stream, plan->d_tdescs, tiles, image); break;
        case 1: hipLaunchKernelGGL((mlf_transpose_kernel<PACK, uint16_t>), grid, block, 0, stream, plan->d_tdescs, tiles, image); break;
        case 2: hipLaunchKernelGGL((mlf_transpose_kernel<PACK, uint32_t>), grid, block, 0, stream, plan->d_tdescs, tiles, image); break;
        case 3: hipLaunchKernelGGL((mlf_transpose_kernel<PACK, uint64_t>), grid, block, 0, stream, plan->d_tdescs, tiles, image); break;
        default: hipLaunchKernelGGL((mlf_transpose_kernel<PACK, u32x4>), grid, block, 0, stream, plan->d_tdescs, tiles, image); break;
      }
      HIP_TRY(hipGetLastError());
    }
  }
  for (uint64_t first = 0; first < plan->n_work; first += (1u << 23)) {
    const uint64_t count = std::min<uint64_t>(1u << 23, plan->n_work - first);
    hipLaunchKernelGGL((mlf_strided_kernel<PACK>), dim3((uint32_t)count), dim3(256), 0, stream, plan->d_descs,
                       plan->d_work + first, image);
    HIP_TRY(hipGetLastError());
  }
  for (uint64_t first = 0; first < plan->n_gwork; first += (1u << 21)) {
    const uint64_t count = std::min<uint64_t>(1u << 21, plan->n_gwork - first);
    if (PACK)
      hipLaunchKernelGGL(mlf_gather_kernel, dim3((uint32_t)(count * kGatherSplit)), dim3(256), 0, stream,
                         plan->d_gwork + first, (uint32_t)(count * kGatherSplit), image);
    else
      hipLaunchKernelGGL(mlf_scatter_kernel, dim3((uint32_t)count), dim3(256), 0, stream, plan->d_gwork + first, image);
    HIP_TRY(hipGetLastError());
  }
  if (plan->blob_size) {
    if (!plan->launched) HIP_TRY(hipEventCreateWithFlags(&plan->launched, hipEventDisableTiming));
    HIP_TRY(hipEventRecord(plan->launched, stream));
  }
  // the image (pack) or its source (unpack) is complete at this point of the stream: the rest of the checksum
  if (plan->has_crc) return crc_fused_finish(&plan->crc, image, stream);
  return MLF_HIP_OK;
}

}  // namespace

extern "C" {

int mlf_plan_crc_values(mlf_plan* plan, uint32_t* out_host, uint64_t n_out) {
  if (!plan || !out_host) return fail(MLF_HIP_BAD_ARG, "null argument");
  if (!plan->has_crc) return fail(MLF_HIP_BAD_ARG, "the plan was created without crc_chunk_kib");
  if (!plan->crc.launched) return fail(MLF_HIP_BAD_ARG, "the plan has not been launched yet");
  if (n_out < plan->crc.n_chunks) return fail(MLF_HIP_BAD_ARG, "output array too small");
  HIP_TRY(hipEventSynchronize(plan->crc.done));
  memcpy(out_host, plan->crc.h_out, plan->crc.n_chunks * sizeof(uint32_t));
  return MLF_HIP_OK;
}

int mlf_pack_launch(const mlf_plan* plan, void* image_dev, void* stream) {
  return launch_plan<true>(plan, static_cast<char*>(image_dev), static_cast<hipStream_t>(stream));
}

int mlf_unpack_launch(const mlf_plan* plan, const void* image_dev, void* stream) {
  return launch_plan<false>(plan, const_cast<char*>(static_cast<const char*>(image_dev)),
                            static_cast<hipStream_t>(stream));
}

}  // extern "C"

// Copy engine between HBM and pageable host memory (a tmpfs mapping or file): a ring of pinned slots, two copy
// streams plus a checksum stream, and a persistent pool of host threads.  Part of the library behind
// include/mlf_hip.h.
#include "mlf_internal.h"

#include <immintrin.h>

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

using namespace mlf;

namespace {

// ---------------------------------------------------------------------------------------------------------
// host thread pool: run(n, fn) executes fn(0..n-1) on the pool's threads plus the caller
// ---------------------------------------------------------------------------------------------------------
class WorkerPool {
 public:
  explicit WorkerPool(unsigned extra_threads) {
    for (unsigned i = 0; i < extra_threads; ++i) threads_.emplace_back([this] { loop(); });
  }
  ~WorkerPool() {
    {
      std::lock_guard<std::mutex> g(m_);
      stop_ = true;
    }
    cv_.notify_all();
    for (auto& t : threads_) t.join();
  }
  unsigned width() const { return (unsigned)threads_.size() + 1; }

  void run(unsigned n, const std::function<void(unsigned)>& fn) {
    if (n == 0) return;
    {
      std::lock_guard<std::mutex> g(m_);
      fn_ = &fn;
      total_ = n;
      next_ = 0;
      pending_ = n;
      ++generation_;
    }
    cv_.notify_all();
    drain();
    std::unique_lock<std::mutex> l(m_);
    done_cv_.wait(l, [this] { return pending_ == 0; });
    fn_ = nullptr;
  }

 private:
  void drain() {
    for (;;) {
      unsigned idx;
      const std::function<void(unsigned)>* fn;
      {
        std::lock_guard<std::mutex> g(m_);
        if (!fn_ || next_ >= total_) return;
        idx = next_++;
        fn = fn_;
      }
      (*fn)(idx);
      {
        std::lock_guard<std::mutex> g(m_);
        if (--pending_ == 0) done_cv_.notify_all();
      }
    }
  }
  void loop() {
    uint64_t seen = 0;
    for (;;) {
      {
        std::unique_lock<std::mutex> l(m_);
        cv_.wait(l, [&] { return stop_ || generation_ != seen; });
        if (stop_) return;
        seen = generation_;
      }
      drain();
    }
  }
  std::vector<std::thread> threads_;
  std::mutex m_;
  std::condition_variable cv_, done_cv_;
  const std::function<void(unsigned)>* fn_ = nullptr;
  unsigned total_ = 0, next_ = 0, pending_ = 0;
  uint64_t generation_ = 0;
  bool stop_ = false;
};

void pool_memcpy(WorkerPool& pool, char* dst, const char* src, size_t n) {
  const unsigned parts = std::max<unsigned>(1, std::min<size_t>(pool.width(), n / ((size_t)1 << 20)));
  size_t per = (n + parts - 1) / parts;
  per = (per + 4095) & ~(size_t)4095;
  pool.run(parts, [&](unsigned i) {
    const size_t off = (size_t)i * per;
    if (off < n) memcpy(dst + off, src + off, std::min(per, n - off));
  });
}

// ---------------------------------------------------------------------------------------------------------
// copy + CRC-32C on the host threads
// ---------------------------------------------------------------------------------------------------------
// The threads that move a pinned slot into the buffer touch every byte of the image anyway, and the crc32
// instruction retires eight bytes per cycle when three independent chains keep it busy: a piece is cut into three
// lanes that are copied (32-byte loads, streaming stores: the destination is written once and not read soon) and
// checksummed side by side, and the lanes' states are joined with two multiplications.  Measured on the MI355X host
// (16 threads, 2 MiB pieces, 24 GiB into a tmpfs mapping): memcpy 190 GB/s, this loop 212 GB/s - against the 56 GB/s
// the link delivers.

// CRC state after `n` more bytes (state in, state out; no initial or final inversion)
inline uint64_t crc_advance(uint64_t s, const char* p, size_t n) {
  for (; n >= 8; n -= 8, p += 8) {
    uint64_t w;
    memcpy(&w, p, 8);
    s = _mm_crc32_u64(s, w);
  }
  while (n--) s = _mm_crc32_u8((uint32_t)s, (unsigned char)*p++);
  return s;
}

// x^(8 * n) for the lane length in use (pieces are of one size but for the last one: looked up once per thread)
inline uint32_t lane_weight(size_t n) {
  thread_local size_t known_n = 0;
  thread_local uint32_t known_x = 0;
  if (n != known_n) {
    known_x = x_pow_bytes(n);
    known_n = n;
  }
  return known_x;
}

// Copies [src, src + n) to dst (dst == nullptr: only reads it) and returns its CRC-32C.
__attribute__((target("avx2,sse4.2"))) uint32_t copy_crc_avx2(char* dst, const char* src, size_t n) {
  const size_t lane = (n / 3) & ~(size_t)63;
  uint64_t c0 = 0xFFFFFFFFu, c1 = 0, c2 = 0;
  if (lane >= 1024) {
    const char *p0 = src, *p1 = src + lane, *p2 = src + 2 * lane;
    const bool copy = dst != nullptr;
    const bool stream = copy && (reinterpret_cast<uintptr_t>(dst) & 31u) == 0;  // (lanes are multiples of 64 bytes)
    char *q0 = dst, *q1 = dst + lane, *q2 = dst + 2 * lane;
#define MLF_LANE(p, q, c)                                                                \
  {                                                                                      \
    if (copy) {                                                                          \
      const __m256i a = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(p + i));      \
      const __m256i b = _mm256_loadu_si256(reinterpret_cast<const __m256i*>(p + i + 32)); \
      if (stream) {                                                                      \
        _mm256_stream_si256(reinterpret_cast<__m256i*>(q + i), a);                       \
        _mm256_stream_si256(reinterpret_cast<__m256i*>(q + i + 32), b);                  \
      } else {                                                                           \
        _mm256_storeu_si256(reinterpret_cast<__m256i*>(q + i), a);                       \
        _mm256_storeu_si256(reinterpret_cast<__m256i*>(q + i + 32), b);                  \
      }                                                                                  \
    }                                                                                    \
    uint64_t w[8];                                                                       \
    memcpy(w, p + i, 64);                                                                \
    c = _mm_crc32_u64(c, w[0]);                                                          \
    c = _mm_crc32_u64(c, w[1]);                                                          \
    c = _mm_crc32_u64(c, w[2]);                                                          \
    c = _mm_crc32_u64(c, w[3]);                                                          \
    c = _mm_crc32_u64(c, w[4]);                                                          \
    c = _mm_crc32_u64(c, w[5]);                                                          \
    c = _mm_crc32_u64(c, w[6]);                                                          \
    c = _mm_crc32_u64(c, w[7]);                                                          \
  }
    for (size_t i = 0; i < lane; i += 64) {
      MLF_LANE(p0, q0, c0)
      MLF_LANE(p1, q1, c1)
      MLF_LANE(p2, q2, c2)
    }
#undef MLF_LANE
    if (stream) _mm_sfence();  // streaming stores are ordered before whatever announces the piece
    const uint32_t x = lane_weight(lane);
    c0 = gf_mul(x, (uint32_t)c0) ^ (uint32_t)c1;
    c0 = gf_mul(x, (uint32_t)c0) ^ (uint32_t)c2;
    src += 3 * lane;
    if (dst) dst += 3 * lane;
    n -= 3 * lane;
  }
  if (dst && n) memcpy(dst, src, n);
  return (uint32_t)crc_advance(c0, src, n) ^ 0xFFFFFFFFu;
}

uint32_t copy_crc(char* dst, const char* src, size_t n) {
  static const bool avx2 = __builtin_cpu_supports("avx2") && __builtin_cpu_supports("sse4.2");
  if (avx2) return copy_crc_avx2(dst, src, n);
  if (dst && n) memcpy(dst, src, n);
  return (uint32_t)crc_advance(0xFFFFFFFFu, src, n) ^ 0xFFFFFFFFu;
}

// A piece of the image that one thread has copied and checksummed
struct CheckedPiece {
  uint64_t image_off, len;
  uint32_t crc;
};

// Where the checksum chunks of a range begin: after `first` bytes (the rest of a chunk that began before the range;
// 0: the range begins on a boundary), then every `chunk` bytes.
struct ChunkGrid {
  uint64_t chunk = 0, first = 0;
  uint64_t index(uint64_t off) const { return first == 0 ? off / chunk : (off < first ? 0 : 1 + (off - first) / chunk); }
  uint64_t next_cut(uint64_t off) const {
    if (off < first) return first;
    return first + ((off - first) / chunk + 1) * chunk;
  }
  uint64_t count(uint64_t nbytes) const {
    if (nbytes == 0) return 0;
    const uint64_t head = std::min(first, nbytes);
    return (head ? 1 : 0) + (nbytes - head + chunk - 1) / chunk;
  }
};

// The pageable end of a transfer: a plain pointer, or a byte range of an open file (pread/pwrite).  Going
// through the file descriptor moves the same page-cache pages as a MAP_SHARED mapping would, without building
// (and later tearing down) one page-table entry per 4 KiB of a buffer that can be 100+ GB.
struct HostEnd {
  char* ptr = nullptr;
  int fd = -1;
  uint64_t file_off = 0;
};

// slot -> host end (to_host) or host end -> slot, split over the pool; returns 0 or an errno value
int pool_host_copy(WorkerPool& pool, const HostEnd& host, uint64_t host_off, char* slot, size_t n, bool to_host) {
  if (host.fd < 0) {
    if (to_host) pool_memcpy(pool, host.ptr + host_off, slot, n);
    else pool_memcpy(pool, slot, host.ptr + host_off, n);
    return 0;
  }
  const unsigned parts = std::max<unsigned>(1, std::min<size_t>(pool.width(), n / ((size_t)1 << 20)));
  size_t per = (n + parts - 1) / parts;
  per = (per + 4095) & ~(size_t)4095;
  std::atomic<int> err{0};
  pool.run(parts, [&](unsigned i) {
    const size_t off = (size_t)i * per;
    if (off >= n) return;
    const size_t len = std::min(per, n - off);
    const int e = to_host ? full_pwrite(host.fd, slot + off, len, host.file_off + host_off + off)
                          : full_pread(host.fd, slot + off, len, host.file_off + host_off + off);
    if (e) err.store(e);
  });
  return err.load();
}

// slot -> host end like pool_host_copy, every thread also taking the CRC-32C of what it moves.  The pieces are cut
// where the checksum chunks of `grid` end, and `out` gets them in image order.
int pool_host_copy_checked(WorkerPool& pool, const HostEnd& host, uint64_t image_off, const char* slot, size_t n,
                           const ChunkGrid& grid, std::vector<CheckedPiece>* out) {
  const unsigned parts = std::max<unsigned>(1, std::min<size_t>(pool.width(), n / ((size_t)1 << 20)));
  size_t per = (n + parts - 1) / parts;
  per = (per + 4095) & ~(size_t)4095;
  std::vector<std::vector<CheckedPiece>> found(parts);
  std::atomic<int> err{0};
  pool.run(parts, [&](unsigned i) {
    size_t off = (size_t)i * per;
    if (off >= n) return;
    const size_t end = std::min(off + per, n);
    while (off < end) {
      const uint64_t at = image_off + off;
      const size_t len = (size_t)std::min<uint64_t>(end - off, grid.next_cut(at) - at);
      uint32_t crc;
      if (host.fd < 0) {
        crc = copy_crc(host.ptr + at, slot + off, len);
      } else {
        crc = copy_crc(nullptr, slot + off, len);
        if (int e = full_pwrite(host.fd, slot + off, len, host.file_off + at)) err.store(e);
      }
      found[i].push_back({at, len, crc});
      off += len;
    }
  });
  for (const auto& list : found) out->insert(out->end(), list.begin(), list.end());
  return err.load();
}

// pieces in image order -> per-chunk values: crc(A || B) = crc(A) * x^(8 |B|) + crc(B)
void fold_pieces(const std::vector<CheckedPiece>& pieces, const ChunkGrid& grid, std::vector<uint32_t>* chunk_crc,
                 std::vector<uint64_t>* chunk_len) {
  for (const CheckedPiece& p : pieces) {
    const uint64_t k = grid.index(p.image_off);
    (*chunk_crc)[k] = (*chunk_len)[k] ? mlf_crc32c_combine((*chunk_crc)[k], p.crc, p.len) : p.crc;
    (*chunk_len)[k] += p.len;
  }
}

}  // namespace

// ---------------------------------------------------------------------------------------------------------
// copy engine
// ---------------------------------------------------------------------------------------------------------
struct mlf_engine {
  int device = 0;
  uint64_t slot_bytes = 0;
  std::vector<char*> slots;
  std::vector<hipEvent_t> slot_done;
  hipStream_t streams[2] = {nullptr, nullptr};
  hipStream_t crc_stream = nullptr;  // checksum kernels run beside the copies, not before them
  // streams that mlf_engine_avoid_streams replaced: handles to them may still be in a caller's hands (the checksum
  // stream is handed out), so they live as long as the engine does
  std::vector<hipStream_t> retired;
  hipEvent_t gate = nullptr;
  CrcScratch crc;  // of the checksum passes that run beside transfers; allocated on first use, grown when too small
  std::unique_ptr<WorkerPool> pool;
  std::mutex busy;  // one transfer at a time per engine
  // checksums of a device-to-host transfer: taken by the host threads as they move the slots (true), or by kernels
  // on crc_stream that read the image once more while it crosses the link (false)
  std::atomic<bool> host_checksums{false};
};

namespace {

// The two kernels of the hardware-queue test (mlf_engine_avoid_streams).  The first keeps one wavefront busy for a
// stated time by the device's constant-rate clock (100 MHz) - bounded by a count as well, so that it ends whatever
// that clock does; the second does nothing but exist.
__global__ void mlf_queue_test_hold(uint64_t ticks, uint32_t* out) {
  const uint64_t t0 = wall_clock64();
  uint32_t n = 0;
  while (wall_clock64() - t0 < ticks && n < (1u << 22)) ++n;
  if (threadIdx.x == 0) *out = n;
}

__global__ void mlf_queue_test_touch(uint32_t* out) {
  if (threadIdx.x == 0) *out = 1u;
}

// Whether work on `s` waits for work enqueued earlier on `busy`: both idle, an event, a 2 ms kernel and another event
// on `busy`, an empty kernel and an event on `s`.  On a hardware queue of its own the empty kernel is done long before
// the 2 ms kernel, behind that kernel it is done after it.  Decided by the device's own time stamps of the three
// events - the empty kernel's completion lies before or after the long kernel's - not by a host clock or a constant.
int waits_behind(hipStream_t s, hipStream_t busy, uint32_t* d_flags, hipEvent_t* ev, bool* shared) {
  HIP_TRY(hipStreamSynchronize(busy));
  HIP_TRY(hipStreamSynchronize(s));
  HIP_TRY(hipEventRecord(ev[0], busy));
  hipLaunchKernelGGL(mlf_queue_test_hold, dim3(1), dim3(64), 0, busy, 200000ull, d_flags);
  HIP_TRY(hipEventRecord(ev[1], busy));
  hipLaunchKernelGGL(mlf_queue_test_touch, dim3(1), dim3(64), 0, s, d_flags + 16);
  HIP_TRY(hipEventRecord(ev[2], s));
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipEventSynchronize(ev[2]));
  HIP_TRY(hipEventSynchronize(ev[1]));
  float held_ms = 0.0f, touched_ms = 0.0f;
  HIP_TRY(hipEventElapsedTime(&held_ms, ev[0], ev[1]));
  HIP_TRY(hipEventElapsedTime(&touched_ms, ev[0], ev[2]));
  *shared = touched_ms >= held_ms;
  return MLF_HIP_OK;
}

}  // namespace

extern "C" {

int mlf_engine_destroy(mlf_engine* e) {
  if (!e) return MLF_HIP_OK;
  for (char* s : e->slots) (void)hipHostFree(s);
  for (hipEvent_t ev : e->slot_done) (void)hipEventDestroy(ev);
  if (e->gate) (void)hipEventDestroy(e->gate);
  for (hipStream_t s : e->streams)
    if (s) (void)hipStreamDestroy(s);
  if (e->crc_stream) {
    (void)hipStreamSynchronize(e->crc_stream);
    (void)hipStreamDestroy(e->crc_stream);
  }
  for (hipStream_t s : e->retired) {
    (void)hipStreamSynchronize(s);
    (void)hipStreamDestroy(s);
  }
  crc_scratch_free(&e->crc);
  delete e;
  return MLF_HIP_OK;
}

int mlf_engine_create(uint64_t slot_bytes, uint32_t n_slots, uint32_t n_threads, mlf_engine** out) {
  if (!out) return fail(MLF_HIP_BAD_ARG, "null out");
  *out = nullptr;
  if (slot_bytes < (1u << 20) || slot_bytes % 4096) return fail(MLF_HIP_BAD_ARG, "slot_bytes must be a multiple of 4096, at least 1 MiB");
  if (n_slots < 2 || n_slots > 64) return fail(MLF_HIP_BAD_ARG, "n_slots must be in [2, 64]");
  if (n_threads < 1 || n_threads > 256) return fail(MLF_HIP_BAD_ARG, "n_threads must be in [1, 256]");
  std::unique_ptr<mlf_engine> e(new mlf_engine());
  e->slot_bytes = slot_bytes;
  int rc = MLF_HIP_OK;
  auto check = [&](hipError_t err, const char* what) {
    if (err != hipSuccess && rc == MLF_HIP_OK) rc = fail(MLF_HIP_RUNTIME, std::string(what) + " failed: " + hipGetErrorString(err));
  };
  check(hipGetDevice(&e->device), "hipGetDevice");
  for (int i = 0; i < 2 && rc == MLF_HIP_OK; ++i)
    check(hipStreamCreateWithFlags(&e->streams[i], hipStreamNonBlocking), "hipStreamCreateWithFlags");
  if (rc == MLF_HIP_OK) check(hipStreamCreateWithFlags(&e->crc_stream, hipStreamNonBlocking), "hipStreamCreateWithFlags");
  if (rc == MLF_HIP_OK) check(hipEventCreateWithFlags(&e->gate, hipEventDisableTiming), "hipEventCreateWithFlags");
  for (uint32_t i = 0; i < n_slots && rc == MLF_HIP_OK; ++i) {
    char* p = nullptr;
    check(hipHostMalloc(reinterpret_cast<void**>(&p), slot_bytes, hipHostMallocDefault), "hipHostMalloc");
    if (rc != MLF_HIP_OK) break;
    memset(p, 0, slot_bytes);  // touch the pages once, outside any timed transfer
    e->slots.push_back(p);
    hipEvent_t ev = nullptr;
    check(hipEventCreateWithFlags(&ev, hipEventDisableTiming), "hipEventCreateWithFlags");
    if (rc == MLF_HIP_OK) e->slot_done.push_back(ev);
  }
  if (rc != MLF_HIP_OK) {
    const std::string keep = last_error();
    mlf_engine_destroy(e.release());
    last_error() = keep;
    return rc;
  }
  e->pool.reset(new WorkerPool(n_threads - 1));
  *out = e.release();
  return MLF_HIP_OK;
}

}  // extern "C"

namespace {

// Copies still in flight when a transfer gives up target the pinned slots: they must have landed before the engine
// (or the next transfer) touches the slots again.  Disarmed on the success path, where the streams are already idle.
struct DrainOnExit {
  mlf_engine* e;
  bool armed = true;
  ~DrainOnExit() {
    if (!armed) return;
    for (hipStream_t s : e->streams) (void)hipStreamSynchronize(s);
  }
};

struct CrcRequest {
  uint64_t chunk_bytes = 0;  // 0: no checksum
  uint32_t* out_host = nullptr;
  uint64_t n_out = 0;
  uint64_t* landed = nullptr;  // progress counter of the caller, or null
  uint64_t first_part = 0;     // bytes up to the first chunk boundary (a piece of a larger data section)
  bool by_host_threads = false;  // whatever the engine's setting
};

// What a device-to-host transfer waits for before its first copy: everything enqueued so far on a stream, or an
// event the caller recorded behind the producing kernel (then later work on the producer's stream does not delay it).
struct Gate {
  void* producer_stream = nullptr;
  hipEvent_t ready = nullptr;
  bool by_event = false;
};

int engine_d2h(mlf_engine* e, const void* src_dev, const HostEnd& host, uint64_t nbytes, const Gate& gate,
               mlf_xfer_stats* stats, const CrcRequest& crc = CrcRequest()) {
  if (!e) return fail(MLF_HIP_BAD_ARG, "null engine");
  if (nbytes && (!src_dev || (host.fd < 0 && !host.ptr))) return fail(MLF_HIP_BAD_ARG, "null pointer");
  std::lock_guard<std::mutex> g(e->busy);
  HIP_TRY(hipSetDevice(e->device));
  const double t0 = now_s();
  hipEvent_t ready = gate.ready;
  if (!gate.by_event) {
    // the copy streams start after whatever the producer has enqueued so far (the pack)
    HIP_TRY(hipEventRecord(e->gate, static_cast<hipStream_t>(gate.producer_stream)));
    ready = e->gate;
  }
  if (ready)
    for (hipStream_t s : e->streams) HIP_TRY(hipStreamWaitEvent(s, ready, 0));
  const char* src = static_cast<const char*>(src_dev);
  if (crc.landed) __atomic_store_n(crc.landed, (uint64_t)0, __ATOMIC_RELEASE);
  const bool want_crc = crc.chunk_bytes != 0 && nbytes != 0;
  const ChunkGrid grid{crc.chunk_bytes, crc.first_part};
  const uint64_t n_crc = want_crc ? grid.count(nbytes) : 0;
  if (want_crc && crc.n_out < n_crc) return fail(MLF_HIP_BAD_ARG, "checksum output too small");
  const bool on_host = want_crc && (crc.by_host_threads || e->host_checksums.load());
  if (want_crc && !on_host && crc.first_part) return fail(MLF_HIP_BAD_ARG, "a first part needs the host threads' checksums");
  std::vector<CheckedPiece> pieces;
  std::vector<uint32_t> chunk_crc(on_host ? n_crc : 0);
  std::vector<uint64_t> chunk_len(on_host ? n_crc : 0, 0);
  struct CrcGuard {  // on every exit path the checksum kernels have finished before the scratch can be used again
    hipStream_t stream;
    bool armed;
    ~CrcGuard() {
      if (armed) (void)hipStreamSynchronize(stream);
    }
  } crc_guard{e->crc_stream, false};
  if (want_crc && !on_host) {
    // the image is complete once the gate has passed and is not modified afterwards, so its checksum can be
    // computed while the link-bound copies run: it costs neither blocking time nor transfer time
    if (ready) HIP_TRY(hipStreamWaitEvent(e->crc_stream, ready, 0));
    crc_guard.armed = true;
    if (int rc = crc_enqueue(src_dev, nbytes, crc.chunk_bytes, crc.n_out, e->crc_stream, &e->crc, true)) return rc;
  }
  const uint64_t slot = e->slot_bytes;
  const uint64_t n_chunks = (nbytes + slot - 1) / slot;
  const uint64_t n_slots = e->slots.size();
  auto issue = [&](uint64_t c) -> int {
    const uint64_t off = c * slot, len = std::min(slot, nbytes - off);
    const uint64_t s = c % n_slots;
    hipStream_t st = e->streams[c & 1];
    HIP_TRY(hipMemcpyAsync(e->slots[s], src + off, len, hipMemcpyDeviceToHost, st));
    HIP_TRY(hipEventRecord(e->slot_done[s], st));
    return MLF_HIP_OK;
  };
  DrainOnExit drain{e};
  for (uint64_t c = 0; c < std::min(n_chunks, n_slots); ++c)
    if (int rc = issue(c)) return rc;
  double wait = 0;
  for (uint64_t c = 0; c < n_chunks; ++c) {
    const uint64_t off = c * slot, len = std::min(slot, nbytes - off);
    const uint64_t s = c % n_slots;
    const double w0 = now_s();
    HIP_TRY(hipEventSynchronize(e->slot_done[s]));
    if (c == 0) wait = now_s() - w0;
    if (on_host) {
      pieces.clear();
      if (int err = pool_host_copy_checked(*e->pool, host, off, e->slots[s], len, grid, &pieces))
        return fail(MLF_HIP_RUNTIME, std::string("pwrite() to the buffer file failed: ") + strerror(err));
      fold_pieces(pieces, grid, &chunk_crc, &chunk_len);
    } else if (int err = pool_host_copy(*e->pool, host, off, e->slots[s], len, true)) {
      return fail(MLF_HIP_RUNTIME, std::string("pwrite() to the buffer file failed: ") + strerror(err));
    }
    if (crc.landed) __atomic_store_n(crc.landed, off + len, __ATOMIC_RELEASE);  // the host threads' stores come first
    if (c + n_slots < n_chunks)
      if (int rc = issue(c + n_slots)) return rc;
  }
  drain.armed = false;  // every chunk's event has been waited for
  if (on_host) {
    std::copy(chunk_crc.begin(), chunk_crc.end(), crc.out_host);
  } else if (want_crc) {
    crc_guard.armed = false;
    if (int rc = crc_finish(&e->crc, e->crc_stream, n_crc, crc.out_host)) return rc;
  }
  if (stats) {
    stats->seconds = now_s() - t0;
    stats->wait_seconds = wait;
    stats->bytes = nbytes;
    stats->chunks = n_chunks;
  }
  return MLF_HIP_OK;
}

int engine_h2d(mlf_engine* e, const HostEnd& host, void* dst_dev, uint64_t nbytes, void* consumer_stream,
               mlf_xfer_stats* stats) {
  if (!e) return fail(MLF_HIP_BAD_ARG, "null engine");
  if (nbytes && (!dst_dev || (host.fd < 0 && !host.ptr))) return fail(MLF_HIP_BAD_ARG, "null pointer");
  std::lock_guard<std::mutex> g(e->busy);
  HIP_TRY(hipSetDevice(e->device));
  const double t0 = now_s();
  char* dst = static_cast<char*>(dst_dev);
  const uint64_t slot = e->slot_bytes;
  const uint64_t n_chunks = (nbytes + slot - 1) / slot;
  const uint64_t n_slots = e->slots.size();
  DrainOnExit drain{e};
  double host_s = 0;  // spent filling slots from the file or the mapping
  for (uint64_t c = 0; c < n_chunks; ++c) {
    const uint64_t off = c * slot, len = std::min(slot, nbytes - off);
    const uint64_t s = c % n_slots;
    if (c >= n_slots) HIP_TRY(hipEventSynchronize(e->slot_done[s]));  // the slot's previous upload has left it
    const double t_read = now_s();
    if (int err = pool_host_copy(*e->pool, host, off, e->slots[s], len, false))
      return fail(MLF_HIP_RUNTIME, std::string("pread() from the buffer file failed: ") + strerror(err));
    host_s += now_s() - t_read;
    hipStream_t st = e->streams[c & 1];
    HIP_TRY(hipMemcpyAsync(dst + off, e->slots[s], len, hipMemcpyHostToDevice, st));
    HIP_TRY(hipEventRecord(e->slot_done[s], st));
  }
  // the consumer (unpack) waits for both copy streams; the host waits too, so the slots are reusable
  for (hipStream_t s : e->streams) {
    HIP_TRY(hipEventRecord(e->gate, s));
    HIP_TRY(hipStreamWaitEvent(static_cast<hipStream_t>(consumer_stream), e->gate, 0));
    HIP_TRY(hipStreamSynchronize(s));
  }
  drain.armed = false;
  if (stats) {
    stats->seconds = now_s() - t0;
    stats->wait_seconds = host_s;
    stats->bytes = nbytes;
    stats->chunks = n_chunks;
  }
  return MLF_HIP_OK;
}

}  // namespace

extern "C" {

int mlf_engine_d2h(mlf_engine* e, const void* src_dev, void* dst_host, uint64_t nbytes, void* producer_stream,
                   mlf_xfer_stats* stats) {
  HostEnd host;
  host.ptr = static_cast<char*>(dst_host);
  Gate gate;
  gate.producer_stream = producer_stream;
  return engine_d2h(e, src_dev, host, nbytes, gate, stats);
}

int mlf_engine_h2d(mlf_engine* e, const void* src_host, void* dst_dev, uint64_t nbytes, void* consumer_stream,
                   mlf_xfer_stats* stats) {
  HostEnd host;
  host.ptr = const_cast<char*>(static_cast<const char*>(src_host));
  return engine_h2d(e, host, dst_dev, nbytes, consumer_stream, stats);
}

int mlf_engine_d2h_crc(mlf_engine* e, const void* src_dev, void* dst_host, uint64_t nbytes, void* producer_stream,
                       uint64_t crc_chunk_bytes, uint32_t* crc_out_host, uint64_t n_crc_out, mlf_xfer_stats* stats) {
  if (crc_chunk_bytes && !crc_out_host) return fail(MLF_HIP_BAD_ARG, "null checksum output");
  HostEnd host;
  host.ptr = static_cast<char*>(dst_host);
  CrcRequest crc;
  crc.chunk_bytes = crc_chunk_bytes;
  crc.out_host = crc_out_host;
  crc.n_out = n_crc_out;
  Gate gate;
  gate.producer_stream = producer_stream;
  return engine_d2h(e, src_dev, host, nbytes, gate, stats, crc);
}

int mlf_engine_d2h_watched(mlf_engine* e, const void* src_dev, void* dst_host, uint64_t nbytes, void* producer_stream,
                           uint64_t crc_chunk_bytes, uint32_t* crc_out_host, uint64_t n_crc_out, uint64_t* landed,
                           mlf_xfer_stats* stats) {
  if (crc_chunk_bytes && !crc_out_host) return fail(MLF_HIP_BAD_ARG, "null checksum output");
  if (reinterpret_cast<uintptr_t>(landed) & 7) return fail(MLF_HIP_BAD_ARG, "progress counter must be 8-byte aligned");
  HostEnd host;
  host.ptr = static_cast<char*>(dst_host);
  CrcRequest crc;
  crc.chunk_bytes = crc_chunk_bytes;
  crc.out_host = crc_out_host;
  crc.n_out = n_crc_out;
  crc.landed = landed;
  Gate gate;
  gate.producer_stream = producer_stream;
  return engine_d2h(e, src_dev, host, nbytes, gate, stats, crc);
}

int mlf_engine_d2h_gated(mlf_engine* e, const void* src_dev, void* dst_host, uint64_t nbytes, void* ready_event,
                         uint64_t crc_chunk_bytes, uint32_t* crc_out_host, uint64_t n_crc_out, uint64_t* landed,
                         mlf_xfer_stats* stats) {
  if (crc_chunk_bytes && !crc_out_host) return fail(MLF_HIP_BAD_ARG, "null checksum output");
  if (reinterpret_cast<uintptr_t>(landed) & 7) return fail(MLF_HIP_BAD_ARG, "progress counter must be 8-byte aligned");
  HostEnd host;
  host.ptr = static_cast<char*>(dst_host);
  CrcRequest crc;
  crc.chunk_bytes = crc_chunk_bytes;
  crc.out_host = crc_out_host;
  crc.n_out = n_crc_out;
  crc.landed = landed;
  Gate gate;
  gate.ready = static_cast<hipEvent_t>(ready_event);
  gate.by_event = true;
  return engine_d2h(e, src_dev, host, nbytes, gate, stats, crc);
}

int mlf_engine_avoid_streams(mlf_engine* e, void* const* busy_streams, uint32_t n_busy, uint32_t* still_shared) {
  if (!e) return fail(MLF_HIP_BAD_ARG, "null engine");
  if (n_busy == 0 || !busy_streams) return fail(MLF_HIP_BAD_ARG, "no stream to avoid");
  std::lock_guard<std::mutex> g(e->busy);
  HIP_TRY(hipSetDevice(e->device));
  // shares a queue with any of the busy streams?
  hipEvent_t ev[3] = {nullptr, nullptr, nullptr};
  auto shares_hardware_queue = [&](hipStream_t s, uint32_t* flags, bool* shared) -> int {
    *shared = false;
    for (uint32_t k = 0; k < n_busy && !*shared; ++k)
      if (int err = waits_behind(s, static_cast<hipStream_t>(busy_streams[k]), flags, ev, shared)) return err;
    return MLF_HIP_OK;
  };
  uint32_t* d_flags = nullptr;
  HIP_TRY(hipMalloc(reinterpret_cast<void**>(&d_flags), 128));
  for (hipEvent_t& e1 : ev)
    if (hipEventCreate(&e1) != hipSuccess) {  // (timing enabled: their time stamps are what is compared)
      for (hipEvent_t e2 : ev)
        if (e2) (void)hipEventDestroy(e2);
      (void)hipFree(d_flags);
      return fail(MLF_HIP_RUNTIME, "hipEventCreate failed");
    }
  std::vector<hipStream_t> rejected;  // candidates that were no better; kept until the end: a destroyed stream's
                                      // queue would be handed out again
  uint32_t left = 0;
  int rc = MLF_HIP_OK;
  hipStream_t* mine[3] = {&e->streams[0], &e->streams[1], &e->crc_stream};
  for (hipStream_t* slot : mine) {
    bool shared = false;
    if ((rc = shares_hardware_queue(*slot, d_flags, &shared))) break;
    for (int attempt = 0; shared && attempt < 8 && rc == MLF_HIP_OK; ++attempt) {
      hipStream_t candidate = nullptr;
      if (hipStreamCreateWithFlags(&candidate, hipStreamNonBlocking) != hipSuccess) {
        rc = fail(MLF_HIP_RUNTIME, "hipStreamCreateWithFlags failed");
        break;
      }
      bool also = false;
      if ((rc = shares_hardware_queue(candidate, d_flags, &also))) {
        rejected.push_back(candidate);
        break;
      }
      if (also) {
        rejected.push_back(candidate);
      } else {
        e->retired.push_back(*slot);  // not destroyed: somebody may still hold its handle, or have work on it
        *slot = candidate;
        shared = false;
      }
    }
    if (rc != MLF_HIP_OK) break;
    left += shared ? 1u : 0u;
  }
  for (hipStream_t s : rejected) (void)hipStreamDestroy(s);
  for (hipEvent_t e1 : ev) (void)hipEventDestroy(e1);
  (void)hipFree(d_flags);
  if (rc == MLF_HIP_OK && still_shared) *still_shared = left;
  return rc;
}

void* mlf_engine_checksum_stream(mlf_engine* e) { return e ? e->crc_stream : nullptr; }

int mlf_engine_set_host_checksums(mlf_engine* e, int on) {
  if (!e) return fail(MLF_HIP_BAD_ARG, "null engine");
  e->host_checksums.store(on != 0);
  return MLF_HIP_OK;
}

int mlf_engine_link_probe(mlf_engine* e, void* dev_buf, uint64_t nbytes, int to_host, double* seconds) {
  if (!e || !dev_buf || !seconds) return fail(MLF_HIP_BAD_ARG, "null argument");
  if (nbytes == 0) return fail(MLF_HIP_BAD_ARG, "nothing to copy");
  std::lock_guard<std::mutex> g(e->busy);
  HIP_TRY(hipSetDevice(e->device));
  char* dev = static_cast<char*>(dev_buf);
  const uint64_t slot = e->slot_bytes, n_chunks = (nbytes + slot - 1) / slot, n_slots = e->slots.size();
  DrainOnExit drain{e};
  HIP_TRY(hipDeviceSynchronize());
  const double t0 = now_s();
  for (uint64_t c = 0; c < n_chunks; ++c) {
    const uint64_t off = c * slot, len = std::min(slot, nbytes - off), s = c % n_slots;
    if (c >= n_slots) HIP_TRY(hipEventSynchronize(e->slot_done[s]));  // the slot's previous copy has finished
    hipStream_t st = e->streams[c & 1];
    if (to_host) HIP_TRY(hipMemcpyAsync(e->slots[s], dev + off, len, hipMemcpyDeviceToHost, st));
    else HIP_TRY(hipMemcpyAsync(dev + off, e->slots[s], len, hipMemcpyHostToDevice, st));
    HIP_TRY(hipEventRecord(e->slot_done[s], st));
  }
  for (hipStream_t s : e->streams) HIP_TRY(hipStreamSynchronize(s));
  drain.armed = false;
  *seconds = now_s() - t0;
  return MLF_HIP_OK;
}

int mlf_engine_d2h_cut(mlf_engine* e, const void* src_dev, void* dst_host, uint64_t nbytes, void* producer_stream,
                       void* ready_event, uint64_t crc_chunk_bytes, uint64_t first_part_bytes, uint32_t* crc_out_host,
                       uint64_t n_crc_out, uint64_t* landed, mlf_xfer_stats* stats) {
  if (!crc_chunk_bytes || !crc_out_host) return fail(MLF_HIP_BAD_ARG, "chunk size and checksum output are required");
  if (first_part_bytes >= crc_chunk_bytes) return fail(MLF_HIP_BAD_ARG, "the first part is shorter than a chunk");
  HostEnd host;
  host.ptr = static_cast<char*>(dst_host);
  CrcRequest crc;
  crc.chunk_bytes = crc_chunk_bytes;
  crc.out_host = crc_out_host;
  crc.n_out = n_crc_out;
  crc.landed = landed;
  crc.first_part = first_part_bytes;
  crc.by_host_threads = true;
  Gate gate;
  if (ready_event) {
    gate.ready = static_cast<hipEvent_t>(ready_event);
    gate.by_event = true;
  } else {
    gate.producer_stream = producer_stream;
  }
  return engine_d2h(e, src_dev, host, nbytes, gate, stats, crc);
}

int mlf_engine_host_copy_cut(mlf_engine* e, void* dst_host, const void* src_host, uint64_t nbytes,
                             uint64_t crc_chunk_bytes, uint64_t first_part_bytes, uint32_t* crc_out_host,
                             uint64_t n_crc_out) {
  if (!e) return fail(MLF_HIP_BAD_ARG, "null engine");
  if (nbytes && (!dst_host || !src_host)) return fail(MLF_HIP_BAD_ARG, "null pointer");
  if (!crc_chunk_bytes || !crc_out_host) return fail(MLF_HIP_BAD_ARG, "chunk size and checksum output are required");
  if (first_part_bytes >= crc_chunk_bytes) return fail(MLF_HIP_BAD_ARG, "the first part is shorter than a chunk");
  const ChunkGrid grid{crc_chunk_bytes, first_part_bytes};
  const uint64_t n_crc = grid.count(nbytes);
  if (n_crc_out < n_crc) return fail(MLF_HIP_BAD_ARG, "checksum output too small");
  std::lock_guard<std::mutex> g(e->busy);  // the threads are the ones a transfer uses
  std::vector<CheckedPiece> pieces;
  std::vector<uint32_t> chunk_crc(n_crc);
  std::vector<uint64_t> chunk_len(n_crc, 0);
  HostEnd host;
  host.ptr = static_cast<char*>(dst_host);
  // a slice at a time, so that the list of pieces stays short whatever the size
  const uint64_t slice = (uint64_t)256 << 20;
  for (uint64_t off = 0; off < nbytes; off += slice) {
    pieces.clear();
    (void)pool_host_copy_checked(*e->pool, host, off, static_cast<const char*>(src_host) + off,
                                 (size_t)std::min(slice, nbytes - off), grid, &pieces);
    fold_pieces(pieces, grid, &chunk_crc, &chunk_len);
  }
  std::copy(chunk_crc.begin(), chunk_crc.end(), crc_out_host);
  return MLF_HIP_OK;
}

int mlf_engine_read_file(mlf_engine* e, int fd, uint64_t file_offset, void* dst_host, uint64_t nbytes) {
  if (!e) return fail(MLF_HIP_BAD_ARG, "null engine");
  if (fd < 0) return fail(MLF_HIP_BAD_ARG, "bad file descriptor");
  if (nbytes && !dst_host) return fail(MLF_HIP_BAD_ARG, "null pointer");
  std::lock_guard<std::mutex> g(e->busy);  // the threads are the ones a transfer uses
  HostEnd host;
  host.fd = fd;
  host.file_off = file_offset;
  const uint64_t slice = (uint64_t)1 << 30;  // (the pool splits a call into at most one part per thread)
  for (uint64_t off = 0; off < nbytes; off += slice)
    if (int err = pool_host_copy(*e->pool, host, off, static_cast<char*>(dst_host) + off,
                                 (size_t)std::min(slice, nbytes - off), false))
      return fail(MLF_HIP_RUNTIME, std::string("pread() from the buffer file failed: ") + strerror(err));
  return MLF_HIP_OK;
}

int mlf_engine_host_copy(mlf_engine* e, void* dst_host, const void* src_host, uint64_t nbytes) {
  if (!e) return fail(MLF_HIP_BAD_ARG, "null engine");
  if (nbytes && (!dst_host || !src_host)) return fail(MLF_HIP_BAD_ARG, "null pointer");
  std::lock_guard<std::mutex> g(e->busy);  // the threads are the ones a transfer uses
  pool_memcpy(*e->pool, static_cast<char*>(dst_host), static_cast<const char*>(src_host), nbytes);
  return MLF_HIP_OK;
}

int mlf_engine_d2h_fd(mlf_engine* e, const void* src_dev, int fd, uint64_t file_offset, uint64_t nbytes,
                      void* producer_stream, mlf_xfer_stats* stats) {
  if (fd < 0) return fail(MLF_HIP_BAD_ARG, "bad file descriptor");
  HostEnd host;
  host.fd = fd;
  host.file_off = file_offset;
  Gate gate;
  gate.producer_stream = producer_stream;
  return engine_d2h(e, src_dev, host, nbytes, gate, stats);
}

int mlf_engine_h2d_fd(mlf_engine* e, int fd, uint64_t file_offset, void* dst_dev, uint64_t nbytes,
                      void* consumer_stream, mlf_xfer_stats* stats) {
  if (fd < 0) return fail(MLF_HIP_BAD_ARG, "bad file descriptor");
  HostEnd host;
  host.fd = fd;
  host.file_off = file_offset;
  return engine_h2d(e, host, dst_dev, nbytes, consumer_stream, stats);
}

}  // extern "C"

// File-backed MAP_SHARED buffer object and host bulk-copy helpers behind the C-ABI in
// include/mlf_buffer.h.  Plain POSIX, no third-party dependencies.
//
// Behaviour follows the reference's native buffer object
// (src/ml_flashpoint/checkpoint_object_manager/buffer_object/buffer_helper.cpp:43-314 and
// buffer_object.cpp:25-197): same system-call sequence, same failure conditions, same message
// fragments; the structure (one POD handle + free functions + thread-local error text) is this
// library's own.
#include "mlf_buffer.h"

#include <errno.h>
#include <fcntl.h>
#include <string.h>
#ifndef _GNU_SOURCE
#define _GNU_SOURCE
#endif
#include <sys/mman.h>
#include <sys/stat.h>
#include <sys/statvfs.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <string>
#include <thread>
#include <vector>

#ifndef MADV_POPULATE_WRITE
#define MADV_POPULATE_WRITE 23  // Linux 5.14; older kernels answer EINVAL and the per-page store below takes over
#endif

struct mlf_buffer {
  std::string id;
  void* ptr = nullptr;
  size_t cap = 0;
  int fd = -1;
  bool writable = false;
  bool closed = true;
};

namespace {

thread_local std::string g_err;

const char* code_name(int code) {
  switch (code) {
    case MLF_INVALID_ARGUMENT: return "INVALID_ARGUMENT";
    case MLF_ALREADY_EXISTS: return "ALREADY_EXISTS";
    case MLF_FAILED_PRECONDITION: return "FAILED_PRECONDITION";
    case MLF_INTERNAL: return "INTERNAL";
    default: return "UNKNOWN";
  }
}

int fail(int code, const std::string& msg) {
  g_err = std::string(code_name(code)) + ": " + msg;
  return code;
}

int fail_errno(const std::string& msg, int err) {
  return fail(MLF_INTERNAL, msg + ": " + strerror(err));
}

// mkdir -p for the directory part of `path`.
int make_parent_dirs(const std::string& path) {
  size_t slash = path.find_last_of('/');
  if (slash == std::string::npos || slash == 0) return 0;
  std::string dir = path.substr(0, slash);
  for (size_t i = 1; i <= dir.size(); ++i) {
    if (i != dir.size() && dir[i] != '/') continue;
    std::string sub = dir.substr(0, i);
    if (mkdir(sub.c_str(), 0777) != 0 && errno != EEXIST) return errno;
  }
  struct stat st;
  if (stat(dir.c_str(), &st) != 0) return errno;
  return S_ISDIR(st.st_mode) ? 0 : ENOTDIR;
}

// A store into a page of a MAP_SHARED file that the file system cannot back (a full tmpfs) does not fail with an
// error code: the process gets SIGBUS.  So a file is never made larger than what its file system can hold at that
// moment.  Returns 0 if `new_size` fits or nothing can be said (no limit reported), else the failure code.
int check_space(int fd, size_t new_size, const std::string& id) {
  struct stat st;
  struct statvfs vfs;
  if (fstat(fd, &st) != 0 || fstatvfs(fd, &vfs) != 0 || vfs.f_blocks == 0) return 0;
  const unsigned long long allocated = (unsigned long long)st.st_blocks * 512ull;
  if (new_size <= allocated) return 0;
  const unsigned long long needed = new_size - allocated;
  const unsigned long long available = (unsigned long long)vfs.f_bavail * (unsigned long long)vfs.f_frsize;
  if (needed <= available) return 0;
  return fail(MLF_INTERNAL, "not enough space on the file system that holds " + id + ": " + std::to_string(needed) +
                                " more bytes needed, " + std::to_string(available) + " available");
}

bool is_open(const mlf_buffer* b) {
  return b && !b->closed && b->ptr != nullptr && b->ptr != MAP_FAILED && b->fd != -1;
}

}  // namespace

extern "C" {

const char* mlf_buffer_last_error(void) { return g_err.c_str(); }

int mlf_buffer_create(const char* object_id, size_t capacity, int overwrite, mlf_buffer** out) {
  if (!object_id || !out) return fail(MLF_INVALID_ARGUMENT, "null argument");
  *out = nullptr;
  std::string id(object_id);
  if (capacity == 0)
    return fail(MLF_INVALID_ARGUMENT, "create_file_and_mmap requires a size greater than 0 for file: " + id);
  if (int e = make_parent_dirs(id))
    return fail(MLF_INTERNAL, "Failed to create directories for: " + id + ": " + strerror(e));

  int flags = O_CREAT | O_RDWR | (overwrite ? O_TRUNC : O_EXCL);
  int fd = open(object_id, flags, 0666);
  if (fd == -1) {
    int e = errno;
    if (e == EEXIST && !overwrite)
      return fail(MLF_ALREADY_EXISTS,
                  "open() failed for file: " + id + ". File already exists and overwrite is set to false.");
    return fail_errno("open() failed for file: " + id, e);
  }
  if (int rc = check_space(fd, capacity, id)) {
    close(fd);
    unlink(object_id);  // it is empty: either just created or just truncated by O_TRUNC
    return rc;
  }
  if (ftruncate(fd, (off_t)capacity) == -1) {
    int e = errno;
    close(fd);
    return fail_errno("ftruncate() failed for file: " + id, e);
  }
  void* p = mmap(nullptr, capacity, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  if (p == MAP_FAILED) {
    int e = errno;
    close(fd);
    return fail_errno("mmap() failed for file: " + id, e);
  }
  mlf_buffer* b = new mlf_buffer();
  b->id = id;
  b->ptr = p;
  b->cap = capacity;
  b->fd = fd;
  b->writable = true;
  b->closed = false;
  *out = b;
  return MLF_OK;
}

int mlf_buffer_open_readonly(const char* object_id, mlf_buffer** out) {
  if (!object_id || !out) return fail(MLF_INVALID_ARGUMENT, "null argument");
  *out = nullptr;
  std::string id(object_id);
  struct stat st;
  if (stat(object_id, &st) == 0 && S_ISDIR(st.st_mode))
    return fail(MLF_INVALID_ARGUMENT, "Path is a directory, not a file: " + id);
  int fd = open(object_id, O_RDONLY);
  if (fd == -1) return fail_errno("open() failed for file: " + id, errno);
  if (fstat(fd, &st) == -1) {
    int e = errno;
    close(fd);
    return fail_errno("fstat() failed for file: " + id, e);
  }
  if (st.st_size == 0) {
    close(fd);
    return fail(MLF_INVALID_ARGUMENT,
                "File cannot be empty, open_file_and_mmap cannot handle zero-sized file: " + id);
  }
  void* p = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_SHARED, fd, 0);
  if (p == MAP_FAILED) {
    int e = errno;
    close(fd);
    return fail_errno("mmap() failed for file: " + id, e);
  }
  mlf_buffer* b = new mlf_buffer();
  b->id = id;
  b->ptr = p;
  b->cap = (size_t)st.st_size;
  b->fd = fd;
  b->writable = false;
  b->closed = false;
  *out = b;
  return MLF_OK;
}

int mlf_buffer_close(mlf_buffer* b, int has_truncate, size_t truncate_size) {
  if (!is_open(b)) return MLF_OK;
  if (!b->writable) has_truncate = 0;  // read-only mappings are never truncated
  std::string errs;
  auto add = [&errs](const std::string& m) {
    if (!errs.empty()) errs += "; ";
    errs += m;
  };
  if (munmap(b->ptr, b->cap) == -1) add(std::string("munmap() failed: ") + strerror(errno));
  if (has_truncate && ftruncate(b->fd, (off_t)truncate_size) == -1)
    add(std::string("ftruncate() failed: ") + strerror(errno));
  if (close(b->fd) == -1) add(std::string("close() failed: ") + strerror(errno));
  b->closed = true;
  b->fd = -1;
  b->ptr = nullptr;
  b->cap = 0;
  if (!errs.empty()) return fail(MLF_INTERNAL, "Errors during unmap_and_close: " + errs);
  return MLF_OK;
}

void mlf_buffer_destroy(mlf_buffer* b) {
  if (!b) return;
  mlf_buffer_close(b, 0, 0);
  delete b;
}

int mlf_buffer_resize(mlf_buffer* b, size_t new_capacity) {
  if (!is_open(b)) return fail(MLF_FAILED_PRECONDITION, "Cannot resize a closed buffer.");
  if (!b->writable) return fail(MLF_FAILED_PRECONDITION, "Cannot resize a read-only buffer.");
  if (new_capacity == 0) return fail(MLF_INVALID_ARGUMENT, "Cannot resize buffer to 0.");
  if (new_capacity == b->cap) return MLF_OK;
  // Same outcome as munmap + ftruncate + mmap (the file and the mapping both get the new size, the address may
  // change), but mremap carries the page-table entries of the surviving range over, so a pooled buffer that is
  // trimmed after one save and grown again for the next is written without taking a minor fault per page.
  const bool shrinking = new_capacity < b->cap;
  if (!shrinking)
    if (int rc = check_space(b->fd, new_capacity, b->id)) return rc;  // the buffer stays as it is
  if (!shrinking && ftruncate(b->fd, (off_t)new_capacity) == -1) return fail_errno("ftruncate() failed during resize", errno);
  void* p = mremap(b->ptr, b->cap, new_capacity, MREMAP_MAYMOVE);
  if (p == MAP_FAILED) {
    int e = errno;
    // fall back to the plain sequence
    if (munmap(b->ptr, b->cap) == -1) return fail_errno("munmap() failed during resize", errno);
    b->ptr = nullptr;
    if (ftruncate(b->fd, (off_t)new_capacity) == -1) {
      b->closed = true;
      return fail_errno("ftruncate() failed during resize", errno);
    }
    p = mmap(nullptr, new_capacity, PROT_READ | PROT_WRITE, MAP_SHARED, b->fd, 0);
    if (p == MAP_FAILED) {
      b->closed = true;
      return fail_errno(std::string("mmap() failed during resize (after mremap: ") + strerror(e) + ")", errno);
    }
  } else if (shrinking && ftruncate(b->fd, (off_t)new_capacity) == -1) {
    int e2 = errno;
    b->ptr = p;
    b->cap = new_capacity;
    return fail_errno("ftruncate() failed during resize", e2);
  }
  b->ptr = p;
  b->cap = new_capacity;
  return MLF_OK;
}

int mlf_buffer_reserve(mlf_buffer* b, size_t offset, size_t nbytes) {
  if (!is_open(b)) return fail(MLF_FAILED_PRECONDITION, "Cannot reserve pages of a closed buffer.");
  if (!b->writable) return fail(MLF_FAILED_PRECONDITION, "Cannot reserve pages of a read-only buffer.");
  if (offset > b->cap || nbytes > b->cap - offset) return fail(MLF_INVALID_ARGUMENT, "range lies outside the buffer");
  if (nbytes == 0) return MLF_OK;
  struct stat st;
  // a pooled buffer that is written for the second time has its pages already: nothing to do, and walking 100 GB of
  // page cache to find that out would cost more than it saves
  if (fstat(b->fd, &st) == 0 && (unsigned long long)st.st_blocks * 512ull >= (unsigned long long)(offset + nbytes))
    return MLF_OK;
  if (fallocate(b->fd, 0, (off_t)offset, (off_t)nbytes) == 0) return MLF_OK;
  const int e = errno;
  if (e == EOPNOTSUPP || e == ENOSYS) return MLF_OK;  // the file system allocates on first touch only: as before
  if (e == ENOSPC)
    return fail(MLF_INTERNAL, "not enough space on the file system that holds " + b->id + " for " +
                                  std::to_string(nbytes) + " more bytes");
  return fail_errno("fallocate() failed for file: " + b->id, e);
}

int mlf_buffer_prefault(mlf_buffer* b, size_t offset, size_t nbytes, int threads) {
  if (int rc = mlf_buffer_reserve(b, offset, nbytes)) return rc;
  if (nbytes == 0) return MLF_OK;
  // page-table entries for the whole range, writable, so that the first stores into it take no fault at all
  const size_t page = 4096;
  char* base = static_cast<char*>(b->ptr);
  const size_t begin = offset / page * page, end = std::min(b->cap, (offset + nbytes + page - 1) / page * page);
  const size_t want = std::max<size_t>(1, std::min<size_t>((size_t)std::max(threads, 1), (end - begin) / ((size_t)64 << 20) + 1));
  size_t per = ((end - begin + want - 1) / want + page - 1) / page * page;
  std::atomic<int> err{0};
  auto run = [&](size_t lo, size_t hi) {
    const size_t step = (size_t)256 << 20;  // bounded calls: a signal or an error shows up between them
    for (size_t at = lo; at < hi && !err.load(); at += step) {
      const size_t len = std::min(step, hi - at);
#ifdef MADV_POPULATE_WRITE
      if (madvise(base + at, len, MADV_POPULATE_WRITE) == 0) {
        // Once more over the same pages, which costs no fault now: the kernel counts a populate as a use of the
        // page, as it counts a read() of it, and at its second use moves the page to the active list - 27 million
        // list moves for a 112 GB buffer, which otherwise fall into the first pread() pass over the file (measured:
        // 40 GB/s for that pass instead of 100 GB/s, one second more for the first restore of a checkpoint).
        (void)madvise(base + at, len, MADV_POPULATE_WRITE);
        continue;
      }
      if (errno != EINVAL && errno != ENOSYS) {
        err.store(errno);
        return;
      }
#endif
      // a kernel without MADV_POPULATE_WRITE: a store that changes nothing, one per page
      for (size_t p = at; p < at + len; p += page)
        __atomic_fetch_or(reinterpret_cast<unsigned char*>(base + p), (unsigned char)0, __ATOMIC_RELAXED);
    }
  };
  std::vector<std::thread> pool;
  for (size_t lo = begin + per; lo < end; lo += per) pool.emplace_back(run, lo, std::min(end, lo + per));
  run(begin, std::min(end, begin + per));
  for (auto& t : pool) t.join();
  if (int e = err.load()) return fail_errno("madvise(MADV_POPULATE_WRITE) failed for file: " + b->id, e);
  return MLF_OK;
}

void* mlf_buffer_data_ptr(const mlf_buffer* b) { return is_open(b) ? b->ptr : nullptr; }
size_t mlf_buffer_capacity(const mlf_buffer* b) { return is_open(b) ? b->cap : 0; }
int mlf_buffer_is_closed(const mlf_buffer* b) { return is_open(b) ? 0 : 1; }
int mlf_buffer_is_readonly(const mlf_buffer* b) { return (b && b->writable) ? 0 : 1; }
const char* mlf_buffer_id(const mlf_buffer* b) { return b ? b->id.c_str() : ""; }
int mlf_buffer_fd(const mlf_buffer* b) { return is_open(b) ? b->fd : -1; }

int mlf_host_parallel_memcpy(void* dst, const void* src, size_t n, int threads) {
  if (n == 0) return MLF_OK;
  if (!dst || !src) return fail(MLF_INVALID_ARGUMENT, "null pointer passed to mlf_host_parallel_memcpy");
  const size_t kMinPerThread = (size_t)4 << 20;
  size_t want = std::max<size_t>(1, std::min<size_t>((size_t)std::max(threads, 1), n / kMinPerThread));
  if (want <= 1) {
    memcpy(dst, src, n);
    return MLF_OK;
  }
  size_t per = (n + want - 1) / want;
  per = (per + 4095) & ~(size_t)4095;
  std::vector<std::thread> pool;
  char* d = static_cast<char*>(dst);
  const char* s = static_cast<const char*>(src);
  for (size_t off = per; off < n; off += per) {
    size_t len = std::min(per, n - off);
    pool.emplace_back([d, s, off, len] { memcpy(d + off, s + off, len); });
  }
  memcpy(d, s, std::min(per, n));
  for (auto& t : pool) t.join();
  return MLF_OK;
}

}  // extern "C"

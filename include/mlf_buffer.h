/*
 * C-ABI of the file-backed shared-memory buffer object and of the host-side bulk copy helpers.
 *
 * A buffer object is a regular file (normally on tmpfs) mapped MAP_SHARED into the process.  It is the
 * destination of a checkpoint save and the source of a restore.  The entry points below are what a
 * language binding binds in place of the reference's pybind11 class `BufferObject`
 * (reference: src/ml_flashpoint/checkpoint_object_manager/buffer_object/bindings.cpp:27-100,
 * buffer_object.h:24-85).
 *
 * Conventions: every function that can fail returns an mlf_status (0 = ok).  On failure a
 * human-readable message is kept per thread and can be fetched with mlf_buffer_last_error(); the
 * text follows the shape "<CODE_NAME>: <message>" that the reference's status strings have, so callers
 * that match on substrings of those messages keep working.  No function throws across the boundary.
 */
#ifndef MLF_BUFFER_H_
#define MLF_BUFFER_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum mlf_status {
  MLF_OK = 0,
  MLF_INVALID_ARGUMENT = 3, /* bad size, directory instead of file, empty file, closed handle */
  MLF_ALREADY_EXISTS = 6,   /* create without overwrite on an existing path */
  MLF_FAILED_PRECONDITION = 9,
  MLF_INTERNAL = 13         /* a system call failed; message carries strerror text */
} mlf_status;

typedef struct mlf_buffer mlf_buffer; /* opaque */

/* Creates (or, with overwrite != 0, truncates and re-creates) the file `object_id`, sizes it to
 * `capacity` bytes and maps it read-write.  Parent directories are created.  Without overwrite an
 * existing path fails with MLF_ALREADY_EXISTS.  A capacity that the file system cannot hold at that
 * moment (free space per fstatvfs) fails with MLF_INTERNAL and leaves no file: stores into pages a full
 * tmpfs cannot back would otherwise end in SIGBUS (the reference has no such check).
 * Replaces BufferObject(object_id, capacity, overwrite): buffer_object.cpp:25-49,
 * buffer_helper.cpp:43-120. */
int mlf_buffer_create(const char* object_id, size_t capacity, int overwrite, mlf_buffer** out);

/* Maps an existing, non-empty regular file read-only; capacity is the file size.
 * Replaces BufferObject(object_id): buffer_object.cpp:52-73, buffer_helper.cpp:122-185. */
int mlf_buffer_open_readonly(const char* object_id, mlf_buffer** out);

/* Unmaps, optionally truncates the file to `truncate_size` bytes (has_truncate != 0), closes the
 * descriptor.  Idempotent; the handle stays valid (in the closed state) until mlf_buffer_destroy.
 * A truncate request on a read-only mapping is ignored.  Every step is attempted even if an earlier
 * one failed; the failures are joined in the error text.
 * Replaces BufferObject::close: buffer_object.cpp:140-176, buffer_helper.cpp:187-271. */
int mlf_buffer_close(mlf_buffer* b, int has_truncate, size_t truncate_size);

/* Closes (without truncation) if still open and frees the handle. Replaces ~BufferObject. */
void mlf_buffer_destroy(mlf_buffer* b);

/* New capacity for file and mapping (mremap, so the surviving range keeps its page-table entries; the
 * data pointer may change).  Fails on closed or read-only handles, on new_capacity == 0, and on growth
 * beyond the free space of the file system, in which case the buffer stays as it was.
 * Replaces BufferObject::resize: buffer_object.cpp:178-197, buffer_helper.cpp:273-314. */
int mlf_buffer_resize(mlf_buffer* b, size_t new_capacity);

/* Accessors (bindings.cpp:43-76).  data_ptr is NULL and capacity 0 once closed. */
/* Makes the file system allocate the pages of [offset, offset + nbytes) now (fallocate) instead of one by one as
 * they are first stored to.  On tmpfs the allocation inside a page fault is serialised (4-7 GB/s whatever the
 * number of writing threads, measured on the MI355X host), fallocate runs at about 20 GB/s and the stores that
 * follow take minor faults only, which do scale with threads; a full file system is reported here, as an error,
 * instead of by SIGBUS later.  Does nothing if the file already has that many allocated bytes.  An addition: the
 * reference leaves allocation to the page faults of its copy_ (buffer_helper.cpp:96-103). */
int mlf_buffer_reserve(mlf_buffer* b, size_t offset, size_t nbytes);

/* mlf_buffer_reserve plus page-table entries: after it, stores into [offset, offset + nbytes) of the mapping take no
 * page fault at all (madvise MADV_POPULATE_WRITE on up to `threads` threads; on kernels without it, one store per page
 * that changes nothing).  Meant for a pool's buffer files right after they are created, off the critical path: the
 * first checkpoint into a fresh 112 GB file otherwise spends 5-6 s allocating pages and 2 s more taking minor faults.
 * The pages are populated twice, so that the kernel has them on its active list before anyone read()s the file (the
 * first pread pass over pages that are not runs at 40 instead of 100 GB/s).
 * The range must not be written by anyone else meanwhile.  An addition: the reference pre-creates its pool files
 * (src/ml_flashpoint/core/buffer_pool.py:324-342) but leaves their pages to the first save. */
int mlf_buffer_prefault(mlf_buffer* b, size_t offset, size_t nbytes, int threads);

void* mlf_buffer_data_ptr(const mlf_buffer* b);
size_t mlf_buffer_capacity(const mlf_buffer* b);
int mlf_buffer_is_closed(const mlf_buffer* b);
int mlf_buffer_is_readonly(const mlf_buffer* b);
const char* mlf_buffer_id(const mlf_buffer* b);
/* The descriptor the mapping was made from (-1 once closed); stays owned by the buffer object. */
int mlf_buffer_fd(const mlf_buffer* b);

/* Message of the last failure on the calling thread ("" if none). */
const char* mlf_buffer_last_error(void);

/* Copies n bytes with up to `threads` worker threads (page-aligned split).  Used for host-resident
 * checkpoint items and for restore staging; stands where the reference relies on torch's intra-op
 * threaded copy_ (src/ml_flashpoint/core/checkpoint_saver.py:443-450,797-800). */
int mlf_host_parallel_memcpy(void* dst, const void* src, size_t n, int threads);

#ifdef __cplusplus
}
#endif
#endif /* MLF_BUFFER_H_ */

/*
 * C-ABI of the MI355X (gfx950) save/restore data path.
 *
 * The reference moves a checkpoint shard with three PyTorch calls per tensor and has no FFI for it:
 *   save    - Tensor.to("cpu") per tensor + one device synchronize
 *             (src/ml_flashpoint/core/checkpoint_saver.py:347-360,
 *              src/ml_flashpoint/adapter/pytorch/memory_storage_writer.py:213-233), then
 *             header + torch.frombuffer(mmap_slice).copy_(tensor) per tensor
 *             (src/ml_flashpoint/core/checkpoint_saver.py:764-800);
 *   restore - read() copy of each record, torch.frombuffer, narrow, target.copy_()
 *             (src/ml_flashpoint/core/checkpoint_loader.py:177-219,300-336).
 * The entry points below are what a binding binds instead.  They work on an "image": the byte-exact data
 * section of one checkpoint object (records `<u32 len><pickled header><payload>` back to back), held in
 * device memory.  Save = pack live tensors into the image, stream the image to the mapped buffer file;
 * restore = stream the file into an image, unpack into live tensors.
 *
 * Conventions: plain pointers and sizes only; every function returns 0 on success or a non-zero code and
 * keeps a message for mlf_hip_last_error() (per thread).  Device pointers are raw HIP device addresses.
 * `stream` arguments are hipStream_t passed as void* (NULL = the default stream).  Handles are opaque.
 * All calls act on the calling thread's current HIP device.
 */
#ifndef MLF_HIP_H_
#define MLF_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLF_MAX_DIMS 8

/* What an item's bytes are copied from (pack) or to (unpack). */
enum mlf_item_kind {
  MLF_ITEM_DEVICE = 0, /* tensor in device memory described by shape/stride (contiguous or not)              */
  MLF_ITEM_BLOB = 1    /* bytes that live in the plan's host blob: record headers, host-resident tensors,     */
                       /* pickled non-tensor objects.  Pack only; ignored by unpack.                          */
};

/* One entry of the descriptor table handed to mlf_plan_create.  The plan keeps a device-resident form of it.
 * `image_off` is where the item's first byte lies in the image.  For MLF_ITEM_DEVICE the logical index space
 * is `shape[0..ndim)`; element (i0..ik) lives at ptr + esz * sum(i_d * stride[d]) on the tensor side and at
 * image_off + esz * sum(i_d * image_stride[d]) on the image side.  On save the image side is the C-contiguous
 * payload the reference writes (checkpoint_saver.py:797-800); on restore it is the requested sub-box of the
 * stored tensor (checkpoint_loader.py:219 narrow_tensor_by_index) and the tensor side is the caller's target,
 * which may itself be a strided view.  ndim == 0 means one element. */
typedef struct mlf_item {
  uint64_t ptr;       /* DEVICE: device address of element 0.  BLOB: byte offset into the host blob.          */
  uint64_t image_off; /* byte offset in the image                                                              */
  uint64_t nbytes;    /* total bytes of the item (numel * elem_size, or blob length)                           */
  uint32_t kind;      /* enum mlf_item_kind                                                                    */
  uint32_t elem_size; /* bytes per element: 1, 2, 4, 8 or 16 (DEVICE only)                                     */
  uint32_t ndim;      /* 0..MLF_MAX_DIMS (DEVICE only)                                                         */
  uint32_t reserved;
  int64_t shape[MLF_MAX_DIMS];
  int64_t stride[MLF_MAX_DIMS];       /* tensor side, in elements                                               */
  int64_t image_stride[MLF_MAX_DIMS]; /* image side, in elements                                                */
} mlf_item;

typedef struct mlf_plan_opts {
  uint32_t tile_bytes;       /* bytes one workgroup copies per work item (multiple of 1024; 0 = default)       */
  uint32_t block_threads;    /* threads per workgroup for the copy kernels (multiple of 64; 0 = default)       */
  uint32_t align_to_tensor;  /* tile cuts sit on a 4 KiB grid of: 0 = image offsets (pack), 1 = tensor addresses (unpack) */
  uint32_t unroll;           /* 16-byte vectors in flight per thread in the copy loop: 1, 2, 4, 8 (0 = default) */
  uint32_t grid_x_log2;      /* 0 = default; k > 0: rows of 2^(k-1) workgroups in the copy kernel's grid (a row may
                                not exceed 2^32 - 1 threads),
                                the rest goes to gridDim.y of the same launch.  Small values are for tests.     */
  uint32_t crc_chunk_kib;    /* 0 = no checksums.  k > 0 (a multiple of 64): every pack / unpack launch of the plan also
                                yields the CRC-32C of every k KiB chunk of the image (the last may be short), read with
                                mlf_plan_crc_values().  Where a contiguous item covers whole 64 KiB pieces of the image, the
                                kernel that copies them also folds their remainders, so those bytes are not read a second
                                time; the rest of the image (record headers, item edges, strided and transposed items, a
                                last partial chunk) is checksummed from the image after it is complete.                   */
} mlf_plan_opts;

typedef struct mlf_plan_info {
  uint64_t n_items;
  uint64_t n_flat_tiles;      /* workgroup work items of the flat (byte-segment) kernel                        */
  uint64_t n_strided_items;   /* items that go through the generic strided kernel                              */
  uint64_t n_strided_work;
  uint64_t n_transposed_items;/* items that go through the LDS-tiled transpose kernel                          */
  uint64_t n_transposed_work;
  uint64_t device_bytes;      /* payload bytes that live in device tensors (P in the roofline figures)         */
  uint64_t blob_bytes;        /* bytes that come from the host blob                                            */
  uint64_t image_bytes;
  uint64_t table_bytes;       /* device memory held by the plan's tables + blob                                */
  uint64_t n_small_items;     /* pieces of at most 1 KiB that are copied one per wavefront                     */
  uint64_t fused_crc_bytes;   /* image bytes whose checksum remainders come out of the copy itself (crc_chunk_kib > 0) */
  uint64_t crc_chunks;        /* values mlf_plan_crc_values() returns                                                   */
} mlf_plan_info;

typedef struct mlf_plan mlf_plan;

/* Message of the last failure on the calling thread ("" if none). */
const char* mlf_hip_last_error(void);

/* Number of visible devices / select the calling thread's device (HIP's current device is per thread). */
int mlf_hip_device_count(int* out);
int mlf_hip_set_device(int device);
/* Free and total device memory in bytes. */
int mlf_hip_mem_info(uint64_t* free_bytes, uint64_t* total_bytes);

/* Builds the device-resident descriptor/work tables for `n_items` items and uploads `host_blob`.
 * Validates that every item lies inside [0, image_bytes) and every blob item inside the blob.
 * The plan stays valid while the tensors' addresses, shapes and strides stay the same; it can be launched
 * any number of times.  Stands where the reference walks its Python list of (WriteItem, tensor) pairs
 * (checkpoint_saver.py:668-682) or ReadItems (checkpoint_loader.py:322-336). */
int mlf_plan_create(const mlf_item* items, uint64_t n_items, const void* host_blob, uint64_t blob_bytes,
                    uint64_t image_bytes, const mlf_plan_opts* opts, mlf_plan** out);
int mlf_plan_destroy(mlf_plan* plan);
int mlf_plan_get_info(const mlf_plan* plan, mlf_plan_info* out);

/* Replaces the bytes of the plan's blob (same size as at creation) for a plan that is kept from one save to the
 * next: the record headers in it repeat, step counters and other host-resident items do not.  The upload is
 * enqueued on `stream` and made to wait for the plan's last launch wherever that ran, so it is ordered behind
 * the kernels that still read the old bytes and ahead of launches enqueued on `stream` afterwards; a launch on
 * another stream must be ordered behind the upload by the caller.  No reference counterpart: the reference
 * rebuilds everything per save (checkpoint_saver.py:622-707); its plan caching (save_strategies.py:182-212) is the
 * model for keeping the tables. */
int mlf_plan_update_blob(mlf_plan* plan, const void* host_blob, uint64_t blob_bytes, void* stream);

/* Save direction: tensors (+ blob) -> image.  Asynchronous on `stream`; the image is complete when the
 * stream reaches the point after this call.  Replaces the per-tensor .to("cpu") staging
 * (checkpoint_saver.py:347-360; memory_storage_writer.py:213-233) and the per-tensor
 * frombuffer().copy_() (checkpoint_saver.py:797-800): afterwards the training stream may go on. */
int mlf_pack_launch(const mlf_plan* plan, void* image_dev, void* stream);

/* Restore direction: image -> tensors.  Asynchronous on `stream`.  Replaces frombuffer + narrow + copy_
 * (checkpoint_loader.py:206-219,331-336). */
int mlf_unpack_launch(const mlf_plan* plan, const void* image_dev, void* stream);

/* Per-chunk CRC-32C values of the image that the plan's most recent mlf_pack_launch / mlf_unpack_launch moved (plans
 * created with crc_chunk_kib > 0): waits for that launch's checksum work and copies ceil(image_bytes / chunk) values
 * to `out_host`.  Same values as mlf_crc32c_device over the image.  On save they go into the object's sidecar; on
 * restore the caller compares them with the sidecar's.  Call it before the plan is launched again.  No reference
 * counterpart (the reference has no checksum). */
int mlf_plan_crc_values(mlf_plan* plan, uint32_t* out_host, uint64_t n_out);

/* CRC-32C (Castagnoli, reflected, init/xorout 0xFFFFFFFF as in RFC 3720) of consecutive `chunk_bytes`
 * pieces of a device buffer; the last chunk may be short.  Writes ceil(nbytes/chunk_bytes) values to
 * `out_host` and returns after they are valid.  The reference has no checksum; this is the integrity check
 * of the copy pipeline (values are kept beside the object, never inside it). */
int mlf_crc32c_device(const void* dev_ptr, uint64_t nbytes, uint64_t chunk_bytes, uint32_t* out_host,
                      uint64_t n_out, void* stream);
/* mlf_crc32c_device for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc); it has no counterpart in the reference.  Same values, but nothing is
 * allocated or freed by the call: the lookup constants and the per-segment values live in a fixed array of
 * 1 056 768 bytes that is part of the library's code object on every device it runs on, the per-chunk values are
 * written to `out_dev` (DEVICE memory of the caller, ceil(nbytes/chunk_bytes) values, 4-byte aligned), and
 * the call only enqueues kernels on `stream`: the values are valid when the stream reaches the point after it.
 * Limit: at most 262 144 segment values per call (segments are 64 KiB to 512 KiB by the size of the buffer and are
 * doubled, while they still divide `chunk_bytes`, until their count fits); more than that, e.g. 16 GiB in 64 KiB
 * chunks, is refused with a message.  All calls on one device share that device's array and every call
 * overwrites it: calls that overlap in time on one device race; calls ordered on one stream do not (replays of a
 * captured graph that holds the call count as calls: the array's address is part of the graph).  Where the array
 * lies on a device is looked up once, by mlf_hip_set_device(device) or else by the first call on that device; that
 * lookup is not for a stream under capture, so call mlf_hip_set_device first (or make one call) before capturing. */
int mlf_crc32c_device_noalloc(const void* dev_ptr, uint64_t nbytes, uint64_t chunk_bytes, uint32_t* out_dev,
                              uint64_t n_out, void* stream);
/* Same function on host memory (SSE4.2), and the combine law crc(A||B) from crc(A), crc(B), len(B). */
uint32_t mlf_crc32c_host(const void* data, uint64_t nbytes);
uint32_t mlf_crc32c_combine(uint32_t crc_a, uint32_t crc_b, uint64_t len_b);
/* Host-only: CRC-32C of every `chunk_bytes` piece of the byte range [file_offset, file_offset + nbytes) of an
 * open file, read with pread() by `threads` threads (no mapping is built, no GPU is touched).  Writes
 * ceil(nbytes/chunk_bytes) values.  Lets recovery discovery check an object against the values recorded when it
 * was saved before choosing it (the reference's discovery, checkpoint_loader.py:340-424, checks presence only). */
int mlf_crc32c_file(int fd, uint64_t file_offset, uint64_t nbytes, uint64_t chunk_bytes, uint32_t* out_host,
                    uint64_t n_out, uint32_t threads);

/* Copy engine: a ring of pinned host slots, two copy streams and a pool of host threads that move data
 * between device memory and pageable host memory (the MAP_SHARED buffer file) at link speed. */
typedef struct mlf_engine mlf_engine;

typedef struct mlf_xfer_stats {
  double seconds;        /* wall time of the call                                                             */
  double wait_seconds;   /* d2h: of which the calling thread spent waiting for the producer stream;           */
                         /* h2d: of which the host threads spent filling the pinned slots (pread / memcpy)    */
  uint64_t bytes;
  uint64_t chunks;
} mlf_xfer_stats;

int mlf_engine_create(uint64_t slot_bytes, uint32_t n_slots, uint32_t n_threads, mlf_engine** out);
int mlf_engine_destroy(mlf_engine* engine);

/* Device -> host.  Waits (on the copy streams, not on the host) for everything enqueued so far on
 * `producer_stream`, then copies `nbytes` from `src_dev` to `dst_host` and returns when the bytes are in
 * place.  `dst_host` is typically BufferObject.get_data_ptr() + 4096 + position
 * (bindings.cpp:59-72; buffer_io.py:342-343).  Replaces the D2H half of Tensor.to("cpu") and the CPU
 * copy_ into the mapping.  Safe to call from a thread other than the one that launched the pack. */
int mlf_engine_d2h(mlf_engine* engine, const void* src_dev, void* dst_host, uint64_t nbytes,
                   void* producer_stream, mlf_xfer_stats* stats);

/* mlf_engine_d2h that also checksums what it sends: CRC-32C of every `crc_chunk_bytes` piece of the source
 * (same definition and constraints as mlf_crc32c_device), computed on a third stream while the copies run, so
 * the check costs no blocking time and no transfer time.  `crc_out_host` receives ceil(nbytes/crc_chunk_bytes)
 * values before the call returns.  No reference counterpart (the reference has no checksum). */
int mlf_engine_d2h_crc(mlf_engine* engine, const void* src_dev, void* dst_host, uint64_t nbytes,
                       void* producer_stream, uint64_t crc_chunk_bytes, uint32_t* crc_out_host,
                       uint64_t n_crc_out, mlf_xfer_stats* stats);

/* mlf_engine_d2h_crc (`crc_chunk_bytes` may be 0: no checksums) that also publishes its progress: whenever a
 * further slot has reached `dst_host`, the number of leading bytes of the range that are in place is stored into
 * `*landed` (8-byte aligned host memory of the caller) with release ordering; a reader that loads it with acquire
 * ordering may read that many bytes of the destination.  0 is stored before the first copy, `nbytes` with the
 * last.  For a sender that forwards an object to its replica while the rest is still crossing the link: the
 * reference hands the buffer to its replication manager only after the whole object is written
 * (checkpoint_saver.py:700-707, replication_manager.py:248-300). */
int mlf_engine_d2h_watched(mlf_engine* engine, const void* src_dev, void* dst_host, uint64_t nbytes,
                           void* producer_stream, uint64_t crc_chunk_bytes, uint32_t* crc_out_host,
                           uint64_t n_crc_out, uint64_t* landed, mlf_xfer_stats* stats);

/* mlf_engine_d2h_watched whose copies (and checksum pass) wait for an event instead of for a stream: `ready_event`
 * is a hipEvent_t (passed as void*) that the caller recorded right behind the kernel that produced the source - the
 * pack - or NULL to start at once.  A transfer that is started from another thread than the one that launched the
 * pack then waits for the pack only, not for whatever the training step has enqueued on that stream since.  No
 * reference counterpart: the reference's device synchronize (memory_storage_writer.py:229-231) waits for everything. */
int mlf_engine_d2h_gated(mlf_engine* engine, const void* src_dev, void* dst_host, uint64_t nbytes, void* ready_event,
                         uint64_t crc_chunk_bytes, uint32_t* crc_out_host, uint64_t n_crc_out, uint64_t* landed,
                         mlf_xfer_stats* stats);

/* Host -> device.  Copies `nbytes` from `src_host` (pageable, e.g. the read-only mapping) to `dst_dev`
 * and makes `consumer_stream` wait for the last chunk, so an unpack launched on it afterwards sees the data.
 * Returns once all chunks are enqueued and the host source is no longer needed.  Replaces BufferIO.read()'s
 * copy plus the pageable H2D inside target.copy_() (buffer_io.py:206; checkpoint_loader.py:335). */
int mlf_engine_h2d(mlf_engine* engine, const void* src_host, void* dst_dev, uint64_t nbytes,
                   void* consumer_stream, mlf_xfer_stats* stats);

/* Measurement aid: moves `nbytes` between `dev_buf` and the engine's own pinned slots over its two copy streams -
 * device to slots (`to_host` != 0) or slots to device - with no host-side copy behind it, and reports the wall time.
 * That is the rate the host link gives this engine's transfers at best; what mlf_engine_d2h / mlf_engine_h2d reach is
 * to be read against it.  The slots' contents are left as they are (to the device go whatever bytes they hold).  No
 * reference counterpart. */
int mlf_engine_link_probe(mlf_engine* engine, void* dev_buf, uint64_t nbytes, int to_host, double* seconds);

/* Moves the engine's streams off the hardware queues of `busy_streams` - the streams the training step runs on.  The HIP
 * runtime spreads a process's streams over a few hardware queues (GPU_MAX_HW_QUEUES, 4 unless the environment says
 * otherwise), and a queue runs its commands in order: a copy stream that shares its queue with a stream that is kept
 * full waits behind that stream's kernels - measured 10-13 GB/s instead of 53-56 beside back-to-back GEMMs.  Which
 * streams share is decided when they are created and cannot be asked for, so it is measured: both streams idle, a
 * 2 ms kernel of one wavefront on a busy stream, an empty kernel on the engine's stream; if that one has to wait, the
 * stream is replaced by a new one that waits for none of them.  Waits for the busy streams to drain (several times):
 * call it at set-up, or in the blocking part of the first save.  `busy_streams` holds `n_busy` raw hipStream_t values
 * (a null entry is the default stream); `still_shared` (may be null) receives the number of the engine's three
 * streams for which no free queue was found.  No reference counterpart. */
int mlf_engine_avoid_streams(mlf_engine* engine, void* const* busy_streams, uint32_t n_busy, uint32_t* still_shared);

/* The stream the engine runs its checksum kernels on (a raw hipStream_t), for checksum calls a caller makes between
 * the engine's transfers (mlf_crc32c_device on pieces of an image): a stream that mlf_engine_avoid_streams has
 * already moved out of the training stream's way.  A later mlf_engine_avoid_streams may give the engine another
 * one; a handle returned earlier stays a valid stream until mlf_engine_destroy. */
void* mlf_engine_checksum_stream(mlf_engine* engine);

/* Who takes the per-chunk CRC-32C of a device-to-host transfer that asks for one (mlf_engine_d2h_crc, _watched,
 * _gated).  on = 0 (the state of a new engine): kernels on the engine's checksum stream read the image once more
 * while it crosses the link.  on != 0: the host threads that move the pinned slots into the destination take the
 * checksums of what they move (crc32 instructions beside the copy loop, three interleaved chains per thread) - no
 * kernel, no second read of the image from device memory; the values are the same.  Takes effect with the next
 * transfer.  No reference counterpart (the reference keeps no checksums). */
int mlf_engine_set_host_checksums(mlf_engine* engine, int on);

/* A device-to-host transfer of a piece of a larger data section, with the checksums of the piece cut where the
 * section's chunks end: the piece's first `first_part_bytes` bytes (less than a chunk; 0: the piece begins on a
 * chunk boundary) belong to a chunk that began before it and get a value of their own, then every
 * `crc_chunk_bytes` bytes one, the last possibly short - (first_part_bytes ? 1 : 0) + ceil((nbytes -
 * first_part_bytes) / crc_chunk_bytes) values for a piece longer than its first part, which the caller joins with
 * its neighbours' by mlf_crc32c_combine.  Always taken by the host threads as they copy (the checksum kernels read
 * whole chunks from their first byte).  The copies wait for `ready_event` (a hipEvent_t) if that is not NULL, else
 * for what `producer_stream` holds at the call; `landed` as in mlf_engine_d2h_watched, or NULL.  For objects that
 * leave the device in several transfers (an image held in pieces, windows, runs of an image around host-resident
 * items).  No reference counterpart. */
int mlf_engine_d2h_cut(mlf_engine* engine, const void* src_dev, void* dst_host, uint64_t nbytes, void* producer_stream,
                       void* ready_event, uint64_t crc_chunk_bytes, uint64_t first_part_bytes, uint32_t* crc_out_host,
                       uint64_t n_crc_out, uint64_t* landed, mlf_xfer_stats* stats);

/* mlf_engine_host_copy that also yields the checksums of what it copies, cut like those of mlf_engine_d2h_cut. */
int mlf_engine_host_copy_cut(mlf_engine* engine, void* dst_host, const void* src_host, uint64_t nbytes,
                             uint64_t crc_chunk_bytes, uint64_t first_part_bytes, uint32_t* crc_out_host,
                             uint64_t n_crc_out);

/* File -> host memory on the engine's threads: `nbytes` from byte `file_offset` of `fd` into `dst_host`, by pread()
 * in as many parts as the engine has threads.  For the host-resident targets of a restore (optimizer state kept in
 * host memory): the reference copies such a record out of its mapping with one `copy_`
 * (checkpoint_loader.py:331-336), which pays a page fault per 4 KiB of a mapping that was made for this one read. */
int mlf_engine_read_file(mlf_engine* engine, int fd, uint64_t file_offset, void* dst_host, uint64_t nbytes);

/* Host -> host on the engine's threads: `nbytes` from `src_host` to `dst_host` (ranges must not overlap).  For
 * checkpoint items that are resident in host memory - the reference copies those into the mapping with torch's
 * intra-op threads (checkpoint_saver.py:443-450,797-800); they do not visit the device here either. */
int mlf_engine_host_copy(mlf_engine* engine, void* dst_host, const void* src_host, uint64_t nbytes);

/* The same two transfers with the pageable end given as a byte range of an open file instead of a pointer:
 * the host threads pwrite()/pread() the pinned slots straight to/from the buffer file (`fd` from
 * mlf_buffer_fd(), `file_offset` = 4096 + position in the data section).  The bytes land in the same page-cache
 * pages a MAP_SHARED mapping shows (buffer_helper.cpp:96-103), but no page-table entry is built or torn down per
 * 4 KiB of the object, which for a 100 GB object costs more than the copy itself. */
int mlf_engine_d2h_fd(mlf_engine* engine, const void* src_dev, int fd, uint64_t file_offset, uint64_t nbytes,
                      void* producer_stream, mlf_xfer_stats* stats);
int mlf_engine_h2d_fd(mlf_engine* engine, int fd, uint64_t file_offset, void* dst_dev, uint64_t nbytes,
                      void* consumer_stream, mlf_xfer_stats* stats);

#ifdef __cplusplus
}
#endif
#endif /* MLF_HIP_H_ */

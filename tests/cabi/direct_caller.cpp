// A caller of the two C-ABI libraries with no Python and no torch in the process: the way a C++ component of the
// reference (its transfer service already links the buffer object) would use them.  One object with a contiguous
// tensor, a transposed view and a record header is packed, checksummed, sent into a buffer file, read back through
// the file descriptor and unpacked into fresh device memory; then the same object once more with the checksums folded
// into the pack and the unpack, a transfer gated on an event, and the checksum entry point that allocates nothing.
// Every stage is compared with bytes built on the host.
//
// Build (gfx950, no GPU needed):  see __graft_entry__.build().   Run on an MI355X:  tests/cabi/_build/direct_caller <dir>
#include "mlf_buffer.h"
#include "mlf_hip.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#define REQUIRE(cond)                                                                      \
  do {                                                                                     \
    if (!(cond)) {                                                                         \
      std::fprintf(stderr, "FAILED %s:%d: %s  [hip: %s] [buffer: %s]\n", __FILE__, __LINE__, #cond, \
                   mlf_hip_last_error(), mlf_buffer_last_error());                         \
      return 1;                                                                            \
    }                                                                                      \
  } while (0)

int main(int argc, char** argv) {
  const std::string dir = argc > 1 ? argv[1] : "/dev/shm";
  int devices = 0;
  REQUIRE(mlf_hip_device_count(&devices) == 0 && devices >= 1);
  REQUIRE(mlf_hip_set_device(0) == 0);

  // host truth: a 300 x 700 float matrix A (840 kB: it covers whole 64 KiB pieces of the image), and a 64 x 48 int16 matrix B that is saved through its transpose
  const int ar = 300, ac = 700, br = 64, bc = 48;
  std::vector<float> a(ar * ac);
  std::vector<int16_t> b(br * bc);
  for (size_t i = 0; i < a.size(); ++i) a[i] = 0.25f * (float)i - 1000.0f;
  for (size_t i = 0; i < b.size(); ++i) b[i] = (int16_t)(i * 7 - 9000);
  const char header[] = "\x05\x00\x00\x00HELLO";  // stands for a <u32 len><pickled header> record prefix: 9 bytes
  const uint64_t hdr = 9, a_bytes = a.size() * 4, b_bytes = b.size() * 2;
  const uint64_t image_bytes = hdr + a_bytes + hdr + b_bytes;  // no padding anywhere: A's payload starts at byte 9

  void *d_a = nullptr, *d_b = nullptr, *d_image = nullptr;
  REQUIRE(hipMalloc(&d_a, a_bytes) == hipSuccess && hipMalloc(&d_b, b_bytes) == hipSuccess);
  REQUIRE(hipMalloc(&d_image, image_bytes + 256) == hipSuccess);
  REQUIRE(hipMemcpy(d_a, a.data(), a_bytes, hipMemcpyHostToDevice) == hipSuccess);
  REQUIRE(hipMemcpy(d_b, b.data(), b_bytes, hipMemcpyHostToDevice) == hipSuccess);
  REQUIRE(hipMemset(d_image, 0xAB, image_bytes + 256) == hipSuccess);

  // descriptor table: header, A (contiguous), header, B^T (shape 48 x 64 with strides 1, 48 over B's memory)
  std::vector<mlf_item> items(4);
  std::memset(items.data(), 0, items.size() * sizeof(mlf_item));
  items[0].kind = MLF_ITEM_BLOB, items[0].ptr = 0, items[0].image_off = 0, items[0].nbytes = hdr;
  items[1].kind = MLF_ITEM_DEVICE, items[1].ptr = (uint64_t)d_a, items[1].image_off = hdr, items[1].nbytes = a_bytes;
  items[1].elem_size = 4, items[1].ndim = 1, items[1].shape[0] = ar * ac, items[1].stride[0] = 1, items[1].image_stride[0] = 1;
  items[2].kind = MLF_ITEM_BLOB, items[2].ptr = 0, items[2].image_off = hdr + a_bytes, items[2].nbytes = hdr;
  items[3].kind = MLF_ITEM_DEVICE, items[3].ptr = (uint64_t)d_b, items[3].image_off = 2 * hdr + a_bytes, items[3].nbytes = b_bytes;
  items[3].elem_size = 2, items[3].ndim = 2, items[3].shape[0] = bc, items[3].shape[1] = br;
  items[3].stride[0] = 1, items[3].stride[1] = bc, items[3].image_stride[0] = br, items[3].image_stride[1] = 1;

  std::vector<unsigned char> want(image_bytes);
  std::memcpy(&want[0], header, hdr);
  std::memcpy(&want[hdr], a.data(), a_bytes);
  std::memcpy(&want[hdr + a_bytes], header, hdr);
  int16_t* bt = reinterpret_cast<int16_t*>(&want[2 * hdr + a_bytes]);  // odd address: written through memcpy below
  for (int i = 0; i < bc; ++i)
    for (int j = 0; j < br; ++j) {
      const int16_t v = b[j * bc + i];
      std::memcpy(reinterpret_cast<unsigned char*>(bt) + 2 * (i * br + j), &v, 2);
    }

  mlf_plan* plan = nullptr;
  REQUIRE(mlf_plan_create(items.data(), items.size(), header, hdr, image_bytes, nullptr, &plan) == 0);
  mlf_plan_info info;
  REQUIRE(mlf_plan_get_info(plan, &info) == 0 && info.image_bytes == image_bytes && info.device_bytes == a_bytes + b_bytes);
  REQUIRE(mlf_pack_launch(plan, d_image, nullptr) == 0);
  REQUIRE(hipDeviceSynchronize() == hipSuccess);
  std::vector<unsigned char> got(image_bytes + 256);
  REQUIRE(hipMemcpy(got.data(), d_image, image_bytes + 256, hipMemcpyDeviceToHost) == hipSuccess);
  REQUIRE(std::memcmp(got.data(), want.data(), image_bytes) == 0);
  for (uint64_t i = image_bytes; i < image_bytes + 256; ++i) REQUIRE(got[i] == 0xAB);  // nothing past the image

  // checksum on the device == checksum on the host
  uint32_t crc_dev = 0;
  REQUIRE(mlf_crc32c_device(d_image, image_bytes, 1 << 20, &crc_dev, 1, nullptr) == 0);
  REQUIRE(crc_dev == mlf_crc32c_host(want.data(), image_bytes));

  // image -> buffer file (metadata block of 4096 bytes in front), with the progress counter; then close and reopen
  const std::string path = dir + "/cabi_direct_caller.distcp";
  mlf_buffer* buf = nullptr;
  REQUIRE(mlf_buffer_create(path.c_str(), 4096 + image_bytes, 1, &buf) == 0);
  REQUIRE(mlf_buffer_reserve(buf, 4096, image_bytes) == 0);
  mlf_engine* engine = nullptr;
  REQUIRE(mlf_engine_create(1 << 20, 2, 2, &engine) == 0);
  void* busy_streams[1] = {nullptr};  // the default stream: the engine's streams move off its hardware queue
  uint32_t still_shared = 9;
  REQUIRE(mlf_engine_avoid_streams(engine, busy_streams, 1, &still_shared) == 0 && still_shared == 0);
  REQUIRE(mlf_engine_checksum_stream(engine) != nullptr);
  uint64_t landed = 7;
  uint32_t crc_sent = 0;
  mlf_xfer_stats stats;
  REQUIRE(mlf_engine_d2h_watched(engine, d_image, static_cast<char*>(mlf_buffer_data_ptr(buf)) + 4096, image_bytes, nullptr,
                                 1 << 20, &crc_sent, 1, &landed, &stats) == 0);
  REQUIRE(landed == image_bytes && stats.bytes == image_bytes && crc_sent == crc_dev);
  REQUIRE(std::memcmp(static_cast<char*>(mlf_buffer_data_ptr(buf)) + 4096, want.data(), image_bytes) == 0);
  REQUIRE(mlf_buffer_close(buf, 1, 4096 + image_bytes) == 0);
  mlf_buffer_destroy(buf);
  REQUIRE(mlf_buffer_open_readonly(path.c_str(), &buf) == 0 && mlf_buffer_capacity(buf) == 4096 + image_bytes);
  uint32_t crc_file = 0;
  REQUIRE(mlf_crc32c_file(mlf_buffer_fd(buf), 4096, image_bytes, 1 << 20, &crc_file, 1, 2) == 0 && crc_file == crc_dev);

  // file -> device through the descriptor, then unpack into zeroed tensors: A whole, B through its transpose again
  REQUIRE(hipMemset(d_image, 0, image_bytes) == hipSuccess && hipMemset(d_a, 0, a_bytes) == hipSuccess &&
          hipMemset(d_b, 0, b_bytes) == hipSuccess);
  REQUIRE(mlf_engine_h2d_fd(engine, mlf_buffer_fd(buf), 4096, d_image, image_bytes, nullptr, &stats) == 0);
  mlf_plan* back = nullptr;
  mlf_plan_opts opts;
  std::memset(&opts, 0, sizeof opts);
  opts.align_to_tensor = 1;
  REQUIRE(mlf_plan_create(items.data(), items.size(), header, hdr, image_bytes, &opts, &back) == 0);
  REQUIRE(mlf_unpack_launch(back, d_image, nullptr) == 0);
  REQUIRE(hipDeviceSynchronize() == hipSuccess);
  std::vector<float> a2(a.size());
  std::vector<int16_t> b2(b.size());
  REQUIRE(hipMemcpy(a2.data(), d_a, a_bytes, hipMemcpyDeviceToHost) == hipSuccess);
  REQUIRE(hipMemcpy(b2.data(), d_b, b_bytes, hipMemcpyDeviceToHost) == hipSuccess);
  REQUIRE(std::memcmp(a2.data(), a.data(), a_bytes) == 0 && std::memcmp(b2.data(), b.data(), b_bytes) == 0);

  // ---- checksums folded into the copy: one value per 64 KiB chunk of the image, from the pack and from the unpack ----
  const uint64_t chunk = 65536, n_chunks = (image_bytes + chunk - 1) / chunk;
  std::vector<uint32_t> chunk_want(n_chunks), chunk_got(n_chunks);
  for (uint64_t k = 0; k < n_chunks; ++k)
    chunk_want[k] = mlf_crc32c_host(want.data() + k * chunk, std::min(chunk, image_bytes - k * chunk));
  mlf_plan_opts fopts;
  std::memset(&fopts, 0, sizeof fopts);
  fopts.crc_chunk_kib = 64;
  mlf_plan* fused = nullptr;
  REQUIRE(hipMemcpy(d_a, a.data(), a_bytes, hipMemcpyHostToDevice) == hipSuccess);
  REQUIRE(hipMemcpy(d_b, b.data(), b_bytes, hipMemcpyHostToDevice) == hipSuccess);
  REQUIRE(hipMemset(d_image, 0xCD, image_bytes + 256) == hipSuccess);
  REQUIRE(mlf_plan_create(items.data(), items.size(), header, hdr, image_bytes, &fopts, &fused) == 0);
  REQUIRE(mlf_plan_get_info(fused, &info) == 0 && info.crc_chunks == n_chunks && info.fused_crc_bytes >= 10 * chunk);
  REQUIRE(mlf_pack_launch(fused, d_image, nullptr) == 0);
  hipEvent_t packed = nullptr;  // what a transfer on another thread would wait for
  REQUIRE(hipEventCreateWithFlags(&packed, hipEventDisableTiming) == hipSuccess && hipEventRecord(packed, nullptr) == hipSuccess);
  REQUIRE(hipDeviceSynchronize() == hipSuccess);
  REQUIRE(mlf_plan_crc_values(fused, chunk_got.data(), n_chunks) == 0 && chunk_got == chunk_want);
  REQUIRE(hipMemcpy(got.data(), d_image, image_bytes + 256, hipMemcpyDeviceToHost) == hipSuccess);
  REQUIRE(std::memcmp(got.data(), want.data(), image_bytes) == 0 && got[image_bytes] == 0xCD);

  // the entry point that allocates nothing: values into caller-provided device memory
  uint32_t* d_vals = nullptr;
  REQUIRE(hipMalloc(reinterpret_cast<void**>(&d_vals), n_chunks * 4) == hipSuccess);
  REQUIRE(mlf_crc32c_device_noalloc(d_image, image_bytes, chunk, d_vals, n_chunks, nullptr) == 0);
  REQUIRE(hipDeviceSynchronize() == hipSuccess);
  REQUIRE(hipMemcpy(chunk_got.data(), d_vals, n_chunks * 4, hipMemcpyDeviceToHost) == hipSuccess && chunk_got == chunk_want);

  // a second buffer file, its pages and page-table entries made ahead; the transfer waits for the event, not the stream
  const std::string path2 = dir + "/cabi_direct_caller_2.distcp";
  mlf_buffer* buf2 = nullptr;
  REQUIRE(mlf_buffer_create(path2.c_str(), 4096 + image_bytes, 1, &buf2) == 0);
  REQUIRE(mlf_buffer_prefault(buf2, 4096, image_bytes, 2) == 0);
  char* dst2 = static_cast<char*>(mlf_buffer_data_ptr(buf2)) + 4096;
  landed = 0;
  std::fill(chunk_got.begin(), chunk_got.end(), 0u);
  REQUIRE(mlf_engine_d2h_gated(engine, d_image, dst2, image_bytes, packed, chunk, chunk_got.data(), n_chunks, &landed, &stats) == 0);
  REQUIRE(landed == image_bytes && chunk_got == chunk_want && std::memcmp(dst2, want.data(), image_bytes) == 0);
  // the same transfer with the checksums taken by the host threads that copy the slots: same bytes, same values
  REQUIRE(mlf_engine_set_host_checksums(engine, 1) == 0);
  std::memset(dst2, 0, image_bytes);
  std::fill(chunk_got.begin(), chunk_got.end(), 0u);
  REQUIRE(mlf_engine_d2h_gated(engine, d_image, dst2, image_bytes, packed, chunk, chunk_got.data(), n_chunks, &landed, &stats) == 0);
  REQUIRE(landed == image_bytes && chunk_got == chunk_want && std::memcmp(dst2, want.data(), image_bytes) == 0);
  REQUIRE(mlf_engine_set_host_checksums(engine, 0) == 0 && mlf_engine_set_host_checksums(nullptr, 1) != 0);
  // the image as two pieces of a data section, cut at an odd byte: the second begins inside a chunk, its first value
  // covers the bytes up to the next boundary; joined, the parts give the values of the whole
  {
    const uint64_t cut = 3 * chunk + 4099, first_part = chunk - cut % chunk;
    std::vector<uint32_t> head(n_chunks), tail(n_chunks + 1);
    std::memset(dst2, 0, image_bytes);
    REQUIRE(mlf_engine_d2h_cut(engine, d_image, dst2, cut, nullptr, packed, chunk, 0, head.data(), head.size(), nullptr, &stats) == 0);
    REQUIRE(mlf_engine_d2h_cut(engine, static_cast<char*>(d_image) + cut, dst2 + cut, image_bytes - cut, nullptr, nullptr, chunk, first_part,
                               tail.data(), tail.size(), &landed, &stats) == 0);
    REQUIRE(landed == image_bytes - cut && std::memcmp(dst2, want.data(), image_bytes) == 0);
    std::vector<uint32_t> joined(n_chunks);
    for (uint64_t k = 0; k < 3; ++k) joined[k] = head[k];
    joined[3] = mlf_crc32c_combine(head[3], tail[0], first_part);
    for (uint64_t k = 4; k < n_chunks; ++k) joined[k] = tail[k - 3];
    REQUIRE(joined == chunk_want);
    // host memory to host memory with the same cut, and a range of the file back into host memory
    std::vector<char> copy(image_bytes - cut);
    std::vector<uint32_t> tail2(n_chunks + 1);
    REQUIRE(mlf_engine_host_copy_cut(engine, copy.data(), want.data() + cut, copy.size(), chunk, first_part, tail2.data(),
                                     tail2.size()) == 0);
    REQUIRE(tail2 == tail && std::memcmp(copy.data(), want.data() + cut, copy.size()) == 0);
    std::fill(copy.begin(), copy.end(), 0);
    REQUIRE(mlf_engine_read_file(engine, mlf_buffer_fd(buf2), 4096 + cut, copy.data(), copy.size()) == 0);
    REQUIRE(std::memcmp(copy.data(), want.data() + cut, copy.size()) == 0);
    std::vector<char> longer(copy.size() + (1 << 20));  // more than the file holds: an error, not a hang
    REQUIRE(mlf_engine_read_file(engine, mlf_buffer_fd(buf2), 4096 + cut, longer.data(), longer.size()) != 0);
  }
  double seconds = 0;
  REQUIRE(mlf_engine_link_probe(engine, d_image, image_bytes, 1, &seconds) == 0 && seconds > 0);

  // unpack with checksums: the values of the image it read, the tensors as they were
  REQUIRE(hipMemset(d_a, 0, a_bytes) == hipSuccess && hipMemset(d_b, 0, b_bytes) == hipSuccess);
  fopts.align_to_tensor = 1;
  mlf_plan* fused_back = nullptr;
  REQUIRE(mlf_plan_create(items.data(), items.size(), header, hdr, image_bytes, &fopts, &fused_back) == 0);
  REQUIRE(mlf_unpack_launch(fused_back, d_image, nullptr) == 0);
  REQUIRE(hipDeviceSynchronize() == hipSuccess);
  std::fill(chunk_got.begin(), chunk_got.end(), 0u);
  REQUIRE(mlf_plan_crc_values(fused_back, chunk_got.data(), n_chunks) == 0 && chunk_got == chunk_want);
  REQUIRE(hipMemcpy(a2.data(), d_a, a_bytes, hipMemcpyDeviceToHost) == hipSuccess);
  REQUIRE(hipMemcpy(b2.data(), d_b, b_bytes, hipMemcpyDeviceToHost) == hipSuccess);
  REQUIRE(std::memcmp(a2.data(), a.data(), a_bytes) == 0 && std::memcmp(b2.data(), b.data(), b_bytes) == 0);
  mlf_plan_destroy(fused);
  mlf_plan_destroy(fused_back);
  REQUIRE(mlf_buffer_close(buf2, 1, 4096 + image_bytes) == 0);
  mlf_buffer_destroy(buf2);
  std::remove(path2.c_str());
  (void)hipFree(d_vals);
  (void)hipEventDestroy(packed);

  // a descriptor that reaches outside the image is refused with a message, nothing is launched
  items[1].image_off = image_bytes - 4;
  mlf_plan* bad = nullptr;
  REQUIRE(mlf_plan_create(items.data(), items.size(), header, hdr, image_bytes, nullptr, &bad) != 0 && bad == nullptr);
  REQUIRE(std::strstr(mlf_hip_last_error(), "does not fit in the image") != nullptr);

  mlf_plan_destroy(plan);
  mlf_plan_destroy(back);
  mlf_engine_destroy(engine);
  mlf_buffer_destroy(buf);
  std::remove(path.c_str());
  (void)hipFree(d_a), (void)hipFree(d_b), (void)hipFree(d_image);
  std::printf("direct C-ABI caller ok: %llu image bytes, crc32c %08x\n", (unsigned long long)image_bytes, crc_dev);
  return 0;
}

/*
 * CPU oracle, part 2: CRC-32C (Castagnoli) restated in plain C.  TEST INFRASTRUCTURE ONLY - nothing shipped
 * links or loads this file.
 *
 * The reference has no checksum, so there is no reference line to follow; the definition is RFC 3720 B.4 /
 * RFC 4960 appendix B: polynomial 0x1EDC6F41, reflected (0x82F63B78), initial value and final xor 0xFFFFFFFF.
 * Two independent routines are given (bit-at-a-time and byte-table); tests pin both against the RFC 3720 B.4
 * vectors and against each other, and pin oracle_crc32c_combine by brute force on short strings.
 */
#include <stddef.h>
#include <stdint.h>

#define POLY_REFLECTED 0x82F63B78u

uint32_t oracle_crc32c_bitwise(const unsigned char* p, size_t n) {
  uint32_t s = 0xFFFFFFFFu;
  for (size_t i = 0; i < n; ++i) {
    s ^= p[i];
    for (int k = 0; k < 8; ++k) s = (s & 1u) ? (s >> 1) ^ POLY_REFLECTED : s >> 1;
  }
  return s ^ 0xFFFFFFFFu;
}

static uint32_t g_table[256];
static int g_table_ready = 0;

static void build_table(void) {
  for (uint32_t v = 0; v < 256; ++v) {
    uint32_t s = v;
    for (int k = 0; k < 8; ++k) s = (s & 1u) ? (s >> 1) ^ POLY_REFLECTED : s >> 1;
    g_table[v] = s;
  }
  g_table_ready = 1;
}

uint32_t oracle_crc32c(const unsigned char* p, size_t n) {
  if (!g_table_ready) build_table();
  uint32_t s = 0xFFFFFFFFu;
  for (size_t i = 0; i < n; ++i) s = g_table[(s ^ p[i]) & 0xFFu] ^ (s >> 8);
  return s ^ 0xFFFFFFFFu;
}

/* CRC of each chunk_bytes piece of p[0..n); out must hold ceil(n/chunk_bytes) values. */
void oracle_crc32c_chunks(const unsigned char* p, size_t n, size_t chunk_bytes, uint32_t* out) {
  size_t k = 0;
  for (size_t off = 0; off < n; off += chunk_bytes, ++k) {
    size_t len = n - off < chunk_bytes ? n - off : chunk_bytes;
    out[k] = oracle_crc32c(p + off, len);
  }
}

/* crc(A||B) from crc(A), crc(B) and len(B): append len(B) zero bytes to A's register the slow way, one zero
 * bit at a time, then xor.  (The init/xorout terms cancel: crc(A||B) = shift(crc(A), 8*len(B)) ^ crc(B).) */
uint32_t oracle_crc32c_combine(uint32_t crc_a, uint32_t crc_b, uint64_t len_b) {
  uint32_t s = crc_a;
  for (uint64_t i = 0; i < 8 * len_b; ++i) s = (s & 1u) ? (s >> 1) ^ POLY_REFLECTED : s >> 1;
  return s ^ crc_b;
}

// Mode B decode on the device: canonical Huffman over weight bytes, MSB-first, blocks of `block` symbols that decode
// independently (stream layout: boilerplate/format/entropy.py:13-18; the reference's device kernel:
// boilerplate/kernels/csrc/huffman_cuda_kernel.cu:12-49, one thread of a 128-thread block per symbol block).
//
// Here one LANE walks one symbol block, so a wave decodes 64 blocks side by side and a workgroup of 256 threads 256 of
// them over one copy of the 2^maxlen-entry table in LDS ((symbol << 8) | length, indexed by the next maxlen bits).
// A lane keeps up to 64 bits of its stream in a register pair and refills 32 at a time with one dword load at the
// stream's own byte alignment (byte-swapped: the stream is big-endian by bit); decoded bytes are collected 16 at a time
// and stored with one 16-byte store (with the raw low bytes of 2-byte formats interleaved: 32 bytes), so a lane's
// stores fill whole lines in the L2 before they go to memory.
//
// Checks of the reference kernel, all kept: a code may not start at or past the block's end bit, nor within the last
// 3 bytes of the stream (a 4-byte peek must fit); a table entry of length 0, or a code that runs past the block's end
// bit, or a block that does not end exactly on its end bit, sets *error and ends the block (the output of that
// block is then undefined, as in the reference, which raises).
#include "bp_common.h"

namespace bp {
namespace {

constexpr int HUFF_THREADS = 64;  // a wave per workgroup: the blocks are few (4096 symbols each) and spread over as many CUs as they can

template <bool RAW>
__global__ __launch_bounds__(HUFF_THREADS) void k_huff_decode(uint8_t* __restrict__ out, const uint8_t* __restrict__ stream, int64_t stream_bytes,
                                                              const int64_t* __restrict__ offsets, int64_t n, int64_t block,
                                                              const int32_t* __restrict__ lut, int maxlen, const uint8_t* __restrict__ raw,
                                                              int32_t* __restrict__ error) {
  extern __shared__ int32_t table[];
  const int table_size = 1 << maxlen;
  for (int i = threadIdx.x; i < table_size; i += HUFF_THREADS) table[i] = lut[i];
  __syncthreads();
  const int64_t b = (int64_t)blockIdx.x * HUFF_THREADS + threadIdx.x;
  const int64_t first = b * block;
  if (first >= n) return;
  const int64_t end = first + (n - first < block ? n - first : block);
  const int64_t stop = offsets[b + 1];
  int64_t pos = offsets[b];
  if (pos < 0 || pos > stop) { *error = 1; return; }
  // bits [pos, pos + have) of the stream sit at the top of `buf`
  uint64_t buf = 0;
  int have = 0;
  // The lane's part of the stream travels in 16-byte pieces, requested one piece (four refills, some 30 symbols) before
  // its first word is wanted: with a few thousand blocks per tensor there are few waves per CU, and a load that a wave
  // waits for is a microsecond in which it decodes nothing. Past the stream's last byte a piece holds zeros (never
  // decoded: a code must start 4 bytes before the end).
  auto load_piece = [&](int64_t byte) -> uint4 {
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (byte + 16 <= stream_bytes) {
      __builtin_memcpy(&v, stream + byte, 16);
    } else {
      uint32_t w[4] = {0u, 0u, 0u, 0u};
      for (int64_t q = byte; q < stream_bytes; ++q) w[(q - byte) >> 2] |= (uint32_t)stream[q] << (8 * (int)((q - byte) & 3));
      v = make_uint4(w[0], w[1], w[2], w[3]);
    }
    return v;
  };
  int64_t piece_byte = pos >> 3;  // the byte `cur` starts at
  uint4 cur = load_piece(piece_byte), nxt = load_piece(piece_byte + 16);
  int words = 4;                  // words of `cur` not yet taken (the next one is cur.x)
  auto refill = [&]() {  // 32 more bits
    if (have > 32) return;
    const uint32_t w = __builtin_bswap32(cur.x);
    cur.x = cur.y;
    cur.y = cur.z;
    cur.z = cur.w;
    buf |= (uint64_t)w << (32 - have);
    have += 32;
    if (--words == 0) {
      cur = nxt;
      piece_byte += 16;
      nxt = load_piece(piece_byte + 16);
      words = 4;
    }
  };
  refill();
  {  // drop the bits of the first byte that precede pos
    const int skip = (int)(pos & 7);
    buf <<= skip;
    have -= skip;
  }
  refill();
  bool bad = false;
  int64_t i = first;
  const bool vec = RAW ? ((((uintptr_t)out + 2 * (uintptr_t)first) & 31) == 0 && ((uintptr_t)(raw + first) & 15) == 0) : ((((uintptr_t)out + (uintptr_t)first) & 15) == 0);
  while (i < end && !bad) {
    const int chunk = end - i < 16 ? (int)(end - i) : 16;
    uint32_t sy[4] = {0u, 0u, 0u, 0u};
    // one symbol into byte j of sy (the reference: pos >= end bit, or byte > stream_bytes - 4 -> invalid). After an
    // invalid code the lane decodes nothing more: it stays inside the table and the stream's pieces whatever it holds.
    auto symbol = [&](int j) {
      if (bad) return;
      if (pos >= stop || (pos >> 3) > stream_bytes - 4) { bad = true; return; }
      const int32_t e = table[(uint32_t)(buf >> (64 - maxlen))];
      const int length = e & 0xff;
      if (!length || length > stop - pos) { bad = true; return; }
      sy[j >> 2] |= (uint32_t)((e >> 8) & 0xff) << (8 * (j & 3));
      buf <<= length;
      have -= length;
      pos += length;
      refill();
    };
    if (chunk == 16) {  // (unrolled: sy stays in registers)
#pragma unroll
      for (int j = 0; j < 16; ++j) symbol(j);
    } else {
      uint32_t t4[4] = {0u, 0u, 0u, 0u};
      for (int j = 0; j < chunk; ++j) {  // the block's last symbols: one at a time into byte 0, moved to its place
        sy[0] = 0u;
        symbol(0);
        const uint32_t v = sy[0] << (8 * (j & 3));
        t4[0] |= (j >> 2) == 0 ? v : 0u;
        t4[1] |= (j >> 2) == 1 ? v : 0u;
        t4[2] |= (j >> 2) == 2 ? v : 0u;
        t4[3] |= (j >> 2) == 3 ? v : 0u;
      }
      sy[0] = t4[0]; sy[1] = t4[1]; sy[2] = t4[2]; sy[3] = t4[3];
    }
    if (bad) break;
    auto sy_word = [&](int q) { return q == 0 ? sy[0] : q == 1 ? sy[1] : q == 2 ? sy[2] : sy[3]; };  // (no indexed access: sy stays in registers)
    if (RAW) {
      if (vec && chunk == 16) {
        const uint4 r = *(const uint4*)(raw + i);
        const uint32_t rr[4] = {r.x, r.y, r.z, r.w};
        uint32_t o[8];
#pragma unroll
        for (int q = 0; q < 4; ++q) {  // bytes r0 s0 r1 s1 | r2 s2 r3 s3
          o[2 * q] = (rr[q] & 0xffu) | ((sy[q] & 0xffu) << 8) | ((rr[q] & 0xff00u) << 8) | ((sy[q] & 0xff00u) << 16);
          o[2 * q + 1] = ((rr[q] >> 16) & 0xffu) | (((sy[q] >> 16) & 0xffu) << 8) | (((rr[q] >> 24) & 0xffu) << 16) | (((sy[q] >> 24) & 0xffu) << 24);
        }
        *(uint4*)(out + 2 * i) = make_uint4(o[0], o[1], o[2], o[3]);
        *(uint4*)(out + 2 * i + 16) = make_uint4(o[4], o[5], o[6], o[7]);
      } else {
        for (int j = 0; j < chunk; ++j) {
          out[2 * (i + j)] = raw[i + j];
          out[2 * (i + j) + 1] = (uint8_t)(sy_word(j >> 2) >> (8 * (j & 3)));
        }
      }
    } else {
      if (vec && chunk == 16) *(uint4*)(out + i) = make_uint4(sy[0], sy[1], sy[2], sy[3]);
      else
        for (int j = 0; j < chunk; ++j) out[i + j] = (uint8_t)(sy_word(j >> 2) >> (8 * (j & 3)));
    }
    i += chunk;
  }
  if (bad || pos != stop) *error = 1;
}

}  // namespace
}  // namespace bp

using namespace bp;

// The checks of check_huffman_layout (boilerplate/kernels/csrc/huffman_validation.h:16-41) that need no copy of device
// memory, and - when the caller hands host copies - the ones on the offsets and the table as well.
extern "C" int bp_huff_decode(uint8_t* out, int64_t out_bytes, const uint8_t* stream, int64_t stream_bytes, const int64_t* offsets,
                              const int64_t* offsets_host, int64_t n, int64_t block, const int32_t* lut, const int32_t* lut_host,
                              int64_t maxlen, const uint8_t* raw, int64_t raw_bytes, int32_t* error, void* hstream) {
  fail(BP_OK, "%s", "");
  if (n < 0 || n > INT64_MAX / 12 || block <= 0 || maxlen <= 0 || maxlen > 12) return fail(BP_ERR_ARG, "invalid Huffman dimensions");
  if (n == 0) return BP_OK;
  if (stream_bytes < 4 || stream_bytes > INT64_MAX / 8) return fail(BP_ERR_ARG, "Huffman stream lacks padding or is too large");
  const int64_t bit_limit = (stream_bytes - 3) * 8;
  if (n > bit_limit) return fail(BP_ERR_ARG, "Huffman output exceeds the available encoded bits");
  const int64_t blocks = n / block + (n % block != 0);
  if (blocks > ((int64_t)1 << 31) - HUFF_THREADS) return fail(BP_ERR_ARG, "too many Huffman blocks");
  if (raw_bytes != 0 && raw_bytes < n) return fail(BP_ERR_ARG, "raw low-byte tensor is too small");
  if (out_bytes < n * (raw_bytes ? 2 : 1)) return fail(BP_ERR_ARG, "Huffman output buffer is too small");
  if (!out || !stream || !offsets || !lut || !error || (raw_bytes && !raw)) return fail(BP_ERR_ARG, "null pointer");
  if (offsets_host) {
    for (int64_t b = 0; b <= blocks; ++b)
      if (offsets_host[b] < 0 || offsets_host[b] > bit_limit) return fail(BP_ERR_ARG, "Huffman offset outside stream");
    for (int64_t b = 0; b < blocks; ++b) {
      const int64_t count = block < n - b * block ? block : n - b * block;
      const int64_t span = offsets_host[b + 1] - offsets_host[b];
      if (span < count || span > count * maxlen) return fail(BP_ERR_ARG, "invalid Huffman block offsets");
    }
  }
  if (lut_host) {
    for (int64_t i = 0; i < ((int64_t)1 << maxlen); ++i)
      if (lut_host[i] < 0 || lut_host[i] > 0xffff || (lut_host[i] & 255) > maxlen) return fail(BP_ERR_ARG, "invalid Huffman lookup entry");
  }
  const unsigned grid = (unsigned)((blocks + HUFF_THREADS - 1) / HUFF_THREADS);
  const size_t lds = sizeof(int32_t) << maxlen;
  if (raw_bytes) hipLaunchKernelGGL(k_huff_decode<true>, dim3(grid), dim3(HUFF_THREADS), lds, (hipStream_t)hstream, out, stream, stream_bytes, offsets, n, block, lut, (int)maxlen, raw, error);
  else hipLaunchKernelGGL(k_huff_decode<false>, dim3(grid), dim3(HUFF_THREADS), lds, (hipStream_t)hstream, out, stream, stream_bytes, offsets, n, block, lut, (int)maxlen, raw, error);
  return check_launch("huff_decode");
}

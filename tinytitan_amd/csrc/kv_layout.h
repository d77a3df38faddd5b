// KV page layout shared by host code and kernels.
//
// A page is one (layer, slot, kv_head) run of `capacity` tokens.  Tokens are
// grouped into blocks of 32; a block is 32 * D halves (16 KiB at D = 256) and
// is stored pre-swizzled so that a wavefront's MFMA operand fragment is one
// fully coalesced 16-byte-per-lane load:
//
//   K block  [d / 8][key 0..31][8 halves]      (key = position % 32)
//       v_mfma_f32_32x32x16_f16 A fragment of step s: lane (key = l % 32,
//       g = l / 32) holds d = 16 s + 8 g + j  ->  1 KiB contiguous per step.
//       v_mfma_f32_16x16x32_f16 reads the same block as 128-byte runs.
//
//   V block  [d 0..D-1][chunk 0..3][8 halves]
//       chunk c = 2 t + g holds keys {16 t + 4 g + (0..3), 16 t + 8 + 4 g + (0..3)}:
//       exactly the keys whose probabilities one lane owns after the S^T MFMA
//       (C layout: lane (n, g), register v -> key 8 (v / 4) + 4 g + v % 4), so
//       P needs no cross-lane movement between the two contractions.
//
// Quantised pages (8 or 4 bits per value, one fp16 scale and bias per token and group of 64
// consecutive dims -- the reference's row format, sources/TinyTitan/Runtime/KVCache/
// KVCacheManager+Validation.swift:30-41, regrouped per block so that the attention kernel's
// loads stay coalesced).  A block is [levels][scales and biases], 32 * D * bits / 8 + 128 * D / 64
// bytes (8704 at D = 256, 8 bits):
//
//   K levels   [d / 16][key 0..31][16 dims]: one byte per dim (8 bits), or two dims per byte, even
//              d in the low nibble (4 bits).  A lane's load is the 16 dims of one key -- 16 bytes
//              at 8 bits -- which feed two contraction steps (dims 0-7, then 8-15, of the lane's
//              unit: the contraction order over d is free as long as the query fragments follow it)
//   K params   [key 0..31][group]{scale, bias}
//   V levels   [j = d / 64][r = d % 32][chunk][h = (d / 32) % 2][8 keys]: a lane's load holds the
//              eight keys of its chunk for dims 64 j + r AND 64 j + 32 + r -- two bytes runs of 8 at
//              8 bits (16 bytes), the low and high nibbles of one run at 4 bits (8 bytes).  Two
//              keys never share a byte, so appending a token rewrites no byte of another token
//   V params   [group][chunk][8] scales, then [group][chunk][8] biases (keys in chunk order)
#pragma once
#include <stddef.h>

#if defined(__HIPCC__)
#define TT_HD __host__ __device__ __forceinline__
#else
#define TT_HD inline
#endif

namespace tt {

constexpr int kBlockTokens = 32;

// Offset in halves of K element (position, d) within its page.
TT_HD size_t k_offset(int head_dim, int position, int d) {
    const size_t block = (size_t)(position / kBlockTokens);
    const int key = position % kBlockTokens;
    return block * (size_t)(kBlockTokens * head_dim) + (size_t)(((d >> 3) * kBlockTokens + key) * 8 + (d & 7));
}

// Chunk (0..3) and lane-local index (0..7) of a key (0..31) inside a V block.
TT_HD int v_chunk_of_key(int key) { return 2 * (key >> 4) + ((key & 7) >> 2); }
TT_HD int v_index_of_key(int key) { return 4 * ((key >> 3) & 1) + (key & 3); }
// Inverse: the key stored at (chunk, index).
TT_HD int v_key_at(int chunk, int index) { return 16 * (chunk >> 1) + 8 * (index >> 2) + 4 * (chunk & 1) + (index & 3); }

// Offset in halves of V element (position, d) within its page.
TT_HD size_t v_offset(int head_dim, int position, int d) {
    const size_t block = (size_t)(position / kBlockTokens);
    const int key = position % kBlockTokens;
    return block * (size_t)(kBlockTokens * head_dim) + (size_t)((d * 4 + v_chunk_of_key(key)) * 8 + v_index_of_key(key));
}

constexpr int kQuantGroup = 64;  // KVCacheManager.quantizationGroupSize

// Bytes of the levels of one block, and of the whole block, of a K or V store.
TT_HD size_t block_level_bytes(int head_dim, int bits) { return (size_t)kBlockTokens * head_dim * bits / 8; }
TT_HD size_t block_bytes(int head_dim, int bits) {
    return bits == 16 ? (size_t)kBlockTokens * head_dim * 2
                      : block_level_bytes(head_dim, bits) + (size_t)kBlockTokens * (head_dim / kQuantGroup) * 4;
}

// Byte offset inside a quantised K block of the byte that holds dim d of `key`.
TT_HD size_t kq_level_byte(int bits, int key, int d) {
    const size_t e = (size_t)(((d >> 4) * kBlockTokens + key) * 16 + (d & 15));
    return bits == 8 ? e : e >> 1;  // 4 bits: nibble d & 1
}
// Same for V; at 4 bits the nibble is (d / 32) & 1.
TT_HD size_t vq_level_byte(int bits, int key, int d) {
    const int c = v_chunk_of_key(key), i = v_index_of_key(key);
    const int run = ((d >> 6) * 32 + (d & 31)) * 4 + c;  // (dim pair, chunk)
    if (bits == 8) return (size_t)((run * 2 + ((d >> 5) & 1)) * 8 + i);
    return (size_t)(run * 8 + i);
}
// Byte offsets of the fp16 scale and bias of (key, group) inside a block.
TT_HD size_t kq_scale_byte(int head_dim, int bits, int key, int group) {
    return block_level_bytes(head_dim, bits) + (size_t)(key * (head_dim / kQuantGroup) + group) * 4;
}
TT_HD size_t kq_bias_byte(int head_dim, int bits, int key, int group) { return kq_scale_byte(head_dim, bits, key, group) + 2; }
TT_HD size_t vq_scale_byte(int head_dim, int bits, int key, int group) {
    return block_level_bytes(head_dim, bits) + (size_t)(group * kBlockTokens + v_chunk_of_key(key) * 8 + v_index_of_key(key)) * 2;
}
TT_HD size_t vq_bias_byte(int head_dim, int bits, int key, int group) {
    return vq_scale_byte(head_dim, bits, key, group) + (size_t)(head_dim / kQuantGroup) * kBlockTokens * 2;
}

}  // namespace tt

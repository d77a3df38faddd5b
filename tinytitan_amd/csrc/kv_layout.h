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

}  // namespace tt

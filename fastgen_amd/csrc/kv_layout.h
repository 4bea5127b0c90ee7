// Where a key's and a value's elements lie inside a cache page.
//
// A page holds P tokens (P % 8 == 0) of one layer; per kv head it has P*hd
// elements of keys and P*hd of values (hd % 8 == 0).  Both are stored in
// 16-byte chunks arranged so that the matrix-core kernels read their operands
// as contiguous runs:
//
//  K: keys in blocks of KB = 16 (8 if P % 16 != 0); inside a block the chunk
//     (key r, head dims 8c..8c+7) lies at ((c * KB) + r) * 8, i.e. chunk-major:
//     the 16 keys' chunks for the same head dims are 256 contiguous bytes,
//     which is what the 16 lanes of an MFMA operand row group read.
//  V: transposed, head dims in blocks of DB = 16 (8 if hd % 16 != 0); inside a
//     block the chunk (dim r, 8 key slots) lies at ((kc * DB) + r) * 8 with kc
//     the key chunk.  If P % 32 == 0 the keys of each group of 32 are stored in
//     the slot order  slot = 8*((k%16)/4) + 4*(k/16) + k%4  (k = key % 32): the
//     8 slots of chunk g are keys 4g..4g+3 and 16+4g..16+4g+3, the keys whose
//     probabilities one lane group holds after the score MFMAs.
#pragma once

struct KvLayout {
  int page_size, hd, kb_shift, db_shift, permuted;  // KB = 1 << kb_shift, DB = 1 << db_shift
  __host__ __device__ KvLayout(int P, int head_dim)
      : page_size(P), hd(head_dim), kb_shift(P % 16 == 0 ? 4 : 3), db_shift(head_dim % 16 == 0 ? 4 : 3),
        permuted(P % 32 == 0) {}
  // element offset of (key kappa in page, head dim d) in the page's K part of one kv head
  __host__ __device__ size_t k_off(int kappa, int d) const {
    const int kb = 1 << kb_shift;
    return ((size_t)(((kappa >> kb_shift) * (hd >> 3) + (d >> 3)) << kb_shift) + (kappa & (kb - 1))) * 8 + (d & 7);
  }
  __host__ __device__ int v_slot(int kappa) const {
    if (!permuted) return kappa;
    const int k = kappa & 31;
    return kappa - k + 8 * ((k & 15) >> 2) + 4 * (k >> 4) + (k & 3);
  }
  __host__ __device__ size_t v_off(int kappa, int d) const {
    const int s = v_slot(kappa);
    return v_chunk_off(s >> 3, d) + (s & 7);
  }
  // first element of the chunk (dim d, key chunk kc)
  __host__ __device__ size_t v_chunk_off(int kc, int d) const {
    const int db = 1 << db_shift;
    return ((size_t)(((d >> db_shift) * (page_size >> 3) + kc) << db_shift) + (d & (db - 1))) * 8;
  }
  // elements between the same chunk of consecutive 32-dim steps of K / consecutive dim blocks of V
  __host__ __device__ size_t k_step32() const { return (size_t)32 << kb_shift; }
  __host__ __device__ size_t v_step_block() const { return (size_t)(page_size >> 3) << (db_shift + 3); }
};

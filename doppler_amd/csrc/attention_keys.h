// Key-range arithmetic of decode attention shared by the attention kernels (attention.hip) and by
// consumers of their split-K partial results (q4k_gemv_chain.hip): how many splits a key range gets,
// and the range itself when the key count is only known on the device.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace dh {

constexpr int kAttnTileKeys = 64;

// What the kernels need to redo the host's key-range arithmetic from a key count in device memory.
struct DynKeys {
  const uint32_t* kv_len_ptr;   // null: everything comes in as launch arguments
  int max_kv_len;               // the count is clamped to this (caches, tables and workspace are sized for it)
  int causal, start_pos;        // start_pos < 0: the query sits at the last key, kv_start + kv_len - 1
  int sliding_window, kv_start, qkv;
  int one_per_cu;               // workgroups per kv head that fill the device once
};
struct KeyRange {
  int kbeg, kend, nsplit, start_pos;
};

// Splits of the key range per kv head.  Fewer, longer workgroups beat more splits once every CU
// has one: a workgroup's next chunk costs well under 1 us, every extra split costs the merge
// kernel and the dispatch more (measured, 32/8 heads, four workgroups per CU against one:
// 3000 keys 12.9 vs 10.4 us, 6000 keys 17.1 vs 12.6, 16384 keys 24.4 vs 20.4, 32768 keys 37.1 vs
// 33.4).  One workgroup per CU, two once that would mean more than 16 chunks each.
__host__ __device__ inline int splits_for(int one_per_cu, int nkeys) {
  const int tiles = nkeys > 0 ? (nkeys + kAttnTileKeys - 1) / kAttnTileKeys : 1;
  const int wgs = tiles <= 16 * one_per_cu ? one_per_cu : 2 * one_per_cu;
  if (tiles <= wgs) return tiles;
  // every workgroup the same number of chunks (the slowest one sets the time), in as few splits
  // as that allows (the merge kernel pays per split)
  const int chunks_each = (tiles + wgs - 1) / wgs;
  return (tiles + chunks_each - 1) / chunks_each;
}
// The largest split count any key count up to max_keys can ask for: the grid of a launch whose key
// count is only known on the device.
__host__ __device__ inline int max_splits_upto(int one_per_cu, int max_keys) {
  const int tiles = max_keys > 0 ? (max_keys + kAttnTileKeys - 1) / kAttnTileKeys : 1;
  if (tiles <= one_per_cu) return tiles;
  return tiles <= 16 * one_per_cu ? one_per_cu : 2 * one_per_cu;
}
// Visible key range [kbeg, kend) relative to kv_start, split count (0: no key is visible) and the
// query's position for a key count read on the device.
__device__ inline KeyRange dyn_key_range(const DynKeys& d) {
  int kv_len = (int)*d.kv_len_ptr;
  kv_len = kv_len < 0 ? 0 : (kv_len > d.max_kv_len ? d.max_kv_len : kv_len);
  KeyRange r;
  r.start_pos = d.start_pos < 0 ? d.kv_start + kv_len - 1 : d.start_pos;
  r.kbeg = 0;
  r.kend = kv_len;
  if (!d.qkv && d.causal) r.kend = min(r.kend, r.start_pos - d.kv_start + 1);
  if (d.sliding_window > 0 && r.start_pos >= d.sliding_window) r.kbeg = max(0, r.start_pos - d.sliding_window + 1 - d.kv_start);
  r.nsplit = r.kend > r.kbeg ? splits_for(d.one_per_cu, r.kend - r.kbeg) : 0;
  return r;
}

// Workgroups per kv head that fill a device of num_cus compute units once.
inline int attn_one_per_cu(int num_cus, int Hkv) {
  const int h = Hkv > 1 ? Hkv : 1;
  return num_cus / h > 1 ? num_cus / h : 1;
}

}  // namespace dh

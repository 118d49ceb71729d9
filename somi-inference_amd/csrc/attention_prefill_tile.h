// The prefill attention kernel on 32 x 32 x 16 matrix tiles (attention_prefill_tile.hip), as somi_attention_prefill
// calls it.  Internal to the library: no extern "C" entry of its own.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define SOMI_PREFILL_TILE_LDS_MAX (112 * 1024)   // dynamic LDS a workgroup of the kernel may ask for (launches with 106 KB are tested)

// Dynamic LDS of a launch with qblk query blocks and ks key splits a workgroup.
int somi_prefill_tile_lds(int D, int qblk, int ks, int max_blocks, int page_size, int window);
// Whether the kernel takes these sizes: head size 64 or 128, pages of 8 keys or more (a power of two), and a block
// table whose visible part fits LDS.
bool somi_prefill_tile_applies(int D, int page_size, int max_blocks, int window);
// Arguments as somi_attention_prefill's.  wide: 256 queries a workgroup, else 128 queries and two key splits.
int somi_prefill_tile(const void* q, int64_t q_stride, const void* kc, const void* vc, const int* block_table,
                      int max_blocks, const int* entry_start, const int* entry_first_pos, const int* entry_len,
                      int n_entries, int max_entry_len, bool wide, int nq, int nkv, int D, int page_size, int window,
                      float scale, void* out, hipStream_t stream);

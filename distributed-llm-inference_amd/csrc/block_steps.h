// A step's layers issued from C: what the caller fills in. The layouts are mirrored field by field
// in dli_amd/parts/native.py (ctypes); change both together.
#pragma once
#include <stdint.h>

#define DLI_MAX_GROUPS 4   // cache groups whose slots and block tables a step may carry
#define DLI_MAX_SHAPES 4   // distinct attention shapes (head size, heads, kv heads) in one model

// What depends on the step's batch and an attention shape: the query tiles of the portions (for
// this shape's tile height), which of them have their keys cut into runs (tile_cut null: none;
// see dli_attention_prefill_bf16) with the memory for that, and the key splits of the
// single-token rows.
struct DliStepShape {
  const int32_t* tile_entry;
  const int32_t* tile_q0;
  int32_t tiles;
  int32_t decode_splits;
  const int32_t* tile_cut;
  float* cut_buf;
  uint32_t* cut_count;
  int32_t cut_tiles;
  int32_t cut_room;   // the most runs of any cut tile
};

// One step: the batch's arrays on the device (as the step context holds them) and the scratch
// buffers that every layer reuses (bfloat16 unless said otherwise; each at least as large as the
// widest layer needs for `rows` rows).
struct DliStepArgs {
  int32_t rows, num_decode, num_entries, page_size, device, pad0;
  const int32_t* positions;
  const int32_t* q_start;
  const int32_t* kv_len;
  const int32_t* slots[DLI_MAX_GROUPS];
  const int32_t* block_tables[DLI_MAX_GROUPS];
  int32_t table_stride[DLI_MAX_GROUPS];
  struct DliStepShape shapes[DLI_MAX_SHAPES];
  float* part_o;    // float32, for the largest requests * heads * splits * head_dim of the shapes
  float* part_ml;   // float32, requests * heads * splits * 2
  void* normed;     // [rows, hidden]
  void* qkv;        // [rows, (heads + 2 kv_heads) * head_dim]
  void* attn;       // [rows, heads * head_dim]
  void* mixed;      // [rows, hidden]
  void* gate_up;    // [rows, 2 * intermediate]
  void* act;        // [rows, intermediate]
  void* ffn_out;    // [rows, hidden]: the last block's feed-forward output, not yet added to x
  void* gemm_workspace;
  int64_t gemm_workspace_bytes;
};

// One pre-norm block (RMSNorm, grouped-query attention with rotary positions over paged keys and
// values, RMSNorm, gated feed-forward) with the cache of the schedule entry that runs it.
struct DliBlockArgs {
  const float* norm1_w;
  const float* norm2_w;
  const void* w_qkv;      // [(heads + 2 kv_heads) * head_dim, hidden]
  const void* b_qkv;      // or null
  const void* w_o;        // [hidden, heads * head_dim]
  const void* b_o;
  const void* w_gate_up;  // [2 * intermediate, hidden], gate rows then up rows
  const void* b_gate_up;
  const void* w_down;     // [hidden, intermediate]
  const void* b_down;
  const float* inv_freq;  // [rotary_dim / 2]
  void* k_pages;
  void* v_pages;
  float eps1, eps2, scale;
  int32_t rotary_dim, hidden, q_heads, kv_heads, head_dim, intermediate, window, group, shape;
  int32_t kind;  // which arrangement of which parts this describes: DLI_BLOCK_PRENORM_RMS_GQA_SILU, the only one
};

// kind: x += attention(rms(x)) with rotary pairs (i, i + dim/2); x += down(silu(gate(rms(x))) * up(rms(x)))
#define DLI_BLOCK_PRENORM_RMS_GQA_SILU 1

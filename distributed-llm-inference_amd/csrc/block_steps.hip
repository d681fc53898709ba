// The layers of a step that holds portions of prompts, issued from one call.
//
// Such a step is launched kernel by kernel (only decode-only steps replay graphs): eleven launches
// a layer. Issued one by one from Python, with the checks and temporaries of each, they cost more
// host time than the GPU needs for a step of a few hundred tokens. This entry point issues the
// same launches, in the same order and with the same arguments, from a loop in C: the caller
// passes the step's arrays and scratch buffers once and an array with one entry per block.
//
// A block here is the pre-norm arrangement of src/dli/model/llama.py:194-213 in bfloat16:
//   x += delta (the previous block's feed-forward output); h = norm1(x)
//   q, k, v = h Wqkv^T (+ b); rotate q, k; write k, v at the tokens' cache slots
//   a = attention over the pages (single-token rows: split-key decode kernel; portions: tiles)
//   x += a Wo^T (+ b); h = norm2(x);  delta = down(silu(gate(h)) * up(h))
// Host code only: every kernel is the one its own entry point launches.
#include "block_steps.h"

#include "common.h"

extern "C" {
int dli_rms_norm(const void* x, const void* delta, const float* weight, void* sum_out, void* out, int rows,
                 int width, float eps, int is_bf16, hipStream_t stream);
int dli_silu_mul(const void* gu, void* out, int rows, int inter, int is_bf16, hipStream_t stream);
int dli_gemm_bf16(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, void* out, int64_t ldo,
                  int64_t rows, int64_t feats, int64_t k, void* workspace, int64_t workspace_bytes, int device,
                  hipStream_t stream);
int dli_gemm_bf16_usable(int64_t rows, int64_t feats, int64_t k, int64_t ldx, int64_t ldw, int64_t ldo, int bias,
                         int64_t workspace_bytes, int device);
int dli_rope_kv_write(void* qkv, int64_t row_stride, const int* positions, const float* inv_freq, int rotary_dim,
                      const int* slots, void* k_pages, void* v_pages, int tokens, int q_heads, int kv_heads,
                      int head_dim, int page_size, int is_bf16, hipStream_t stream);
int dli_attention_mfma_supports(int head_dim, int page_size);
int dli_attention_decode_bf16(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages, void* out,
                              int64_t out_stride, float* part_o, float* part_ml, const int* kv_len,
                              const int* block_tables, int table_stride, int requests, int q_heads, int kv_heads,
                              int head_dim, int page_size, float scale, int window, int splits, hipStream_t stream);
int dli_attention_prefill_bf16(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages, void* out,
                               int64_t out_stride, const int* q_start, const int* kv_len, const int* block_tables,
                               int table_stride, const int* tile_entry, const int* tile_q0, int tiles, int q_heads,
                               int kv_heads, int head_dim, int page_size, float scale, int window, const int* tile_cut,
                               int cut_tiles, int cut_room, float* cut_buf, unsigned* cut_count, hipStream_t stream);
}

namespace {

bool block_is_sane(const DliBlockArgs& b, const DliStepArgs& s) {
  if (b.kind != DLI_BLOCK_PRENORM_RMS_GQA_SILU) return false;  // the loop below computes this arrangement only
  if (b.norm1_w == nullptr || b.norm2_w == nullptr || b.w_qkv == nullptr || b.w_o == nullptr ||
      b.w_gate_up == nullptr || b.w_down == nullptr || b.inv_freq == nullptr || b.k_pages == nullptr ||
      b.v_pages == nullptr)
    return false;
  if (b.hidden <= 0 || b.q_heads <= 0 || b.kv_heads <= 0 || b.head_dim <= 0 || b.intermediate <= 0 ||
      b.q_heads % b.kv_heads != 0 || b.rotary_dim <= 0 || b.rotary_dim > b.head_dim || b.window < 0)
    return false;
  if (b.group < 0 || b.group >= DLI_MAX_GROUPS || b.shape < 0 || b.shape >= DLI_MAX_SHAPES) return false;
  if (s.slots[b.group] == nullptr || s.block_tables[b.group] == nullptr || s.table_stride[b.group] <= 0) return false;
  const DliStepShape& sh = s.shapes[b.shape];
  if (s.num_entries > s.num_decode && (sh.tiles <= 0 || sh.tile_entry == nullptr || sh.tile_q0 == nullptr)) return false;
  if (sh.tile_cut != nullptr && (b.window > 0 || sh.cut_tiles <= 0 || sh.cut_room < 2 || sh.cut_buf == nullptr || sh.cut_count == nullptr))
    return false;
  if (s.num_decode > 0 && (sh.decode_splits < 1 || (sh.decode_splits > 1 && (s.part_o == nullptr || s.part_ml == nullptr))))
    return false;
  return dli_attention_mfma_supports(b.head_dim, s.page_size) != 0;
}

}  // namespace

// x: bfloat16 [rows, hidden] (contiguous rows), the residual stream after the embedding; on return
// it holds every residual sum but the last block's feed-forward output, which lies in
// step->ffn_out (the caller's final norm adds it). Returns DLI_ERR_ARGUMENT, with nothing
// launched, if an argument does not fit or the vendor library has no kernel for one of the
// products at this number of rows (the caller then runs the step part by part).
extern "C" int dli_prenorm_blocks_bf16(void* x, const DliBlockArgs* blocks, int n_blocks, const DliStepArgs* step,
                                       hipStream_t stream) {
  if (n_blocks <= 0 || step == nullptr || step->rows <= 0) return DLI_OK;
  const DliStepArgs& s = *step;
  if (x == nullptr || blocks == nullptr || s.positions == nullptr || s.q_start == nullptr || s.kv_len == nullptr ||
      s.normed == nullptr || s.qkv == nullptr || s.attn == nullptr || s.mixed == nullptr || s.gate_up == nullptr ||
      s.act == nullptr || s.ffn_out == nullptr || s.num_decode < 0 || s.num_entries < s.num_decode ||
      s.num_decode > s.rows || s.page_size <= 0 || s.gemm_workspace_bytes < 0)
    return DLI_ERR_ARGUMENT;
  for (int i = 0; i < n_blocks; ++i) {
    const DliBlockArgs& b = blocks[i];
    if (!block_is_sane(b, s)) return DLI_ERR_ARGUMENT;
    const int64_t h = b.hidden, qkv_w = (int64_t)(b.q_heads + 2 * b.kv_heads) * b.head_dim,
                  q_w = (int64_t)b.q_heads * b.head_dim, inter = b.intermediate;
    const int64_t ws = s.gemm_workspace_bytes;
    if (!dli_gemm_bf16_usable(s.rows, qkv_w, h, h, h, qkv_w, b.b_qkv != nullptr, ws, s.device) ||
        !dli_gemm_bf16_usable(s.rows, h, q_w, q_w, q_w, h, b.b_o != nullptr, ws, s.device) ||
        !dli_gemm_bf16_usable(s.rows, 2 * inter, h, h, h, 2 * inter, b.b_gate_up != nullptr, ws, s.device) ||
        !dli_gemm_bf16_usable(s.rows, h, inter, inter, inter, h, b.b_down != nullptr, ws, s.device))
      return DLI_ERR_ARGUMENT;
  }
#define STEP(call)                       \
  do {                                   \
    const int status_ = (call);          \
    if (status_ != DLI_OK) return status_ == DLI_ERR_ARGUMENT ? DLI_ERR_LAUNCH : status_; \
  } while (0)
  const void* delta = nullptr;
  for (int i = 0; i < n_blocks; ++i) {
    const DliBlockArgs& b = blocks[i];
    const DliStepShape& sh = s.shapes[b.shape];
    const int64_t h = b.hidden, qkv_w = (int64_t)(b.q_heads + 2 * b.kv_heads) * b.head_dim,
                  q_w = (int64_t)b.q_heads * b.head_dim, inter = b.intermediate;
    STEP(dli_rms_norm(x, delta, b.norm1_w, delta != nullptr ? x : nullptr, s.normed, s.rows, b.hidden, b.eps1, 1, stream));
    STEP(dli_gemm_bf16(s.normed, h, b.w_qkv, h, b.b_qkv, s.qkv, qkv_w, s.rows, qkv_w, h, s.gemm_workspace,
                       s.gemm_workspace_bytes, s.device, stream));
    STEP(dli_rope_kv_write(s.qkv, qkv_w, s.positions, b.inv_freq, b.rotary_dim, s.slots[b.group], b.k_pages, b.v_pages,
                           s.rows, b.q_heads, b.kv_heads, b.head_dim, s.page_size, 1, stream));
    if (s.num_decode > 0)
      STEP(dli_attention_decode_bf16(s.qkv, qkv_w, b.k_pages, b.v_pages, s.attn, q_w, s.part_o, s.part_ml, s.kv_len,
                                     s.block_tables[b.group], s.table_stride[b.group], s.num_decode, b.q_heads,
                                     b.kv_heads, b.head_dim, s.page_size, b.scale, b.window, sh.decode_splits, stream));
    if (s.num_entries > s.num_decode)
      STEP(dli_attention_prefill_bf16(s.qkv, qkv_w, b.k_pages, b.v_pages, s.attn, q_w, s.q_start, s.kv_len,
                                      s.block_tables[b.group], s.table_stride[b.group], sh.tile_entry, sh.tile_q0,
                                      sh.tiles, b.q_heads, b.kv_heads, b.head_dim, s.page_size, b.scale, b.window,
                                      sh.tile_cut, sh.cut_tiles, sh.cut_room, sh.cut_buf, sh.cut_count, stream));
    STEP(dli_gemm_bf16(s.attn, q_w, b.w_o, q_w, b.b_o, s.mixed, h, s.rows, h, q_w, s.gemm_workspace,
                       s.gemm_workspace_bytes, s.device, stream));
    STEP(dli_rms_norm(x, s.mixed, b.norm2_w, x, s.normed, s.rows, b.hidden, b.eps2, 1, stream));
    STEP(dli_gemm_bf16(s.normed, h, b.w_gate_up, h, b.b_gate_up, s.gate_up, 2 * inter, s.rows, 2 * inter, h,
                       s.gemm_workspace, s.gemm_workspace_bytes, s.device, stream));
    STEP(dli_silu_mul(s.gate_up, s.act, s.rows, b.intermediate, 1, stream));
    STEP(dli_gemm_bf16(s.act, inter, b.w_down, inter, b.b_down, s.ffn_out, h, s.rows, h, inter, s.gemm_workspace,
                       s.gemm_workspace_bytes, s.device, stream));
    delta = s.ffn_out;
  }
#undef STEP
  return DLI_OK;
}

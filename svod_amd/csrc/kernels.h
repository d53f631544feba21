// Launchers of the gfx950 kernels; the op layer (ops.cpp) is their only caller.
#pragma once
#include <hip/hip_runtime_api.h>
#include <stdint.h>

namespace svodk {

// The prologue: tk/src/kernels/heads.rs:40-125 (heads_body).
struct HeadsArgs {
  const void *qkv;  // [rows, (heads + 2*kv_heads) * d] bf16
  const void *q_w;  // [d] or null
  const void *k_w;  // [d] or null
  const void *cos;  // [t | rows, d/2] or null
  const void *sin;
  void *q;  // [rows, heads, d]
  void *k;  // [rows, kv_heads, d]
  void *v;
  int64_t rows;  // live batches * t
  int32_t t, heads, kv_heads, d;
  float eps;
  int32_t rope;  // 0 none, 1 tables by position [t, d/2], 2 by token [rows, d/2]
  int32_t f16;   // every 16-bit operand is f16, not bf16
};
hipError_t launch_heads(const HeadsArgs &a, hipStream_t stream);
// Head sizes the prologue kernel is built for.
bool heads_supports(int32_t d);

// Row norms: tk/src/kernels/rows.rs:41-115 (norm_body).
struct NormArgs {
  const void *x;         // [rows, d]
  const void *residual;  // [rows, d] or null: normalize x + residual, the sum written to `sum`
  const void *w;         // [d]
  const void *b;         // [d] or null (LayerNorm only)
  void *out;             // [rows, d]
  void *sum;             // [rows, d] with a residual
  int64_t rows;          // live rows
  int32_t d;
  double eps;
  int32_t layer;  // LayerNorm (1) or RMSNorm (0)
  int32_t f16;    // every operand is f16, not bf16
};
hipError_t launch_norm(const NormArgs &a, hipStream_t stream);
// Row widths the norm kernel is built for.
bool norm_supports(int64_t d);

// linear with the rope epilogue: tk/src/kernels/gemm.rs (gemm_body, finish :604-645, turn :666-716).
struct LinearArgs {
  const void *x;     // [rows, k]
  const void *w;     // [n, k]
  const void *bias;  // [n] or null
  const void *cos;   // [seq, head_dim / 2] or null: no turn
  const void *sin;
  void *y;           // [rows, n], or the window's first element in a wider output
  int64_t y_ld;      // elements from an output row to the next: n, or the wider output's channels
  int64_t rows;      // live batches * seq
  int32_t n, k;
  int32_t seq;       // row r is the token at position r % seq
  int32_t heads, head_dim;  // the first heads * head_dim columns are turned
  int32_t f16;
  int32_t tile;      // the workgroup's output tile: 256 (8 waves) or 128 (4 waves), linear_tile_of's answer
};
hipError_t launch_linear(const LinearArgs &a, hipStream_t stream);
// Shapes the GEMM kernel takes (n a multiple of 8, k a multiple of 32), and head sizes it turns.
bool linear_supports(int64_t n, int64_t k);
bool linear_turns(int32_t head_dim);
// The output tile of a call: 128 where 256 x 256 tiles would be fewer than half the compute units `units`, unless
// linear_tile() has named one for every call (0: by the shape again).  linear_tile returns the setting.
int linear_tile_of(int64_t rows, int64_t n, int units);
int linear_tile(int32_t tile);

// Flash attention forward: tk/src/kernels/attention.rs:466-924 (attention_body).
struct AttnArgs {
  const void *q;  // [batch, t, heads, d] bf16
  const void *k;  // [batch, tk, kv_heads, d]
  const void *v;
  void *o;               // [batch, t, heads, d]
  const void *key_lens;  // [batch] i32/i64 or null
  const void *key_mask;  // [batch, tk] u8/i32 or null
  int32_t lens_i64;      // key_lens holds 64-bit integers
  // [batch] i32 or null: place p of the launch works on batch row row_order[p] (a permutation;
  // out-of-range entries are clamped).  Results do not depend on it; the order of work does.
  const void *row_order;
  int32_t mask_bytes;    // element size of key_mask: 1 or 4
  int32_t batch;         // live batches
  int32_t t, tk, heads, kv_heads, d;
  int32_t causal;
  float scale;
  int32_t f16;  // the operands are f16, not bf16
  // Key splits (FaCfg::splits, tk/src/kernels/attention.rs:19-21, 487-492): with splits > 1 each
  // split writes its partial state instead of `o`: o_part [splits, batch, t, heads, d],
  // m_part and l_part [splits, batch, t, heads], all f32; launch_combine merges them.
  int32_t splits;
  float *o_part, *m_part, *l_part;
  // Elements from a token's row to the next in q and in k/v; 0 = dense (heads * d, kv_heads * d).
  // A fused projection read in place (tk/src/ops/attention.rs:104-122) has its own row for both.
  int64_t q_row_elems, kv_row_elems;
  // Attn::window (tk/src/ops/attention.rs:64-65): query i sees keys [i - win_left, i + win_right];
  // win_left < 0 = no window.
  int32_t win_left, win_right;
  // Attn::chunk (tk/src/ops/attention.rs:39-50, 66-68): query i sees the keys of chunk i / chunk_size,
  // of the chunk_left chunks before it (< 0 = every earlier one) and the chunk_right after.
  // chunk_size 0 = no chunk mask.
  int32_t chunk_size, chunk_left, chunk_right;
  // Attn::seg_start (tk/src/ops/attention.rs:69-71): [batch, t] i32 or i64 segment starts,
  // non-decreasing along t; query i does not see keys before seg_start[b, i].  Null = none.
  const void *seg_start;
  int32_t seg_i64;
  // Attn::bias (tk/src/ops/attention.rs:82-85): [batch or 1, heads, t, tk] of the operands' type,
  // rows unpadded, added to the scaled scores before the masks.  Null = none.
  const void *bias;
  int32_t bias_per_batch;
  // Cache (tk/src/ops/attention.rs:39-56).  kv_head_start: the first of this attention's kv_heads
  // in a cache row of kv_row_elems / d heads.  row_map: [batch] i32 or i64 cache row per batch
  // lane, null = row b.  k_app / v_app: [batch, app_rows, kv_heads, d] scored after the tk cached
  // keys, the first app_lens[b] of them visible (all without app_lens); app_rows <= 64.
  int32_t cached;
  int32_t kv_head_start;
  const void *row_map;
  int32_t row_map_i64;
  int32_t cache_rows;  // k's leading dim: mapped rows are clamped into it
  const void *k_app, *v_app;
  int32_t app_rows;
  const void *app_lens;
  int32_t app_lens_i64;
};
hipError_t launch_attention(const AttnArgs &a, hipStream_t stream);

// combine_splits: tk/src/kernels/attention.rs:948-1014.
struct CombineArgs {
  const float *o_part, *m_part, *l_part;
  void *o;       // [rows, d] bf16 or f16
  int64_t rows;  // batch * t * heads
  int32_t d, splits;
  int32_t f16;
};
hipError_t launch_combine(const CombineArgs &a, hipStream_t stream);
// The library's own device memory for the partial states of a split call that brings no workspace:
// a file-scope array of kSplitScratchBytes per GPU.  `*ptr` is the current device's copy (its
// address is looked up on the first call on that device), `*bytes` its size.  Allocates nothing.
constexpr int64_t kSplitScratchBytes = 8ll << 20;
hipError_t split_scratch(void **ptr, int64_t *bytes);
bool attention_supports(int32_t d);
// Whether launch_attention runs `a` on grouped tiles: the heads of a KV head's group side by side
// in one query tile (a decoder step under GQA: no causal or per-row mask, group * t <= 128).
bool attention_groups(const AttnArgs &a);
// The decoder step's kernel (decode_kernel.hip): a call without causal or per-row masks or a bias whose (batch,
// KV head) has at most kDecodeRows query rows (group * t) streams K and V past them in registers instead of
// running key tiles through LDS.  launch_attention takes that path by itself; splits, caches, appended rows, key
// lengths and key masks mean what they mean to the tile kernel.
constexpr int kDecodeRows = 4;         // the most the kernel is built for
constexpr int kDecodeRowsDefault = 2;  // the most it takes unasked: up to there it has beaten the tile kernel where measured
bool attention_decodes(const AttnArgs &a);
// The most rows that path takes, 0..kDecodeRows (0: every call runs key tiles): see svodk_tune_decode.
void attention_decode_rows(int32_t rows);
int32_t attention_decode_limit();
hipError_t launch_decode(const AttnArgs &a, hipStream_t stream);
// One head size's kernels each (launch_attention picks by AttnArgs::d).
hipError_t launch_attention_d32(const AttnArgs &a, hipStream_t stream);
hipError_t launch_attention_d48(const AttnArgs &a, hipStream_t stream);
hipError_t launch_attention_d64(const AttnArgs &a, hipStream_t stream);
hipError_t launch_attention_d128(const AttnArgs &a, hipStream_t stream);
hipError_t launch_attention_d256(const AttnArgs &a, hipStream_t stream);
// order[p] = the batch row with the p-th most keys (ties by row), for AttnArgs::row_order.  `keys` is
// [n] lengths (tk < 0; elements of 4 or 8 bytes) or an [n, tk] key mask (elements of 1 or 4 bytes).
constexpr int32_t kMaxOrderedRows = 8192;
hipError_t launch_order_rows(const void *keys, int32_t elem_bytes, int32_t n, int32_t tk, int32_t *order,
                             hipStream_t stream);
// Tuning of the streaming form (workgroups that walk runs of query tiles): see svodk_tune_streaming.
void attention_stream_slots(int32_t slots);
// The set of shared counters the next streaming launch takes (and takes it): the sets in turn.
uint32_t next_queue_set();
// Text of the tile configuration launch_attention picks for `a` (for chosen()).
const char *attention_config(const AttnArgs &a);

}  // namespace svodk

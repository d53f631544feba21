/*
 * svodk — C ABI of the MI355X (gfx950) implementation of Svod's `tk`
 * flash-attention forward op and of the attention prologue ("heads").
 *
 * Every entry point replaces one item of the reference's op layer; the
 * citation beside it is into the reference checkout.  The library follows the
 * op layer's contract: an op either launches a kernel, or says that the
 * caller's graph must run and why, or rejects arguments the graph would
 * reject too (tk/src/ops/mod.rs:1-4).  It computes nothing on the host and
 * allocates no device memory: the caller owns every buffer.
 *
 * All pointers in tensor descriptors are DEVICE pointers (dense, row-major,
 * in the layouts the reference op takes), 16-byte aligned for the 16-bit tensors
 * and the workspace (the kernels move them in 128-bit pieces) and aligned to
 * their element for integers and masks; an address off that answers
 * SVODK_ERR_ARGUMENT.  Launches are enqueued on the HIP
 * stream given and return without synchronising.
 */
#ifndef SVODK_H
#define SVODK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SVODK_ABI_VERSION 8

/* Element types of a tensor descriptor. */
typedef enum svodk_dtype {
  SVODK_BF16 = 0,
  SVODK_F16 = 1,
  SVODK_F32 = 2,
  SVODK_I32 = 3,
  SVODK_I64 = 4,
  SVODK_BOOL = 5 /* one byte per element, nonzero = true */
} svodk_dtype;

/*
 * What an op call did.  Mirrors the three outcomes of the reference op layer:
 *   0   a kernel was enqueued             (Plan::Kernel, tk/src/ops/shape.rs:19-24)
 *   > 0 the caller's graph must run, why  (Plan::Graph(Fallback), shape.rs:26-39)
 *   < 0 the arguments are invalid         (ops::Error, tk/src/ops/mod.rs:132-157)
 */
typedef enum svodk_status {
  SVODK_KERNEL = 0,
  SVODK_GRAPH_TARGET = 1,   /* Fallback::Target: no gfx950 device / no kernels for it */
  SVODK_GRAPH_DTYPE = 2,    /* Fallback::Dtype: f32, or a type without a kernel here */
  SVODK_GRAPH_SYMBOLIC = 3, /* Fallback::Symbolic: a live batch that is not a leading bound */
  SVODK_GRAPH_SHAPE = 4,    /* Fallback::Shape: a shape the kernels do not cover */
  SVODK_GRAPH_CONFIG = 5,   /* Fallback::Config: an option no kernel config here holds */
  SVODK_ERR_SHAPE = -1,     /* Error::Shape */
  SVODK_ERR_DTYPE = -2,     /* Error::Dtype */
  SVODK_ERR_HEADS = -3,     /* Error::Heads */
  SVODK_ERR_LAUNCH = -4,    /* Error::Launch: aliased parameters, a HIP error */
  SVODK_ERR_ARGUMENT = -5   /* a null or malformed descriptor (no reference counterpart:
                               Rust's type system rules these out) */
} svodk_status;

/* A dense row-major device tensor.  `rank` <= 4; unused dims are ignored. */
typedef struct svodk_tensor {
  void *data;
  int32_t dtype; /* svodk_dtype */
  int32_t rank;
  int64_t shape[4];
} svodk_tensor;

/* KeyMask of tk/src/ops/attention.rs:29-37. */
typedef enum svodk_key_mask {
  SVODK_KEYS_NONE = 0,
  SVODK_KEYS_LENS = 1, /* [B] integer valid-key counts (I32 or I64) */
  SVODK_KEYS_BOOL = 2  /* [B, Tk] BOOL or integer, nonzero = attended; rows are NOT padded */
} svodk_key_mask;

/*
 * Cache of tk/src/ops/attention.rs:39-56: k and v are caches [rows, Tk, H_all, D]
 * holding several layers' heads (a decoder step's self or cross attention).
 * Query head h reads cache head head_start + h / (H / kv_heads) of cache row
 * row_map[b] (row b without a map).  `k_app`/`v_app` [B, n, kv_heads, D] are keys
 * and values scored after the cached prefix (the tokens the step projected, not
 * yet written to the cache): they need SVODK_KEYS_LENS naming the prefix, n is
 * at most a key block (64) and only the first app_lens[b] of them are seen
 * (all without app_lens).  Masks other than the key lengths do not reach them.
 */
typedef struct svodk_cache {
  int64_t head_start, kv_heads;
  const svodk_tensor *row_map;  /* [B] I32 or I64, or NULL */
  const svodk_tensor *k_app;    /* both or neither */
  const svodk_tensor *v_app;
  const svodk_tensor *app_lens; /* [B] I32 or I64, or NULL; needs k_app */
} svodk_cache;

/*
 * Attn of tk/src/ops/attention.rs:60-86.  Zero-initialise, then set fields.
 * Windows, chunk masks, segment starts (I32 or I64, non-decreasing along T)
 * an additive bias (of the operands' type, rows unpadded; with appended rows
 * its last dim counts them, their columns last) and a cache have kernels.
 * Every combination runs, a cache under a window, a chunk mask or segment starts
 * included (the ranges hide cached keys only; appended rows answer to app_lens alone);
 * more than 64 appended rows answer SVODK_GRAPH_CONFIG.
 *
 * `splits` > 1 asks for key splits (tk/src/ops/attention.rs:76-79, 280-302): the
 * count is capped at the number of 64-key blocks of Tk (split_ranked, :405-410);
 * each split leaves a partial state in `workspace` and combine_splits
 * (tk/src/kernels/attention.rs:984-1014) merges them into `out`.  The reference
 * op allocates those partial tensors itself; this library allocates nothing,
 * so the caller lends `workspace` (svodk_attention_workspace says how many
 * bytes).  A named count without a large enough workspace answers
 * SVODK_GRAPH_CONFIG.  `splits` = 1 keeps the keys whole.  `splits` = 0 (None)
 * lets the library choose, as the reference's tuner would: it splits calls with
 * few query tiles and many keys (a decoder step) when the workspace
 * svodk_attention_workspace asks for is lent, and keeps the keys whole without it.
 */
typedef struct svodk_attn {
  int32_t causal;
  int32_t key_kind; /* svodk_key_mask */
  const svodk_tensor *keys;
  int32_t has_window;
  int64_t window_left, window_right;
  int32_t has_chunk;
  int64_t chunk_size;
  int32_t chunk_has_left;
  int64_t chunk_left, chunk_right;
  const svodk_tensor *seg_start; /* [B, T] integers or NULL */
  const svodk_cache *cache;      /* or NULL */
  const svodk_tensor *bias;      /* [B|1, H, T, Tk] or NULL */
  int32_t splits;                /* 0 = None: the library chooses */
  int32_t has_scale;
  float scale; /* used when has_scale; else 1/sqrt(D) */
  /* Batch::Var of tk/src/kernels/mod.rs:221-259: buffers hold `q.shape[0]`
   * batches, only the first `batch_live` are computed and written.
   * <= 0 means all of them. */
  int32_t batch_live;
  void *workspace; /* device scratch for key splits, or NULL */
  int64_t workspace_bytes;
  /* [B] I32 or NULL, no counterpart in the reference's Attn: the order in which the launch takes
   * the batch rows (place p works on row row_order[p]).  It must be a permutation of 0..B-1: its
   * contents are device data that no host check reads, so an order that names a row twice computes
   * that row twice and leaves the rows it skips UNWRITTEN (entries out of range are clamped into the
   * batch, never followed out of the tensors).  With a permutation results do not depend on it.
   * svodk_order_rows fills one from the key lengths (always a permutation); a model computes it once
   * per batch and passes it to every layer's call.  Under a bound batch (0 < batch_live < B) the
   * order is IGNORED and the rows run as they come: an order of all B rows would name rows past the
   * live ones. */
  const svodk_tensor *row_order;
} svodk_attn;

/* Qkv of tk/src/ops/heads.rs:19-31. */
typedef struct svodk_qkv {
  int32_t heads, kv_heads, head_dim;
  const svodk_tensor *q_norm; /* [head_dim] or NULL */
  const svodk_tensor *k_norm; /* [head_dim] or NULL */
  double eps;
  const svodk_tensor *cos; /* [1|B, T, 1, head_dim/2] or NULL (both or neither) */
  const svodk_tensor *sin;
  int32_t batch_live; /* as in svodk_attn */
} svodk_qkv;

/*
 * ops::attention (tk/src/ops/attention.rs:100-103 -> attend, :126-303).
 * q [B,T,H,D], k and v [B,Tk,Hkv,D], out [B,T,H,D], all of one 16-bit type.
 * Query head h reads KV head h / (H / Hkv).  A query no key reaches comes out
 * as zeros (tk/src/kernels/attention.rs:974-980).
 */
int svodk_attention(const svodk_tensor *q, const svodk_tensor *k, const svodk_tensor *v, const svodk_attn *opts,
                    const svodk_tensor *out, void *hip_stream);

/*
 * svodk_attention for callers that cannot allocate device memory (code under HIP graph capture, a
 * serving loop with a fixed memory plan, a harness that forbids hipMalloc).  It has no counterpart
 * in the reference, whose op allocates the partial tensors of a split call itself
 * (tk/src/ops/attention.rs:285-293).  Same operands, options, checks, kernels and results as
 * svodk_attention; the one difference is where the partial states of a split call live: in a
 * static device array of the library, svodk_noalloc_scratch_bytes() (8 MiB) on each GPU the library
 * runs on, held until the process ends.  `opts->workspace` is ignored.  The call and everything
 * under it allocate nothing.  With `splits` = 0 the count is chosen as if a workspace had been lent
 * and then lowered to what the array holds (down to one split: the call runs unsplit, as
 * svodk_attention runs it without a workspace).  A call whose NAMED splits need more than the array
 * holds answers SVODK_ERR_ARGUMENT and launches nothing; svodk_attention_workspace says how much a
 * call needs.  Every call on a GPU shares that GPU's
 * array: calls that overlap on one GPU (two streams, two threads) race on it and must be ordered
 * by the caller.  Nothing in the array has to start at zero (a split call writes every partial
 * state its merge reads).
 */
int svodk_attention_noalloc(const svodk_tensor *q, const svodk_tensor *k, const svodk_tensor *v, const svodk_attn *opts,
                            const svodk_tensor *out, void *hip_stream);
int64_t svodk_noalloc_scratch_bytes(void);

/*
 * ops::attention_packed (tk/src/ops/attention.rs:104-122): attention over a fused
 * projection qkv [B, T, (heads + 2*kv_heads)*D] of queries, keys and values side
 * by side, read in place; out [B, T, heads, D].  No cache.  Bit-identical to
 * svodk_attention on the three split tensors (tk/src/test/unit/ops.rs:519-521).
 */
int svodk_attention_packed(const svodk_tensor *qkv, int32_t heads, int32_t kv_heads, const svodk_attn *opts,
                           const svodk_tensor *out, void *hip_stream);

/*
 * The batch rows in descending order of their key counts, ties by row: order[p] = the row with
 * the p-th most keys, for svodk_attn.row_order.  `keys` is what the call's key mask is: [B] lengths
 * (I32 or I64) or a [B, Tk] mask (BOOL or I32), a row of which counts up to its last visible key.
 * No counterpart in the reference, whose grid takes the rows as they come: workgroups are
 * dispatched in launch order, so a variable-length batch whose rows run grouped by length keeps a
 * CU's workgroups in step and ends on its short tiles (BGE-M3-shaped batches: 3 % less kernel time
 * with operands cold in HBM, 8-12 % with operands still in the Infinity Cache).  order [B] I32,
 * B <= 8192.  One small launch on the stream.
 */
int svodk_order_rows(const svodk_tensor *keys, const svodk_tensor *order, void *hip_stream);

/*
 * Bytes of `workspace` svodk_attention needs for these operands and options:
 * the f32 partial tensors o_part [splits, B, T, H, D], m_part and l_part
 * [splits, B, T, H] of tk/src/ops/attention.rs:285-293, for the split count the
 * call would run with; 0 when it would not split.  Pure, no device.
 */
int64_t svodk_attention_workspace(const svodk_tensor *q, const svodk_tensor *k, const svodk_attn *opts);

/*
 * ops::heads (tk/src/ops/heads.rs:37-102).
 * qkv [B,T,(heads+2*kv_heads)*head_dim] -> q [B,T,heads,D], k and v
 * [B,T,kv_heads,D]: q and k RMS-normalised over the head where a weight is
 * given, then rotated (halves paired) where tables are given; v copied.
 */
int svodk_heads(const svodk_tensor *qkv, const svodk_qkv *opts, const svodk_tensor *q, const svodk_tensor *k,
                const svodk_tensor *v, void *hip_stream);

/*
 * Rotary of tk/src/ops/linear.rs:47-58: the output's first `heads` heads of `head_dim` columns are
 * turned by the tables' row of the token's position, halves paired as in svodk_heads; tables
 * [1, T, 1, head_dim/2] of the operands' type.
 */
typedef struct svodk_rotary {
  const svodk_tensor *cos, *sin;
  int32_t heads, head_dim;
} svodk_rotary;

/* Act of tk/src/ops/mod.rs (the activation of a Linear). */
typedef enum svodk_act { SVODK_ACT_NONE = 0, SVODK_ACT_GELU = 1, SVODK_ACT_SILU = 2 } svodk_act;

/*
 * Linear of tk/src/ops/linear.rs:24-45.  Zero-initialise, then set fields.  This library's GEMM
 * carries a bias and the rope; an activation, a gated weight, a residual, a scale (the rest of the
 * reference's GEMM family) answer SVODK_GRAPH_CONFIG, as does a rope with a head size other than 64
 * or 128 (no tile of the kernel holds its heads: the reference then rotates on the graph after a
 * plain kernel, tk/src/ops/linear.rs:176-184).
 */
typedef struct svodk_linear_opts {
  const svodk_tensor *bias; /* [N] or NULL */
  int32_t act;              /* svodk_act */
  int32_t gated;
  const svodk_tensor *residual; /* [B, T, N] or NULL */
  int32_t has_scale;
  float scale;
  const svodk_rotary *rope; /* or NULL */
  int32_t batch_live;       /* as in svodk_attn */
  /* Linear::into (tk/src/ops/linear.rs:40-42), the `out=` of a fused projection: with has_into the
   * call's `out` is the wider tensor [lead..., C] and the result is stored into its channels
   * into_at .. into_at + N; the other channels are left as they are.  into_at + N <= C
   * (tk/src/ops/mod.rs:459-477).  The kernel stores 16 bytes a lane: a window whose start or whose
   * row is not a multiple of 8 elements answers SVODK_GRAPH_CONFIG (the reference then runs the
   * plain kernel and lets the graph store the window, :96-103). */
  int32_t has_into;
  int64_t into_at;
} svodk_linear_opts;

/*
 * ops::linear (tk/src/ops/linear.rs:60-231) for a fused projection: x [B, T, K] . w [N, K]^T
 * (+ bias) -> out [B, T, N] (or channels of a wider out, see has_into), the rope applied in the GEMM's store (tk/src/kernels/gemm.rs:604-645,
 * 666-716): a model without QK norms gets its rotated queries and keys and its plain values from the
 * projection itself and needs no svodk_heads pass (svodk_attention_packed then reads `out` in place).
 * f32 accumulators, one rounding at the store.  N a multiple of 8 (tk/src/ops/shape.rs:133-136);
 * K a multiple of 32 here (others answer SVODK_GRAPH_SHAPE).
 */
int svodk_linear(const svodk_tensor *x, const svodk_tensor *w, const svodk_linear_opts *opts, const svodk_tensor *out,
                 void *hip_stream);
/* shape::linear (tk/src/ops/shape.rs:120-139) as a pure function: x_dims [.., K], n the output's columns. */
int svodk_plan_linear(int32_t has_target, const int32_t *dtypes, int32_t n_dtypes, const int64_t *x_dims, int32_t x_rank,
                      int64_t n);

/*
 * ops::layer_norm, add_layer_norm, rms_norm, add_rms_norm (tk/src/ops/norm.rs:16-42 -> norm, :44-98):
 *   layer: (x - mean) * rsqrt(var + eps) * w + b      rms: x * rsqrt(mean(x^2) + eps) * w
 * over the last dim of x [..., D], in f32, rounded once to x's type.  The add_ forms normalize
 * x + residual and also write that sum, rounded to x's type first, to `sum`.  w and b are [D];
 * b may be NULL; every operand has x's 16-bit type.  D is a multiple of 256 in 256..4096 (the
 * reference stops at 2048); other widths answer SVODK_GRAPH_SHAPE.  `batch_live` is as in
 * the attention options: <= 0 runs every batch.
 */
int svodk_layer_norm(const svodk_tensor *x, const svodk_tensor *w, const svodk_tensor *b, double eps, int32_t batch_live,
                     const svodk_tensor *out, void *hip_stream);
int svodk_add_layer_norm(const svodk_tensor *x, const svodk_tensor *residual, const svodk_tensor *w,
                         const svodk_tensor *b, double eps, int32_t batch_live, const svodk_tensor *sum,
                         const svodk_tensor *out, void *hip_stream);
int svodk_rms_norm(const svodk_tensor *x, const svodk_tensor *w, double eps, int32_t batch_live, const svodk_tensor *out,
                   void *hip_stream);
int svodk_add_rms_norm(const svodk_tensor *x, const svodk_tensor *residual, const svodk_tensor *w, double eps,
                       int32_t batch_live, const svodk_tensor *sum, const svodk_tensor *out, void *hip_stream);

/*
 * The shape gates as pure functions, no device needed
 * (shape::attention, tk/src/ops/shape.rs:189-206; shape::heads, :209-218;
 * gate, :92-99).  `has_target` stands for "the default device has kernels".
 * `dtypes` are those of every operand (q, k, v[, bias] / qkv[, weights, tables]).
 * `q_dims`/`k_dims` NULL means a symbolic dim past the batch.
 */
int svodk_plan_attention(int32_t has_target, const int32_t *dtypes, int32_t n_dtypes, const int64_t *q_dims,
                         const int64_t *k_dims, int32_t causal, int32_t bias);
int svodk_plan_heads(int32_t has_target, const int32_t *dtypes, int32_t n_dtypes, const int64_t *x_dims, int32_t x_rank,
                     int32_t head_dim);
/* shape::norm (tk/src/ops/shape.rs:221-231). */
int svodk_plan_norm(int32_t has_target, const int32_t *dtypes, int32_t n_dtypes, const int64_t *x_dims, int32_t x_rank);

/*
 * A tuning knob in place of the reference's per-shape tuner (tk/src/tune.rs): attention calls
 * with head size 64, no key mask tensor, no window and no splits can run as "streaming"
 * workgroups that each walk a run of query tiles, the next tile's keys loading under the
 * current tile's last steps.  n > 0 = stream, n workgroups per XCD (96 fills an MI355X);
 * n <= 0 (the default) = a workgroup per tile.  Process-wide.  Results are bit-equal either way.
 *
 * A streaming launch hands out its tiles through one of SVODK_STREAMING_SETS sets of counters in
 * device memory, taken in turn at enqueue time and put back to zero by the launch's last
 * workgroup: at most SVODK_STREAMING_SETS streaming launches may be in flight at once on a device,
 * and a launch that dies midway leaves its set dirty for the launch that meets it next.  A call on
 * a stream that is being captured never streams (a graph's replays would all use the set the
 * capture took, and overlapping replays would share it): it runs a workgroup per tile.
 */
#define SVODK_STREAMING_SETS 256
void svodk_tune_streaming(int32_t workgroups_per_xcd);
/*
 * No counterpart in the reference.  A decoder step (an attention call without causal or per-row masks or a bias
 * whose KV heads each serve at most SVODK_DECODE_ROWS query rows, heads / kv_heads * T) streams K and V through
 * registers past its rows instead of running 64-key tiles through LDS: such a call is bound by the bytes of K and V
 * in flight, not by arithmetic.  `rows` = the most rows a KV head may serve for a call to go that way, 0 ..
 * SVODK_DECODE_ROWS; 0 = every call runs key tiles; SVODK_DECODE_ROWS_DEFAULT until a call says otherwise.
 * Process-wide.  Results of the two paths agree to the op's tolerance, not bit for bit: they sum in different orders.
 */
#define SVODK_DECODE_ROWS 4
#define SVODK_DECODE_ROWS_DEFAULT 2
void svodk_tune_decode(int32_t rows);
/*
 * No counterpart in the reference, whose tuner picks a GEMM's tile by measurement (tk/src/tune.rs, GemmCfg of
 * tk/src/ops/config/gemm.rs).  svodk_linear runs 256 x 256 output tiles by 8 waves, or 128 x 128 tiles by 4 waves
 * where the larger tile would make fewer workgroups than half the device's compute units (a projection of few
 * rows).  `tile` = 256 or 128 names the tile of every later call, 0 gives the choice back to the shape.
 * Process-wide.  The two tiles give the same bits: a column's k-steps are summed in the same order.
 */
void svodk_tune_linear(int32_t tile);
/* The set the next streaming launch would take, and takes it (no device work): for tests of the
 * assignment.  No counterpart in the reference. */
uint32_t svodk_streaming_next_set(void);

/*
 * ops::supported (tk/src/ops/mod.rs:164-166): 1 when the current HIP device is
 * a gfx950 this library has kernels for.
 */
int svodk_supported(void);

/*
 * ops::chosen (tk/src/ops/mod.rs:83-118): what the last op on THIS thread
 * ran, as text — `Kernel { op: "attention", family: "flash_attention", cfg: "..." }`
 * or `Graph { op: "attention", why: Dtype }`.  Empty before any op ran.
 * The pointer stays valid until the thread's next op call.
 */
const char *svodk_last_chosen(void);

/* The message of the last negative status on this thread (Display of ops::Error). */
const char *svodk_last_error(void);

/* Name of a status code, e.g. "Fallback::Shape". */
const char *svodk_status_name(int status);

int svodk_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* SVODK_H */

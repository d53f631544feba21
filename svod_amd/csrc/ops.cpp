// The op layer of the gfx950 library: what Svod's `svod_tk::ops::{attention, heads}`
// do on the host before a kernel runs — validate, plan "kernel or graph", record
// what was chosen, launch — restated in C++ behind the C ABI of include/svodk.h.
//
// Contract kept from the reference (tk/src/ops/mod.rs:1-4): an op launches a
// kernel, or names why the caller's graph must run, or rejects what the graph
// would also reject.  Validation comes first and never touches the device, so
// it behaves the same on a machine without a GPU.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <atomic>
#include <string>

#include "../../include/svodk.h"
#include "kernels.h"

namespace {

// ---- per-thread records: ops::chosen (tk/src/ops/mod.rs:83-118) and the last error.
thread_local std::string g_chosen;
thread_local std::string g_error;

const char *fallback_name(int why) {
  switch (why) {
    case SVODK_GRAPH_TARGET: return "Target";
    case SVODK_GRAPH_DTYPE: return "Dtype";
    case SVODK_GRAPH_SYMBOLIC: return "Symbolic";
    case SVODK_GRAPH_SHAPE: return "Shape";
    case SVODK_GRAPH_CONFIG: return "Config";
    default: return "?";
  }
}

// ran_graph (mod.rs:115-118).
int ran_graph(const char *op, int why) {
  g_chosen = std::string("Graph { op: \"") + op + "\", why: " + fallback_name(why) + " }";
  return why;
}

// ran (mod.rs:110-113).
void ran(const char *op, const char *family, const char *cfg) {
  g_chosen = std::string("Kernel { op: \"") + op + "\", family: \"" + family + "\", cfg: \"" + cfg + "\" }";
}

int fail(int status, const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_error = buf;
  return status;
}

const char *dtype_name(int32_t d) {
  switch (d) {
    case SVODK_BF16: return "BFloat16";
    case SVODK_F16: return "Float16";
    case SVODK_F32: return "Float32";
    case SVODK_I32: return "Int32";
    case SVODK_I64: return "Int64";
    case SVODK_BOOL: return "Bool";
    default: return "?";
  }
}

size_t dtype_bytes(int32_t d) {
  switch (d) {
    case SVODK_BF16:
    case SVODK_F16: return 2;
    case SVODK_F32:
    case SVODK_I32: return 4;
    case SVODK_I64: return 8;
    case SVODK_BOOL: return 1;
    default: return 0;
  }
}

std::string fmt_shape(const svodk_tensor *t) {
  std::string s = "[";
  for (int i = 0; i < t->rank; i++) {
    if (i) s += ", ";
    s += std::to_string((long long)t->shape[i]);
  }
  return s + "]";
}

bool well_formed(const svodk_tensor *t) {
  if (t == nullptr || t->rank < 0 || t->rank > 4 || dtype_bytes(t->dtype) == 0) return false;
  for (int i = 0; i < t->rank; i++)
    if (t->shape[i] < 0) return false;
  return true;
}

int64_t numel(const svodk_tensor *t) {
  int64_t n = 1;
  for (int i = 0; i < t->rank; i++) n *= t->shape[i];
  return n;
}

bool same_shape(const svodk_tensor *a, const svodk_tensor *b) {
  if (a->rank != b->rank) return false;
  for (int i = 0; i < a->rank; i++)
    if (a->shape[i] != b->shape[i]) return false;
  return true;
}

bool is_int(int32_t d) { return d == SVODK_I32 || d == SVODK_I64; }

// What the kernels assume of a device address: 16-bit tensors are read and written in 128-bit pieces
// (and filled into LDS 16 bytes a lane), integers and masks at their element's size.
size_t alignment_of(const svodk_tensor *t) {
  return (t->dtype == SVODK_BF16 || t->dtype == SVODK_F16) ? 16 : dtype_bytes(t->dtype);
}

// The first of `tensors` (nulls skipped) whose address is off its alignment, or -1.
int misaligned(const svodk_tensor *const *tensors, int n) {
  for (int i = 0; i < n; i++) {
    const svodk_tensor *t = tensors[i];
    if (t != nullptr && t->data != nullptr && ((uintptr_t)t->data & (alignment_of(t) - 1)) != 0) return i;
  }
  return -1;
}

// launch::aliasing (tk/src/launch.rs:227-246): no parameter the kernel writes
// shares memory with another.  Here a parameter is a byte range.
struct Span {
  const char *name;
  const void *data;
  size_t bytes;
  bool written;
};

int check_aliasing(const char *op, const Span *spans, int n) {
  for (int i = 0; i < n; i++) {
    for (int j = i + 1; j < n; j++) {
      const Span &a = spans[i], &b = spans[j];
      if (!(a.written || b.written) || a.data == nullptr || b.data == nullptr || a.bytes == 0 || b.bytes == 0) continue;
      const char *a0 = (const char *)a.data, *b0 = (const char *)b.data;
      if (a0 < b0 + b.bytes && b0 < a0 + a.bytes)
        return fail(SVODK_ERR_LAUNCH, "%s: parameters %s and %s share memory", op, a.name, b.name);
    }
  }
  return 0;
}

// ---- the target: ops::supported / planner (mod.rs:161-197), without the cost probes.
// The library is built for gfx950 alone; any other device has no kernels.
bool device_is_gfx950(int device) {
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) != hipSuccess) return false;
  return std::strncmp(prop.gcnArchName, "gfx950", 6) == 0;
}

bool current_device_has_kernels() {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0) {
    (void)hipGetLastError();
    return false;
  }
  // 0 unknown, 1 yes, 2 no; two threads that both find it unknown ask the runtime twice and store the same answer.
  static std::atomic<int> known[64];
  if (device >= 64) return device_is_gfx950(device);
  int state = known[device].load(std::memory_order_acquire);
  if (state == 0) {
    state = device_is_gfx950(device) ? 1 : 2;
    known[device].store(state, std::memory_order_release);
  }
  return state == 1;
}

// The compute units of the current device (256 on an MI355X), asked once a device.
int current_device_units() {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0) {
    (void)hipGetLastError();
    return 256;
  }
  static std::atomic<int> known[64];
  int units = device < 64 ? known[device].load(std::memory_order_acquire) : 0;
  if (units == 0) {
    if (hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || units <= 0) {
      (void)hipGetLastError();
      units = 256;
    }
    if (device < 64) known[device].store(units, std::memory_order_release);
  }
  return units;
}

// ---- shape gates (tk/src/ops/shape.rs).
// gate (L92-99): a target with kernels, every operand the same 16-bit type the
// target has a matrix core for: gfx950 has one for bf16 and for f16, and both have kernels here.
int gate(bool has_target, const int32_t *dtypes, int n) {
  if (!has_target) return SVODK_GRAPH_TARGET;
  if (n <= 0) return SVODK_GRAPH_DTYPE;
  const int32_t first = dtypes[0];
  if (!(first == SVODK_BF16 || first == SVODK_F16)) return SVODK_GRAPH_DTYPE;
  for (int i = 0; i < n; i++)
    if (dtypes[i] != first) return SVODK_GRAPH_DTYPE;
  return 0;
}

// shape::attention (L189-206).  attention_ranked lists configs for head sizes
// that tile the matrix atom; here the candidates are the head sizes the HIP
// kernel is instantiated for.
int plan_attention(bool has_target, const int32_t *dtypes, int n, const int64_t *q, const int64_t *k, bool causal,
                   bool bias) {
  (void)causal;
  (void)bias;
  if (int why = gate(has_target, dtypes, n)) return why;
  if (q == nullptr || k == nullptr) return SVODK_GRAPH_SYMBOLIC;
  for (int i = 0; i < 4; i++)
    if (q[i] == 0 || k[i] == 0) return SVODK_GRAPH_SHAPE;
  if (q[3] > 0x7fffffff || !svodk::attention_supports((int32_t)q[3])) return SVODK_GRAPH_SHAPE;
  return 0;
}

// shape::heads (L209-218) with heads_candidates (tk/src/ops/config/norm.rs:8-13):
// rank 3, no empty dim, head size a power of two in 16..=256.
int plan_heads(bool has_target, const int32_t *dtypes, int n, const int64_t *x, int rank, int32_t d) {
  if (int why = gate(has_target, dtypes, n)) return why;
  if (x == nullptr) return SVODK_GRAPH_SYMBOLIC;
  if (rank != 3) return SVODK_GRAPH_SHAPE;
  for (int i = 0; i < 3; i++)
    if (x[i] == 0) return SVODK_GRAPH_SHAPE;
  const bool pow2 = d > 0 && (d & (d - 1)) == 0;
  if (!(pow2 && d >= 16 && d <= 256) || !svodk::heads_supports(d)) return SVODK_GRAPH_SHAPE;
  return 0;
}

// shape::norm (L221-231) with norm_candidates (tk/src/ops/config/norm.rs:19-24): the reduced dim a
// multiple of 256 from 256 on, no empty dim.  The reference stops at 2048 (64 elements a lane of
// its 32-lane warp); a 64-lane wave holds 4096 the same way, so the kernel here goes that far.
int plan_norm(bool has_target, const int32_t *dtypes, int n, const int64_t *x, int rank) {
  if (int why = gate(has_target, dtypes, n)) return why;
  if (x == nullptr) return SVODK_GRAPH_SYMBOLIC;
  if (rank < 1) return SVODK_GRAPH_SHAPE;
  for (int i = 0; i < rank; i++)
    if (x[i] == 0) return SVODK_GRAPH_SHAPE;
  if (!svodk::norm_supports(x[rank - 1])) return SVODK_GRAPH_SHAPE;
  return 0;
}

const char *OP_ATTN = "attention";
const char *OP_HEADS = "heads";

}  // namespace

extern "C" {

int svodk_abi_version(void) { return SVODK_ABI_VERSION; }

const char *svodk_last_chosen(void) { return g_chosen.c_str(); }

const char *svodk_last_error(void) { return g_error.c_str(); }

const char *svodk_status_name(int status) {
  switch (status) {
    case SVODK_KERNEL: return "Kernel";
    case SVODK_GRAPH_TARGET: return "Fallback::Target";
    case SVODK_GRAPH_DTYPE: return "Fallback::Dtype";
    case SVODK_GRAPH_SYMBOLIC: return "Fallback::Symbolic";
    case SVODK_GRAPH_SHAPE: return "Fallback::Shape";
    case SVODK_GRAPH_CONFIG: return "Fallback::Config";
    case SVODK_ERR_SHAPE: return "Error::Shape";
    case SVODK_ERR_DTYPE: return "Error::Dtype";
    case SVODK_ERR_HEADS: return "Error::Heads";
    case SVODK_ERR_LAUNCH: return "Error::Launch";
    case SVODK_ERR_ARGUMENT: return "Error::Argument";
    default: return "?";
  }
}

int svodk_supported(void) { return current_device_has_kernels() ? 1 : 0; }

int svodk_plan_attention(int32_t has_target, const int32_t *dtypes, int32_t n_dtypes, const int64_t *q_dims,
                         const int64_t *k_dims, int32_t causal, int32_t bias) {
  return plan_attention(has_target != 0, dtypes, n_dtypes, q_dims, k_dims, causal != 0, bias != 0);
}

int svodk_plan_heads(int32_t has_target, const int32_t *dtypes, int32_t n_dtypes, const int64_t *x_dims, int32_t x_rank,
                     int32_t head_dim) {
  return plan_heads(has_target != 0, dtypes, n_dtypes, x_dims, x_rank, head_dim);
}

// split_ranked of tk/src/ops/attention.rs:405-410 for this library's one tile shape: a named
// count is capped at the 64-key blocks of tk; one leaves the keys unsplit.  With none named the
// reference lets its tuner choose "among one, two, the counts around two blocks per SM and the
// block count" (tk/src/ops/attention.rs:76-79) by measurement; here a rule stands where the
// tuner would: enough splits for about two workgroups a CU (512 on an MI355X), each with at
// least 8 key blocks.  Measured on decode and short-query shapes (kernel + merge, microseconds,
// unsplit -> rule's count): 16 workgroups x 128 blocks 101.6 -> 24.2 (16 splits), 32 x 128
// 151.5 -> 29.8 (16), 64 x 32 28.7 -> 16.8 (4), 64 x 64 82.7 -> 37.6 (8), 256 x 64 86.2 -> 67.4
// (2), 320 x 24 32.7 -> 28.6 (2); from 640 workgroups on the rule answers one, which is fastest.
// A window, a chunk mask or segment starts leave a tile few of the keys: the rule keeps those whole.
static int split_count(const svodk_attn *opts, int64_t batch, int64_t t, int64_t heads, int64_t kv_heads, int64_t tk) {
  const int32_t asked = opts->splits;
  const int64_t most = tk > 0 ? (tk + 63) / 64 : 1;
  if (asked == 1) return 1;
  if (asked > 1) return (int)(asked < most ? asked : most);
  if (opts->has_window || opts->has_chunk || opts->seg_start != nullptr) return 1;
  const int64_t group = kv_heads > 0 ? heads / kv_heads : 1;
  // A decoder step of a few rows a KV head streams its keys (svodk::attention_decodes): a workgroup a (batch, KV
  // head, split), splits of at least four key blocks, as many as bring the launch to about a thousand workgroups
  // (one row) or five hundred (more): enough of them resident for the bytes in flight, few enough that their
  // streams do not thrash the memory's open pages.
  if (!opts->causal && opts->bias == nullptr && group * t >= 1 && group * t <= svodk::attention_decode_limit()) {
    const int64_t units = kv_heads * batch;
    if (units <= 0) return 1;
    const int64_t target = group * t == 1 ? 1024 : 512;
    const int64_t wanted = (target + units / 2) / units, fits = most / 4;
    const int64_t n = wanted < fits ? wanted : fits;
    return (int)(n < 1 ? 1 : (n > 64 ? 64 : n));
  }
  // A decoder step under GQA runs a KV head's whole group in one tile (svodk::attention_groups).
  const bool grouped = group > 1 && !opts->causal && group * t <= 128;
  const int64_t workgroups = grouped ? kv_heads * batch : (t + 127) / 128 * heads * batch;
  if (workgroups <= 0) return 1;
  const int64_t wanted = (512 + workgroups / 2) / workgroups;  // rounded
  const int64_t fits = most / 8;
  const int64_t n = wanted < fits ? wanted : fits;
  return (int)(n < 1 ? 1 : (n > 64 ? 64 : n));
}

// attend (tk/src/ops/attention.rs:126-303): attention of q, k and v, or of the `packed` operand
// they are views of.
// `own_scratch`: the partial states of a split call go to the library's static device array instead
// of a lent workspace (svodk_attention_noalloc).
static int attend(const svodk_tensor *q, const svodk_tensor *k, const svodk_tensor *v, const svodk_tensor *packed,
                  const svodk_attn *opts, const svodk_tensor *out, void *hip_stream, bool own_scratch = false) {
  const char *op = OP_ATTN;
  if (!well_formed(q) || !well_formed(k) || !well_formed(v) || !well_formed(out) || opts == nullptr)
    return fail(SVODK_ERR_ARGUMENT, "%s: a null or malformed tensor descriptor", op);
  // L131: q is [B, T, H, D].
  if (q->rank != 4)
    return fail(SVODK_ERR_SHAPE, "%s: q has shape %s, expected [B, T, H, D]", op, fmt_shape(q).c_str());
  // L132-138: k is [B, Tk, H_kv, D] ([rows, ...] under a cache's row map); v has k's shape.
  const svodk_cache *cache = opts->cache;
  const bool mapped = cache != nullptr && cache->row_map != nullptr;
  const bool batch_fits = k->rank == 4 && (k->shape[0] == q->shape[0] || mapped);
  if (!(k->rank == 4 && batch_fits && k->shape[3] == q->shape[3])) {
    if (mapped)
      return fail(SVODK_ERR_SHAPE, "%s: k has shape %s, expected [rows, Tk, H_kv, %lld]", op, fmt_shape(k).c_str(),
                  (long long)q->shape[3]);
    return fail(SVODK_ERR_SHAPE, "%s: k has shape %s, expected [%lld, Tk, H_kv, %lld]", op, fmt_shape(k).c_str(),
                (long long)q->shape[0], (long long)q->shape[3]);
  }
  if (!same_shape(v, k))
    return fail(SVODK_ERR_SHAPE, "%s: v has shape %s, expected %s", op, fmt_shape(v).c_str(), fmt_shape(k).c_str());
  // L139-141: k and v share q's type.
  if (k->dtype != q->dtype)
    return fail(SVODK_ERR_DTYPE, "%s: k is %s, the input is %s", op, dtype_name(k->dtype), dtype_name(q->dtype));
  if (v->dtype != q->dtype)
    return fail(SVODK_ERR_DTYPE, "%s: v is %s, the input is %s", op, dtype_name(v->dtype), dtype_name(q->dtype));
  // L142-145: whole groups of query heads per KV head.
  const int64_t heads = q->shape[2], kv_heads = cache ? cache->kv_heads : k->shape[2];
  if (!(kv_heads > 0 && heads % kv_heads == 0))
    return fail(SVODK_ERR_HEADS, "%s: %lld query heads are not a multiple of %lld key/value heads", op,
                (long long)heads, (long long)kv_heads);
  // L146-170: the cache's head range lies in the row; its map, appended rows and their counts fit the batch.
  int64_t appended = 0;
  if (cache != nullptr) {
    if (!(cache->head_start >= 0 && cache->head_start + cache->kv_heads <= k->shape[2]))
      return fail(SVODK_ERR_SHAPE, "%s: k has shape %s, expected [rows, Tk, >= %lld, %lld]", op, fmt_shape(k).c_str(),
                  (long long)(cache->head_start + cache->kv_heads), (long long)q->shape[3]);
    if (cache->row_map != nullptr) {
      if (!well_formed(cache->row_map)) return fail(SVODK_ERR_ARGUMENT, "%s: row map descriptor malformed", op);
      if (!(cache->row_map->rank == 1 && cache->row_map->shape[0] == q->shape[0]))
        return fail(SVODK_ERR_SHAPE, "%s: row map has shape %s, expected [%lld]", op,
                    fmt_shape(cache->row_map).c_str(), (long long)q->shape[0]);
      if (!is_int(cache->row_map->dtype))
        return fail(SVODK_ERR_DTYPE, "%s: row map is %s, the input is an integer type", op,
                    dtype_name(cache->row_map->dtype));
    }
    if ((cache->k_app != nullptr) != (cache->v_app != nullptr))
      return fail(SVODK_ERR_ARGUMENT, "%s: appended keys and values come together", op);
    if (cache->k_app != nullptr) {
      const svodk_tensor *both[2] = {cache->k_app, cache->v_app};
      const char *names[2] = {"appended k", "appended v"};
      if (!well_formed(both[0]) || !well_formed(both[1]))
        return fail(SVODK_ERR_ARGUMENT, "%s: appended rows descriptor malformed", op);
      const int64_t rows = both[0]->rank == 4 && both[0]->shape[1] > 0 ? both[0]->shape[1] : 0;
      for (int i = 0; i < 2; i++) {
        const svodk_tensor *x = both[i];
        const bool fits = rows > 0 && x->rank == 4 && x->shape[0] == q->shape[0] && x->shape[1] == rows &&
                          x->shape[2] == kv_heads && x->shape[3] == q->shape[3];
        if (!fits)
          return fail(SVODK_ERR_SHAPE, "%s: %s has shape %s, expected [%lld, %lld, %lld, %lld]", op, names[i],
                      fmt_shape(x).c_str(), (long long)q->shape[0], (long long)(rows > 0 ? rows : 1),
                      (long long)kv_heads, (long long)q->shape[3]);
        if (x->dtype != q->dtype)
          return fail(SVODK_ERR_DTYPE, "%s: %s is %s, the input is %s", op, names[i], dtype_name(x->dtype),
                      dtype_name(q->dtype));
      }
      if (opts->key_kind != SVODK_KEYS_LENS)
        return fail(SVODK_ERR_SHAPE, "%s: key lens has shape [], expected [B] with appended rows", op);
      appended = rows;
    }
    if (cache->app_lens != nullptr) {
      if (!well_formed(cache->app_lens)) return fail(SVODK_ERR_ARGUMENT, "%s: appended lens descriptor malformed", op);
      if (!(cache->k_app != nullptr && cache->app_lens->rank == 1 && cache->app_lens->shape[0] == q->shape[0]))
        return fail(SVODK_ERR_SHAPE, "%s: appended lens has shape %s, expected [%lld] with appended rows", op,
                    fmt_shape(cache->app_lens).c_str(), (long long)q->shape[0]);
      if (!is_int(cache->app_lens->dtype))
        return fail(SVODK_ERR_DTYPE, "%s: appended lens is %s, the input is an integer type", op,
                    dtype_name(cache->app_lens->dtype));
    }
  }
  // L174-186: the key mask's shape.
  const svodk_tensor *lens = nullptr, *bools = nullptr;
  if (opts->key_kind == SVODK_KEYS_LENS) {
    if (!well_formed(opts->keys)) return fail(SVODK_ERR_ARGUMENT, "%s: key lens descriptor missing", op);
    if (!(opts->keys->rank == 1 && opts->keys->shape[0] == q->shape[0]))
      return fail(SVODK_ERR_SHAPE, "%s: key lens has shape %s, expected [%lld]", op, fmt_shape(opts->keys).c_str(),
                  (long long)q->shape[0]);
    lens = opts->keys;
  } else if (opts->key_kind == SVODK_KEYS_BOOL) {
    if (!well_formed(opts->keys)) return fail(SVODK_ERR_ARGUMENT, "%s: key mask descriptor missing", op);
    if (!(opts->keys->rank == 2 && opts->keys->shape[0] == q->shape[0] && opts->keys->shape[1] == k->shape[1]))
      return fail(SVODK_ERR_SHAPE, "%s: key mask has shape %s, expected [%lld, %lld]", op,
                  fmt_shape(opts->keys).c_str(), (long long)q->shape[0], (long long)k->shape[1]);
    bools = opts->keys;
  } else if (opts->key_kind != SVODK_KEYS_NONE) {
    return fail(SVODK_ERR_ARGUMENT, "%s: unknown key mask kind %d", op, opts->key_kind);
  }
  // L187-190: segment starts are [B, T].
  if (opts->seg_start != nullptr) {
    if (!well_formed(opts->seg_start)) return fail(SVODK_ERR_ARGUMENT, "%s: seg start descriptor malformed", op);
    if (!(opts->seg_start->rank == 2 && opts->seg_start->shape[0] == q->shape[0] &&
          opts->seg_start->shape[1] == q->shape[1]))
      return fail(SVODK_ERR_SHAPE, "%s: seg start has shape %s, expected [%lld, %lld]", op,
                  fmt_shape(opts->seg_start).c_str(), (long long)q->shape[0], (long long)q->shape[1]);
  }
  // L193-203: a bias is [B | 1, H, T, Tk].
  if (opts->bias != nullptr) {
    if (!well_formed(opts->bias)) return fail(SVODK_ERR_ARGUMENT, "%s: bias descriptor malformed", op);
    const svodk_tensor *bt = opts->bias;
    const bool fits = bt->rank == 4 && (bt->shape[0] == q->shape[0] || bt->shape[0] == 1) && bt->shape[1] == heads &&
                      bt->shape[2] == q->shape[1] && bt->shape[3] == k->shape[1] + appended;
    if (!fits)
      return fail(SVODK_ERR_SHAPE, "%s: bias has shape %s, expected [%lld | 1, %lld, %lld, %lld]", op,
                  fmt_shape(bt).c_str(), (long long)q->shape[0], (long long)heads, (long long)q->shape[1],
                  (long long)(k->shape[1] + appended));
  }
  // The output the reference op allocates itself (tk/src/ops/mod.rs:423-429):
  // here the caller's, so its shape and type are checked like an operand's.
  if (!same_shape(out, q))
    return fail(SVODK_ERR_SHAPE, "%s: out has shape %s, expected %s", op, fmt_shape(out).c_str(),
                fmt_shape(q).c_str());
  if (out->dtype != q->dtype)
    return fail(SVODK_ERR_DTYPE, "%s: out is %s, the input is %s", op, dtype_name(out->dtype), dtype_name(q->dtype));
  if (lens != nullptr && !is_int(lens->dtype))
    return fail(SVODK_ERR_DTYPE, "%s: key lens is %s, the input is an integer type", op, dtype_name(lens->dtype));
  if (bools != nullptr && !(bools->dtype == SVODK_BOOL || bools->dtype == SVODK_I32))
    return fail(SVODK_ERR_DTYPE, "%s: key mask is %s, the input is Bool or Int32", op, dtype_name(bools->dtype));
  const int64_t cap = q->shape[0];
  if (opts->batch_live > cap)
    return fail(SVODK_ERR_SHAPE, "%s: live batch %d exceeds the capacity %lld", op, opts->batch_live, (long long)cap);

  // L205-208: the plan.  A chunk mask plans as a causal one.
  int32_t dtypes[4] = {q->dtype, k->dtype, v->dtype, opts->bias ? opts->bias->dtype : 0};
  const int why = plan_attention(current_device_has_kernels(), dtypes, opts->bias ? 4 : 3, q->shape, k->shape,
                                 opts->causal || opts->has_chunk, opts->bias != nullptr);
  if (why != 0) return ran_graph(op, why);
  // Options the reference's kernel holds and this library's does not: no
  // config here holds them (the reference's own use of Fallback::Config, L210-214).
  // L209-214: no config holds more appended rows than a key block.
  if (appended > 64) return ran_graph(op, SVODK_GRAPH_CONFIG);
  if (opts->has_window && (opts->window_left < 0 || opts->window_right < 0))
    return fail(SVODK_ERR_ARGUMENT, "%s: a negative window reach", op);
  // Chunk { size, left, right } of tk/src/ops/attention.rs:39-50: usize fields, a size of at least 1.
  if (opts->has_chunk && (opts->chunk_size <= 0 || opts->chunk_right < 0 || (opts->chunk_has_left && opts->chunk_left < 0)))
    return fail(SVODK_ERR_ARGUMENT, "%s: a chunk mask needs a positive size and non-negative reaches", op);
  if (opts->seg_start != nullptr && !(opts->seg_start->dtype == SVODK_I32 || opts->seg_start->dtype == SVODK_I64))
    return fail(SVODK_ERR_DTYPE, "%s: seg start is %s, the input is Int32 or Int64", op,
                dtype_name(opts->seg_start->dtype));
  const int64_t t = q->shape[1], tk = k->shape[1], d = q->shape[3];
  if (t > 0x7fffffff || tk > 0x7fffffff || heads > 0xffff || cap > 0x7fffffff)
    return ran_graph(op, SVODK_GRAPH_SHAPE);
  {
    // A fill addresses the 64 rows of one key block with 32-bit byte offsets from the block's own base
    // (which is 64-bit), and the launch counts its workgroups in 31 bits: shapes past either keep the graph.
    const int64_t row_elems = packed ? (heads + 2 * kv_heads) * d : k->shape[2] * d;
    const int64_t tiles = (t + 127) / 128 * heads * cap;
    if (row_elems * 2 * 64 > 0x7fffffffLL || tiles * 64 > 0x7ffffff0LL)
      return ran_graph(op, SVODK_GRAPH_SHAPE);
  }

  // A packed operand is one parameter (L268): its views overlap one another by construction.
  const size_t packed_bytes = packed ? (size_t)numel(packed) * 2 : 0;
  Span spans[6] = {{packed ? "qkv" : "q", packed ? packed->data : q->data, packed ? packed_bytes : (size_t)numel(q) * 2,
                    false},
                   {"k", packed ? nullptr : k->data, packed ? 0 : (size_t)numel(k) * 2, false},
                   {"v", packed ? nullptr : v->data, packed ? 0 : (size_t)numel(v) * 2, false},
                   {"o", out->data, (size_t)numel(out) * 2, true},
                   {"key_lens", lens ? lens->data : nullptr, lens ? (size_t)numel(lens) * dtype_bytes(lens->dtype) : 0,
                    false},
                   {"key_mask", bools ? bools->data : nullptr,
                    bools ? (size_t)numel(bools) * dtype_bytes(bools->dtype) : 0, false}};
  if (q->data == nullptr || k->data == nullptr || v->data == nullptr || out->data == nullptr ||
      (lens && lens->data == nullptr) || (bools && bools->data == nullptr) ||
      (opts->seg_start && opts->seg_start->data == nullptr) || (opts->bias && opts->bias->data == nullptr))
    return fail(SVODK_ERR_ARGUMENT, "%s: a null device pointer", op);
  {
    // 128-bit loads, stores and LDS fills on the 16-bit tensors; a bias row is read element-wise where
    // it is not 8-byte aligned, so its base needs its element's alignment only.
    const svodk_tensor *checked[10] = {q, k, v, out, lens, bools, opts->seg_start,
                                       cache ? cache->row_map : nullptr, cache ? cache->k_app : nullptr,
                                       cache ? cache->v_app : nullptr};
    const char *names[10] = {"q", "k", "v", "out", "key lens", "key mask", "seg start", "row map", "appended k", "appended v"};
    const int bad = misaligned(checked, 10);
    if (bad >= 0)
      return fail(SVODK_ERR_ARGUMENT, "%s: %s is not %zu-byte aligned", op, names[bad], alignment_of(checked[bad]));
    if (opts->bias != nullptr && ((uintptr_t)opts->bias->data & 1u) != 0)
      return fail(SVODK_ERR_ARGUMENT, "%s: bias is not 2-byte aligned", op);
    if (cache && cache->app_lens && cache->app_lens->data &&
        ((uintptr_t)cache->app_lens->data & (dtype_bytes(cache->app_lens->dtype) - 1)) != 0)
      return fail(SVODK_ERR_ARGUMENT, "%s: appended lens is not aligned to its element", op);
    if (opts->workspace != nullptr && ((uintptr_t)opts->workspace & 15u) != 0)
      return fail(SVODK_ERR_ARGUMENT, "%s: the workspace is not 16-byte aligned", op);
  }
  if (int rc = check_aliasing(op, spans, 6)) return rc;
  if (opts->seg_start != nullptr) {
    const svodk_tensor *seg = opts->seg_start;
    Span pair[2] = {{"seg_start", seg->data, (size_t)numel(seg) * dtype_bytes(seg->dtype), false}, spans[3]};
    if (int rc = check_aliasing(op, pair, 2)) return rc;
  }

  svodk::AttnArgs a{};
  a.q = q->data;
  a.k = k->data;
  a.v = v->data;
  a.o = out->data;
  a.key_lens = lens ? lens->data : nullptr;
  a.key_mask = bools ? bools->data : nullptr;
  a.lens_i64 = lens && lens->dtype == SVODK_I64;
  a.mask_bytes = bools ? (int32_t)dtype_bytes(bools->dtype) : 0;
  a.batch = opts->batch_live > 0 ? opts->batch_live : (int32_t)cap;
  a.t = (int32_t)t;
  a.tk = (int32_t)tk;
  a.heads = (int32_t)heads;
  a.kv_heads = (int32_t)kv_heads;
  a.d = (int32_t)d;
  a.causal = opts->causal != 0;
  // L230: the default scale is 1/sqrt(D) in f32.
  a.scale = opts->has_scale ? opts->scale : 1.0f / std::sqrt((float)d);
  a.f16 = q->dtype == SVODK_F16;
  // The window's reaches, capped where they no longer hide anything (and stay 32-bit).
  a.win_left = -1;
  if (opts->has_window) {
    a.win_left = (int32_t)std::min<int64_t>(opts->window_left, t + tk);
    a.win_right = (int32_t)std::min<int64_t>(opts->window_right, t + tk);
  }
  // The chunk mask's reaches, capped the same way: past the last chunk they hide nothing.
  if (opts->has_chunk) {
    const int64_t chunks = (t + tk) / opts->chunk_size + 2;
    a.chunk_size = (int32_t)std::min<int64_t>(opts->chunk_size, t + tk + 1);
    a.chunk_left = opts->chunk_has_left ? (int32_t)std::min<int64_t>(opts->chunk_left, chunks) : -1;
    a.chunk_right = (int32_t)std::min<int64_t>(opts->chunk_right, chunks);
    if (t + tk > 0x3fffffff) return ran_graph(op, SVODK_GRAPH_SHAPE);  // chunk edges stay 32-bit
  }
  if (opts->bias != nullptr) {
    Span pair[2] = {{"bias", opts->bias->data, (size_t)numel(opts->bias) * 2, false}, spans[3]};
    if (int rc = check_aliasing(op, pair, 2)) return rc;
    a.bias = opts->bias->data;
    a.bias_per_batch = opts->bias->shape[0] != 1 || cap == 1;
  }
  if (opts->seg_start != nullptr) {
    a.seg_start = opts->seg_start->data;
    a.seg_i64 = opts->seg_start->dtype == SVODK_I64;
  }
  if (opts->row_order != nullptr) {
    const svodk_tensor *ro = opts->row_order;
    if (!well_formed(ro)) return fail(SVODK_ERR_ARGUMENT, "%s: row order descriptor malformed", op);
    if (!(ro->rank == 1 && ro->shape[0] == q->shape[0]))
      return fail(SVODK_ERR_SHAPE, "%s: row order has shape %s, expected [%lld]", op, fmt_shape(ro).c_str(),
                  (long long)q->shape[0]);
    if (ro->dtype != SVODK_I32)
      return fail(SVODK_ERR_DTYPE, "%s: row order is %s, the input is Int32", op, dtype_name(ro->dtype));
    if (ro->data == nullptr) return fail(SVODK_ERR_ARGUMENT, "%s: a null device pointer", op);
    Span pair[2] = {{"row_order", ro->data, (size_t)numel(ro) * 4, false}, spans[3]};
    if (int rc = check_aliasing(op, pair, 2)) return rc;
    // Under a bound batch the order must name live rows only: an order of the whole capacity does not.
    if (a.batch == cap) a.row_order = ro->data;
  }
  if (packed != nullptr) a.q_row_elems = a.kv_row_elems = (heads + 2 * kv_heads) * d;
  if (cache != nullptr) {
    a.cached = 1;
    a.kv_row_elems = k->shape[2] * d;  // a cache row holds every layer's heads
    a.kv_head_start = (int32_t)cache->head_start;
    if (cache->row_map != nullptr) {
      if (cache->row_map->data == nullptr) return fail(SVODK_ERR_ARGUMENT, "%s: a null device pointer", op);
      if (k->shape[0] > 0x7fffffff) return ran_graph(op, SVODK_GRAPH_SHAPE);
      a.row_map = cache->row_map->data;
      a.row_map_i64 = cache->row_map->dtype == SVODK_I64;
      a.cache_rows = (int32_t)k->shape[0];
      Span pair[2] = {{"row_map", a.row_map, (size_t)numel(cache->row_map) * dtype_bytes(cache->row_map->dtype), false},
                      spans[3]};
      if (int rc = check_aliasing(op, pair, 2)) return rc;
    }
    if (cache->k_app != nullptr) {
      if (cache->k_app->data == nullptr || cache->v_app->data == nullptr ||
          (cache->app_lens != nullptr && cache->app_lens->data == nullptr))
        return fail(SVODK_ERR_ARGUMENT, "%s: a null device pointer", op);
      const svodk_tensor *apps[2] = {cache->k_app, cache->v_app};
      for (const svodk_tensor *x : apps) {
        Span pair[2] = {{"appended rows", x->data, (size_t)numel(x) * 2, false}, spans[3]};
        if (int rc = check_aliasing(op, pair, 2)) return rc;
      }
      a.k_app = cache->k_app->data;
      a.v_app = cache->v_app->data;
      a.app_rows = (int32_t)appended;
      if (cache->app_lens != nullptr) {
        a.app_lens = cache->app_lens->data;
        a.app_lens_i64 = cache->app_lens->dtype == SVODK_I64;
        Span pair[2] = {{"appended lens", a.app_lens, (size_t)numel(cache->app_lens) * dtype_bytes(cache->app_lens->dtype),
                         false},
                        spans[3]};
        if (int rc = check_aliasing(op, pair, 2)) return rc;
      }
    }
  }
  // L280-302: key splits.  The partial tensors live in the caller's workspace.
  a.splits = split_count(opts, a.batch, t, heads, kv_heads, tk);
  void *workspace = opts->workspace;
  if (a.splits > 1 && own_scratch) {
    // The library's own array holds the partial states.  A split count the rule chose is lowered to
    // what the array holds (down to one, as svodk_attention does without a workspace); a count the
    // caller named is refused when it does not fit, not shrunk.
    const int64_t per_split = (int64_t)a.batch * t * heads * (d + 2) * 4;
    int64_t have = 0;
    const hipError_t e = svodk::split_scratch(&workspace, &have);
    if (e != hipSuccess) return fail(SVODK_ERR_LAUNCH, "%s: the static scratch: %s", op, hipGetErrorString(e));
    if (opts->splits <= 0 && (int64_t)a.splits * per_split > have)
      a.splits = (int32_t)std::max<int64_t>(1, per_split > 0 ? have / per_split : 1);
    const int64_t need = (int64_t)a.splits * per_split;
    if (a.splits > 1 && need > have)
      return fail(SVODK_ERR_ARGUMENT,
                  "%s: %d key splits of %lld rows need %lld bytes of partial states, the static scratch holds %lld", op,
                  a.splits, (long long)((int64_t)a.batch * t * heads), (long long)need, (long long)have);
  } else if (a.splits > 1) {
    const int64_t rows = (int64_t)a.batch * t * heads;
    int64_t need = (int64_t)a.splits * rows * (d + 2) * 4;
    const bool lent = opts->workspace != nullptr && opts->workspace_bytes >= need;
    // Splits the caller named need their workspace; splits of the rule's own are dropped without it.
    if (!lent && opts->splits > 1) return ran_graph(op, SVODK_GRAPH_CONFIG);
    if (!lent) a.splits = 1, need = 0;
  }
  if (a.splits > 1) {
    const int64_t rows = (int64_t)a.batch * t * heads;
    const int64_t need = (int64_t)a.splits * rows * (d + 2) * 4;
    Span ws[2] = {{"workspace", workspace, (size_t)need, true}, {"o", out->data, (size_t)numel(out) * 2, true}};
    if (int rc = check_aliasing(op, ws, 2)) return rc;
    for (int i = 0; i < 3; i++) {
      Span pair[2] = {{"workspace", workspace, (size_t)need, true}, spans[i]};
      if (int rc = check_aliasing(op, pair, 2)) return rc;
    }
    a.o_part = (float *)workspace;
    a.m_part = a.o_part + (int64_t)a.splits * rows * d;
    a.l_part = a.m_part + (int64_t)a.splits * rows;
  }
  ran(op, "flash_attention", svodk::attention_config(a));
  hipError_t e = svodk::launch_attention(a, (hipStream_t)hip_stream);
  if (e != hipSuccess) return fail(SVODK_ERR_LAUNCH, "%s: %s", op, hipGetErrorString(e));
  if (a.splits > 1) {
    svodk::CombineArgs c{};
    c.o_part = a.o_part;
    c.m_part = a.m_part;
    c.l_part = a.l_part;
    c.o = out->data;
    c.rows = (int64_t)a.batch * t * heads;
    c.d = a.d;
    c.splits = a.splits;
    c.f16 = a.f16;
    ran(op, "combine_splits", "NormCfg { br: 4 }");
    e = svodk::launch_combine(c, (hipStream_t)hip_stream);
    if (e != hipSuccess) return fail(SVODK_ERR_LAUNCH, "%s: %s", op, hipGetErrorString(e));
  }
  return SVODK_KERNEL;
}

int svodk_attention(const svodk_tensor *q, const svodk_tensor *k, const svodk_tensor *v, const svodk_attn *opts,
                    const svodk_tensor *out, void *hip_stream) {
  return attend(q, k, v, nullptr, opts, out, hip_stream);
}

int svodk_attention_noalloc(const svodk_tensor *q, const svodk_tensor *k, const svodk_tensor *v, const svodk_attn *opts,
                            const svodk_tensor *out, void *hip_stream) {
  return attend(q, k, v, nullptr, opts, out, hip_stream, /*own_scratch=*/true);
}

int64_t svodk_noalloc_scratch_bytes(void) { return svodk::kSplitScratchBytes; }

// attention_packed (tk/src/ops/attention.rs:104-122).
int svodk_attention_packed(const svodk_tensor *qkv, int32_t heads, int32_t kv_heads, const svodk_attn *opts,
                           const svodk_tensor *out, void *hip_stream) {
  const char *op = OP_ATTN;
  if (!well_formed(qkv) || !well_formed(out) || opts == nullptr)
    return fail(SVODK_ERR_ARGUMENT, "%s: a null or malformed tensor descriptor", op);
  // L109: whole groups of query heads per KV head.
  if (!(kv_heads > 0 && heads >= 0 && heads % kv_heads == 0))
    return fail(SVODK_ERR_HEADS, "%s: %lld query heads are not a multiple of %lld key/value heads", op,
                (long long)heads, (long long)kv_heads);
  // L110-114: qkv is [B, T, slots * D] and a packed call has no cache.
  const int64_t slots = (int64_t)heads + 2 * kv_heads;
  if (!(qkv->rank == 3 && qkv->shape[2] > 0 && qkv->shape[2] % slots == 0))
    return fail(SVODK_ERR_SHAPE, "%s: qkv has shape %s, expected [B, T, slots·D]", op, fmt_shape(qkv).c_str());
  if (opts->cache != nullptr)
    return fail(SVODK_ERR_SHAPE, "%s: qkv has shape %s, expected [B, T, slots·D] with no cache", op,
                fmt_shape(qkv).c_str());
  // L115-121: the three views of the fused row.
  const int64_t d = qkv->shape[2] / slots;
  uint16_t *base = (uint16_t *)qkv->data;
  svodk_tensor q = {base, qkv->dtype, 4, {qkv->shape[0], qkv->shape[1], heads, d}};
  svodk_tensor k = {base ? base + (int64_t)heads * d : nullptr, qkv->dtype, 4, {qkv->shape[0], qkv->shape[1], kv_heads, d}};
  svodk_tensor v = {base ? base + ((int64_t)heads + kv_heads) * d : nullptr, qkv->dtype, 4,
                    {qkv->shape[0], qkv->shape[1], kv_heads, d}};
  return attend(&q, &k, &v, qkv, opts, out, hip_stream);
}

void svodk_tune_streaming(int32_t workgroups_per_xcd) { svodk::attention_stream_slots(workgroups_per_xcd); }
void svodk_tune_decode(int32_t rows) { svodk::attention_decode_rows(rows); }
void svodk_tune_linear(int32_t tile) { svodk::linear_tile(tile); }
uint32_t svodk_streaming_next_set(void) { return svodk::next_queue_set(); }

// The batch rows by descending key count, for svodk_attn.row_order (no counterpart in the reference,
// whose grid fixes what a block computes and leaves the order of blocks to the hardware).
int svodk_order_rows(const svodk_tensor *keys, const svodk_tensor *order, void *hip_stream) {
  const char *op = "order_rows";
  if (!well_formed(keys) || !well_formed(order))
    return fail(SVODK_ERR_ARGUMENT, "%s: a null or malformed tensor descriptor", op);
  const bool mask = keys->rank == 2;
  if (!((keys->rank == 1 || mask) && order->rank == 1 && order->shape[0] == keys->shape[0]))
    return fail(SVODK_ERR_SHAPE, "%s: keys %s and order %s, expected [B] or [B, Tk] and [B]", op,
                fmt_shape(keys).c_str(), fmt_shape(order).c_str());
  if (mask ? !(keys->dtype == SVODK_BOOL || keys->dtype == SVODK_I32) : !is_int(keys->dtype))
    return fail(SVODK_ERR_DTYPE, "%s: keys are %s, the input is %s", op, dtype_name(keys->dtype),
                mask ? "Bool or Int32" : "an integer type");
  if (order->dtype != SVODK_I32)
    return fail(SVODK_ERR_DTYPE, "%s: order is %s, the output is Int32", op, dtype_name(order->dtype));
  if (keys->shape[0] > svodk::kMaxOrderedRows || (mask && keys->shape[1] > 0x7fffffff))
    return fail(SVODK_ERR_SHAPE, "%s: %lld rows, at most %d", op, (long long)keys->shape[0], svodk::kMaxOrderedRows);
  if (!current_device_has_kernels()) return ran_graph(op, SVODK_GRAPH_TARGET);
  if (keys->data == nullptr || order->data == nullptr) return fail(SVODK_ERR_ARGUMENT, "%s: a null device pointer", op);
  Span spans[2] = {{"keys", keys->data, (size_t)numel(keys) * dtype_bytes(keys->dtype), false},
                   {"order", order->data, (size_t)numel(order) * 4, true}};
  if (int rc = check_aliasing(op, spans, 2)) return rc;
  ran(op, "order_rows", "one workgroup");
  const hipError_t e = svodk::launch_order_rows(keys->data, (int32_t)dtype_bytes(keys->dtype), (int32_t)keys->shape[0],
                                                mask ? (int32_t)keys->shape[1] : -1, (int32_t *)order->data,
                                                (hipStream_t)hip_stream);
  if (e != hipSuccess) return fail(SVODK_ERR_LAUNCH, "%s: %s", op, hipGetErrorString(e));
  return SVODK_KERNEL;
}

// The workspace of a split call (tk/src/ops/attention.rs:285-293).
int64_t svodk_attention_workspace(const svodk_tensor *q, const svodk_tensor *k, const svodk_attn *opts) {
  if (!well_formed(q) || !well_formed(k) || opts == nullptr || q->rank != 4 || k->rank != 4) return 0;
  const int64_t batch = opts->batch_live > 0 ? opts->batch_live : q->shape[0];
  const int64_t kv_heads = opts->cache != nullptr ? opts->cache->kv_heads : k->shape[2];
  const int splits = split_count(opts, batch, q->shape[1], q->shape[2], kv_heads, k->shape[1]);
  if (splits <= 1) return 0;
  return (int64_t)splits * batch * q->shape[1] * q->shape[2] * (q->shape[3] + 2) * 4;
}

// heads (tk/src/ops/heads.rs:37-102).
int svodk_heads(const svodk_tensor *qkv, const svodk_qkv *opts, const svodk_tensor *q, const svodk_tensor *k,
                const svodk_tensor *v, void *hip_stream) {
  const char *op = OP_HEADS;
  if (!well_formed(qkv) || !well_formed(q) || !well_formed(k) || !well_formed(v) || opts == nullptr)
    return fail(SVODK_ERR_ARGUMENT, "%s: a null or malformed tensor descriptor", op);
  const int64_t heads = opts->heads, kv_heads = opts->kv_heads, d = opts->head_dim;
  // L44: whole groups of query heads per KV head.
  if (!(kv_heads > 0 && heads >= 0 && heads % kv_heads == 0))
    return fail(SVODK_ERR_HEADS, "%s: %lld query heads are not a multiple of %lld key/value heads", op,
                (long long)heads, (long long)kv_heads);
  if (d <= 0) return fail(SVODK_ERR_ARGUMENT, "%s: head_dim %lld", op, (long long)d);
  const int64_t slots = heads + 2 * kv_heads;
  // L45-47: qkv is [B, T, slots*d].
  if (!(qkv->rank == 3 && qkv->shape[2] == slots * d))
    return fail(SVODK_ERR_SHAPE, "%s: qkv has shape %s, expected [B, T, %lld\xc2\xb7%lld]", op, fmt_shape(qkv).c_str(),
                (long long)slots, (long long)d);
  // L48-53: the norm weights are [d].
  const svodk_tensor *norms[2] = {opts->q_norm, opts->k_norm};
  const char *norm_names[2] = {"q norm", "k norm"};
  for (int i = 0; i < 2; i++) {
    if (norms[i] == nullptr) continue;
    if (!well_formed(norms[i])) return fail(SVODK_ERR_ARGUMENT, "%s: %s descriptor malformed", op, norm_names[i]);
    if (!(norms[i]->rank == 1 && norms[i]->shape[0] == d))
      return fail(SVODK_ERR_SHAPE, "%s: %s has shape %s, expected [%lld]", op, norm_names[i],
                  fmt_shape(norms[i]).c_str(), (long long)d);
  }
  // L54-63: tables are [1, T, 1, d/2] by position or [B, T, 1, d/2] by token.
  if ((opts->cos == nullptr) != (opts->sin == nullptr))
    return fail(SVODK_ERR_ARGUMENT, "%s: cos and sin come together", op);
  bool per_batch = false;
  if (opts->cos != nullptr) {
    const svodk_tensor *c = opts->cos, *s = opts->sin;
    if (!well_formed(c) || !well_formed(s)) return fail(SVODK_ERR_ARGUMENT, "%s: rope descriptor malformed", op);
    const bool tail = c->rank == 4 && c->shape[1] == qkv->shape[1] && c->shape[2] == 1 && c->shape[3] == d / 2;
    const bool fits = tail && (c->shape[0] == 1 || c->shape[0] == qkv->shape[0]);
    if (!fits)
      return fail(SVODK_ERR_SHAPE, "%s: cos has shape %s, expected [1, %lld, 1, %lld] or [%lld, %lld, 1, %lld]", op,
                  fmt_shape(c).c_str(), (long long)qkv->shape[1], (long long)(d / 2), (long long)qkv->shape[0],
                  (long long)qkv->shape[1], (long long)(d / 2));
    if (!same_shape(s, c))
      return fail(SVODK_ERR_SHAPE, "%s: sin has shape %s, expected %s", op, fmt_shape(s).c_str(),
                  fmt_shape(c).c_str());
    // L80: by token when the leading dim is not the constant 1.
    per_batch = c->shape[0] != 1;
  }
  // The outputs the reference op allocates itself (L89-91), here the caller's.
  const int64_t want_q[4] = {qkv->shape[0], qkv->shape[1], heads, d};
  const int64_t want_kv[4] = {qkv->shape[0], qkv->shape[1], kv_heads, d};
  const svodk_tensor *outs[3] = {q, k, v};
  const char *out_names[3] = {"q", "k", "v"};
  for (int i = 0; i < 3; i++) {
    const int64_t *want = i == 0 ? want_q : want_kv;
    bool fits = outs[i]->rank == 4;
    for (int j = 0; fits && j < 4; j++) fits = outs[i]->shape[j] == want[j];
    if (!fits)
      return fail(SVODK_ERR_SHAPE, "%s: %s has shape %s, expected [%lld, %lld, %lld, %lld]", op, out_names[i],
                  fmt_shape(outs[i]).c_str(), (long long)want[0], (long long)want[1], (long long)want[2],
                  (long long)want[3]);
    if (outs[i]->dtype != qkv->dtype)
      return fail(SVODK_ERR_DTYPE, "%s: %s is %s, the input is %s", op, out_names[i], dtype_name(outs[i]->dtype),
                  dtype_name(qkv->dtype));
  }
  const int64_t cap = qkv->shape[0];
  if (opts->batch_live > cap)
    return fail(SVODK_ERR_SHAPE, "%s: live batch %d exceeds the capacity %lld", op, opts->batch_live, (long long)cap);

  // L65-72: a weight or table off the stream dtype keeps the graph.
  int32_t dtypes[5];
  int n = 0;
  dtypes[n++] = qkv->dtype;
  if (opts->q_norm) dtypes[n++] = opts->q_norm->dtype;
  if (opts->k_norm) dtypes[n++] = opts->k_norm->dtype;
  if (opts->cos) dtypes[n++] = opts->cos->dtype;
  if (opts->sin) dtypes[n++] = opts->sin->dtype;
  const int why = plan_heads(current_device_has_kernels(), dtypes, n, qkv->shape, qkv->rank, (int32_t)d);
  if (why != 0) return ran_graph(op, why);
  const int64_t t = qkv->shape[1];
  if (t > 0x7fffffff || heads > 0x7fff || kv_heads > 0x7fff) return ran_graph(op, SVODK_GRAPH_SHAPE);

  const size_t table_bytes = opts->cos ? (size_t)numel(opts->cos) * 2 : 0;
  Span spans[8] = {{"qkv", qkv->data, (size_t)numel(qkv) * 2, false},
                   {"q_w", opts->q_norm ? opts->q_norm->data : nullptr, (size_t)d * 2, false},
                   {"k_w", opts->k_norm ? opts->k_norm->data : nullptr, (size_t)d * 2, false},
                   {"cos", opts->cos ? opts->cos->data : nullptr, table_bytes, false},
                   {"sin", opts->sin ? opts->sin->data : nullptr, table_bytes, false},
                   {"q", q->data, (size_t)numel(q) * 2, true},
                   {"k", k->data, (size_t)numel(k) * 2, true},
                   {"v", v->data, (size_t)numel(v) * 2, true}};
  if (qkv->data == nullptr || q->data == nullptr || k->data == nullptr || v->data == nullptr ||
      (opts->q_norm && opts->q_norm->data == nullptr) || (opts->k_norm && opts->k_norm->data == nullptr) ||
      (opts->cos && (opts->cos->data == nullptr || opts->sin->data == nullptr)))
    return fail(SVODK_ERR_ARGUMENT, "%s: a null device pointer", op);
  {
    const svodk_tensor *checked[8] = {qkv, opts->q_norm, opts->k_norm, opts->cos, opts->sin, q, k, v};
    const int bad = misaligned(checked, 8);
    if (bad >= 0) return fail(SVODK_ERR_ARGUMENT, "%s: %s is not 16-byte aligned", op, spans[bad].name);
  }
  if (int rc = check_aliasing(op, spans, 8)) return rc;

  svodk::HeadsArgs a{};
  a.qkv = qkv->data;
  a.q_w = opts->q_norm ? opts->q_norm->data : nullptr;
  a.k_w = opts->k_norm ? opts->k_norm->data : nullptr;
  a.cos = opts->cos ? opts->cos->data : nullptr;
  a.sin = opts->sin ? opts->sin->data : nullptr;
  a.q = q->data;
  a.k = k->data;
  a.v = v->data;
  const int64_t live = opts->batch_live > 0 ? opts->batch_live : cap;
  a.rows = live * t;
  a.t = (int32_t)t;
  a.heads = (int32_t)heads;
  a.kv_heads = (int32_t)kv_heads;
  a.d = (int32_t)d;
  a.eps = (float)opts->eps;
  a.rope = opts->cos ? (per_batch ? 2 : 1) : 0;
  a.f16 = qkv->dtype == SVODK_F16;
  ran(op, "heads", "NormCfg { lanes_per_head: d/16, block: 256 }");
  const hipError_t e = svodk::launch_heads(a, (hipStream_t)hip_stream);
  if (e != hipSuccess) return fail(SVODK_ERR_LAUNCH, "%s: %s", op, hipGetErrorString(e));
  return SVODK_KERNEL;
}

// norm (tk/src/ops/norm.rs:44-98): LayerNorm or RMSNorm over the last dim of x, after a residual
// add when there is one.
static int norm(bool layer, const svodk_tensor *x, const svodk_tensor *residual, const svodk_tensor *w,
                const svodk_tensor *b, double eps, int32_t batch_live, const svodk_tensor *sum, const svodk_tensor *out,
                void *hip_stream) {
  const char *op = layer ? "layer_norm" : "rms_norm";
  if (!well_formed(x) || !well_formed(w) || !well_formed(out) || (b && !well_formed(b)) ||
      (residual && !well_formed(residual)) || (sum && !well_formed(sum)))
    return fail(SVODK_ERR_ARGUMENT, "%s: a null or malformed tensor descriptor", op);
  if ((residual != nullptr) != (sum != nullptr))
    return fail(SVODK_ERR_ARGUMENT, "%s: the sum comes with a residual and only with one", op);
  // L54-60: x is [..., D]; w and b are [D].
  if (x->rank < 1) return fail(SVODK_ERR_SHAPE, "%s: x has shape %s, expected [..., D]", op, fmt_shape(x).c_str());
  const int64_t d = x->shape[x->rank - 1];
  const svodk_tensor *vecs[2] = {w, b};
  const char *vec_names[2] = {"w", "b"};
  for (int i = 0; i < 2; i++)
    if (vecs[i] != nullptr && !(vecs[i]->rank == 1 && vecs[i]->shape[0] == d))
      return fail(SVODK_ERR_SHAPE, "%s: %s has shape %s, expected [%lld]", op, vec_names[i], fmt_shape(vecs[i]).c_str(),
                  (long long)d);
  // L61-64: the residual has x's shape.
  if (residual != nullptr && !same_shape(residual, x))
    return fail(SVODK_ERR_SHAPE, "%s: residual has shape %s, expected %s", op, fmt_shape(residual).c_str(),
                fmt_shape(x).c_str());
  // The outputs the reference op allocates itself (L88-89): here the caller's.
  const svodk_tensor *outs[2] = {out, sum};
  const char *out_names[2] = {"out", "sum"};
  for (int i = 0; i < 2; i++) {
    if (outs[i] == nullptr) continue;
    if (!same_shape(outs[i], x))
      return fail(SVODK_ERR_SHAPE, "%s: %s has shape %s, expected %s", op, out_names[i], fmt_shape(outs[i]).c_str(),
                  fmt_shape(x).c_str());
    if (outs[i]->dtype != x->dtype)
      return fail(SVODK_ERR_DTYPE, "%s: %s is %s, the input is %s", op, out_names[i], dtype_name(outs[i]->dtype),
                  dtype_name(x->dtype));
  }
  const int64_t cap = x->shape[0];
  if (batch_live > cap)
    return fail(SVODK_ERR_SHAPE, "%s: live batch %d exceeds the capacity %lld", op, batch_live, (long long)cap);

  // L66-71: the plan over every operand's type.
  int32_t dtypes[4];
  int n = 0;
  dtypes[n++] = x->dtype;
  if (residual) dtypes[n++] = residual->dtype;
  dtypes[n++] = w->dtype;
  if (b) dtypes[n++] = b->dtype;
  const int why = plan_norm(current_device_has_kernels(), dtypes, n, x->shape, x->rank);
  if (why != 0) return ran_graph(op, why);

  const size_t bytes = (size_t)numel(x) * 2;
  Span spans[6] = {{"x", x->data, bytes, false},
                   {"residual", residual ? residual->data : nullptr, residual ? bytes : 0, false},
                   {"w", w->data, (size_t)d * 2, false},
                   {"b", b ? b->data : nullptr, b ? (size_t)d * 2 : 0, false},
                   {"out", out->data, bytes, true},
                   {"sum", sum ? sum->data : nullptr, sum ? bytes : 0, true}};
  if (x->data == nullptr || w->data == nullptr || out->data == nullptr || (b && b->data == nullptr) ||
      (residual && residual->data == nullptr) || (sum && sum->data == nullptr))
    return fail(SVODK_ERR_ARGUMENT, "%s: a null device pointer", op);
  {
    const svodk_tensor *checked[6] = {x, residual, w, b, out, sum};
    const int bad = misaligned(checked, 6);
    if (bad >= 0) return fail(SVODK_ERR_ARGUMENT, "%s: %s is not 16-byte aligned", op, spans[bad].name);
  }
  if (int rc = check_aliasing(op, spans, 6)) return rc;

  svodk::NormArgs a{};
  a.x = x->data;
  a.residual = residual ? residual->data : nullptr;
  a.w = w->data;
  a.b = (layer && b) ? b->data : nullptr;
  a.out = out->data;
  a.sum = sum ? sum->data : nullptr;
  // L74-76: the rows are every dim before the last; a bound leading batch runs its live part.
  const int64_t per_batch = x->rank > 1 ? numel(x) / (cap * d) : 1;
  a.rows = x->rank > 1 ? (batch_live > 0 ? batch_live : cap) * per_batch : 1;
  a.d = (int32_t)d;
  a.eps = eps;
  a.layer = layer;
  a.f16 = x->dtype == SVODK_F16;
  ran(op, op, "NormCfg { br: 4 }");
  const hipError_t e = svodk::launch_norm(a, (hipStream_t)hip_stream);
  if (e != hipSuccess) return fail(SVODK_ERR_LAUNCH, "%s: %s", op, hipGetErrorString(e));
  return SVODK_KERNEL;
}

int svodk_layer_norm(const svodk_tensor *x, const svodk_tensor *w, const svodk_tensor *b, double eps, int32_t batch_live,
                     const svodk_tensor *out, void *hip_stream) {
  return norm(true, x, nullptr, w, b, eps, batch_live, nullptr, out, hip_stream);
}

int svodk_add_layer_norm(const svodk_tensor *x, const svodk_tensor *residual, const svodk_tensor *w,
                         const svodk_tensor *b, double eps, int32_t batch_live, const svodk_tensor *sum,
                         const svodk_tensor *out, void *hip_stream) {
  if (residual == nullptr || sum == nullptr)
    return fail(SVODK_ERR_ARGUMENT, "layer_norm: add_layer_norm needs a residual and a sum");
  return norm(true, x, residual, w, b, eps, batch_live, sum, out, hip_stream);
}

int svodk_rms_norm(const svodk_tensor *x, const svodk_tensor *w, double eps, int32_t batch_live, const svodk_tensor *out,
                   void *hip_stream) {
  return norm(false, x, nullptr, w, nullptr, eps, batch_live, nullptr, out, hip_stream);
}

int svodk_add_rms_norm(const svodk_tensor *x, const svodk_tensor *residual, const svodk_tensor *w, double eps,
                       int32_t batch_live, const svodk_tensor *sum, const svodk_tensor *out, void *hip_stream) {
  if (residual == nullptr || sum == nullptr)
    return fail(SVODK_ERR_ARGUMENT, "rms_norm: add_rms_norm needs a residual and a sum");
  return norm(false, x, residual, w, nullptr, eps, batch_live, sum, out, hip_stream);
}

// shape::linear (tk/src/ops/shape.rs:120-139): the gate, a reduced dim, columns in vector runs
// of 8, rows; then this library's own: the k-columns in whole stages of the kernel's ring.
static int plan_linear(bool has_target, const int32_t *dtypes, int n_dtypes, const int64_t *x, int rank, int64_t n) {
  if (int why = gate(has_target, dtypes, n_dtypes)) return why;
  if (x == nullptr) return SVODK_GRAPH_SYMBOLIC;
  if (rank < 1) return SVODK_GRAPH_SHAPE;
  int64_t rows = 1;
  for (int i = 0; i + 1 < rank; i++) rows *= x[i];
  if (n % 8 != 0 || rows == 0 || n <= 0) return SVODK_GRAPH_SHAPE;
  if (!svodk::linear_supports(n, x[rank - 1])) return SVODK_GRAPH_SHAPE;
  return 0;
}

int svodk_plan_linear(int32_t has_target, const int32_t *dtypes, int32_t n_dtypes, const int64_t *x_dims, int32_t x_rank,
                      int64_t n) {
  return plan_linear(has_target != 0, dtypes, n_dtypes, x_dims, x_rank, n);
}

// linear (tk/src/ops/linear.rs:60-231).
int svodk_linear(const svodk_tensor *x, const svodk_tensor *w, const svodk_linear_opts *opts, const svodk_tensor *out,
                 void *hip_stream) {
  const char *op = "linear";
  if (!well_formed(x) || !well_formed(w) || !well_formed(out) || opts == nullptr)
    return fail(SVODK_ERR_ARGUMENT, "%s: a null or malformed tensor descriptor", op);
  // L66-68: x is [..., K], w is [N, K] of x's type.
  if (x->rank < 1) return fail(SVODK_ERR_SHAPE, "%s: x has shape %s, expected [..., K]", op, fmt_shape(x).c_str());
  const int64_t k = x->shape[x->rank - 1];
  if (!(w->rank == 2 && w->shape[1] == k))
    return fail(SVODK_ERR_SHAPE, "%s: w has shape %s, expected [N, %lld]", op, fmt_shape(w).c_str(), (long long)k);
  if (w->dtype != x->dtype)
    return fail(SVODK_ERR_DTYPE, "%s: w is %s, the input is %s", op, dtype_name(w->dtype), dtype_name(x->dtype));
  // L69-73: a gated weight holds gate rows over up rows.
  int64_t n = w->shape[0];
  if (opts->gated) {
    if (n % 2 != 0) return fail(SVODK_ERR_SHAPE, "%s: w has shape %s, expected [2N, %lld]", op, fmt_shape(w).c_str(), (long long)k);
    n /= 2;
  }
  // L74-77: the bias is [rows of w].
  if (opts->bias != nullptr) {
    if (!well_formed(opts->bias)) return fail(SVODK_ERR_ARGUMENT, "%s: bias descriptor malformed", op);
    if (!(opts->bias->rank == 1 && opts->bias->shape[0] == w->shape[0]))
      return fail(SVODK_ERR_SHAPE, "%s: bias has shape %s, expected [%lld]", op, fmt_shape(opts->bias).c_str(),
                  (long long)w->shape[0]);
  }
  // The output the reference op allocates itself (L203-206): [lead..., N] of x's type.
  // With `into` (L40-42, tk/src/ops/mod.rs:459-477) it is the caller's wider tensor [lead..., C], channels
  // into_at .. into_at + N of which take the result.
  const int64_t out_ld = out->rank >= 1 ? out->shape[out->rank - 1] : 0;
  bool out_fits = out->rank == x->rank &&
                  (opts->has_into ? (opts->into_at >= 0 && opts->into_at + n <= out_ld) : out_ld == n);
  for (int i = 0; out_fits && i + 1 < x->rank; i++) out_fits = out->shape[i] == x->shape[i];
  // L79-82: the residual has the output's shape.
  if (opts->residual != nullptr) {
    if (!well_formed(opts->residual)) return fail(SVODK_ERR_ARGUMENT, "%s: residual descriptor malformed", op);
    bool fits = opts->residual->rank == x->rank && opts->residual->shape[x->rank - 1] == n;
    for (int i = 0; fits && i + 1 < x->rank; i++) fits = opts->residual->shape[i] == x->shape[i];
    if (!fits) return fail(SVODK_ERR_SHAPE, "%s: residual has shape %s, expected [lead..., %lld]", op,
                           fmt_shape(opts->residual).c_str(), (long long)n);
  }
  // L83-93: a rope wants x [B, T, K] under a plain weight, whole even heads inside N, tables [1, T, 1, d/2].
  const svodk_rotary *rope = opts->rope;
  if (rope != nullptr) {
    if (!(x->rank == 3 && !opts->gated))
      return fail(SVODK_ERR_SHAPE, "%s: x has shape %s, expected [B, T, K] under a plain weight", op, fmt_shape(x).c_str());
    const bool fits = rope->head_dim > 0 && rope->head_dim % 2 == 0 && rope->heads >= 0 &&
                      (int64_t)rope->heads * rope->head_dim <= n;
    if (!fits)
      return fail(SVODK_ERR_SHAPE, "%s: w has shape %s, expected [>= %d\xc2\xb7%d, %lld] of even heads", op,
                  fmt_shape(w).c_str(), rope->heads, rope->head_dim, (long long)k);
    const svodk_tensor *tables[2] = {rope->cos, rope->sin};
    const char *names[2] = {"cos", "sin"};
    for (int i = 0; i < 2; i++) {
      if (!well_formed(tables[i])) return fail(SVODK_ERR_ARGUMENT, "%s: %s descriptor malformed", op, names[i]);
      const svodk_tensor *tb = tables[i];
      if (!(tb->rank == 4 && tb->shape[0] == 1 && tb->shape[1] == x->shape[1] && tb->shape[2] == 1 &&
            tb->shape[3] == rope->head_dim / 2))
        return fail(SVODK_ERR_SHAPE, "%s: %s has shape %s, expected [1, %lld, 1, %d]", op, names[i], fmt_shape(tb).c_str(),
                    (long long)x->shape[1], rope->head_dim / 2);
    }
  }
  if (!out_fits && opts->has_into)
    return fail(SVODK_ERR_SHAPE, "%s: into has shape %s, expected [lead..., %lld] widened to hold channels %lld.. past the last axis",
                op, fmt_shape(out).c_str(), (long long)n, (long long)opts->into_at);
  if (!out_fits)
    return fail(SVODK_ERR_SHAPE, "%s: out has shape %s, expected [lead..., %lld]", op, fmt_shape(out).c_str(), (long long)n);
  if (out->dtype != x->dtype)
    return fail(SVODK_ERR_DTYPE, "%s: out is %s, the input is %s", op, dtype_name(out->dtype), dtype_name(x->dtype));
  const int64_t cap = x->shape[0];
  if (opts->batch_live > cap)
    return fail(SVODK_ERR_SHAPE, "%s: live batch %d exceeds the capacity %lld", op, opts->batch_live, (long long)cap);

  // L107-127: the plan over every operand's type.
  int32_t dtypes[4];
  int nd = 0;
  dtypes[nd++] = x->dtype;
  dtypes[nd++] = w->dtype;
  if (opts->bias) dtypes[nd++] = opts->bias->dtype;
  if (opts->residual) dtypes[nd++] = opts->residual->dtype;
  const int why = plan_linear(current_device_has_kernels(), dtypes, nd, x->shape, x->rank, n);
  if (why != 0) return ran_graph(op, why);
  // The parts of the reference's GEMM family this library has no kernel for keep the graph; so does a
  // turn beside an activation, a residual or a scale (L135-141: the graph rotates before them).
  if (opts->act != SVODK_ACT_NONE || opts->gated || opts->residual != nullptr || opts->has_scale)
    return ran_graph(op, SVODK_GRAPH_CONFIG);
  if (rope != nullptr) {
    // L142-143: tables off the stream dtype leave the turn to the graph.
    if (rope->cos->dtype != x->dtype || rope->sin->dtype != x->dtype) return ran_graph(op, SVODK_GRAPH_DTYPE);
    // L176-184: no tile turns heads of this size.
    if (!svodk::linear_turns(rope->head_dim)) return ran_graph(op, SVODK_GRAPH_CONFIG);
  }
  // tk/src/ops/mod.rs:475-476: a window the kernel's 16-byte stores cannot land in is the graph's to store.
  if (opts->has_into && (opts->into_at % 8 != 0 || out_ld % 8 != 0)) return ran_graph(op, SVODK_GRAPH_CONFIG);
  int64_t lead = 1;
  for (int i = 1; i + 1 < x->rank; i++) lead *= x->shape[i];
  const int64_t live = x->rank > 1 ? (opts->batch_live > 0 ? opts->batch_live : cap) : 1;
  const int64_t rows = x->rank > 1 ? live * lead : 1;
  if (n > 0x7fffffff || (rope && x->shape[1] > 0x7fffffff)) return ran_graph(op, SVODK_GRAPH_SHAPE);

  const size_t table_bytes = rope ? (size_t)numel(rope->cos) * 2 : 0;
  Span spans[6] = {{"x", x->data, (size_t)numel(x) * 2, false},
                   {"w", w->data, (size_t)numel(w) * 2, false},
                   {"bias", opts->bias ? opts->bias->data : nullptr, opts->bias ? (size_t)numel(opts->bias) * 2 : 0, false},
                   {"cos", rope ? rope->cos->data : nullptr, table_bytes, false},
                   {"sin", rope ? rope->sin->data : nullptr, table_bytes, false},
                   {"out", out->data, (size_t)numel(out) * 2, true}};
  if (x->data == nullptr || w->data == nullptr || out->data == nullptr || (opts->bias && opts->bias->data == nullptr) ||
      (rope && (rope->cos->data == nullptr || rope->sin->data == nullptr)))
    return fail(SVODK_ERR_ARGUMENT, "%s: a null device pointer", op);
  for (const Span &sp : spans)
    if (sp.data != nullptr && ((uintptr_t)sp.data & 15u) != 0)
      return fail(SVODK_ERR_ARGUMENT, "%s: %s is not 16-byte aligned", op, sp.name);
  if (int rc = check_aliasing(op, spans, 6)) return rc;

  svodk::LinearArgs a{};
  a.x = x->data;
  a.w = w->data;
  a.bias = opts->bias ? opts->bias->data : nullptr;
  a.cos = rope ? rope->cos->data : nullptr;
  a.sin = rope ? rope->sin->data : nullptr;
  a.y = (uint16_t *)out->data + (opts->has_into ? opts->into_at : 0);
  a.y_ld = opts->has_into ? out_ld : n;
  a.rows = rows;
  a.n = (int32_t)n;
  a.k = (int32_t)k;
  a.seq = rope ? (int32_t)x->shape[1] : 1;
  a.heads = rope ? rope->heads : 0;
  a.head_dim = rope ? rope->head_dim : 0;
  a.f16 = x->dtype == SVODK_F16;
  a.tile = svodk::linear_tile_of(rows, n, current_device_units());
  if (a.tile == 128)
    ran(op, "gemm", rope ? "GemmCfg { bm: 128, bn: 128, bk: 64, stages: 2, warps: [4, 1], epilogue: { bias, rope } }"
                         : "GemmCfg { bm: 128, bn: 128, bk: 64, stages: 2, warps: [4, 1], epilogue: { bias } }");
  else
    ran(op, "gemm", rope ? "GemmCfg { bm: 256, bn: 256, bk: 64, stages: 2, warps: [4, 2], epilogue: { bias, rope } }"
                         : "GemmCfg { bm: 256, bn: 256, bk: 64, stages: 2, warps: [4, 2], epilogue: { bias } }");
  const hipError_t e = svodk::launch_linear(a, (hipStream_t)hip_stream);
  if (e != hipSuccess) return fail(SVODK_ERR_LAUNCH, "%s: %s", op, hipGetErrorString(e));
  return SVODK_KERNEL;
}

int svodk_plan_norm(int32_t has_target, const int32_t *dtypes, int32_t n_dtypes, const int64_t *x_dims, int32_t x_rank) {
  return plan_norm(has_target != 0, dtypes, n_dtypes, x_dims, x_rank);
}

}  // extern "C"

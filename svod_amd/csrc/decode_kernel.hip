// The decoder step of flash attention for gfx950: a call whose (batch, KV head) has at most four query rows
// (one new token, or a few, for the heads of a KV head's group), without a causal or per-row mask or a bias.
//
// Such a call is a stream of K and V past a handful of queries (tk/src/kernels/attention.rs:466-924 is the
// program whose results it reproduces; nothing in it is a matrix product worth a matrix instruction): its time is
// the bytes of K and V over what the memory system delivers, and what it delivers is set by the bytes a compute
// unit has in flight.  The tile kernel holds 48 KiB a compute unit in its LDS rings and waits for each step's
// fills before the next; here every lane loads its 16 bytes of a key row straight into registers, several
// rows ahead, with no LDS and no barrier in the loop, and a compute unit holds a few hundred KiB in flight.
//
//   a key row of D elements is shared by D/8 lanes (16 bytes each); a wave instruction covers 512/D rows
//   score:   v_dot2_f32 over the lane's four pairs, summed over the row's lanes by DPP
//   softmax: every lane runs the online form over the keys of its own place in the wave, in the exponent's
//            units (scores scaled first, L365-370); probabilities stay f32 where the tile program rounds them
//            to the operands' type for its second matrix product (L432-444)
//   at the end the places of a wave, then the waves of the workgroup, merge their states (m, l, o) as key
//   splits do (L948-1014), and the workgroup writes the output rows, or with key splits its partial state for
//   combine_kernel (L899-921).
#include <hip/hip_runtime.h>

#include <atomic>

#include "kernels.h"

namespace svodk {
namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNoKey = -1e30f;   // the running maximum before any key: finite, so that its differences are numbers
constexpr int kMaxWaves = 8;       // waves a workgroup
constexpr int kAhead = 2;          // passes a lane works on at a time, with as many more in flight

// What the kernel takes: AttnArgs without the fields a decoder step does not have.
struct DecodeArgs {
  const uint16_t *q, *k, *v;
  uint16_t *o;
  const void *key_lens, *key_mask;
  const void *row_map;
  const uint16_t *k_app, *v_app;
  const void *app_lens;
  float *o_part, *m_part, *l_part;
  int64_t q_row_elems, kv_row_elems;
  int32_t lens_i64, mask_bytes, row_map_i64, app_lens_i64;
  int32_t batch, t, tk, heads, kv_heads, group;
  int32_t splits, cached, kv_head_start, cache_rows, app_rows;
  float scale;
};

template <bool F16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  f32x2 f = {lo, hi};
  if constexpr (F16)
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
  else
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}
// The two 16-bit values of a word as f32.
template <bool F16>
__device__ __forceinline__ f32x2 unpack2(uint32_t x) {
  if constexpr (F16) {
    return __builtin_convertvector(__builtin_bit_cast(f16x2, x), f32x2);
  } else {
    return f32x2{__uint_as_float(x << 16), __uint_as_float(x & 0xffff0000u)};
  }
}
// c + a.lo * b.lo + a.hi * b.hi
template <bool F16>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
  if constexpr (F16)
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
  else
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
}
// x of the lane a DPP control names.
template <int CTRL>
__device__ __forceinline__ float moved(float x) {
  return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(x), CTRL, 0xf, 0xf, true));
}
// x summed over the LANES (4, 8, 16 or 32) neighbouring lanes that share a key row; every one of them gets the sum.
template <int LANES>
__device__ __forceinline__ float sum_over(float x) {
  x += moved<0xB1>(x);                              // quad_perm [1,0,3,2]
  x += moved<0x4E>(x);                              // quad_perm [2,3,0,1]
  if constexpr (LANES >= 8) x += moved<0x141>(x);   // row_half_mirror
  if constexpr (LANES >= 16) x += moved<0x140>(x);  // row_mirror
  if constexpr (LANES >= 32) x += __shfl_xor(x, 16, 64);
  return x;
}

// The online-softmax state of one query row over some of the keys: the lane's eight output columns.
struct State {
  float m, l, acc[8];
};
// `a` takes in `b` (the merge of two key splits, L948-1014).
__device__ __forceinline__ void merge(State &a, const State &b) {
#pragma clang fp contract(off)  // the products and sums as written, wherever this is inlined
  const float m = __builtin_fmaxf(a.m, b.m);
  const float wa = __builtin_amdgcn_exp2f(a.m - m), wb = __builtin_amdgcn_exp2f(b.m - m);
  a.m = m;
  a.l = a.l * wa + b.l * wb;
#pragma unroll
  for (int j = 0; j < 8; j++) a.acc[j] = a.acc[j] * wa + b.acc[j] * wb;
}

// The workgroup's program for `nw` waves, for the kernels below to inline.
template <int D, int R, bool F16, bool SPLIT>
__device__ __forceinline__ void decode_body(const DecodeArgs &p, const int nw) {
#if defined(__HIP_DEVICE_COMPILE__)
  // No contraction beyond the fused multiply-adds written out below: the library's kernel (its wave count a launch
  // argument) and a code object's (four waves, known to the compiler) are then the same arithmetic bit for bit.
#pragma clang fp contract(off)
  constexpr int kWide = D == 48 ? 64 : D;
  constexpr int LPK = kWide / 8;   // lanes a key row
  constexpr int KPI = 64 / LPK;    // key rows a wave instruction
  constexpr int U = kAhead;  // the same for every R: a row's arithmetic does not depend on how many rows share the keys
  __shared__ float merged[kMaxWaves][R][LPK][10];

  const int wg = (int)__builtin_amdgcn_workgroup_id_x();
  const int split = SPLIT ? wg % p.splits : 0;
  const int unit = SPLIT ? wg / p.splits : wg;
  const int b = unit / p.kv_heads;
  const int kvh = unit - b * p.kv_heads;
  const int tid = (int)__builtin_amdgcn_workitem_id_x();
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pos = lane % LPK;   // which 16 bytes of a row
  const int slot = lane / LPK;  // which row of a wave instruction
  const bool pos_ok = 8 * pos < D;

  // L533-536: len = min(key_lens[b], tk).
  const int tk = p.tk;
  int len = tk;
  if (p.key_lens != nullptr) {
    long long n = p.lens_i64 ? ((const long long *)p.key_lens)[b] : (long long)((const int *)p.key_lens)[b];
    n = n < 0 ? 0 : n;
    len = n < (long long)tk ? (int)n : tk;
  }
  // L609-612: a split takes an even share of the 64-key blocks below the length.
  int k0 = 0, k1 = len;
  if (SPLIT) {
    const int n = (len + 63) / 64;
    k0 = (int)((int64_t)n * split / p.splits) * 64;
    k1 = min(len, (int)((int64_t)n * (split + 1) / p.splits) * 64);
  }
  // L544-550: a cache is read at the batch lane's row of it, from the launch's first head on.
  int64_t kv_row = b;
  int kv_col = kvh;
  if (p.cached) {
    if (p.row_map != nullptr) {
      const long long x = p.row_map_i64 ? ((const long long *)p.row_map)[b] : (long long)((const int *)p.row_map)[b];
      kv_row = x < 0 ? 0 : (x < p.cache_rows ? x : p.cache_rows - 1);
    }
    kv_col += p.kv_head_start;
  }

  // The rows: row r is token r % t of the group's head r / t (a grouped tile's order).
  const int rows = p.group * p.t;
  uint32_t qf[R][4];
  int64_t out_row[R];
#pragma unroll
  for (int r = 0; r < R; r++) {
    const int rr = min(r, rows - 1);
    const int in_group = rr / p.t;
    const int q_row = rr - in_group * p.t;
    const int q_head = kvh * p.group + in_group;
    out_row[r] = ((int64_t)b * p.t + q_row) * p.heads + q_head;
    const uint16_t *at = p.q + ((int64_t)b * p.t + q_row) * p.q_row_elems + (int64_t)q_head * D + 8 * pos;
    u32x4 x = {0, 0, 0, 0};
    if (pos_ok && r < rows) x = *reinterpret_cast<const u32x4 *>(at);
#pragma unroll
    for (int i = 0; i < 4; i++) qf[r][i] = x[i];
  }

  const float c_exp = p.scale * kLog2e;  // L619
  State st[R];
#pragma unroll
  for (int r = 0; r < R; r++) {
    st[r].m = kNoKey;
    st[r].l = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) st[r].acc[j] = 0.0f;
  }

  // Keys [from, to) of rows `row_elems` apart at kb / vb (this lane's 16 bytes of the first row), `mask` their
  // visibility bytes or words (null: all visible).  A pass of the workgroup is nw * KPI rows; a lane works on U
  // passes at a time and has the next U in flight meanwhile.  The workgroup starts `turn` such chunks into the
  // range and wraps: the softmax does not care where it starts, and the memory does.  Rows of a cache are very
  // often a power of two apart, and so are the batch rows; workgroups that all walk from key 0 then ask the same
  // few memory channels for their rows at the same time (a [64, 512, 128, 64] cache read one layer's 32 heads at a
  // time: 3.8 TB/s from key 0, 5.2 with the starts spread; rows 20 or 80 KiB apart stream the same either way).
  auto stream = [&](const uint16_t *kb, const uint16_t *vb, int64_t row_elems, int from, int to, const void *mask,
                    int mask_bytes, uint32_t turn) {
    const int pass = nw * KPI;
    struct Rows {
      u32x4 k[U], v[U];
      int seen[U];
    };
    auto load = [&](Rows &x, int key0) {
#pragma unroll
      for (int u = 0; u < U; u++) {
        const int key = key0 + u * pass;
        const bool there = key < to;
        x.k[u] = u32x4{0, 0, 0, 0};
        x.v[u] = u32x4{0, 0, 0, 0};
        x.seen[u] = there ? 1 : 0;
        if (there && pos_ok) {
          x.k[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(kb + (int64_t)key * row_elems));
          x.v[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(vb + (int64_t)key * row_elems));
        }
        if (there && mask != nullptr)
          x.seen[u] = mask_bytes == 1 ? (int)((const uint8_t *)mask)[key] : ((const int *)mask)[key];
      }
    };
    // The softmax and the second product of the U passes in `x`.
    auto work = [&](Rows &x) {
      float e[U][R];
#pragma unroll
      for (int u = 0; u < U; u++) {
        const bool seen = x.seen[u] != 0;
        if (mask != nullptr && !seen) x.v[u] = u32x4{0, 0, 0, 0};  // a hidden row weighs nothing, whatever it holds
#pragma unroll
        for (int r = 0; r < R; r++) {
          float s = 0.0f;
#pragma unroll
          for (int i = 0; i < 4; i++) s = dot2<F16>(x.k[u][i], qf[r][i], s);
          s = sum_over<LPK>(s);
          e[u][r] = seen ? s * c_exp : -__builtin_inff();
        }
      }
#pragma unroll
      for (int r = 0; r < R; r++) {
        float m = st[r].m;
#pragma unroll
        for (int u = 0; u < U; u++) m = __builtin_fmaxf(m, e[u][r]);
        const float corr = __builtin_amdgcn_exp2f(st[r].m - m);
        st[r].m = m;
        st[r].l *= corr;
#pragma unroll
        for (int j = 0; j < 8; j++) st[r].acc[j] *= corr;
        float pr[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
          pr[u] = __builtin_amdgcn_exp2f(e[u][r] - m);
          st[r].l += pr[u];
        }
#pragma unroll
        for (int u = 0; u < U; u += 2) {
          const float held[2] = {pr[u], pr[u + 1]};
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const f32x2 a = unpack2<F16>(x.v[u][i]), c = unpack2<F16>(x.v[u + 1][i]);
            st[r].acc[2 * i] = __builtin_fmaf(held[0], a[0], st[r].acc[2 * i]);
            st[r].acc[2 * i + 1] = __builtin_fmaf(held[0], a[1], st[r].acc[2 * i + 1]);
            st[r].acc[2 * i] = __builtin_fmaf(held[1], c[0], st[r].acc[2 * i]);
            st[r].acc[2 * i + 1] = __builtin_fmaf(held[1], c[1], st[r].acc[2 * i + 1]);
          }
        }
      }
    };
    // Two sets of rows take turns: one is worked on while the other is on its way.
    if (from + wave * KPI >= to) return;  // no chunk holds a row of this wave's
    const int chunk = U * pass, chunks = (to - from + chunk - 1) / chunk;
    const int first = (int)(turn % (uint32_t)chunks);
    // This lane's first row of the i-th chunk the workgroup takes; past the last chunk, a row that is not there.
    auto row_of = [&](int i) {
      if (i >= chunks) return to;
      int c = first + i;
      if (c >= chunks) c -= chunks;
      return from + c * chunk + wave * KPI + slot;
    };
    Rows one, two;
    load(one, row_of(0));
    for (int i = 0; i < chunks; i += 2) {
      load(two, row_of(i + 1));
      work(one);
      load(one, row_of(i + 2));
      if (i + 1 < chunks) work(two);
    }
  };

  {
    const int64_t at = (kv_row * tk) * p.kv_row_elems + (int64_t)kv_col * D + 8 * pos;
    const void *mask = nullptr;
    if (p.key_mask != nullptr) mask = (const uint8_t *)p.key_mask + (int64_t)b * tk * p.mask_bytes;
    // Turned by where the keys lie (the cache row, and the split's share of it), not by who asks: a batch lane
    // mapped to another cache row reads it as that row's own lane would.  The heads of a row stay in step:
    // their pieces of a key row lie side by side.
    stream(p.k + at, p.v + at, p.kv_row_elems, k0, k1, mask, p.mask_bytes, (uint32_t)kv_row * 7u + (uint32_t)split * 3u);
  }
  // The appended rows (L739-755, L827-846): scored by the last split after the cached keys, the first
  // app_lens[b] of them visible, from tensors of their own.
  if (p.cached && p.k_app != nullptr && (!SPLIT || split == p.splits - 1)) {
    int seen = p.app_rows;
    if (p.app_lens != nullptr) {
      const long long n = p.app_lens_i64 ? ((const long long *)p.app_lens)[b] : (long long)((const int *)p.app_lens)[b];
      seen = (int)(n < 0 ? 0 : (n < seen ? n : seen));
    }
    const int64_t at = ((int64_t)b * p.app_rows * p.kv_heads + kvh) * D + 8 * pos;
    stream(p.k_app + at, p.v_app + at, (int64_t)p.kv_heads * D, 0, seen, nullptr, 1, 0u);
  }

  // The places of a wave that share output columns (lanes LPK apart) merge, then the waves.
#pragma unroll
  for (int r = 0; r < R; r++) {
#pragma unroll
    for (int step = LPK; step < 64; step <<= 1) {
      State other;
      other.m = __shfl_xor(st[r].m, step, 64);
      other.l = __shfl_xor(st[r].l, step, 64);
#pragma unroll
      for (int j = 0; j < 8; j++) other.acc[j] = __shfl_xor(st[r].acc[j], step, 64);
      merge(st[r], other);
    }
    if (slot == 0) {
      float *at = merged[wave][r][pos];
      at[0] = st[r].m;
      at[1] = st[r].l;
#pragma unroll
      for (int j = 0; j < 8; j++) at[2 + j] = st[r].acc[j];
    }
  }
  __syncthreads();
  if (wave != 0 || slot != 0 || !pos_ok) return;
#pragma unroll
  for (int r = 0; r < R; r++) {
    if (r >= rows) break;
    State all = st[r];
    for (int w = 1; w < nw; w++) {
      State other;
      const float *at = merged[w][r][pos];
      other.m = at[0];
      other.l = at[1];
#pragma unroll
      for (int j = 0; j < 8; j++) other.acc[j] = at[2 + j];
      merge(all, other);
    }
    if (SPLIT) {
      // L899-921: the accumulator as it stands, the maximum in the exponent's units, the sum.
      const int64_t at = (int64_t)split * p.batch * p.t * p.heads + out_row[r];
      if (pos == 0) {
        p.m_part[at] = all.m;
        p.l_part[at] = all.l;
      }
      f32x4 *to = reinterpret_cast<f32x4 *>(p.o_part + at * D + 8 * pos);
      to[0] = f32x4{all.acc[0], all.acc[1], all.acc[2], all.acc[3]};
      to[1] = f32x4{all.acc[4], all.acc[5], all.acc[6], all.acc[7]};
    } else {
      // L892-898: out = o / (l == 0 ? 1 : l).
      const float inv = 1.0f / (all.l == 0.0f ? 1.0f : all.l);
      u32x4 out;
#pragma unroll
      for (int i = 0; i < 4; i++) out[i] = pack2<F16>(all.acc[2 * i] * inv, all.acc[2 * i + 1] * inv);
      *reinterpret_cast<u32x4 *>(p.o + out_row[r] * D + 8 * pos) = out;
    }
  }
#endif  // __HIP_DEVICE_COMPILE__
}

#if !defined(SVODK_CODE_OBJECT)  // the library's kernel and its launch: not part of a code object build
template <int D, int R, bool F16, bool SPLIT>
__global__ __launch_bounds__(kMaxWaves * 64) void decode_kernel(const DecodeArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  decode_body<D, R, F16, SPLIT>(p, (int)(__builtin_amdgcn_workgroup_size_x() >> 6));
#endif
}

template <int D, int R, bool F16>
hipError_t launch_r(const DecodeArgs &p, int waves, hipStream_t stream) {
  const int64_t grid = (int64_t)p.batch * p.kv_heads * p.splits;
  if (grid == 0) return hipSuccess;
  if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
  if (p.splits > 1)
    hipLaunchKernelGGL((decode_kernel<D, R, F16, true>), dim3((uint32_t)grid), dim3(waves * 64), 0, stream, p);
  else
    hipLaunchKernelGGL((decode_kernel<D, R, F16, false>), dim3((uint32_t)grid), dim3(waves * 64), 0, stream, p);
  return hipGetLastError();
}

template <int D>
hipError_t launch_d(const DecodeArgs &p, int rows, int waves, bool f16, hipStream_t stream) {
  if (rows <= 1) return f16 ? launch_r<D, 1, true>(p, waves, stream) : launch_r<D, 1, false>(p, waves, stream);
  if (rows <= 2) return f16 ? launch_r<D, 2, true>(p, waves, stream) : launch_r<D, 2, false>(p, waves, stream);
  return f16 ? launch_r<D, 4, true>(p, waves, stream) : launch_r<D, 4, false>(p, waves, stream);
}

std::atomic<int> g_decode_rows{kDecodeRowsDefault};

}  // namespace

void attention_decode_rows(int32_t rows) {
  g_decode_rows.store(rows < 0 ? 0 : (rows > kDecodeRows ? kDecodeRows : rows), std::memory_order_relaxed);
}

int32_t attention_decode_limit() { return g_decode_rows.load(std::memory_order_relaxed); }

bool attention_decodes(const AttnArgs &a) {
  const bool ranged = a.win_left >= 0 || a.chunk_size > 0 || a.seg_start != nullptr;
  if (a.causal || ranged || a.bias != nullptr || a.kv_heads <= 0 || a.heads % a.kv_heads != 0) return false;
  const int64_t rows = (int64_t)(a.heads / a.kv_heads) * a.t;
  return rows >= 1 && rows <= g_decode_rows.load(std::memory_order_relaxed);
}

hipError_t launch_decode(const AttnArgs &a, hipStream_t stream) {
  DecodeArgs p;
  p.q = (const uint16_t *)a.q;
  p.k = (const uint16_t *)a.k;
  p.v = (const uint16_t *)a.v;
  p.o = (uint16_t *)a.o;
  p.key_lens = a.key_lens;
  p.key_mask = a.key_mask;
  p.row_map = a.row_map;
  p.k_app = (const uint16_t *)a.k_app;
  p.v_app = (const uint16_t *)a.v_app;
  p.app_lens = a.app_lens;
  p.o_part = a.o_part;
  p.m_part = a.m_part;
  p.l_part = a.l_part;
  p.q_row_elems = a.q_row_elems > 0 ? a.q_row_elems : (int64_t)a.heads * a.d;
  p.kv_row_elems = a.kv_row_elems > 0 ? a.kv_row_elems : (int64_t)a.kv_heads * a.d;
  p.lens_i64 = a.lens_i64;
  p.mask_bytes = a.mask_bytes;
  p.row_map_i64 = a.row_map_i64;
  p.app_lens_i64 = a.app_lens_i64;
  p.batch = a.batch;
  p.t = a.t;
  p.tk = a.tk;
  p.heads = a.heads;
  p.kv_heads = a.kv_heads;
  p.group = a.heads / a.kv_heads;
  p.splits = a.splits > 1 ? a.splits : 1;
  p.cached = a.cached;
  p.kv_head_start = a.kv_head_start;
  p.cache_rows = a.cache_rows;
  p.app_rows = a.app_rows;
  p.scale = a.scale;
  if (p.splits > 1 && (a.o_part == nullptr || a.m_part == nullptr || a.l_part == nullptr)) return hipErrorInvalidValue;
  const int rows = p.group * p.t;
  // Few workgroups take eight waves each, so that the launch still has its bytes in flight.
  const int64_t grid = (int64_t)p.batch * p.kv_heads * p.splits;
  const int waves = grid >= 256 ? 4 : kMaxWaves;
  switch (a.d) {
    case 32: return launch_d<32>(p, rows, waves, a.f16 != 0, stream);
    case 48: return launch_d<48>(p, rows, waves, a.f16 != 0, stream);
    case 64: return launch_d<64>(p, rows, waves, a.f16 != 0, stream);
    case 128: return launch_d<128>(p, rows, waves, a.f16 != 0, stream);
    case 256: return launch_d<256>(p, rows, waves, a.f16 != 0, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace svodk

#else  // SVODK_CODE_OBJECT
}  // namespace
}  // namespace svodk
// ---------------------------------------------------------------------------------------------
// The same program as kernels a loader outside the HIP runtime can run (a flat argument record, static LDS, no
// dispatch packet: the workgroup is 256 threads, which the kernel cannot ask and therefore fixes).  One kernel an
// instantiation, svodk_decode_d<D>_r<rows>_<type>_s<split>, all with one record.  Buffers, an address of 0 for what
// a call does not have: q, k, v, o, key_lens, key_mask, row_map, k_app, v_app, app_lens, then the partial states of
// a split call o_part, m_part, l_part.  Scalars: batch, t, tk, heads, kv_heads, scale_bits, lens_i64, mask_bytes (1 or
// 4), q_row_elems, kv_row_elems (0: heads * D and kv_heads * D), splits, cached, kv_head_start, row_map_i64,
// cache_rows, app_rows, app_lens_i64.  Launch: batch * kv_heads * (s ? splits : 1) workgroups of 256 threads; r is
// the least of 1, 2, 4 that holds heads / kv_heads * t.
// ---------------------------------------------------------------------------------------------
#define SVODK_DECODE_ENTRY(D, R, T, F16, S)                                                                           \
  extern "C" __global__ __launch_bounds__(256) void svodk_decode_d##D##_r##R##_##T##_s##S(                            \
      const uint16_t *__restrict__ q, const uint16_t *__restrict__ k, const uint16_t *__restrict__ v,                 \
      uint16_t *__restrict__ o, const void *__restrict__ key_lens, const void *__restrict__ key_mask,                 \
      const void *__restrict__ row_map, const uint16_t *__restrict__ k_app, const uint16_t *__restrict__ v_app,       \
      const void *__restrict__ app_lens, float *__restrict__ o_part, float *__restrict__ m_part,                      \
      float *__restrict__ l_part, int32_t batch, int32_t t, int32_t tk, int32_t heads, int32_t kv_heads,              \
      int32_t scale_bits, int32_t lens_i64, int32_t mask_bytes, int32_t q_row_elems, int32_t kv_row_elems,            \
      int32_t splits, int32_t cached, int32_t kv_head_start, int32_t row_map_i64, int32_t cache_rows,                 \
      int32_t app_rows, int32_t app_lens_i64) {                                                                       \
    if (batch <= 0 || t <= 0 || tk < 0 || kv_heads <= 0 || heads < kv_heads) return;                                  \
    svodk::DecodeArgs p;                                                                                              \
    p.q = q, p.k = k, p.v = v, p.o = o, p.key_lens = key_lens, p.key_mask = key_mask, p.row_map = row_map;            \
    p.k_app = k_app, p.v_app = v_app, p.app_lens = app_lens, p.o_part = o_part, p.m_part = m_part, p.l_part = l_part; \
    p.q_row_elems = q_row_elems > 0 ? q_row_elems : heads * D;                                                        \
    p.kv_row_elems = kv_row_elems > 0 ? kv_row_elems : kv_heads * D;                                                  \
    p.lens_i64 = lens_i64, p.mask_bytes = mask_bytes, p.row_map_i64 = row_map_i64, p.app_lens_i64 = app_lens_i64;     \
    p.batch = batch, p.t = t, p.tk = tk, p.heads = heads, p.kv_heads = kv_heads, p.group = heads / kv_heads;          \
    p.splits = (S) && splits > 1 ? splits : 1, p.cached = cached, p.kv_head_start = kv_head_start;                    \
    p.cache_rows = cache_rows, p.app_rows = app_rows, p.scale = __builtin_bit_cast(float, scale_bits);                \
    svodk::decode_body<D, R, F16, (S) != 0>(p, 4);                                                                    \
  }
#define SVODK_DECODE_ROWS_OF(D, T, F16, S) \
  SVODK_DECODE_ENTRY(D, 1, T, F16, S) SVODK_DECODE_ENTRY(D, 2, T, F16, S) SVODK_DECODE_ENTRY(D, 4, T, F16, S)
#define SVODK_DECODE_FAMILY(D)                                              \
  SVODK_DECODE_ROWS_OF(D, bf16, false, 0) SVODK_DECODE_ROWS_OF(D, bf16, false, 1) \
  SVODK_DECODE_ROWS_OF(D, f16, true, 0) SVODK_DECODE_ROWS_OF(D, f16, true, 1)
SVODK_DECODE_FAMILY(32) SVODK_DECODE_FAMILY(48) SVODK_DECODE_FAMILY(64) SVODK_DECODE_FAMILY(128) SVODK_DECODE_FAMILY(256)
#endif  // SVODK_CODE_OBJECT

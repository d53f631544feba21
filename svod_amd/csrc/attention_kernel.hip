// Flash attention forward for gfx950 (MI355X): o = softmax(q k^T scale) v over
// sequence-major heads, q [B,T,H,D], k/v [B,Tk,Hkv,D], bf16 in, f32 state.
//
// The algorithm is the reference tile program's (tk/src/kernels/attention.rs):
// a block owns BQ query rows of one head, streams BKV-key blocks of K and V
// through an LDS ring, and carries the online-softmax state (m, l, o) with the
// lazy rescale of L373-427 (a row adopts a new maximum only when it grew by
// more than 8 in log2 units), the `raw_max` score form of L60-65/L400-431 (the
// maximum kept in raw score units, the scale applied inside the exponent's
// fused multiply-add) and the `skip_rescale` form of L56-59.  Hidden scores are
// -inf before the maximum (L637-697), a row no key reaches is zeros (L974-980).
//
// The mapping onto CDNA4 is this file's own.  Both products run TRANSPOSED on
// v_mfma_f32_32x32x16_bf16 so that a query is a lane:
//   S^T[keys, q] = K[keys, d] . Q^T[d, q]      A = K rows from LDS, B = Q in registers
//   O^T[d, q]   += V^T[d, keys] . P^T[keys, q]  A = V^T through ds_read_b64_tr_b16,
//                                               B = P, straight from S^T's registers
// In the 32x32 accumulator lane l holds column l%32 and rows 8(i/4)+4(l/32)+i%4,
// so lane l and lane l^32 together hold all scores of query l%32: the row
// maximum and sum are in-lane folds plus ONE v_permlane32_swap, and (m, l, corr)
// are plain per-lane scalars for the rescale of O^T.  P feeds the second
// product as its B operand without leaving registers: B wants, per lane, 8
// consecutive k-indices of column l%32, and the contraction index is ours to
// order, so V^T's fragments are fetched in the key order P's registers have.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "kernels.h"

namespace svodk {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define LDS_PTR(T) T __attribute__((address_space(3))) *

constexpr int kBkv = 64;           // keys per ring slot
constexpr int kWaveRows = 32;      // query rows a wave owns: the N of the MFMA atom
constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kRescaleAbove = 8.0f;  // tk/src/kernels/attention.rs:379

// A ring slot holds a [64 keys, D] tile of K and one of V, rows unpadded
// (D*2 bytes), filled by buffer_load_dwordx4 ... lds: a wave instruction lands
// 64 consecutive 16-byte chunks, so the only freedom is WHICH global chunk a
// lane fetches.  Each row's chunks are therefore stored XOR-permuted, with a
// permutation chosen per tile so that its read pattern touches every bank once:
//   K is read one chunk per lane, 16 consecutive rows at the same logical chunk
//     (ds_read_b128 serves 16 lanes a cycle): chunk ^ sK(row) with sK distinct
//     over 16 rows modulo the 256-byte bank period;
//   V is read transposed, 4 consecutive rows x 64 contiguous bytes per 32 lanes
//     (ds_read_b64_tr_b16): the 64-byte group index ^ sV(row) with sV distinct
//     over 4 rows modulo the period.
template <int D>
struct Tile {
  static constexpr int kRowBytes = D * 2;
  static constexpr int kCpr = D / 8;  // 16-byte chunks per row
  static constexpr int kBytes = kBkv * kRowBytes;
  static constexpr int kStage = 2 * kBytes;  // K then V
  static constexpr int kInstrs = kBytes / 1024;  // wave-wide 1 KiB fills per tile
  __device__ static constexpr int swz_k(int row) { return D == 64 ? ((row >> 1) & 7) : (row & 15); }
  // In units of 64-byte groups (4 chunks).
  __device__ static constexpr int swz_v(int row) { return D == 64 ? ((row >> 1) & 1) : (row & 3); }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  f32x2 f = {lo, hi};
  bf16x2 b = __builtin_convertvector(f, bf16x2);
  return __builtin_bit_cast(uint32_t, b);
}

// `x` of this lane and of its partner in the other half-wave (lane l <-> l^32),
// in an order that differs between the halves: v_permlane32_swap hands lanes
// < 32 (own, partner) and lanes >= 32 (partner, own).  Callers fold the pair
// with a commutative op.
struct Pair {
  float a, b;
};
__device__ __forceinline__ Pair both_halves(float x) {
  const uint32_t u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return {__uint_as_float(r[0]), __uint_as_float(r[1])};
}

// A raw buffer over `bytes` bytes at `base`: loads past the end return zero,
// which is how rows at and past a batch's key length read (the bounded views
// of tk/src/kernels/attention.rs:551-560).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, int64_t bytes) {
  const int64_t clamped = bytes < 0 ? 0 : (bytes > 0xffffffffLL ? 0xffffffffLL : bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)(uint32_t)clamped, 0x00020000);
}

template <int D, int NW, bool CAUSAL>
__global__ __launch_bounds__(NW * 64) void flash_fwd_kernel(
    const uint16_t *__restrict__ q, const uint16_t *__restrict__ k, const uint16_t *__restrict__ v,
    uint16_t *__restrict__ o, const void *__restrict__ key_lens, const void *__restrict__ key_mask, int32_t lens_i64,
    int32_t mask_bytes, int32_t t, int32_t tk, int32_t heads, int32_t kv_heads, int32_t nqt, float scale) {
  // The body is device code only: the host pass needs the kernel's handle, not its
  // instructions (and drops the whole instantiation over the LDS-fill builtins).
#if defined(__HIP_DEVICE_COMPILE__)
  using TL = Tile<D>;
  constexpr int BQ = NW * kWaveRows;
  constexpr int KS = D / 16;  // k-steps of the score product
  constexpr int DB = D / 32;  // 32-row blocks of O^T
  constexpr int CH = TL::kInstrs / NW;  // fills per wave per tile
  static_assert(TL::kInstrs % NW == 0, "the tile fills in whole wave instructions per wave");

  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

  const int tid = __builtin_amdgcn_workitem_id_x();
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;   // half-wave: the k-chunk of MFMA operands
  const int ln = lane & 31;  // the query column this lane owns

  // grid x = query tile fastest, then head, then batch (attention.rs:512,523).
  const int bid = __builtin_amdgcn_workgroup_id_x();
  const int order = bid % nqt;
  const int h = (bid / nqt) % heads;
  const int b = bid / (nqt * heads);
  // Where later queries see more keys the last query blocks run first (L524-528).
  const int qt = CAUSAL ? (nqt - 1 - order) : order;
  const int q_off = qt * BQ;
  const int kvh = h / (heads / kv_heads);  // L548

  // L533-536: len = min(key_lens[b], tk).
  int len = tk;
  if (key_lens != nullptr) {
    long long n = lens_i64 ? ((const long long *)key_lens)[b] : (long long)((const int *)key_lens)[b];
    n = n < 0 ? 0 : n;
    len = n < (long long)tk ? (int)n : tk;
  }
  // L596-608: key blocks some query of the tile sees.
  int end = (tk + kBkv - 1) / kBkv;
  if (CAUSAL) end = min(end, (q_off + BQ + kBkv - 1) / kBkv);
  if (key_lens != nullptr) end = min(end, (len + kBkv - 1) / kBkv);

  const int64_t q_row_stride = (int64_t)heads * D;
  const int kv_row_bytes = kv_heads * D * 2;
  const uint8_t *k_base = (const uint8_t *)(k + ((int64_t)b * tk * kv_heads + kvh) * D);
  const uint8_t *v_base = (const uint8_t *)(v + ((int64_t)b * tk * kv_heads + kvh) * D);
  // Bytes of this (batch, kv head)'s rows below the length, measured from its first row.
  const int64_t kv_bytes = len > 0 ? (int64_t)(len - 1) * kv_row_bytes + D * 2 : 0;

  // ---- Q fragments: B operand of the score product, resident for the block.
  const int wave_first_row = q_off + wave * kWaveRows;
  const int my_row = wave_first_row + ln;
  bf16x8 qf[KS];
  {
    const uint16_t *q_ptr = q + ((int64_t)b * t + my_row) * q_row_stride + (int64_t)h * D + g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      u32x4 w = {0, 0, 0, 0};
      if (my_row < t) w = *reinterpret_cast<const u32x4 *>(q_ptr + ks * 16);
      qf[ks] = __builtin_bit_cast(bf16x8, w);
    }
  }

  // ---- ring fill: this wave's share of a tile, CH wave-wide 1 KiB fills of K and of V.
  // Fill j lands on rows [j*rows_per, ...): lane i at physical chunk i % kCpr of row i / kCpr.
  constexpr int kRowsPer = 64 / TL::kCpr;
  int k_src[CH], v_src[CH];
#pragma unroll
  for (int i = 0; i < CH; i++) {
    const int j = wave + NW * i;
    const int row = j * kRowsPer + lane / TL::kCpr;
    const int pc = lane % TL::kCpr;
    k_src[i] = row * kv_row_bytes + ((pc ^ TL::swz_k(row)) << 4);
    v_src[i] = row * kv_row_bytes + ((pc ^ (TL::swz_v(row) << 2)) << 4);
  }
  auto fill = [&](int blk, int stage) {
    const int64_t off = (int64_t)blk * kBkv * kv_row_bytes;
    const __amdgpu_buffer_rsrc_t kr = make_rsrc(k_base + off, kv_bytes - off);
    const __amdgpu_buffer_rsrc_t vr = make_rsrc(v_base + off, kv_bytes - off);
    uint8_t *ks = smem + stage * TL::kStage;
#pragma unroll
    for (int i = 0; i < CH; i++) {
      const int j = wave + NW * i;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, (LDS_PTR(void))(ks + j * 1024), 16, k_src[i], 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, (LDS_PTR(void))(ks + TL::kBytes + j * 1024), 16, v_src[i], 0, 0, 0);
    }
  };

  // ---- per-lane LDS offsets of the operand reads.
  // K fragment (kb, ks): row 32kb + ln, logical chunk 2ks + g.
  int k_read[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) k_read[ks] = ln * TL::kRowBytes + (((2 * ks + g) ^ TL::swz_k(ln)) << 4);
  // V^T fragment (kb, tt, half, db): lanes 4j..4j+3 of a 16-lane group supply row j
  // (four 4-element runs), lane i of the group receives column i of those 4 rows.
  const int vq = (lane & 15) >> 2;                        // row within the group of 4
  const int vc = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);  // chunk within the 64-byte group
  int v_read[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
    v_read[db] = (4 * g + vq) * TL::kRowBytes + ((db ^ TL::swz_v(vq)) << 6) + (vc << 4) + ((lane & 1) << 3);

  // ---- online softmax state.  m in RAW score units (raw_max form).
  const bool positive = scale > 0.0f;
  const float c_exp = scale * kLog2e;  // L619
  // With a non-positive scale the maximum does not commute with it: the scores
  // are scaled first and m lives in the exponent's units (L365-370).
  const float unit = positive ? c_exp : 1.0f;
  const float limit = kRescaleAbove / unit;
  float m_run = -1e30f, l_run = 0.0f;
  f32x16 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[db][i] = 0.0f;

  if (end > 0) fill(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's fills have landed
  __syncthreads();

  auto step = [&](int blk, auto stage_c) {
    constexpr int stage = decltype(stage_c)::value;
    const int k0 = blk * kBkv;
    if (blk + 1 < end) fill(blk + 1, stage ^ 1);

    const uint8_t *ks_ = smem + stage * TL::kStage;
    const uint8_t *vs_ = ks_ + TL::kBytes;
    // A causal wave past its last visible key has nothing to add from this block.
    const bool idle = CAUSAL && k0 > wave_first_row + kWaveRows - 1;
    if (!idle) {
      // ---- S^T = K . Q^T
      f32x16 s[2];
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
#pragma unroll
        for (int i = 0; i < 16; i++) s[kb][i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          const u32x4 w = *reinterpret_cast<const u32x4 *>(ks_ + k_read[ks] + kb * 32 * TL::kRowBytes);
          s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w), qf[ks], s[kb], 0, 0, 0);
        }
      }
      if (!positive) {
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
          for (int i = 0; i < 16; i++) s[kb][i] *= c_exp;
      }

      // ---- masks (L641-697) as one 64-bit word per lane: bit j = key k0 + j is kept.
      // The length and the key mask give a wave-uniform word; causality a per-lane one.
      uint64_t kbits = ~0ull;
      if (key_mask != nullptr) {
        const int key = k0 + lane;
        bool vis = false;
        if (key < tk) {
          const int64_t at = (int64_t)b * tk + key;
          vis = mask_bytes == 1 ? ((const uint8_t *)key_mask)[at] != 0 : ((const int *)key_mask)[at] != 0;
        }
        kbits = __builtin_amdgcn_ballot_w64(vis);
      }
      if (k0 + kBkv > len) kbits &= (len > k0) ? (~0ull >> (64 - (len - k0))) : 0ull;
      const bool diagonal = CAUSAL && (k0 + kBkv - 1 > wave_first_row);
      if (kbits != ~0ull || diagonal) {
        uint64_t mine = kbits;
        if (diagonal) {
          const int seen = my_row - k0 + 1;  // keys k0 .. my_row
          mine &= seen >= 64 ? ~0ull : (seen <= 0 ? 0ull : (~0ull >> (64 - seen)));
        }
        mine >>= 4 * g;
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
          const uint32_t word = kb ? (uint32_t)(mine >> 32) : (uint32_t)mine;
#pragma unroll
          for (int i = 0; i < 16; i++) {
            const int rel = 8 * (i / 4) + (i % 4);  // key k0 + 32kb + 4g + rel
            s[kb][i] = ((word >> rel) & 1u) ? s[kb][i] : -INFINITY;
          }
        }
      }

      // ---- row maximum: in-lane tree, then the other half-wave's.
      float t8[8];
#pragma unroll
      for (int i = 0; i < 8; i++) t8[i] = fmaxf(fmaxf(s[0][2 * i], s[0][2 * i + 1]), fmaxf(s[1][2 * i], s[1][2 * i + 1]));
      float bm = fmaxf(fmaxf(fmaxf(t8[0], t8[1]), fmaxf(t8[2], t8[3])), fmaxf(fmaxf(t8[4], t8[5]), fmaxf(t8[6], t8[7])));
      {
        const Pair p = both_halves(bm);
        bm = fmaxf(p.a, p.b);
      }

      // ---- lazy rescale (L418-431).
      const float m_max = fmaxf(m_run, bm);
      const bool grows = limit < (m_max - m_run);
      const float m_new = grows ? m_max : m_run;
      const float corr = fast_exp2((m_run - m_new) * unit);
      const float m_exp = m_new * unit;
      m_run = m_new;

      // ---- p = 2^(s*unit - m*unit), held as bf16 (L432-435); the row sum adds the
      // probabilities as held, two per v_dot2 (the `truncate_p` form's rule, L436-444,
      // applied to the rounded values), in four independent chains.
      float bs[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      uint32_t pk[2][8];
      const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          const float p0 = fast_exp2(__builtin_fmaf(s[kb][i], unit, -m_exp));
          const float p1 = fast_exp2(__builtin_fmaf(s[kb][i + 1], unit, -m_exp));
          const uint32_t w = pack2(p0, p1);
          pk[kb][i / 2] = w;
          bs[(i / 2) & 3] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), ones, bs[(i / 2) & 3], false);
        }
      }
      l_run = l_run * corr + ((bs[0] + bs[1]) + (bs[2] + bs[3]));

      // ---- O^T rescale, skipped by a wave whose rows all kept their maximum (L56-59).
      if (__builtin_amdgcn_ballot_w64(corr != 1.0f) != 0) {
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
          for (int i = 0; i < 16; i++) acc[db][i] *= corr;
      }

      // ---- O^T += V^T . P^T
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
          u32x4 pw = {pk[kb][4 * tt], pk[kb][4 * tt + 1], pk[kb][4 * tt + 2], pk[kb][4 * tt + 3]};
          const bf16x8 pf = __builtin_bit_cast(bf16x8, pw);
#pragma unroll
          for (int db = 0; db < DB; db++) {
            const uint8_t *at = vs_ + v_read[db] + (32 * kb + 16 * tt) * TL::kRowBytes;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(at));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(at + 8 * TL::kRowBytes));
            typedef __attribute__((ext_vector_type(8))) short s16x8;
            const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pf, acc[db], 0, 0, 0);
          }
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the next tile's fills have landed
    __syncthreads();
  };

  int blk = 0;
  for (; blk + 2 <= end; blk += 2) {
    step(blk, std::integral_constant<int, 0>{});
    step(blk + 1, std::integral_constant<int, 1>{});
  }
  if (blk < end) step(blk, std::integral_constant<int, 0>{});

  // ---- out = o / (l == 0 ? 1 : l), bounded store (L892-898, L974-980).
  const Pair lp = both_halves(l_run);
  const float l_tot = lp.a + lp.b;
  const float inv = 1.0f / (l_tot == 0.0f ? 1.0f : l_tot);
  if (my_row < t) {
    uint16_t *o_ptr = o + ((int64_t)b * t + my_row) * q_row_stride + (int64_t)h * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; db++) {
#pragma unroll
      for (int c = 0; c < 4; c++) {
        u32x2 w;
        w[0] = pack2(acc[db][4 * c] * inv, acc[db][4 * c + 1] * inv);
        w[1] = pack2(acc[db][4 * c + 2] * inv, acc[db][4 * c + 3] * inv);
        *reinterpret_cast<u32x2 *>(o_ptr + 32 * db + 8 * c) = w;
      }
    }
  }
#endif  // __HIP_DEVICE_COMPILE__
}

template <int D, int NW, bool CAUSAL>
hipError_t launch(const AttnArgs &a, hipStream_t stream) {
  using TL = Tile<D>;
  constexpr int BQ = NW * kWaveRows;
  const int nqt = (a.t + BQ - 1) / BQ;
  const int64_t blocks = (int64_t)nqt * a.heads * a.batch;
  if (blocks == 0) return hipSuccess;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
  constexpr int smem = 2 * TL::kStage;
  // The fills address a (batch, kv head)'s rows with 32-bit byte offsets.
  if ((int64_t)a.tk * a.kv_heads * a.d * 2 > 0x7fffffffLL) return hipErrorInvalidValue;
  auto kernel = flash_fwd_kernel<D, NW, CAUSAL>;
  static bool configured = false;  // one attribute call per instantiation
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return e;
    configured = true;
  }
  hipLaunchKernelGGL(kernel, dim3((uint32_t)blocks), dim3(NW * 64), smem, stream, (const uint16_t *)a.q,
                     (const uint16_t *)a.k, (const uint16_t *)a.v, (uint16_t *)a.o, a.key_lens, a.key_mask, a.lens_i64,
                     a.mask_bytes, a.t, a.tk, a.heads, a.kv_heads, nqt, a.scale);
  return hipGetLastError();
}

template <int D>
hipError_t launch_d(const AttnArgs &a, hipStream_t stream) {
  return a.causal ? launch<D, 4, true>(a, stream) : launch<D, 4, false>(a, stream);
}

}  // namespace

bool attention_supports(int32_t d) { return d == 64 || d == 128; }

const char *attention_config(const AttnArgs &a) {
  (void)a;
  return "FaCfg { bq: 128, bkv: 64, stages: 2, splits: 1, forms: { raw_max, skip_rescale }, warp_rows: 32, core: "
         "mfma_f32_32x32x16_bf16 }";
}

hipError_t launch_attention(const AttnArgs &a, hipStream_t stream) {
  switch (a.d) {
    case 64: return launch_d<64>(a, stream);
    case 128: return launch_d<128>(a, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace svodk

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
//
// The loop is software-pipelined by one key block inside each wave: while the
// VALU turns S(j) into P(j), the matrix pipe computes S(j+1) and O += P(j) V(j).
// On this part a 32x32x16 MFMA leaves room for about four simple VALU
// instructions beside it, and one wave cannot issue faster than about one
// instruction per five cycles, so the step's instructions are laid out as
// "one MFMA, a share of the VALU work, the LDS reads two MFMAs ahead".
#include <hip/hip_runtime.h>

#include <atomic>

#include "kernels.h"

namespace svodk {
#if !defined(SVODK_CODE_OBJECT)
// Workgroups per XCD of the streaming form (<= 0: a workgroup per query tile instead), and the
// streaming launches so far: each takes the next set of shared counters.
extern std::atomic<int> g_stream_slots;
extern std::atomic<uint32_t> g_queue_turn;
uint32_t next_queue_set();  // the counter set of the next streaming launch: the sets in turn
#endif
namespace {

// The kernel's body is compiled for the device only (see flash_fwd_kernel): to the host pass
// the helpers below have no caller.
#if !defined(__HIP_DEVICE_COMPILE__) || defined(SVODK_HEAD)  // nor, to a part of the build, what other parts use
#pragma clang diagnostic ignored "-Wunused-function"
#pragma clang diagnostic ignored "-Wunused-variable"
#pragma clang diagnostic ignored "-Wunused-const-variable"
#pragma clang diagnostic ignored "-Wunneeded-internal-declaration"
#pragma clang diagnostic ignored "-Wunused-template"
#endif

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) int i32x4;

#define LDS_PTR(T) T __attribute__((address_space(3))) *

constexpr int kBkv = 64;       // keys per ring slot
constexpr int kScannedBlocks = 256;  // key blocks (16384 keys) of a key mask row scanned up front
constexpr int kWaveRows = 32;  // query rows a wave owns: the N of the MFMA atom
constexpr int kXcds = 8;       // accelerator dies of an MI355X, each with its own L2
constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kRescaleAbove = 8.0f;  // tk/src/kernels/attention.rs:379

// The library's build compiles this file once per head size (SVODK_HEAD = 32, 48, 64, 128: that
// size's instantiations) and once for what does not depend on it (SVODK_HEAD = 0), side by side;
// without the macro one translation unit holds everything.
#if defined(SVODK_HEAD)
#define SVODK_HAS_HEAD(D) (SVODK_HEAD == (D))
#define SVODK_HAS_COMMON (SVODK_HEAD == 0)
#else
#define SVODK_HAS_HEAD(D) 1
#define SVODK_HAS_COMMON 1
#endif

// A ring slot holds a [64 keys, D] tile, rows unpadded (D*2 bytes), filled by
// buffer_load_dwordx4 ... lds: a wave instruction lands 64 consecutive 16-byte
// chunks, so the only freedom is WHICH global chunk a lane fetches.  Each row's
// chunks are therefore stored XOR-permuted, with a permutation chosen per tile
// so that its read pattern touches every bank once:
//   K is read one chunk per lane, 16 consecutive rows at the same logical chunk
//     (ds_read_b128 serves 16 lanes a cycle): chunk ^ sK(row) with sK distinct
//     over 16 rows modulo the 256-byte bank period;
//   V is read transposed, 4 consecutive rows x 64 contiguous bytes per 32 lanes
//     (ds_read_b64_tr_b16): the 64-byte group index ^ sV(row) with sV distinct
//     over 4 rows modulo the period.
// K runs one block ahead of V, so each has its own pair of slots:
// LDS = [K slot 0][K slot 1][V slot 0][V slot 1].
// A head of 48 takes the 64-wide tile: a row's last two chunks are never fetched (their lanes
// read past the descriptor's bound and land zeros), the score product stops at the third
// k-step, and the second half of O^T's second row block is dropped at the store.
template <int D>
struct Tile {
  static constexpr int kWide = D == 48 ? 64 : D;  // the head size the tile is laid out for
  static constexpr int kRowBytes = kWide * 2;
  static constexpr int kCpr = kWide / 8;   // 16-byte chunk places per row of the tile
  static constexpr int kChunks = D / 8;    // chunks a row holds in memory
  static constexpr int kBytes = kBkv * kRowBytes;
  static constexpr int kLds = 4 * kBytes;
  static constexpr int kInstrs = kBytes / 1024;  // wave-wide 1 KiB fills per tile
  // 32 wide: rows are 64 bytes, four to the bank period, so 16 rows at one logical chunk spread over
  // the period's 16 chunk places when the chunk is xor-ed with row / 4; a V row is one 64-byte
  // group and four consecutive rows are the whole period as they lie.
  // 256 wide: rows are two bank periods, every row starts on a period, and row & 15 spreads 16 rows
  // over the 16 chunk places of a half row as it does for 128.
  __device__ static constexpr int swz_k(int row) {
    return kWide == 32 ? ((row >> 2) & 3) : kWide == 64 ? ((row >> 1) & 7) : (row & 15);
  }
  // In units of 64-byte groups (4 chunks).
  __device__ static constexpr int swz_v(int row) {
    return kWide == 32 ? 0 : kWide == 64 ? ((row >> 1) & 1) : (row & 3);
  }
  // The byte offset, from a fill instruction's first row, of what the lane at chunk place `pc` of
  // tile row `row` fetches: logical chunk pc ^ swizzle of that row of memory, or an offset past any
  // descriptor's bound where the row has no such chunk.
  // `ahead` rows lie between the fill instruction's first row and the tile row the swizzle is the one of
  // (a wave's later fills of a tile, where they do not share the first's swizzle).
  __device__ static int source(int row, int pc, int row_bytes, bool v, int ahead = 0) {
    const int chunk = pc ^ (v ? swz_v(row + ahead) << 2 : swz_k(row + ahead));
    return chunk < kChunks ? row * row_bytes + (chunk << 4) : (int)0xfffffff0u;
  }
  // A wave's fills of a tile are NW instructions apart; where that is not a whole period of the swizzle
  // (16 rows) its even and odd fills have a swizzle each.
  __device__ static constexpr int sources(int nw) { return (nw * (64 / kCpr)) % 16 == 0 ? 1 : 2; }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float max3(float a, float b, float c) {
  return __builtin_fmaxf(__builtin_fmaxf(a, b), c);
}

// Two f32 values as a pair of the operands' 16-bit type, rounded to nearest even
// (tk/src/interp.rs:37-50).
template <bool F16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  f32x2 f = {lo, hi};
  if constexpr (F16) {
    f16x2 h = __builtin_convertvector(f, f16x2);
    return __builtin_bit_cast(uint32_t, h);
  } else {
    bf16x2 b = __builtin_convertvector(f, bf16x2);
    return __builtin_bit_cast(uint32_t, b);
  }
}

// D = A . B + C on the 32x32x16 atom of the operands' type: A 32 rows x 16, B 16 x 32 columns,
// eight 16-bit values a lane each.
template <bool F16>
__device__ __forceinline__ f32x16 mma(const u32x4 &a, const u32x4 &b, const f32x16 &c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
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

// A raw buffer descriptor over `bytes` bytes at `base` (stride 0, 32-bit raw format): loads
// past the end return zero, which is how rows at and past a batch's key length read (the
// bounded views of tk/src/kernels/attention.rs:551-560).
// Both arguments are the same in every lane (a descriptor lives in scalar registers).  The bound is `bytes`
// clamped to [0, 2^32 - 1] on the scalar unit: written as comparisons of the 64-bit value the compiler does it on
// the VALU (v_cmp_*_i64 on broadcast operands), six vector instructions a descriptor in a loop whose VALU port is
// what bounds it.
__device__ __forceinline__ i32x4 make_rsrc(const void *base, int64_t bytes) {
  const uint64_t addr = (uint64_t)(uintptr_t)base;
  const int lo = (int)(uint32_t)(uint64_t)bytes, hi = (int)(bytes >> 32);
  int bound;
  asm("s_cmp_lt_i32 %1, 0\n\ts_cselect_b32 %0, 0, %2\n\ts_cmp_gt_i32 %1, 0\n\ts_cselect_b32 %0, -1, %0"
      : "=&s"(bound)
      : "s"(hi), "s"(lo)
      : "scc");
  i32x4 r;
  r[0] = (int)(uint32_t)addr;
  r[1] = (int)(uint32_t)((addr >> 32) & 0xffffu);
  r[2] = bound;
  r[3] = 0x00020000;
  return r;
}

// What a kernel's wave state is compiled for.
constexpr unsigned kStream = 1;  // a workgroup walks several query tiles
constexpr unsigned kRanged = 2;  // per-row key ranges: window, chunk mask, segment starts
constexpr unsigned kBiased = 4;  // an additive bias joins the scaled scores

// Everything a wave carries through the key loop.
template <int D, int NW, bool F16, unsigned FLAGS>
struct Wave {
  static constexpr int KS = D / 16;               // k-steps of the score product
  static constexpr int DB = Tile<D>::kWide / 32;  // 32-row blocks of O^T
  static constexpr int CH = Tile<D>::kInstrs / NW;  // fills per wave per tile
  // block constants
  const uint8_t *k_base, *v_base;
  int64_t kv_bytes;  // bytes of this (batch, kv head)'s rows below the length
  int kv_row_bytes;
  int end;           // key blocks the query tile sees
  int len, tk;
  const void *key_mask;
  int64_t mask_row;  // b * tk
  int mask_bytes;
  int lds0;          // LDS byte address of the ring
  int wave, lane, g;
  int wave_first_row, my_row;
  bool positive;  // the maximum is kept in raw score units: a positive scale and no bias (L368-370)
  // An additive bias (Attn::bias): this lane's row of it, at the tile's first key, and the keys
  // (from there) the row holds.  Unused unless `biased`.
  const uint16_t *bias_row;
  int bias_keys;
  bool my_row_ok;  // this lane's query row exists (rows past t read no bias)
  float c_exp, unit, limit;
  // Per-row key ranges (a window, a chunk mask, segment starts: tk/src/ops/attention.rs:64-71):
  // this lane's query sees keys [row_lo, row_hi] only, a causal mask already folded into row_hi.
  // Both are non-decreasing in the row, so the wave's first and last rows bound every row's:
  // lo_last, hi_first and hi_last are theirs.  All unused unless `ranged`.
  static constexpr bool ranged = (FLAGS & kRanged) != 0;
  static constexpr bool biased = (FLAGS & kBiased) != 0;
  int row_lo, row_hi;
  int lo_last, hi_first, hi_last;
  // per-lane addressing
  // global byte offsets of this lane's chunk in this wave's fills of a tile (one per swizzle phase)
  static constexpr int NS = Tile<D>::sources(NW);
  int k_src[NS], v_src[NS];
  int k_read[KS], v_read[DB];
  // state
  u32x4 qf[KS];
  f32x16 acc[DB];
  float m_run, l_run;
  int mask_next;
  // A key mask whose row was scanned at the start (rows of up to kScannedBlocks blocks): the
  // blocks' 64-bit words, one copy a wave, in LDS after the ring.  Otherwise the words are read a
  // lane a key, two blocks ahead of their use (mask_next).
  bool scanned;
  LDS_PTR(uint64_t) mask_words;
  // A streaming workgroup's next item (STREAM; nxt_end = 0: none): this item's
  // last steps request its first blocks.  The next item's blocks follow this item's at an even
  // position of the ring (end_even = end rounded up), so every item starts in slot 0.
  const uint8_t *nxt_k, *nxt_v;
  int64_t nxt_bytes;
  int nxt_end, end_even;
};

// The fills are issued as raw instructions: the compiler's wait-count pass treats an LDS fill
// it knows about as aliasing every later LDS read and would park the wave on the NEXT tile's
// fills in the middle of the current tile.  The kernel waits for them itself (vmcnt(0) before
// the barrier that ends a step).  m0 carries the LDS address of a wave instruction's 1 KiB.
template <int D, int NW, bool F16, unsigned FLAGS>
__device__ __forceinline__ void fill_tile(const Wave<D, NW, F16, FLAGS> &w, const uint8_t *base, int64_t bytes, int blk,
                                          int lds_at, const int (&src)[Tile<D>::sources(NW)], int row_bytes) {
  // This wave's fills of a tile are NW instructions apart; the swizzle repeats with that period (or
  // with twice it), so they share the lanes' offsets and differ in the descriptor's base.
  constexpr int kRowsPer = 64 / Tile<D>::kCpr;  // rows a wave instruction covers
  constexpr int NS = Tile<D>::sources(NW);
  static_assert((NS * NW * kRowsPer) % 16 == 0, "the swizzle repeats over a wave's fills");
  const int64_t off = (int64_t)blk * kBkv * row_bytes;
  const i32x4 r = make_rsrc(base + off, bytes - off);
#pragma unroll
  for (int i = 0; i < Wave<D, NW, F16, FLAGS>::CH; i++) {
    int voff = src[i % NS] + (NW * i * kRowsPer) * row_bytes;
    if constexpr (D == 48) voff = src[i % NS] == (int)0xfffffff0u ? src[i % NS] : voff;  // a chunk the row does not have
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_at + (w.wave + NW * i) * 1024), "v"(voff), "s"(r)
                 : "memory");
  }
}
// Block `n` of the stream of blocks that starts with this item's: the item's own while n < end,
// then (past the padding to an even count) the next item's.  Nothing past either.
template <int D, int NW, bool F16, unsigned FLAGS>
__device__ __forceinline__ void fill_k(const Wave<D, NW, F16, FLAGS> &w, int n, int slot) {
  const int at = w.lds0 + slot * Tile<D>::kBytes;
  if (n < w.end)
    fill_tile<D, NW>(w, w.k_base, w.kv_bytes, n, at, w.k_src, w.kv_row_bytes);
  else if ((FLAGS & kStream) && n >= w.end_even && n - w.end_even < w.nxt_end)
    fill_tile<D, NW>(w, w.nxt_k, w.nxt_bytes, n - w.end_even, at, w.k_src, w.kv_row_bytes);
}
template <int D, int NW, bool F16, unsigned FLAGS>
__device__ __forceinline__ void fill_v(const Wave<D, NW, F16, FLAGS> &w, int n, int slot) {
  const int at = w.lds0 + (2 + slot) * Tile<D>::kBytes;
  if (n < w.end)
    fill_tile<D, NW>(w, w.v_base, w.kv_bytes, n, at, w.v_src, w.kv_row_bytes);
  else if ((FLAGS & kStream) && n >= w.end_even && n - w.end_even < w.nxt_end)
    fill_tile<D, NW>(w, w.nxt_v, w.nxt_bytes, n - w.end_even, at, w.v_src, w.kv_row_bytes);
}

// A key mask row is read 64 keys (one per lane) a block, one block ahead: the load is issued
// before that block's fills and is long back when the block's step needs it.
template <int D, int NW, bool F16, unsigned FLAGS>
__device__ __forceinline__ int mask_lane(const Wave<D, NW, F16, FLAGS> &w, int blk) {
  const int key = blk * kBkv + w.lane;
  if (w.key_mask == nullptr || key >= w.tk) return 0;
  const int64_t at = w.mask_row + key;
  return w.mask_bytes == 1 ? (int)((const uint8_t *)w.key_mask)[at] : ((const int *)w.key_mask)[at];
}

// S^T = K . Q^T of the key block in K slot `slot`, as 32 scalars: sv[16kb + i] is the score of
// key 32kb + 8(i/4) + 4g + i%4 (sub-registers of the two accumulators: no moves).
template <int D, int NW, bool F16, unsigned FLAGS>
__device__ __forceinline__ void scores(const Wave<D, NW, F16, FLAGS> &w, const uint8_t *smem, int slot, float (&sv)[32]) {
  using TL = Tile<D>;
  const uint8_t *ks_ = smem + slot * TL::kBytes;
  const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  f32x16 s0 = zero, s1 = zero;
#pragma unroll
  for (int ks = 0; ks < Wave<D, NW, F16, FLAGS>::KS; ks++) {
    const u32x4 a0 = *reinterpret_cast<const u32x4 *>(ks_ + w.k_read[ks]);
    const u32x4 a1 = *reinterpret_cast<const u32x4 *>(ks_ + w.k_read[ks] + 32 * TL::kRowBytes);
    s0 = mma<F16>(a0, w.qf[ks], s0);
    s1 = mma<F16>(a1, w.qf[ks], s1);
  }
#pragma unroll
  for (int i = 0; i < 16; i++) {
    sv[i] = s0[i];
    sv[16 + i] = s1[i];
  }
}

// The wave-uniform part of block `blk`'s mask: bit j = key 64 blk + j is below the length and
// kept by the key mask (`word` is this lane's key-mask element of the block).
template <int D, int NW, bool F16, unsigned FLAGS>
__device__ __forceinline__ uint64_t uniform_bits(const Wave<D, NW, F16, FLAGS> &w, int blk, int word) {
  const int k0 = blk * kBkv;
  uint64_t kbits = ~0ull;
  if (w.key_mask != nullptr) {
    if (w.scanned) {
      const uint64_t x = w.mask_words[blk];  // the same address in every lane
      kbits = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)x) |
              (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(x >> 32)) << 32;
    } else {
      kbits = __builtin_amdgcn_ballot_w64(word != 0);
    }
  }
  if (k0 + kBkv > w.len) kbits &= (w.len > k0) ? (~0ull >> (64 - (w.len - k0))) : 0ull;
  return kbits;
}

// The 32 bias elements this lane's scores of the 64 keys from `first` on take, as 16 packed
// pairs: keys first + 32 kb + 8 c + 4 g + {0..3}.  Keys past the row read as zero (their scores are hidden anyway).
template <int D, int NW, bool F16, unsigned FLAGS>
__device__ __forceinline__ void load_bias(const Wave<D, NW, F16, FLAGS> &w, int first, bool row_ok, uint32_t (&bw)[16]) {
  const int k0 = first + 4 * w.g;
  const bool aligned = ((uintptr_t)w.bias_row & 7u) == 0;  // wave-uniform when every row is: checked per lane
#pragma unroll
  for (int c = 0; c < 8; c++) {
    const int key = k0 + 32 * (c / 4) + 8 * (c % 4);
    uint32_t lo = 0, hi = 0;
    if (row_ok && aligned && key + 3 < w.bias_keys) {
      const u32x2 x = *reinterpret_cast<const u32x2 *>(w.bias_row + key);
      lo = x[0];
      hi = x[1];
    } else if (row_ok) {
      const uint32_t e0 = key + 0 < w.bias_keys ? w.bias_row[key + 0] : 0u;
      const uint32_t e1 = key + 1 < w.bias_keys ? w.bias_row[key + 1] : 0u;
      const uint32_t e2 = key + 2 < w.bias_keys ? w.bias_row[key + 2] : 0u;
      const uint32_t e3 = key + 3 < w.bias_keys ? w.bias_row[key + 3] : 0u;
      lo = e0 | e1 << 16;
      hi = e2 | e3 << 16;
    }
    bw[2 * c] = lo;
    bw[2 * c + 1] = hi;
  }
}

// biased() of L358-362: s = fma(bias, log2(e), s) on the scaled scores, before the masks.
template <bool F16>
__device__ __forceinline__ void add_bias(const uint32_t (&bw)[16], float (&sv)[32]) {
#pragma unroll
  for (int i = 0; i < 32; i++) {
    const uint32_t pair = bw[i / 2];
    const uint16_t e = (uint16_t)((i & 1) ? pair >> 16 : pair & 0xffffu);
    float x;
    if (F16) {
      x = (float)__builtin_bit_cast(_Float16, e);
    } else {
      const uint32_t wide = (uint32_t)e << 16;
      x = __builtin_bit_cast(float, wide);
    }
    sv[i] = __builtin_fmaf(x, kLog2e, sv[i]);
  }
}

// Whether a mask edge crosses block `blk` for this wave (L698-733).
template <int D, int NW, bool CAUSAL, bool F16, unsigned FLAGS>
__device__ __forceinline__ bool on_edge(const Wave<D, NW, F16, FLAGS> &w, int blk, uint64_t kbits) {
  const int k0 = blk * kBkv;
  if (kbits != ~0ull) return true;
  // L715-731: a range's right edge for the wave's first row, its left edge for the last.
  if (w.ranged) return k0 + kBkv - 1 > w.hi_first || k0 < w.lo_last;
  return CAUSAL && (k0 + kBkv - 1 > w.wave_first_row);
}

// Scores whose bit of `mine` is clear become -inf; bit 8 (i / 4) + i % 4 (+ 32 for the second
// half) is this lane's score i: the key that many places past the lane's first.
__device__ __forceinline__ void hide_scores(uint64_t mine, float (&sv)[32]) {
  const uint32_t lo = (uint32_t)mine, hi = (uint32_t)(mine >> 32);
#pragma unroll
  for (int i = 0; i < 16; i++) {
    const int rel = 8 * (i / 4) + (i % 4);  // key k0 + 32kb + 4g + rel
    sv[i] = ((lo >> rel) & 1u) ? sv[i] : -INFINITY;
    sv[16 + i] = ((hi >> rel) & 1u) ? sv[16 + i] : -INFINITY;
  }
}

// Scales (a non-positive scale only) and masks (L641-697) the scores of block `blk`: hidden
// scores become -inf.  `kbits` is the uniform word; causality adds a per-lane one.
template <int D, int NW, bool CAUSAL, bool F16, unsigned FLAGS>
__device__ __forceinline__ void mask_scores(const Wave<D, NW, F16, FLAGS> &w, int blk, uint64_t kbits, float (&sv)[32]) {
  const int k0 = blk * kBkv;
  uint64_t mine = kbits;
  if (w.ranged) {
    // Keys k0 .. row_hi are seen from above and those from row_lo on from below (L659-695).
    const int seen = w.row_hi - k0 + 1;
    mine &= seen >= 64 ? ~0ull : (seen <= 0 ? 0ull : (~0ull >> (64 - seen)));
    const int below = w.row_lo - k0;
    mine &= below <= 0 ? ~0ull : (below >= 64 ? 0ull : (~0ull << below));
  } else if (CAUSAL && (k0 + kBkv - 1 > w.wave_first_row)) {
    const int seen = w.my_row - k0 + 1;  // keys k0 .. my_row are seen
    mine &= seen >= 64 ? ~0ull : (seen <= 0 ? 0ull : (~0ull >> (64 - seen)));
  }
  hide_scores(mine >> (4 * w.g), sv);
}

// The row maximum of a block's scores: in-lane tree of three-way folds, then the other
// half-wave's.
__device__ __forceinline__ float row_max(const float (&sv)[32]) {
  float t[11];
#pragma unroll
  for (int i = 0; i < 10; i++) t[i] = max3(sv[3 * i], sv[3 * i + 1], sv[3 * i + 2]);
  t[10] = __builtin_fmaxf(sv[30], sv[31]);
  const float u0 = max3(t[0], t[1], t[2]), u1 = max3(t[3], t[4], t[5]), u2 = max3(t[6], t[7], t[8]);
  const float bm = max3(max3(u0, u1, u2), t[9], t[10]);
  const Pair p = both_halves(bm);
  return __builtin_fmaxf(p.a, p.b);
}

// Half a block's probabilities: p = 2^(s*unit - m*unit) for 16 scores, summed unrounded in
// four chains, then held as bf16 (L432-444).
template <bool F16>
__device__ __forceinline__ void probabilities(const float *sv, float unit, float m_exp, float (&bs)[4],
                                              uint32_t *pk) {
#pragma unroll
  for (int i = 0; i < 16; i += 4) {
    const float p0 = fast_exp2(__builtin_fmaf(sv[i], unit, -m_exp));
    const float p1 = fast_exp2(__builtin_fmaf(sv[i + 1], unit, -m_exp));
    const float p2 = fast_exp2(__builtin_fmaf(sv[i + 2], unit, -m_exp));
    const float p3 = fast_exp2(__builtin_fmaf(sv[i + 3], unit, -m_exp));
    bs[0] += p0;
    bs[1] += p1;
    bs[2] += p2;
    bs[3] += p3;
    pk[i / 2] = pack2<F16>(p0, p1);
    pk[i / 2 + 1] = pack2<F16>(p2, p3);
  }
}

// O^T += V^T . P^T over 32 keys (half a block): chunks c of 16 keys, fragment registers 4c..4c+3.
template <int D, int NW, bool F16, unsigned FLAGS>
__device__ __forceinline__ void accumulate(Wave<D, NW, F16, FLAGS> &w, const uint8_t *vs_, int half, const uint32_t *pk) {
  using TL = Tile<D>;
#pragma unroll
  for (int c = 0; c < 2; c++) {
    const u32x4 pw = {pk[4 * c], pk[4 * c + 1], pk[4 * c + 2], pk[4 * c + 3]};

#pragma unroll
    for (int db = 0; db < Wave<D, NW, F16, FLAGS>::DB; db++) {
      const uint8_t *at = vs_ + w.v_read[db] + (32 * half + 16 * c) * TL::kRowBytes;
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(at));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(at + 8 * TL::kRowBytes));
      const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      w.acc[db] = mma<F16>(__builtin_bit_cast(u32x4, both), pw, w.acc[db]);
    }
  }
}

// The running maximum's update for a block whose row maximum is `bm`: the lazy rescale of
// L418-431, and the O^T rescale that a wave skips when all its rows kept their maximum
// (L56-59).  Returns the exponent's offset m*unit; `corr` is the correction of l.
template <int D, int NW, bool F16, unsigned FLAGS>
__device__ __forceinline__ float adopt_maximum(Wave<D, NW, F16, FLAGS> &w, float bm, float &corr) {
  const float m_max = __builtin_fmaxf(w.m_run, bm);
  const bool grows = w.limit < (m_max - w.m_run);
  const float m_new = grows ? m_max : w.m_run;
  corr = fast_exp2((w.m_run - m_new) * w.unit);
  w.m_run = m_new;
  if (__builtin_amdgcn_ballot_w64(corr != 1.0f) != 0) {
#pragma unroll
    for (int db = 0; db < Wave<D, NW, F16, FLAGS>::DB; db++) w.acc[db] *= corr;
  }
  return m_new * w.unit;
}

// Keeps the computation of `x` where the source has it: instruction selection is otherwise free
// to let arithmetic without side effects drift past the fences between slots.
__device__ __forceinline__ void pin(float &x) { asm volatile("" : "+v"(x)); }

// One unit of the exponentials: two scores to two probabilities (p = 2^(s*unit - m*unit)),
// each added unrounded to a row-sum chain, the pair held as bf16 (L432-444).
template <bool F16>
__device__ __forceinline__ uint32_t p_unit(float s_a, float s_b, float unit, float m_exp, float &sum_a, float &sum_b) {
  const float pa = fast_exp2(__builtin_fmaf(s_a, unit, -m_exp));
  const float pb = fast_exp2(__builtin_fmaf(s_b, unit, -m_exp));
  sum_a += pa;
  sum_b += pb;
  return pack2<F16>(pa, pb);
}

// The hot step: block `blk` (parity PAR = blk & 1: V(blk) in V slot PAR, K(blk+1) in K slot
// PAR^1) when block blk+1 is this wave's too, no mask edge crosses it and the scale is
// positive.  `sv` holds S(blk) and `bm` its row maximum; S(blk+1) goes to `nv`, its maximum to
// `bm`.
//
// The step is written as a sequence of slots, one matrix instruction each, fenced so that the
// compiler keeps their order: the LDS fragment a matrix instruction reads was requested four
// slots earlier, and each slot carries its share of the VALU work, so that the matrix pipe
// never waits for the VALU's whole job.  2 KS slots compute S(blk+1) beside the exponentials
// of keys 0..31; 2 DB slots add P V of keys 0..31 beside the exponentials of keys 32..63;
// 2 DB slots add P V of keys 32..63 beside the row maximum of S(blk+1).
template <int D, int NW, int PAR, bool F16, unsigned FLAGS>
__device__ __forceinline__ void hot_step(Wave<D, NW, F16, FLAGS> &w, const uint8_t *smem, int blk, const float (&sv)[32],
                                         float (&nv)[32], float &bm) {
  using TL = Tile<D>;
  constexpr int KS = Wave<D, NW, F16, FLAGS>::KS, DB = Wave<D, NW, F16, FLAGS>::DB;
  constexpr int NQK = 2 * KS;  // score slots
  constexpr int NPV = 4 * DB;  // P V slots, half of them per 32 keys
  const uint8_t *ks_ = smem + (PAR ^ 1) * TL::kBytes;
  const uint8_t *vs_ = smem + (2 + PAR) * TL::kBytes;
  // Score fragment f: key half kb = f & 1, k-step ks = f >> 1.
  auto k_frag = [&](int f) -> u32x4 {
    return *reinterpret_cast<const u32x4 *>(ks_ + w.k_read[f >> 1] + (f & 1) * 32 * TL::kRowBytes);
  };
  // P V fragment j: 16-key chunk c = j / DB (0..3), d-block db = j % DB.
  auto v_frag = [&](int j) -> s16x8 {
    const uint8_t *at = vs_ + w.v_read[j % DB] + 16 * (j / DB) * TL::kRowBytes;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(at));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(at + 8 * TL::kRowBytes));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };

  u32x4 kf[4];
#pragma unroll
  for (int f = 0; f < 4; f++) kf[f] = k_frag(f);
  fill_v<D, NW>(w, blk + 1, PAR ^ 1);
  fill_k<D, NW>(w, blk + 2, PAR);
  w.mask_next = 0;  // hot steps run without a key mask only
  float corr;
  const float m_exp = adopt_maximum<D, NW>(w, bm, corr);
  __builtin_amdgcn_sched_barrier(0);

  float bs[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  uint32_t pk[16];
  s16x8 vf[4];
  const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  f32x16 s0 = zero, s1 = zero;
  // ---- S(blk+1) beside the probabilities of keys 0..31 (8 units over NQK slots).
#pragma unroll
  for (int i = 0; i < NQK; i++) {
    if (i & 1)
      s1 = mma<F16>(kf[i & 3], w.qf[i >> 1], s1);
    else
      s0 = mma<F16>(kf[i & 3], w.qf[i >> 1], s0);
    if (i + 4 < NQK)
      kf[i & 3] = k_frag(i + 4);
    else
      vf[(i + 4 - NQK) & 3] = v_frag(i + 4 - NQK);
#pragma unroll
    for (int u = 8 * i / NQK; u < 8 * (i + 1) / NQK; u++)
      pk[u] = p_unit<F16>(sv[2 * u], sv[2 * u + 1], w.unit, m_exp, bs[(2 * u) & 3], bs[(2 * u + 1) & 3]);
    if (8 * i / NQK < 8 * (i + 1) / NQK) {
#pragma unroll
      for (int x = 0; x < 4; x++) pin(bs[x]);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int i = 0; i < 16; i++) {
    nv[i] = s0[i];
    nv[16 + i] = s1[i];
  }
  // ---- O += P V of keys 0..31 beside the probabilities of keys 32..63, then O += P V of keys
  // 32..63 beside the row maximum of S(blk+1).
  float t[11];
#pragma unroll
  for (int j = 0; j < NPV; j++) {
    const int c = j / DB;
    const u32x4 pw = {pk[4 * c], pk[4 * c + 1], pk[4 * c + 2], pk[4 * c + 3]};
    w.acc[j % DB] = mma<F16>(__builtin_bit_cast(u32x4, vf[j & 3]), pw, w.acc[j % DB]);
    if (j + 4 < NPV) vf[j & 3] = v_frag(j + 4);
    if (j < NPV / 2) {
#pragma unroll
      for (int u = 8 + 16 * j / NPV; u < 8 + 16 * (j + 1) / NPV; u++)
        pk[u] = p_unit<F16>(sv[2 * u], sv[2 * u + 1], w.unit, m_exp, bs[(2 * u) & 3], bs[(2 * u + 1) & 3]);
#pragma unroll
      for (int x = 0; x < 4; x++) pin(bs[x]);
    } else {
      // The row maximum's first level, ten three-way folds and one two-way, over these slots.
      const int jj = j - NPV / 2;
#pragma unroll
      for (int x = 11 * jj / (NPV / 2); x < 11 * (jj + 1) / (NPV / 2); x++)
      {
        t[x] = x < 10 ? max3(nv[3 * x], nv[3 * x + 1], nv[3 * x + 2]) : __builtin_fmaxf(nv[30], nv[31]);
        pin(t[x]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  {
    const float u0 = max3(t[0], t[1], t[2]), u1 = max3(t[3], t[4], t[5]), u2 = max3(t[6], t[7], t[8]);
    const Pair p = both_halves(max3(max3(u0, u1, u2), t[9], t[10]));
    bm = __builtin_fmaxf(p.a, p.b);
  }
  w.l_run = w.l_run * corr + ((bs[0] + bs[1]) + (bs[2] + bs[3]));
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the fills issued this step have landed
  __syncthreads();
}

// The general step, for the blocks at the edges: any block, a next block or none, masks, any
// scale.  Slots are picked at run time.  `sv` holds the masked S(blk) and `bm` its row maximum;
// on exit they hold block blk+1's (when this wave has one).
template <int D, int NW, bool CAUSAL, bool F16, unsigned FLAGS>
__device__ __forceinline__ void edge_step(Wave<D, NW, F16, FLAGS> &w, const uint8_t *smem, int blk, int my_end, float (&sv)[32],
                                          float &bm) {
  using TL = Tile<D>;
  const int par = blk & 1;
  const bool more = blk + 1 < my_end;
  const uint64_t kbits_next = uniform_bits<D, NW>(w, blk + 1, w.mask_next);
  // The next block's bias is asked for first: it has this block's P.V to arrive under.
  uint32_t bw[16];
  if (w.biased && more) load_bias<D, NW>(w, (blk + 1) * kBkv, w.my_row_ok, bw);
  fill_v<D, NW>(w, blk + 1, par ^ 1);
  if (!w.scanned && blk + 2 < w.end) w.mask_next = mask_lane<D, NW>(w, blk + 2);
  fill_k<D, NW>(w, blk + 2, par);
  float corr;
  const float m_exp = adopt_maximum<D, NW>(w, bm, corr);

  const uint8_t *vs_ = smem + (2 + par) * TL::kBytes;
  float bs[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  uint32_t pk[16];
  probabilities<F16>(sv, w.unit, m_exp, bs, pk);
  probabilities<F16>(sv + 16, w.unit, m_exp, bs, pk + 8);
  accumulate<D, NW>(w, vs_, 0, pk);
  accumulate<D, NW>(w, vs_, 1, pk + 8);
  w.l_run = w.l_run * corr + ((bs[0] + bs[1]) + (bs[2] + bs[3]));
  if (more) {
    scores<D, NW>(w, smem, par ^ 1, sv);
    if (!w.positive) {
#pragma unroll
      for (int i = 0; i < 32; i++) sv[i] *= w.c_exp;
    }
    if (w.biased) add_bias<F16>(bw, sv);
    if (on_edge<D, NW, CAUSAL>(w, blk + 1, kbits_next)) mask_scores<D, NW, CAUSAL>(w, blk + 1, kbits_next, sv);
    bm = row_max(sv);
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the fills issued this step have landed
  __syncthreads();
}

// A step of a wave with nothing to compute: fills and the barrier only.
template <int D, int NW, bool F16, unsigned FLAGS>
__device__ __forceinline__ void idle_step(Wave<D, NW, F16, FLAGS> &w, int blk) {
  const int par = blk & 1;
  fill_v<D, NW>(w, blk + 1, par ^ 1);
  fill_k<D, NW>(w, blk + 2, par);
  __builtin_amdgcn_s_waitcnt(0x0f70);
  __syncthreads();
}

// n / d for n < 2^32 with rcp = floor(2^32 / d) (2^32 - 1 for d = 1) from the host: the
// estimate is the quotient or one less.
__device__ __forceinline__ uint32_t div_by(uint32_t n, uint32_t d, uint32_t rcp) {
  const uint32_t q = __umulhi(n, rcp);
  return n - q * d >= d ? q + 1 : q;
}

// Launch geometry the host works out once: sizes and their reciprocals for div_by.
struct Geometry {
  uint32_t unit_size, unit_rcp;  // workgroups of a (batch, KV head): group * nqt
  uint32_t nqt, nqt_rcp;         // query tiles
  uint32_t kv_heads, kvh_rcp;
  uint32_t group;                // heads / kv_heads
  uint32_t units;                // kv_heads * batch
};
// The key splits of a launch that has them, and where their partial states go.
struct Splits {
  uint32_t count, rcp;
  float *o_part, *m_part, *l_part;
  uint32_t nbatch;
};

// The per-row masks (the RANGED instantiations) and the bias (the BIASED ones) of a launch that
// has them.
struct Ranges {
  int32_t win_left, win_right;  // win_left < 0: no window; the host caps both at t + tk
  int32_t chunk_size;           // 0: no chunk mask (Chunk of tk/src/ops/attention.rs:39-50)
  int32_t chunk_left;           // < 0: every earlier chunk
  int32_t chunk_right;          // the host caps it at the chunks of the keys
  const void *seg_start;        // [B, T] integers or null
  int32_t seg_i64;
  const uint16_t *bias;         // [B or 1, H, T, bias_cols] of the operands' type, or null
  int32_t bias_per_batch;
  int32_t bias_cols;            // Tk, plus the appended rows
  // The cache of a launch that has one (the CACHED instantiations; tk/src/ops/attention.rs:39-56).
  int32_t kv_head_start;        // the first of the launch's kv heads in a cache row
  const void *row_map;          // [B] cache row per batch lane, or null: row b
  int32_t row_map_i64;
  int32_t cache_rows;           // rows of the cache: a mapped row is held inside them
  const uint16_t *k_app, *v_app;  // [B, app_rows, kv_heads, D] scored after the cached keys, or null
  int32_t app_rows;             // at most a key block
  const void *app_lens;         // [B] visible appended rows, or null: all
  int32_t app_lens_i64;
};

// GROUPED: the query tile's rows are (head of the KV head's group, query) pairs instead of 128
// queries of one head, for calls whose whole group fits a tile (a decoder step: heads / kv_heads
// * T <= 128).  The group's heads then share one pass over their K and V instead of one each.
// The workgroup's whole program, for the kernels below to inline: `smem` is the workgroup's LDS (the
// ring, and behind it the scanned key mask words of a launch with a key mask).  Device code only:
// the host pass needs a kernel's handle, not its instructions (and would drop the whole
// instantiation over the LDS-fill instructions).
#if defined(__HIP_DEVICE_COMPILE__)
template <int D, int NW, bool CAUSAL, bool SPLIT, bool RANGED, bool BIASED, bool CACHED, bool GROUPED, bool F16>
__device__ __forceinline__ void flash_fwd_body(
    uint8_t *smem, uint32_t unit_size, uint32_t unit_rcp, uint32_t nqt_u, uint32_t nqt_rcp, uint32_t kvh_u,
    uint32_t kvh_rcp, uint32_t units, uint32_t heads_group, const void *__restrict__ key_lens,
    const int32_t *__restrict__ row_order, int32_t t, uint32_t tk_lens64, const uint16_t *__restrict__ q,
    const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, uint16_t *__restrict__ o,
    const void *__restrict__ key_mask, int32_t mask_bytes, float scale, const Splits &sp, int32_t q_row_elems,
    int32_t kv_row_elems, const Ranges &rg) {
  // Two of the arguments are packed: heads | group << 16, and tk | (key_lens is 64-bit) << 31.
  const Geometry geo = {unit_size, unit_rcp, nqt_u, nqt_rcp, kvh_u, kvh_rcp, heads_group >> 16, units};
  const int heads = (int)(heads_group & 0xffffu);
  const int tk = (int)(tk_lens64 & 0x7fffffffu);
  const bool lens_i64 = (tk_lens64 >> 31) != 0;
  using TL = Tile<D>;
  using W = Wave<D, NW, F16, (RANGED ? kRanged : 0u) | (BIASED ? kBiased : 0u)>;
  constexpr int BQ = NW * kWaveRows;
  constexpr int KS = W::KS, DB = W::DB;
  static_assert(TL::kInstrs % NW == 0, "the tile fills in whole wave instructions per wave");

  // A unit of work is one (batch, KV head): the query tiles of the heads that share its K and
  // V.  Workgroups are dealt to the 8 XCDs round-robin, each XCD with its own L2, so the units
  // are dealt to the XCDs round-robin too and a unit's workgroups all land on one XCD: they
  // meet in one L2 instead of being spread over all eight.  (The reference's grid is query
  // tile fastest, then head, then batch, attention.rs:512,523; the order within a unit is that.)
  const uint32_t wg = __builtin_amdgcn_workgroup_id_x();
  const uint32_t local = wg / kXcds;
  const uint32_t round = div_by(local, geo.unit_size, geo.unit_rcp);
  const uint32_t within = local - round * geo.unit_size;
  uint32_t head_in_group = div_by(within, geo.nqt, geo.nqt_rcp);
  int order = (int)(within - head_in_group * geo.nqt);
  if (CAUSAL && !GROUPED) {
    // An XCD deals its workgroups to its four shader engines strictly in turn, and one whose engine
    // is full holds back all behind it.  Head after head, every fourth tile of a causal unit (the
    // longest of each four) would go to the same engine; with the group's heads side by side for
    // each tile, neighbours cost the same and the engines fill and drain in step.
    order = (int)(within / geo.group);
    head_in_group = within - (uint32_t)order * geo.group;
  }
  // Which unit of a round an XCD takes turns with the round: with a power-of-two head count a
  // fixed deal would hand an XCD the same heads in every batch row, i.e. always the same 128-byte
  // residues of every K, V, Q and O row, and the XCD whose residues share a memory channel with
  // other traffic then runs a tenth behind the rest (measured: whichever XCD read bytes 384..511
  // of every KiB); turned, every XCD reads every residue and they finish together.
  const uint32_t unit = round * kXcds + (wg + round) % kXcds;
  if (unit >= geo.units) return;
  const int b_place = (int)div_by(unit, geo.kv_heads, geo.kvh_rcp);
  const int kvh = (int)(unit - (uint32_t)b_place * geo.kv_heads);  // L548: query head h reads KV head h / (heads / kv_heads)
  const int h = kvh * (int)geo.group + (int)head_in_group;
  // Which batch row a workgroup takes is free (the reference's grid fixes what is computed, not
  // when): with an order from the caller, place p of the launch works on row row_order[p], so
  // that rows with more keys can go first and the launch ends on its short tiles.
  int b = b_place;
  if (row_order != nullptr) b = row_order[b_place];
  // Everything the first loads and fills take from the argument record (past the words that arrive in
  // registers with the wave) is asked for HERE, while the row's number is on its way: left to the
  // compiler those loads sit behind the wait for it, and a workgroup's start is three scalar memory
  // round trips (the row, the arguments, the length) where two will do.
  asm volatile("" : "+s"(b) : "s"(q), "s"(k), "s"(v), "s"(o), "s"(key_mask), "s"(mask_bytes), "s"(scale), "s"(q_row_elems),
               "s"(kv_row_elems));
  if (row_order != nullptr) {
    const int nbatch = (int)div_by(geo.units, geo.kv_heads, geo.kvh_rcp);
    b = min(max(b, 0), nbatch - 1);
  }
  // Grid x of the reference is order * splits + split (L523); geo.nqt counts those.
  int split = 0, tile = order, nqt = (int)geo.nqt;
  if (SPLIT) {
    tile = (int)div_by((uint32_t)order, sp.count, sp.rcp);
    split = order - tile * (int)sp.count;
    nqt = (int)div_by(geo.nqt, sp.count, sp.rcp);
  }
  // Where later queries see more keys the last query blocks run first (L524-528).
  const int qt = CAUSAL ? (nqt - 1 - tile) : tile;
  const int q_off = qt * BQ;

  W w;
  const int tid = __builtin_amdgcn_workitem_id_x();
  w.lane = tid & 63;
  w.wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  w.g = w.lane >> 5;           // half-wave: the k-chunk of MFMA operands
  const int ln = w.lane & 31;  // the query column this lane owns

  // L533-536: len = min(key_lens[b], tk).
  int len = tk;
  if (key_lens != nullptr) {
    long long n = lens_i64 ? ((const long long *)key_lens)[b] : (long long)((const int *)key_lens)[b];
    n = n < 0 ? 0 : n;
    len = n < (long long)tk ? (int)n : tk;
  }

  // Elements from a token's row to the next: heads * D and kv_heads * D for separate q, k, v;
  // the fused projection's row for operands read in place (tk/src/ops/attention.rs:104-122).
  const int64_t q_row_stride = q_row_elems;
  const int64_t o_row_stride = (int64_t)heads * D;
  const int row = q_off + w.wave * kWaveRows + ln;  // this lane's row of the tile
  static_assert(!GROUPED || (!CAUSAL && !RANGED), "grouped tiles take no per-row masks");
  // This lane's query: row q_row of head q_head, when there is one.
  int q_row = row, q_head = h;
  bool q_ok = row < t;
  if (GROUPED) {
    const int in_group = row / t;
    q_row = row - in_group * t;
    q_ok = in_group < (int)geo.group;
    q_head = kvh * (int)geo.group + min(in_group, (int)geo.group - 1);
  }

  // L584-608: key blocks [first, end) hold every key some query of the tile sees.
  int first = 0, end = (tk + kBkv - 1) / kBkv;
  if (CAUSAL) end = min(end, (q_off + BQ + kBkv - 1) / kBkv);
  if (RANGED) {
    // This lane's row sees keys [lo, hi] (L659-695); rows past t stand in for row t - 1 where a
    // table is read.  Everything is monotonic in the row, so the tile's first row gives its
    // first block and its last row the end (L580-606).
    const int64_t row_abs = q_off + w.wave * kWaveRows + ln;
    int64_t lo = 0, hi = tk - 1;
    if (rg.win_left >= 0) {
      lo = max(lo, row_abs - rg.win_left);
      hi = min(hi, row_abs + rg.win_right);
      first = max(q_off - rg.win_left, 0) / kBkv;
      end = min(end, (q_off + BQ + rg.win_right + kBkv - 1) / kBkv);
    }
    if (rg.chunk_size > 0) {
      const int64_t cq = row_abs / rg.chunk_size;
      hi = min(hi, (cq + rg.chunk_right + 1) * rg.chunk_size - 1);
      const int cq1 = (q_off + BQ - 1) / rg.chunk_size;
      end = (int)min((int64_t)end, ((int64_t)(cq1 + 1 + rg.chunk_right) * rg.chunk_size + (kBkv - 1)) / kBkv);
      if (rg.chunk_left >= 0) {
        lo = max(lo, (max(cq, (int64_t)rg.chunk_left) - rg.chunk_left) * rg.chunk_size);
        const int cq0 = q_off / rg.chunk_size;
        first = max(first, (int)((int64_t)(max(cq0, rg.chunk_left) - rg.chunk_left) * rg.chunk_size / kBkv));
      }
    }
    if (rg.seg_start != nullptr) {
      auto start_of = [&](int64_t r) -> int64_t {
        const int64_t at = (int64_t)b * t + min(r, (int64_t)t - 1);
        const long long x = rg.seg_i64 ? ((const long long *)rg.seg_start)[at] : (long long)((const int *)rg.seg_start)[at];
        return x < 0 ? 0 : (x > tk ? tk : x);
      };
      lo = max(lo, start_of(row_abs));
      first = max(first, (int)(start_of(q_off) / kBkv));
    }
    if (CAUSAL) hi = min(hi, row_abs);
    w.row_lo = (int)lo;
    w.row_hi = (int)max(hi, (int64_t)-1);
  }
  if (key_lens != nullptr) end = min(end, (len + kBkv - 1) / kBkv);
  end = max(end, first);
  // L609-612: a split takes an even share of those blocks.  From here on the kernel works in
  // the split's own frame: keys, lengths and query rows count from the split's first key.
  if (SPLIT) {
    const uint32_t n = (uint32_t)(end - first);
    const int s_first = first + (int)div_by(n * (uint32_t)split, sp.count, sp.rcp);
    end = first + (int)div_by(n * (uint32_t)(split + 1), sp.count, sp.rcp);
    first = s_first;
  }
  const int first_key = first * kBkv;
  end -= first;
  len = max(len - first_key, 0);
  w.end = end;
  w.len = len;
  w.tk = tk - first_key;
  w.key_mask = key_mask;
  w.mask_row = (int64_t)b * tk + first_key;
  w.mask_bytes = mask_bytes;
  w.wave_first_row = q_off + w.wave * kWaveRows - first_key;
  w.my_row = w.wave_first_row + ln;
  w.my_row_ok = q_ok;
  if (BIASED) {
    // L566-571: the bias of this (batch or 0, head), this lane's row, from the tile's first key on.
    const int64_t brow = ((int64_t)(rg.bias_per_batch ? b : 0) * heads + q_head) * t + min(q_row, t - 1);
    w.bias_row = rg.bias + brow * rg.bias_cols + first_key;
    w.bias_keys = rg.bias_cols - first_key;
  }
  if (RANGED) {
    w.row_lo -= first_key;
    w.row_hi -= first_key;
    w.lo_last = __builtin_amdgcn_readlane(w.row_lo, kWaveRows - 1);
    w.hi_first = __builtin_amdgcn_readlane(w.row_hi, 0);
    w.hi_last = __builtin_amdgcn_readlane(w.row_hi, kWaveRows - 1);
  }

  w.kv_row_bytes = kv_row_elems * 2;
  // L544-550: a cache is read at the batch lane's row of it, from the launch's first head on.
  int64_t kv_row = b;
  int kv_col = kvh;
  if (CACHED) {
    if (rg.row_map != nullptr) {
      // The map is device data nobody has checked: a row outside the cache reads its nearest row
      // instead of memory that is not there.
      const long long x = rg.row_map_i64 ? ((const long long *)rg.row_map)[b] : (long long)((const int *)rg.row_map)[b];
      kv_row = x < 0 ? 0 : (x < rg.cache_rows ? x : rg.cache_rows - 1);
    }
    kv_col += rg.kv_head_start;
  }
  w.k_base = (const uint8_t *)(k + (kv_row * tk + first_key) * kv_row_elems + (int64_t)kv_col * D);
  w.v_base = (const uint8_t *)(v + (kv_row * tk + first_key) * kv_row_elems + (int64_t)kv_col * D);
  w.kv_bytes = len > 0 ? (int64_t)(len - 1) * w.kv_row_bytes + D * 2 : 0;
  w.lds0 = (int)(uintptr_t)(LDS_PTR(uint8_t))(smem);

  // ---- this wave's share of a tile fill: CH wave-wide 1 KiB instructions, NW apart.  Fill j
  // lands on rows [j*rows_per, ...): lane i at physical chunk i % kCpr of row i / kCpr.
  constexpr int kRowsPer = 64 / TL::kCpr;
  {
    const int row = w.wave * kRowsPer + w.lane / TL::kCpr;
    const int pc = w.lane % TL::kCpr;
#pragma unroll
    for (int j = 0; j < W::NS; j++) {
      w.k_src[j] = TL::source(row, pc, w.kv_row_bytes, false, j * NW * kRowsPer);
      w.v_src[j] = TL::source(row, pc, w.kv_row_bytes, true, j * NW * kRowsPer);
    }
  }
  // ---- Q fragments: B operand of the score product, resident for the block.
  {
    const uint16_t *q_ptr = q + ((int64_t)b * t + q_row) * q_row_stride + (int64_t)q_head * D + w.g * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      u32x4 x = {0, 0, 0, 0};
      if (q_ok) x = *reinterpret_cast<const u32x4 *>(q_ptr + ks * 16);
      w.qf[ks] = x;
    }
  }
  // ---- the first eight blocks' elements of a key mask row that is scanned up front (see below) are asked for
  // now, a lane a key, straight into this wave's stretch of LDS: behind the Q loads and ahead of the fills in
  // the memory counter's order, so that the scan can wait for them with the fills still in flight.
  w.mask_words = (LDS_PTR(uint64_t))(smem + TL::kLds) + w.wave * kScannedBlocks;
  const bool scan_early = key_mask != nullptr && end <= kScannedBlocks && end > 0;
  if (scan_early) {
    const uint8_t *row = (const uint8_t *)key_mask + w.mask_row * mask_bytes;
    const i32x4 r = make_rsrc(row, (int64_t)w.tk * mask_bytes);  // keys past the row read as hidden
    const int at = (int)(uintptr_t)(w.mask_words);
    // Block i lies 64 elements further on: the instruction's own offset, which the LDS address takes as well as the
    // memory address (block i's 256 bytes of LDS start at m0 + that offset).
    const int voff = w.lane * mask_bytes;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      if (mask_bytes == 1)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_ubyte %1, %2, 0 offen offset:%3 lds"
                     :
                     : "s"(at + i * 256 - i * kBkv), "v"(voff), "s"(r), "n"(i * kBkv)
                     : "memory");
      else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen offset:%3 lds"
                     :
                     : "s"(at + i * 256 - i * kBkv * 4), "v"(voff), "s"(r), "n"(i * kBkv * 4)
                     : "memory");
    }
  }
  // ---- K(0), V(0), K(1): everything below runs in the shadow of their flight.
  w.nxt_end = 0;  // one item a workgroup
  w.end_even = end;
  w.nxt_k = w.nxt_v = nullptr;
  w.nxt_bytes = 0;
  const int fills_out = W::CH * (end > 1 ? 3 : end > 0 ? 2 : 0);
  fill_k<D, NW>(w, 0, 0);
  fill_v<D, NW>(w, 0, 0);
  fill_k<D, NW>(w, 1, 1);
  // A key mask row of up to kScannedBlocks blocks is scanned now, under the fills' flight: every
  // wave ballots each block's 64 keys into a word of its own LDS copy.  The scan also says where
  // the row's last visible key is (later blocks are skipped, like blocks past a length) and how
  // many leading blocks hide nothing (those take the hot loop).  A longer row's words are read two
  // blocks ahead of their use instead.
  w.scanned = key_mask != nullptr && end <= kScannedBlocks;
  int word0 = 0, lead_open = 0, seen_end = 0;
  w.mask_next = 0;
  if (w.scanned) {
    bool open = true;
    int visible = 0, last_key = 0;  // keys the row shows, and the place after the last of them
    // A row of up to eight blocks keeps its words in scalar registers until it is known to need them: a padding
    // mask (the usual case) turns into a length below and never reads them.
    const bool few = end <= 8;
    uint64_t kept[8];
    for (int base = 0; base < end; base += 8) {
      // Eight blocks' elements in flight together: every lane loads (a key past the row's end, or a block
      // past the tile's, loads the row's first element and drops it), so that no branch stands between the
      // loads and a single wait brings them in.
      int words[8];
      if (base == 0 && scan_early) {
        // Asked for ahead of the fills: everything issued before the fills is back when no more than the fills are out.
        constexpr int kCh = W::CH;
        if (fills_out == 3 * kCh)
          asm volatile("s_waitcnt vmcnt(%0)" : : "n"(3 * kCh) : "memory");
        else if (fills_out == 2 * kCh)
          asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * kCh) : "memory");
        else
          asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
        LDS_PTR(const int) raw = (LDS_PTR(const int))(w.mask_words);
#pragma unroll
        for (int i = 0; i < 8; i++) words[i] = raw[i * 64 + w.lane];
        // The words go where the elements lay: every element is in a register before the first word is written.
        asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
      } else if (w.mask_bytes == 1) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
          const int key = (base + i) * kBkv + w.lane;
          const bool there = base + i < end && key < w.tk;
          const int x = (int)((const uint8_t *)w.key_mask)[w.mask_row + (there ? key : 0)];
          words[i] = there ? x : 0;
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; i++) {
          const int key = (base + i) * kBkv + w.lane;
          const bool there = base + i < end && key < w.tk;
          const int x = ((const int *)w.key_mask)[w.mask_row + (there ? key : 0)];
          words[i] = there ? x : 0;
        }
      }
#pragma unroll
      for (int i = 0; i < 8; i++) {
        if (base + i >= end) break;
        const uint64_t bits = __builtin_amdgcn_ballot_w64(words[i] != 0);
        kept[i] = bits;
        if (!few && w.lane == 0) w.mask_words[base + i] = bits;
        if (bits != 0) {
          seen_end = base + i + 1;
          last_key = (base + i) * kBkv + 64 - __builtin_clzll(bits);
        }
        visible += __builtin_popcountll(bits);
        open = open && bits == ~0ull;
        lead_open += open ? 1 : 0;
      }
    }
    end = min(end, seen_end);
    w.end = end;
    if (visible == last_key) {
      // The row shows exactly its first `last_key` keys (a padding mask): that is a length, and
      // from here on the row runs as one with a length does: no mask word per block, rows past
      // the length never fetched.
      len = min(len, last_key);
      w.len = len;
      w.key_mask = nullptr;
      w.scanned = false;
      w.kv_bytes = len > 0 ? (int64_t)(len - 1) * w.kv_row_bytes + D * 2 : 0;
    } else if (few && w.lane == 0) {
#pragma unroll
      for (int i = 0; i < 8; i++)
        if (i < end) w.mask_words[i] = kept[i];
    }
  } else if (key_mask != nullptr) {
    word0 = mask_lane<D, NW>(w, 0);
    w.mask_next = mask_lane<D, NW>(w, 1);
  }

  // ---- per-lane LDS offsets of the operand reads.
  // K fragment (kb, ks): row 32kb + ln, logical chunk 2ks + g.
#pragma unroll
  for (int ks = 0; ks < KS; ks++) w.k_read[ks] = ln * TL::kRowBytes + (((2 * ks + w.g) ^ TL::swz_k(ln)) << 4);
  // V^T fragment: lanes 4j..4j+3 of a 16-lane group supply row j (four 4-element runs),
  // lane i of the group receives column i of those 4 rows.
  const int vq = (w.lane & 15) >> 2;                             // row within the group of 4
  const int vc = 2 * ((w.lane >> 4) & 1) + ((w.lane & 3) >> 1);  // chunk within the 64-byte group
#pragma unroll
  for (int db = 0; db < DB; db++)
    w.v_read[db] = (4 * w.g + vq) * TL::kRowBytes + ((db ^ TL::swz_v(vq)) << 6) + (vc << 4) + ((w.lane & 1) << 3);

  // ---- online softmax state.  m in RAW score units (raw_max form) when the scale is positive;
  // otherwise the maximum does not commute with it: the scores are scaled first and m lives
  // in the exponent's units (L365-370).
  w.positive = scale > 0.0f && !BIASED;
  w.c_exp = scale * kLog2e;  // L619
  w.unit = w.positive ? w.c_exp : 1.0f;
  w.limit = kRescaleAbove / w.unit;
  w.m_run = -1e30f;
  w.l_run = 0.0f;
  const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int db = 0; db < DB; db++) w.acc[db] = zero;

  // A wait the compiler knows of: it covers the Q loads too, so that no wait of its own for
  // them lands inside the loop, where it would also wait out the fills in flight.
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();

  // ---- the first block's scores, masked, and their row maximum.
  // A causal wave past its last visible key has nothing to add from a block: it only keeps
  // filling and meeting the barriers.  Blocks [0, my_end) are this wave's.
  int my_end = end;
  if (RANGED || CAUSAL) {
    // The last key the wave's last row sees; negative: the blocks lie past every row's reach.
    const int last_seen = RANGED ? w.hi_last : w.wave_first_row + kWaveRows - 1;
    my_end = min(end, last_seen < 0 ? 0 : last_seen / kBkv + 1);
  }

  float sv[32], nv[32];  // S of the current and of the next block, swapping roles each hot step
  float bm = -INFINITY;
#pragma unroll
  for (int i = 0; i < 32; i++) sv[i] = nv[i] = 0.0f;
  if (my_end > 0) {
    uint32_t bw[16];
    if (BIASED) load_bias<D, NW>(w, 0, q_ok, bw);
    scores<D, NW>(w, smem, 0, sv);
    if (!w.positive) {
#pragma unroll
      for (int i = 0; i < 32; i++) sv[i] *= w.c_exp;
    }
    if (BIASED) add_bias<F16>(bw, sv);
    const uint64_t kbits0 = uniform_bits<D, NW>(w, 0, word0);
    if (on_edge<D, NW, CAUSAL>(w, 0, kbits0)) mask_scores<D, NW, CAUSAL>(w, 0, kbits0, sv);
    bm = row_max(sv);
  }
  // Step 0 refills the K slot those scores were read from: every wave has read it first.
  __syncthreads();

  // Blocks [0, full) are crossed by no mask edge for this wave: they lie below the length and,
  // for a causal wave, below its first row's diagonal.  A key mask puts every block on the
  // edge path.  Step j is hot when block j+1 is such a block.
  int full = 0;
  if (w.positive && (w.key_mask == nullptr || w.scanned)) {
    full = min(my_end, len / kBkv);
    if (w.scanned) full = min(full, lead_open);
    if (RANGED)
      full = min(full, w.hi_first < 0 ? 0 : (w.hi_first + 1) / kBkv);
    else if (CAUSAL)
      full = min(full, (w.wave_first_row + 1) / kBkv);
  }
  int blk = 0;
  if (RANGED) {
    // A range's left edge crosses the blocks below the last row's first key: general steps, an
    // even number of them so that the hot pairs start on an even block.
    const int below = w.lo_last;
    const int lead = min(my_end, below <= 0 ? 0 : ((below + kBkv - 1) / kBkv + 1) & ~1);
    for (; blk < lead; blk++) edge_step<D, NW, CAUSAL>(w, smem, blk, my_end, sv, bm);
  }
  for (; blk + 2 < full; blk += 2) {
    hot_step<D, NW, 0>(w, smem, blk, sv, nv, bm);
    hot_step<D, NW, 1>(w, smem, blk + 1, nv, sv, bm);
  }
  for (; blk < my_end; blk++) edge_step<D, NW, CAUSAL>(w, smem, blk, my_end, sv, bm);
  for (; blk < end; blk++) idle_step<D, NW>(w, blk);

  // ---- the appended rows (L739-755, L827-846): one more block of keys, from their own tensors,
  // which only the last split scores; the first `seen` of them are visible and no other mask
  // reaches them.  Every wave is past the last step's barrier, so the ring is free.
  if (CACHED) {
    if (rg.k_app != nullptr && (!SPLIT || split == (int)sp.count - 1)) {
      int seen = rg.app_rows;
      if (rg.app_lens != nullptr) {
        const long long n = rg.app_lens_i64 ? ((const long long *)rg.app_lens)[b] : (long long)((const int *)rg.app_lens)[b];
        seen = (int)(n < 0 ? 0 : (n < seen ? n : seen));
      }
      const int app_row_bytes = (int)geo.kv_heads * D * 2;
      const int64_t at = ((int64_t)b * rg.app_rows * geo.kv_heads + kvh) * D;
      const int64_t bytes = seen > 0 ? (int64_t)(seen - 1) * app_row_bytes + D * 2 : 0;  // hidden rows read as zeros
      {
        const int frow = w.wave * kRowsPer + w.lane / TL::kCpr;
        const int pc = w.lane % TL::kCpr;
        int k_src[W::NS], v_src[W::NS];
#pragma unroll
        for (int j = 0; j < W::NS; j++) {
          k_src[j] = TL::source(frow, pc, app_row_bytes, false, j * NW * kRowsPer);
          v_src[j] = TL::source(frow, pc, app_row_bytes, true, j * NW * kRowsPer);
        }
        fill_tile<D, NW>(w, (const uint8_t *)(rg.k_app + at), bytes, 0, w.lds0, k_src, app_row_bytes);
        fill_tile<D, NW>(w, (const uint8_t *)(rg.v_app + at), bytes, 0, w.lds0 + 2 * TL::kBytes, v_src, app_row_bytes);
      }
      uint32_t bw[16];
      if (BIASED) load_bias<D, NW>(w, tk - first_key, q_ok, bw);  // their columns come last (L84-85)
      __builtin_amdgcn_s_waitcnt(0x0f70);
      __syncthreads();
      scores<D, NW>(w, smem, 0, sv);
      if (!w.positive) {
#pragma unroll
        for (int i = 0; i < 32; i++) sv[i] *= w.c_exp;
      }
      if (BIASED) add_bias<F16>(bw, sv);
      const uint64_t visible = seen >= 64 ? ~0ull : ((1ull << seen) - 1);
      if (visible != ~0ull) hide_scores(visible >> (4 * w.g), sv);
      bm = row_max(sv);
      float corr;
      const float m_exp = adopt_maximum<D, NW>(w, bm, corr);
      const uint8_t *vs_ = smem + 2 * TL::kBytes;
      float bs[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      uint32_t pk[16];
      probabilities<F16>(sv, w.unit, m_exp, bs, pk);
      probabilities<F16>(sv + 16, w.unit, m_exp, bs, pk + 8);
      accumulate<D, NW>(w, vs_, 0, pk);
      accumulate<D, NW>(w, vs_, 1, pk + 8);
      w.l_run = w.l_run * corr + ((bs[0] + bs[1]) + (bs[2] + bs[3]));
    }
  }

  const Pair lp = both_halves(w.l_run);
  const float l_tot = lp.a + lp.b;
  if (SPLIT) {
    // ---- the split's partial state (L899-921): the accumulator as it stands, the maximum in
    // the exponent's units (L848-853) and the sum.
    if (q_ok) {
      const int64_t at = (((int64_t)split * sp.nbatch + b) * t + q_row) * heads + q_head;
      if (w.g == 0) {
        sp.m_part[at] = w.positive ? w.m_run * w.c_exp : w.m_run;
        sp.l_part[at] = l_tot;
      }
      float *o_ptr = sp.o_part + at * D + 4 * w.g;
#pragma unroll
      for (int db = 0; db < DB; db++) {
#pragma unroll
        for (int c = 0; c < 4; c++) {
          if (32 * db + 8 * c >= D) continue;  // the tile's columns past the head
          const f32x4 x = {w.acc[db][4 * c], w.acc[db][4 * c + 1], w.acc[db][4 * c + 2], w.acc[db][4 * c + 3]};
          *reinterpret_cast<f32x4 *>(o_ptr + 32 * db + 8 * c) = x;
        }
      }
    }
    return;
  }
  // ---- out = o / (l == 0 ? 1 : l), bounded store (L892-898, L974-980).
  const float inv = 1.0f / (l_tot == 0.0f ? 1.0f : l_tot);
  // A lane holds four consecutive columns of its row per register quad and its partner in the other half-wave
  // the next four: the halves trade quads (v_permlane32_swap), so that each lane stores eight columns, 128 bits
  // at a time: the lower half the even runs of eight, the upper half the odd ones.
  uint16_t *o_ptr = o + ((int64_t)b * t + q_row) * o_row_stride + (int64_t)q_head * D + 8 * w.g;
#pragma unroll
  for (int db = 0; db < DB; db++) {
#pragma unroll
    for (int c = 0; c < 4; c += 2) {
      if (32 * db + 8 * c >= D) continue;  // the tile's columns past the head (a head of 48: its last 16)
      uint32_t x[2], y[2];
#pragma unroll
      for (int e = 0; e < 2; e++) {
        x[e] = pack2<F16>(w.acc[db][4 * c + 2 * e] * inv, w.acc[db][4 * c + 2 * e + 1] * inv);
        y[e] = pack2<F16>(w.acc[db][4 * c + 4 + 2 * e] * inv, w.acc[db][4 * c + 5 + 2 * e] * inv);
      }
      // swap(x, y): {lower: own x, upper: the partner's y}, {lower: the partner's x, upper: own y}.
      const auto lo = __builtin_amdgcn_permlane32_swap(x[0], y[0], false, false);
      const auto hi = __builtin_amdgcn_permlane32_swap(x[1], y[1], false, false);
      const u32x4 out = {lo[0], hi[0], lo[1], hi[1]};
      if (q_ok) *reinterpret_cast<u32x4 *>(o_ptr + 32 * db + 8 * c) = out;
    }
  }
}
#endif  // __HIP_DEVICE_COMPILE__

template <int D, int NW, bool CAUSAL, bool SPLIT, bool RANGED, bool BIASED, bool CACHED, bool GROUPED, bool F16>
__global__ __launch_bounds__(NW * 64, (D <= 64 && !BIASED && !(RANGED && CACHED)) ? 3 : (D <= 128 ? 2 : 1)) void flash_fwd_kernel(
    uint32_t unit_size, uint32_t unit_rcp, uint32_t nqt_u, uint32_t nqt_rcp, uint32_t kvh_u, uint32_t kvh_rcp,
    uint32_t units, uint32_t heads_group, const void *__restrict__ key_lens, const int32_t *__restrict__ row_order,
    int32_t t, uint32_t tk_lens64, const uint16_t *__restrict__ q, const uint16_t *__restrict__ k,
    const uint16_t *__restrict__ v, uint16_t *__restrict__ o, const void *__restrict__ key_mask, int32_t mask_bytes,
    float scale, Splits sp, int32_t q_row_elems, int32_t kv_row_elems, Ranges rg) {
#if defined(__HIP_DEVICE_COMPILE__)
  // The first 14 dwords of the arguments (up to tk_lens64) arrive in registers with the wave
  // (kernarg preload, scalars and pointers only): they are what the workgroup's coordinates,
  // its batch row and its length need, so none of those waits for an argument load.
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  flash_fwd_body<D, NW, CAUSAL, SPLIT, RANGED, BIASED, CACHED, GROUPED, F16>(
      smem, unit_size, unit_rcp, nqt_u, nqt_rcp, kvh_u, kvh_rcp, units, heads_group, key_lens, row_order, t, tk_lens64,
      q, k, v, o, key_mask, mask_bytes, scale, sp, q_row_elems, kv_row_elems, rg);
#endif
}

#if !defined(SVODK_CODE_OBJECT)  // the library's kernels and their launches: not part of a code object build
// ---------------------------------------------------------------------------------------------
// The streaming form: a workgroup walks query tiles (items) one after another as a single stream
// of key blocks.  The last steps of an item fill the ring with the next item's first blocks, and
// the next item's Q rows are already staged in LDS, so an item starts without the launch, the
// argument loads, the first fills' flight and the output drain that a workgroup of its own pays;
// with 1 to 8 key blocks an item (BGE-M3) those are a third of its time.  Each XCD has a list of
// items; a workgroup starts with two of them by its index and takes the rest from the list's
// shared counter, one item ahead of need (the oldest workgroup of a CU wins the arbitration for
// its SIMDs and runs half again as fast as the youngest, so fixed runs would end far apart).
// ---------------------------------------------------------------------------------------------

// Key blocks of query tile `qt` of a batch row with `len` keys (L596-608), at least 1 (a tile
// with no visible block still takes one step, of a block whose keys are all hidden).
template <int NW, bool CAUSAL>
__device__ __forceinline__ int item_blocks(int qt, int len, int tk, bool has_lens) {
  constexpr int BQ = NW * kWaveRows;
  int end = (tk + kBkv - 1) / kBkv;
  if (CAUSAL) end = min(end, (qt * BQ + BQ + kBkv - 1) / kBkv);
  if (has_lens) end = min(end, (len + kBkv - 1) / kBkv);
  return max(end, 1);
}

// The key length of batch row b, b wave-uniform, as a scalar load: inside the item loop a vector
// load would bring a vmcnt wait that also sits out the fills and stores in flight.
__device__ __forceinline__ int len_of_uniform(const void *key_lens, bool lens_i64, int tk, int b) {
  if (key_lens == nullptr) return tk;
  auto word = [&](int byte) {
    int x;
    asm volatile("s_load_dword %0, %1, %2\n\ts_waitcnt lgkmcnt(0)" : "=s"(x) : "s"(key_lens), "s"(byte) : "memory");
    return x;
  };
  long long n;
  if (lens_i64)
    n = (long long)(((uint64_t)(uint32_t)word(b * 8 + 4) << 32) | (uint32_t)word(b * 8));
  else
    n = (long long)word(b * 4);
  n = n < 0 ? 0 : n;
  return n < (long long)tk ? (int)n : tk;
}

// The shared counters of one XCD's item list in one launch.  `next` counts the items handed out
// beyond every workgroup's first two, `done` the workgroups that have left; the last to leave
// puts both back to zero for the launch that gets this set next.  Launches take the sets in
// turn, so a set is met again only kQueueSets launches later.
struct alignas(64) TileQueue {
  uint32_t next, done;
};
constexpr int kQueueSets = 256;
#if SVODK_HAS_HEAD(64)  // the streaming form exists at head size 64 only
__device__ __attribute__((unused)) TileQueue g_tile_queues[kQueueSets][kXcds];
#else
extern __device__ TileQueue g_tile_queues[kQueueSets][kXcds];  // named by the template, never instantiated here
#endif

template <int D, int NW, bool CAUSAL, bool F16>
__global__ __launch_bounds__(NW * 64, 3) void flash_stream_kernel(
    uint32_t unit_size, uint32_t unit_rcp, uint32_t nqt_u, uint32_t nqt_rcp, uint32_t kvh_u, uint32_t kvh_rcp,
    uint32_t units, uint32_t heads_group, const void *__restrict__ key_lens, const uint16_t *__restrict__ q, int32_t t,
    uint32_t tk_lens64, const uint16_t *__restrict__ k, const uint16_t *__restrict__ v,
    uint16_t *__restrict__ o, float scale, int32_t q_row_elems, int32_t kv_row_elems, uint32_t slots,
    uint32_t queue_set, const int32_t *__restrict__ row_order) {
#if defined(__HIP_DEVICE_COMPILE__)
  const Geometry geo = {unit_size, unit_rcp, nqt_u, nqt_rcp, kvh_u, kvh_rcp, heads_group >> 16, units};
  const int heads = (int)(heads_group & 0xffffu);
  const int tk = (int)(tk_lens64 & 0x7fffffffu);
  const bool lens_i64 = (tk_lens64 >> 31) != 0;
  using TL = Tile<D>;
  using W = Wave<D, NW, F16, kStream>;
  constexpr int BQ = NW * kWaveRows;
  constexpr int KS = W::KS, DB = W::DB;
  constexpr int kStageRows = 1024 / TL::kRowBytes;                  // rows a wave instruction stages
  constexpr int kStageInstrs = kWaveRows * TL::kRowBytes / 1024;    // per wave and item
  constexpr int kStageBytes = BQ * TL::kRowBytes;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  uint8_t *stage = smem + TL::kLds;  // [BQ rows][D] of the next item's Q
  // Two words after the stage: the counter's answers, written by wave 0, read by every wave.
  LDS_PTR(uint32_t) answers = (LDS_PTR(uint32_t))(smem + TL::kLds + kStageBytes);

  W w;
  const int tid = __builtin_amdgcn_workitem_id_x();
  w.lane = tid & 63;
  w.wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  w.g = w.lane >> 5;
  const int ln = w.lane & 31;

  // ---- this workgroup's place: XCD `xcd` (workgroups are dealt over the XCDs in turn), number
  // `slot` of `slots` on it.  Items of the XCD's list: unit r of the list is (batch, kv head)
  // number r * 8 + xcd; a unit's items run head-in-group major, then query tile in launch order.
  const uint32_t wg = __builtin_amdgcn_workgroup_id_x();
  const uint32_t xcd = wg % kXcds, slot = wg / kXcds;
  const uint32_t units_here = geo.units > xcd ? (geo.units - xcd + kXcds - 1) / kXcds : 0;
  const uint32_t total = units_here * geo.unit_size;
  TileQueue *queue = &g_tile_queues[queue_set][xcd];
  // Every workgroup of the launch comes by here exactly once, after its last look at `next`.
  auto leave = [&]() {
    // The lane number afresh, not a register kept from the kernel's start.
    const uint32_t lane_now = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    if (w.wave == 0 && lane_now == 0) {
      const uint32_t before = __hip_atomic_fetch_add(&queue->done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (before == slots - 1) {
        __hip_atomic_store(&queue->next, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&queue->done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  };
  if (slot >= total) {
    leave();
    return;
  }

  // ---- call constants
  const int64_t o_row_stride = (int64_t)heads * D;
  w.tk = tk;
  w.key_mask = nullptr;
  w.scanned = false;
  w.mask_row = 0;
  w.mask_bytes = 0;
  w.mask_next = 0;
  w.kv_row_bytes = kv_row_elems * 2;
  w.lds0 = (int)(uintptr_t)(LDS_PTR(uint8_t))(smem);
  constexpr int kRowsPer = 64 / TL::kCpr;
  {
    const int row = w.wave * kRowsPer + w.lane / TL::kCpr;
    const int pc = w.lane % TL::kCpr;
#pragma unroll
    for (int j = 0; j < W::NS; j++) {
      w.k_src[j] = TL::source(row, pc, w.kv_row_bytes, false, j * NW * kRowsPer);
      w.v_src[j] = TL::source(row, pc, w.kv_row_bytes, true, j * NW * kRowsPer);
    }
  }
#pragma unroll
  for (int ks = 0; ks < KS; ks++) w.k_read[ks] = ln * TL::kRowBytes + (((2 * ks + w.g) ^ TL::swz_k(ln)) << 4);
  const int vq = (w.lane & 15) >> 2;
  const int vc = 2 * ((w.lane >> 4) & 1) + ((w.lane & 3) >> 1);
#pragma unroll
  for (int db = 0; db < DB; db++)
    w.v_read[db] = (4 * w.g + vq) * TL::kRowBytes + ((db ^ TL::swz_v(vq)) << 6) + (vc << 4) + ((w.lane & 1) << 3);
  w.positive = scale > 0.0f;
  w.c_exp = scale * kLog2e;
  w.unit = w.positive ? w.c_exp : 1.0f;
  w.limit = kRescaleAbove / w.unit;

  // An item of the list: where its rows and keys are.
  struct Item {
    int b, h, q_off, len, end;
    const uint8_t *k_base, *v_base;
    int64_t kv_bytes;
  };
  auto item = [&](uint32_t s) -> Item {
    Item it;
    const uint32_t round = div_by(s, geo.unit_size, geo.unit_rcp);
    const uint32_t unit = round * kXcds + xcd;
    const uint32_t within = s - round * geo.unit_size;
    const uint32_t head_in_group = div_by(within, geo.nqt, geo.nqt_rcp);
    const int order = (int)(within - head_in_group * geo.nqt);
    const int b_place = (int)div_by(unit, geo.kv_heads, geo.kvh_rcp);
    const int kvh = (int)(unit - (uint32_t)b_place * geo.kv_heads);
    it.h = kvh * (int)geo.group + (int)head_in_group;
    // The batch row of this place of the launch (AttnArgs::row_order), by scalar load like the length.
    it.b = b_place;
    if (row_order != nullptr) {
      int x;
      asm volatile("s_load_dword %0, %1, %2\n\ts_waitcnt lgkmcnt(0)" : "=s"(x) : "s"(row_order), "s"(b_place * 4) : "memory");
      const int nbatch = (int)div_by(geo.units, geo.kv_heads, geo.kvh_rcp);
      it.b = min(max(x, 0), nbatch - 1);
    }
    const int qt = CAUSAL ? (int)geo.nqt - 1 - order : order;  // L524-528: longest first under a causal mask
    it.q_off = qt * BQ;
    it.len = len_of_uniform(key_lens, lens_i64, tk, it.b);
    it.end = item_blocks<NW, CAUSAL>(qt, it.len, tk, key_lens != nullptr);
    it.k_base = (const uint8_t *)(k + (int64_t)it.b * tk * kv_row_elems + (int64_t)kvh * D);
    it.v_base = (const uint8_t *)(v + (int64_t)it.b * tk * kv_row_elems + (int64_t)kvh * D);
    it.kv_bytes = it.len > 0 ? (int64_t)(it.len - 1) * w.kv_row_bytes + D * 2 : 0;
    return it;
  };
  // This wave's rows of an item's Q, global -> LDS: rows past t read as zeros.
  const int stage_lds = w.lds0 + TL::kLds + w.wave * kWaveRows * TL::kRowBytes;
  const int q_row_bytes = q_row_elems * 2;
  auto stage_q = [&](const Item &it) {
    // The lane's offset is worked out afresh each time (the empty asm keeps the compiler from
    // carrying it, and spilling it, across the item loop).
    int lane = w.lane;
    asm volatile("" : "+v"(lane));
    const int stage_src = (lane / TL::kCpr) * q_row_bytes + (lane % TL::kCpr) * 16;
    const int row0 = it.q_off + w.wave * kWaveRows;
    const uint8_t *base = (const uint8_t *)q + ((int64_t)it.b * t + row0) * q_row_bytes + (int64_t)it.h * (D * 2);
    const int64_t rows = (int64_t)t - row0;
    const int64_t bytes = rows > 0 ? (rows - 1) * q_row_bytes + D * 2 : 0;
#pragma unroll
    for (int i = 0; i < kStageInstrs; i++) {
      const int64_t skip = (int64_t)(i * kStageRows) * q_row_bytes;
      const i32x4 r = make_rsrc(base + skip, bytes - skip);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                   :
                   : "s"(stage_lds + i * 1024), "v"(stage_src), "s"(r)
                   : "memory");
    }
  };

  // ---- the first item: K(0), V(0), K(1) and its Q rows in flight, then everything lands.
  Item cur = item(slot);
  auto adopt = [&](const Item &it) {
    int lane = w.lane;
    asm volatile("" : "+v"(lane));
    const int ln = lane & 31;
    w.k_base = it.k_base;
    w.v_base = it.v_base;
    w.kv_bytes = it.kv_bytes;
    w.end = it.end;
    w.end_even = (it.end + 1) & ~1;
    w.len = it.len;
    w.wave_first_row = it.q_off + w.wave * kWaveRows;
    w.my_row = w.wave_first_row + ln;
  };
  adopt(cur);
  w.nxt_end = 0;
  w.nxt_k = w.nxt_v = nullptr;
  w.nxt_bytes = 0;
  fill_k<D, NW>(w, 0, 0);
  fill_v<D, NW>(w, 0, 0);
  fill_k<D, NW>(w, 1, 1);
  stage_q(cur);
  w.m_run = -1e30f;
  w.l_run = 0.0f;
  const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int db = 0; db < DB; db++) w.acc[db] = zero;
  // The second item is fixed as well; the counter hands out the items from 2 * slots on.
  bool more_items = slot + slots < total;
  Item nxt = cur;
  if (more_items) nxt = item(slot + slots);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();

  for (uint32_t round = 0;; round++) {
    // ---- the item after this one: its first blocks ride this item's last steps.
    w.nxt_end = more_items ? nxt.end : 0;
    w.nxt_k = nxt.k_base;
    w.nxt_v = nxt.v_base;
    w.nxt_bytes = nxt.kv_bytes;
    // ---- the item after that: wave 0 asks the counter now and passes the answer on through LDS
    // before the barrier below; every wave reads it after this item's steps.
    uint32_t answer = 0;
    const bool asking = more_items && w.wave == 0;
    if (asking && w.lane == 0)
      answer = __hip_atomic_fetch_add(&queue->next, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // ---- this item's Q rows from the stage to registers; the stage is then free for the next
    // item's rows, which have the whole item to arrive.
    {
      int lane = w.lane;
      asm volatile("" : "+v"(lane));
      const uint8_t *mine = stage + (w.wave * kWaveRows + (lane & 31)) * TL::kRowBytes + (lane >> 5) * 16;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) w.qf[ks] = *reinterpret_cast<const u32x4 *>(mine + ks * 32);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the reads are done before the refill is issued
      if (more_items) stage_q(nxt);
    }
    const int end = w.end;
    int my_end = end;
    if (CAUSAL) {
      const int last_seen = w.wave_first_row + kWaveRows - 1;
      my_end = min(end, last_seen / kBkv + 1);
    }
    float sv[32], nv[32];
    float bm = -INFINITY;
    {
      scores<D, NW>(w, smem, 0, sv);
      if (!w.positive) {
#pragma unroll
        for (int i = 0; i < 32; i++) sv[i] *= w.c_exp;
      }
      const uint64_t kbits0 = uniform_bits<D, NW>(w, 0, 0);
      if (on_edge<D, NW, CAUSAL>(w, 0, kbits0)) mask_scores<D, NW, CAUSAL>(w, 0, kbits0, sv);
      bm = row_max(sv);
    }
    if (asking && w.lane == 0) answers[round & 1] = answer;
    // Step 0 refills the K slot those scores were read from: every wave has read it first.
    __syncthreads();

    int full = 0;
    if (w.positive) {
      full = min(my_end, w.len / kBkv);
      if (CAUSAL) full = min(full, (w.wave_first_row + 1) / kBkv);
    }
    int blk = 0;
    for (; blk + 2 < full; blk += 2) {
      hot_step<D, NW, 0>(w, smem, blk, sv, nv, bm);
      hot_step<D, NW, 1>(w, smem, blk + 1, nv, sv, bm);
    }
    for (; blk < my_end; blk++) edge_step<D, NW, CAUSAL>(w, smem, blk, my_end, sv, bm);
    // Steps with nothing to compute: a causal wave past its diagonal, and the padding of an odd
    // item, which keeps the next item's blocks in the slots a first item's would be in.
    const int steps = more_items ? w.end_even : end;
    for (; blk < steps; blk++) idle_step<D, NW>(w, blk);

    // ---- out = o / (l == 0 ? 1 : l), bounded store (L892-898, L974-980).  The stores fly under
    // the next item's first step.
    {
      const Pair lp = both_halves(w.l_run);
      const float l_tot = lp.a + lp.b;
      const float inv = 1.0f / (l_tot == 0.0f ? 1.0f : l_tot);
      if (w.my_row < t) {
        uint16_t *o_ptr = o + ((int64_t)cur.b * t + w.my_row) * o_row_stride + (int64_t)cur.h * D + 4 * w.g;
#pragma unroll
        for (int db = 0; db < DB; db++) {
#pragma unroll
          for (int c = 0; c < 4; c++) {
            u32x2 x;
            x[0] = pack2<F16>(w.acc[db][4 * c] * inv, w.acc[db][4 * c + 1] * inv);
            x[1] = pack2<F16>(w.acc[db][4 * c + 2] * inv, w.acc[db][4 * c + 3] * inv);
            *reinterpret_cast<u32x2 *>(o_ptr + 32 * db + 8 * c) = x;
          }
        }
      }
      w.m_run = -1e30f;
      w.l_run = 0.0f;
#pragma unroll
      for (int db = 0; db < DB; db++) w.acc[db] = zero;
    }
    if (!more_items) break;
    // Every step ends in a barrier and an item has at least one, so wave 0's answer is there.
    const uint32_t after = 2 * slots + (uint32_t)__builtin_amdgcn_readfirstlane((int)answers[round & 1]);
    cur = nxt;
    adopt(cur);
    more_items = after < total;
    if (more_items) nxt = item(after);
  }
  leave();
#endif  // __HIP_DEVICE_COMPILE__
}

template <int D, int NW, bool CAUSAL, bool F16>
hipError_t launch_stream(const AttnArgs &a, hipStream_t stream, int64_t slots, const Geometry &geo, int64_t q_row,
                         int64_t kv_row) {
  using TL = Tile<D>;
  constexpr int smem = TL::kLds + NW * kWaveRows * TL::kRowBytes + 16;  // ring, Q stage, two words
  auto kernel = flash_stream_kernel<D, NW, CAUSAL, F16>;
  static std::atomic<uint64_t> configured{0};
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  const uint64_t bit = device < 64 ? 1ull << device : 0;
  if ((configured.load(std::memory_order_acquire) & bit) == 0) {
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return e;
    configured.fetch_or(bit, std::memory_order_release);
  }
  const uint32_t heads_group = (uint32_t)a.heads | geo.group << 16;
  const uint32_t tk_lens64 = (uint32_t)a.tk | (a.lens_i64 ? 0x80000000u : 0u);
  hipLaunchKernelGGL(kernel, dim3((uint32_t)(slots * kXcds)), dim3(NW * 64), smem, stream, geo.unit_size, geo.unit_rcp,
                     geo.nqt, geo.nqt_rcp, geo.kv_heads, geo.kvh_rcp, geo.units, heads_group, a.key_lens,
                     (const uint16_t *)a.q, a.t, tk_lens64, (const uint16_t *)a.k, (const uint16_t *)a.v,
                     (uint16_t *)a.o, a.scale, (int32_t)q_row, (int32_t)kv_row, (uint32_t)slots,
                     next_queue_set(), (const int32_t *)a.row_order);
  return hipGetLastError();
}

template <int D, int NW, bool CAUSAL, bool SPLIT, bool RANGED, bool BIASED, bool CACHED, bool GROUPED, bool F16>
hipError_t launch(const AttnArgs &a, hipStream_t stream) {
  using TL = Tile<D>;
  constexpr int BQ = NW * kWaveRows;
  const int splits = SPLIT ? a.splits : 1;
  // grid x: query tile * splits + split (L512, L523); a grouped call has one tile a KV head.
  const int nqt = (GROUPED ? 1 : (a.t + BQ - 1) / BQ) * splits;
  const int64_t blocks = (int64_t)nqt * a.heads * a.batch;
  if (blocks == 0) return hipSuccess;
  if (blocks > 0x7ffffff0LL) return hipErrorInvalidConfiguration;
  // The ring, and behind it the words of a scanned key mask row (a copy a wave).
  constexpr int kMaskLds = NW * kScannedBlocks * 8;
  const int smem = TL::kLds + (a.key_mask != nullptr ? kMaskLds : 0);
  const int64_t q_row = a.q_row_elems > 0 ? a.q_row_elems : (int64_t)a.heads * a.d;
  const int64_t kv_row = a.kv_row_elems > 0 ? a.kv_row_elems : (int64_t)a.kv_heads * a.d;
  // A fill addresses the rows of one key block with 32-bit byte offsets from the block's 64-bit base.
  if (kv_row * 2 * kBkv > 0x7fffffffLL || q_row > 0x7fffffffLL) return hipErrorInvalidValue;
  auto kernel = flash_fwd_kernel<D, NW, CAUSAL, SPLIT, RANGED, BIASED, CACHED, GROUPED, F16>;
  // The LDS ring is above the default limit of a launch: one attribute call per instantiation
  // and device, from whichever thread gets there first (a second call is harmless).
  static std::atomic<uint64_t> configured{0};  // a bit per device ordinal, devices past 63 always ask
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  const uint64_t bit = device < 64 ? 1ull << device : 0;
  if ((configured.load(std::memory_order_acquire) & bit) == 0) {
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            TL::kLds + kMaskLds);
    if (e != hipSuccess) return e;
    configured.fetch_or(bit, std::memory_order_release);
  }
  // Units of work (batch, KV head) are dealt over the XCDs in whole rounds; the workgroups of
  // a round's missing units exit at once.
  const int64_t unit_size = (int64_t)(GROUPED ? 1 : a.heads / a.kv_heads) * nqt;
  const int64_t units = (int64_t)a.kv_heads * a.batch;
  const int64_t grid = (units + kXcds - 1) / kXcds * kXcds * unit_size;
  if (grid > 0x7fffffffLL) return hipErrorInvalidConfiguration;
  auto rcp = [](uint32_t d) { return d == 1 ? 0xffffffffu : (uint32_t)((1ull << 32) / d); };
  Geometry geo;
  geo.unit_size = (uint32_t)unit_size;
  geo.unit_rcp = rcp(geo.unit_size);
  geo.nqt = (uint32_t)nqt;
  geo.nqt_rcp = rcp(geo.nqt);
  geo.kv_heads = (uint32_t)a.kv_heads;
  geo.kvh_rcp = rcp(geo.kv_heads);
  geo.group = (uint32_t)(a.heads / a.kv_heads);
  geo.units = (uint32_t)units;
  if (a.heads > 0xffff) return hipErrorInvalidConfiguration;  // heads and group share an argument
  // The streaming form, where asked for and where it has a kernel (head size 64, lengths or no
  // key mask, no window, no splits): `knob` workgroups per XCD, each walking its run of tiles.
  // It is never chosen unasked: measured, it has not beaten a workgroup per tile.
  if constexpr (D == 64 && !SPLIT && !RANGED && !BIASED && !CACHED && !GROUPED) {
    const int knob = g_stream_slots.load(std::memory_order_relaxed);
    if (knob > 0 && a.key_mask == nullptr) {
      // A captured launch would keep its counter set for every replay, and replays that overlap
      // (two graphs, one graph on two streams) would then share it: a capturing stream gets a
      // workgroup per tile, which needs no counters.
      hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
      e = hipStreamIsCapturing(stream, &capturing);
      if (e != hipSuccess) return e;
      if (capturing == hipStreamCaptureStatusNone)
        return launch_stream<D, NW, CAUSAL, F16>(a, stream, knob, geo, q_row, kv_row);
    }
  }
  const uint32_t heads_group = (uint32_t)a.heads | geo.group << 16;
  const uint32_t tk_lens64 = (uint32_t)a.tk | (a.lens_i64 ? 0x80000000u : 0u);
  Splits sp;
  sp.count = (uint32_t)splits;
  sp.rcp = rcp(sp.count);
  sp.o_part = a.o_part;
  sp.m_part = a.m_part;
  sp.l_part = a.l_part;
  sp.nbatch = (uint32_t)a.batch;
  if (splits > 1 && (a.o_part == nullptr || a.m_part == nullptr || a.l_part == nullptr)) return hipErrorInvalidValue;
  Ranges rg;
  rg.win_left = a.win_left;
  rg.win_right = a.win_right;
  rg.chunk_size = a.chunk_size;
  rg.chunk_left = a.chunk_left;
  rg.chunk_right = a.chunk_right;
  rg.seg_start = a.seg_start;
  rg.seg_i64 = a.seg_i64;
  rg.bias = (const uint16_t *)a.bias;
  rg.bias_per_batch = a.bias_per_batch;
  rg.bias_cols = a.tk + a.app_rows;
  rg.kv_head_start = a.kv_head_start;
  rg.row_map = a.row_map;
  rg.row_map_i64 = a.row_map_i64;
  rg.cache_rows = a.cache_rows;
  rg.k_app = (const uint16_t *)a.k_app;
  rg.v_app = (const uint16_t *)a.v_app;
  rg.app_rows = a.app_rows;
  rg.app_lens = a.app_lens;
  rg.app_lens_i64 = a.app_lens_i64;
  hipLaunchKernelGGL(kernel, dim3((uint32_t)grid), dim3(NW * 64), smem, stream, geo.unit_size, geo.unit_rcp, geo.nqt,
                     geo.nqt_rcp, geo.kv_heads, geo.kvh_rcp, geo.units, heads_group, a.key_lens,
                     (const int32_t *)a.row_order, a.t, tk_lens64, (const uint16_t *)a.q, (const uint16_t *)a.k,
                     (const uint16_t *)a.v, (uint16_t *)a.o, a.key_mask, a.mask_bytes, a.scale, sp, (int32_t)q_row,
                     (int32_t)kv_row, rg);
  return hipGetLastError();
}

template <int D, bool RANGED, bool BIASED, bool CACHED, bool F16>
hipError_t launch_s(const AttnArgs &a, hipStream_t stream) {
  if constexpr (!RANGED) {
    if (attention_groups(a)) {
      return a.splits > 1 ? launch<D, 4, false, true, false, BIASED, CACHED, true, F16>(a, stream)
                          : launch<D, 4, false, false, false, BIASED, CACHED, true, F16>(a, stream);
    }
  }
  if (a.splits > 1)
    return a.causal ? launch<D, 4, true, true, RANGED, BIASED, CACHED, false, F16>(a, stream)
                    : launch<D, 4, false, true, RANGED, BIASED, CACHED, false, F16>(a, stream);
  return a.causal ? launch<D, 4, true, false, RANGED, BIASED, CACHED, false, F16>(a, stream)
                  : launch<D, 4, false, false, RANGED, BIASED, CACHED, false, F16>(a, stream);
}

template <int D, bool F16>
hipError_t launch_t(const AttnArgs &a, hipStream_t stream) {
  // A window, a chunk mask or segment starts: the instantiations with per-row key ranges.
  const bool ranged = a.win_left >= 0 || a.chunk_size > 0 || a.seg_start != nullptr;
  const bool biased = a.bias != nullptr;
  if (a.cached) {
    // A cache under per-row ranges (Attn allows every combination, tk/src/ops/attention.rs:60-86): the ranges
    // hide cached keys only, the appended rows answer to their own count (tk/src/test/unit/attention.rs:138-141).
    if (ranged) return biased ? launch_s<D, true, true, true, F16>(a, stream) : launch_s<D, true, false, true, F16>(a, stream);
    return biased ? launch_s<D, false, true, true, F16>(a, stream) : launch_s<D, false, false, true, F16>(a, stream);
  }
  if (biased) return ranged ? launch_s<D, true, true, false, F16>(a, stream) : launch_s<D, false, true, false, F16>(a, stream);
  return ranged ? launch_s<D, true, false, false, F16>(a, stream) : launch_s<D, false, false, false, F16>(a, stream);
}

template <int D>
hipError_t launch_d(const AttnArgs &a, hipStream_t stream) {
  return a.f16 ? launch_t<D, true>(a, stream) : launch_t<D, false>(a, stream);
}

#if SVODK_HAS_COMMON
// The batch rows in descending order of their key counts, ties by row: order[p] = the row with
// the p-th most keys.  A row's count is its length, or with a [n, tk] key mask the place after its
// last visible key (what a tile's key blocks run to).  One workgroup; a thread ranks its rows
// against all of them in LDS.
__global__ __launch_bounds__(256) void order_rows_kernel(const void *__restrict__ keys, int32_t elem_bytes, int32_t n,
                                                         int32_t tk, int32_t *__restrict__ order) {
  extern __shared__ int32_t lens_sh[];
  if (tk < 0) {
    for (int i = threadIdx.x; i < n; i += 256) {
      const long long x = elem_bytes == 8 ? ((const long long *)keys)[i] : (long long)((const int *)keys)[i];
      lens_sh[i] = (int32_t)(x < 0 ? 0 : (x > 0x7fffffffLL ? 0x7fffffffLL : x));
    }
  } else {
    // A wave a row at a time: the highest key any lane finds visible.
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = wave; i < n; i += 4) {
      int last = 0;
      for (int j = lane; j < tk; j += 64) {
        const int64_t at = (int64_t)i * tk + j;
        const int x = elem_bytes == 1 ? (int)((const uint8_t *)keys)[at] : ((const int *)keys)[at];
        if (x != 0) last = j + 1;
      }
#pragma unroll
      for (int m = 32; m >= 1; m >>= 1) last = max(last, __shfl_xor(last, m, 64));
      if (lane == 0) lens_sh[i] = last;
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += 256) {
    const int32_t mine = lens_sh[i];
    int ahead = 0;
    for (int j = 0; j < n; j++) {
      const int32_t other = lens_sh[j];
      ahead += (other > mine || (other == mine && j < i)) ? 1 : 0;
    }
    order[ahead] = i;
  }
}
#endif  // SVODK_HAS_COMMON

}  // namespace

#if SVODK_HAS_HEAD(32)
hipError_t launch_attention_d32(const AttnArgs &a, hipStream_t stream) { return launch_d<32>(a, stream); }
#endif
#if SVODK_HAS_HEAD(48)
hipError_t launch_attention_d48(const AttnArgs &a, hipStream_t stream) { return launch_d<48>(a, stream); }
#endif
#if SVODK_HAS_HEAD(64)
hipError_t launch_attention_d64(const AttnArgs &a, hipStream_t stream) { return launch_d<64>(a, stream); }
#endif
#if SVODK_HAS_HEAD(128)
hipError_t launch_attention_d128(const AttnArgs &a, hipStream_t stream) { return launch_d<128>(a, stream); }
#endif
#if SVODK_HAS_HEAD(256)
hipError_t launch_attention_d256(const AttnArgs &a, hipStream_t stream) { return launch_d<256>(a, stream); }
#endif

#if SVODK_HAS_COMMON
std::atomic<int> g_stream_slots{0};
std::atomic<uint32_t> g_queue_turn{0};
uint32_t next_queue_set() { return g_queue_turn.fetch_add(1u, std::memory_order_relaxed) % (uint32_t)kQueueSets; }

hipError_t launch_order_rows(const void *keys, int32_t elem_bytes, int32_t n, int32_t tk, int32_t *order,
                             hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  if (n > kMaxOrderedRows) return hipErrorInvalidValue;
  hipLaunchKernelGGL(order_rows_kernel, dim3(1), dim3(256), (size_t)n * 4, stream, keys, elem_bytes, n, tk, order);
  return hipGetLastError();
}

bool attention_supports(int32_t d) { return d == 32 || d == 48 || d == 64 || d == 128 || d == 256; }

bool attention_groups(const AttnArgs &a) {
  const bool ranged = a.win_left >= 0 || a.chunk_size > 0 || a.seg_start != nullptr;
  const int64_t group = a.kv_heads > 0 ? a.heads / a.kv_heads : 1;
  return group > 1 && !a.causal && !ranged && group * a.t <= 128;
}

void attention_stream_slots(int32_t slots) { g_stream_slots.store(slots, std::memory_order_relaxed); }

const char *attention_config(const AttnArgs &a) {
  if (attention_decodes(a))
    return a.splits > 1 ? "FaCfg { rows: 4, lanes_per_key: d / 8, splits: n, core: v_dot2_f32, keys streamed through registers }"
                        : "FaCfg { rows: 4, lanes_per_key: d / 8, splits: 1, core: v_dot2_f32, keys streamed through registers }";
  static const char *const kCfg[2][2] = {
      {"FaCfg { bq: 128, bkv: 64, stages: 2, splits: 1, forms: { raw_max, skip_rescale }, warp_rows: 32, core: "
       "mfma_f32_32x32x16_bf16 }",
       "FaCfg { bq: 128, bkv: 64, stages: 2, splits: n, forms: { raw_max, skip_rescale }, warp_rows: 32, core: "
       "mfma_f32_32x32x16_bf16 }"},
      {"FaCfg { bq: 128, bkv: 64, stages: 2, splits: 1, forms: { raw_max, skip_rescale }, warp_rows: 32, core: "
       "mfma_f32_32x32x16_f16 }",
       "FaCfg { bq: 128, bkv: 64, stages: 2, splits: n, forms: { raw_max, skip_rescale }, warp_rows: 32, core: "
       "mfma_f32_32x32x16_f16 }"}};
  return kCfg[a.f16 ? 1 : 0][a.splits > 1 ? 1 : 0];
}

hipError_t launch_attention(const AttnArgs &a, hipStream_t stream) {
  if (attention_decodes(a)) return launch_decode(a, stream);  // a decoder step: no key tiles, a stream of K and V
  switch (a.d) {
    case 32: return launch_attention_d32(a, stream);
    case 48: return launch_attention_d48(a, stream);
    case 64: return launch_attention_d64(a, stream);
    case 128: return launch_attention_d128(a, stream);
    case 256: return launch_attention_d256(a, stream);
    default: return hipErrorInvalidValue;
  }
}
#endif  // SVODK_HAS_COMMON

}  // namespace svodk

#else  // SVODK_CODE_OBJECT
// ---------------------------------------------------------------------------------------------
// The same program as kernels a loader outside the HIP runtime can run: the reference's device
// layer loads an AMDGPU code object, finds `<name>.kd`, and launches it with a flat argument
// record (device/src/amd/program.rs:77-266, 403-414, 655-675; device/src/hcq.rs:1262-1285):
//   * buffers are 8-byte addresses, every scalar a 4-byte integer, in parameter order at their
//     natural alignment; nothing hidden follows them (the record is kernarg_size bytes, zeroed);
//   * LDS is what the kernel descriptor says (group_segment_fixed_size): static, no launch-time size;
//   * no dispatch packet pointer: the kernel may know its workgroup and lane, not the grid's or
//     the workgroup's size (ENABLE_SGPR_DISPATCH_PTR must be clear);
//   * the launch names workgroup COUNTS and the workgroup's threads.
// So these take plain dimensions and work the launch geometry out themselves (three unsigned
// divisions a workgroup), the scale travels as its bit pattern, and arguments are not preloaded
// into registers (a loader that writes its own user registers hands over the record's address only).
//
// Parameters follow the reference kernel's order (tk/src/kernels/attention.rs:308-327, 452-459):
// q, k, v, o, then key_lens ([batch] i32, or address 0 for none) or, for the `_mask` kernels,
// key_mask ([batch, tk] bytes, a key visible where its byte is not 0: a Bool tensor as it lies in
// memory), then the scalars batch, t, tk, heads, kv_heads, scale_bits.  Launch: workgroups
// [ceil(batch * kv_heads, 8) * (heads / kv_heads) * ceil(t / 128), 1, 1] of [256, 1, 1] threads.
// The host side's checks are the caller's: heads a multiple of kv_heads, heads < 65536, dimensions
// positive, 64 rows of k or v within 2^31 bytes (kv_heads * D < 2^24).
// ---------------------------------------------------------------------------------------------
#if defined(__HIP_DEVICE_COMPILE__)
// floor(2^32 / d) for div_by, or one less where d divides 2^32 (the estimate stays within one).
__device__ __forceinline__ uint32_t rcp_for(uint32_t d) { return d <= 1 ? 0xffffffffu : 0xffffffffu / d; }

template <int D, bool CAUSAL, bool F16>
__device__ __forceinline__ void attention_entry(uint8_t *smem, const uint16_t *q, const uint16_t *k, const uint16_t *v,
                                                uint16_t *o, const void *key_lens, const void *key_mask, int32_t batch,
                                                int32_t t, int32_t tk, int32_t heads, int32_t kv_heads,
                                                int32_t scale_bits) {
  constexpr int NW = 4;
  if (batch <= 0 || t <= 0 || tk < 0 || kv_heads <= 0 || heads < kv_heads) return;
  const uint32_t group = (uint32_t)heads / (uint32_t)kv_heads;
  const uint32_t nqt = ((uint32_t)t + NW * kWaveRows - 1) / (NW * kWaveRows);
  const uint32_t units = (uint32_t)kv_heads * (uint32_t)batch;
  const uint32_t span = group * nqt;  // a unit's workgroups
  const Splits sp = {1u, 0xffffffffu, nullptr, nullptr, nullptr, (uint32_t)batch};
  Ranges rg = {};
  rg.win_left = -1;
  rg.chunk_left = -1;
  flash_fwd_body<D, NW, CAUSAL, false, false, false, false, false, F16>(
      smem, span, rcp_for(span), nqt, rcp_for(nqt), (uint32_t)kv_heads, rcp_for((uint32_t)kv_heads), units,
      (uint32_t)heads | group << 16, key_lens, nullptr, t, (uint32_t)tk, q, k, v, o, key_mask, 1,
      __builtin_bit_cast(float, scale_bits), sp, heads * D, kv_heads * D, rg);
}
#endif

// ---- every form the library has, one kernel an instantiation (svodk_attention_full_d<D>_<type>_
// c<causal>s<split>r<ranged>b<biased>k<cached>g<grouped>), all with one record.  Buffers, in the
// reference kernel's order (tk/src/kernels/attention.rs:308-327, 452-459), an address of 0 for what
// a call does not have: q, k, v, o, key_lens, key_mask, seg_start, row_map, k_app, v_app, app_lens,
// bias, then the partial states of a split call o_part, m_part, l_part.  Scalars: batch, t, tk,
// heads, kv_heads, scale_bits, lens_i64, mask_bytes (1 or 4), q_row_elems, kv_row_elems (0: heads * D
// and kv_heads * D; a fused projection's or a cache's row otherwise), splits, win_left (< 0: no
// window), win_right, chunk_size (0: none), chunk_left (< 0: every earlier chunk), chunk_right,
// seg_i64, bias_per_batch, kv_head_start, row_map_i64, cache_rows, app_rows, app_lens_i64.
// A kernel reads what its flags name and ignores the rest.  Launch: ceil(batch * kv_heads, 8) * per
// workgroups of 256 threads, per = (g ? 1 : heads / kv_heads) * (g ? 1 : ceil(t / 128)) * (s ? splits : 1).
// LDS: the ring and the scanned mask words.  The caller keeps the op layer's checks, the caps on the
// window's and the chunks' reaches included (at most t + tk, and the chunks of t + tk).
#define SVODK_FULL_PARAMS                                                                                             \
  const uint16_t *__restrict__ q, const uint16_t *__restrict__ k, const uint16_t *__restrict__ v,                     \
      uint16_t *__restrict__ o, const void *__restrict__ key_lens, const void *__restrict__ key_mask,                 \
      const void *__restrict__ seg_start, const void *__restrict__ row_map, const uint16_t *__restrict__ k_app,       \
      const uint16_t *__restrict__ v_app, const void *__restrict__ app_lens, const uint16_t *__restrict__ bias,       \
      float *__restrict__ o_part, float *__restrict__ m_part, float *__restrict__ l_part, int32_t batch, int32_t t,   \
      int32_t tk, int32_t heads, int32_t kv_heads, int32_t scale_bits, int32_t lens_i64, int32_t mask_bytes,          \
      int32_t q_row_elems, int32_t kv_row_elems, int32_t splits, int32_t win_left, int32_t win_right,                 \
      int32_t chunk_size, int32_t chunk_left, int32_t chunk_right, int32_t seg_i64, int32_t bias_per_batch,           \
      int32_t kv_head_start, int32_t row_map_i64, int32_t cache_rows, int32_t app_rows, int32_t app_lens_i64
#define SVODK_FULL_ARGS                                                                                               \
  q, k, v, o, key_lens, key_mask, seg_start, row_map, k_app, v_app, app_lens, bias, o_part, m_part, l_part, batch, t, \
      tk, heads, kv_heads, scale_bits, lens_i64, mask_bytes, q_row_elems, kv_row_elems, splits, win_left, win_right,  \
      chunk_size, chunk_left, chunk_right, seg_i64, bias_per_batch, kv_head_start, row_map_i64, cache_rows, app_rows, \
      app_lens_i64

#if defined(__HIP_DEVICE_COMPILE__)
template <int D, bool CAUSAL, bool SPLIT, bool RANGED, bool BIASED, bool CACHED, bool GROUPED, bool F16>
__device__ __forceinline__ void attention_entry_full(uint8_t *smem, SVODK_FULL_PARAMS) {
  constexpr int NW = 4;
  if (batch <= 0 || t <= 0 || tk < 0 || kv_heads <= 0 || heads < kv_heads) return;
  const uint32_t group = (uint32_t)heads / (uint32_t)kv_heads;
  const uint32_t count = SPLIT ? (uint32_t)(splits > 0 ? splits : 1) : 1u;
  const uint32_t nqt = (GROUPED ? 1u : ((uint32_t)t + NW * kWaveRows - 1) / (NW * kWaveRows)) * count;
  const uint32_t units = (uint32_t)kv_heads * (uint32_t)batch;
  const uint32_t span = (GROUPED ? 1u : group) * nqt;
  const Splits sp = {count, rcp_for(count), o_part, m_part, l_part, (uint32_t)batch};
  Ranges rg = {};
  rg.win_left = RANGED ? win_left : -1;
  rg.win_right = win_right;
  rg.chunk_size = RANGED ? chunk_size : 0;
  rg.chunk_left = chunk_left;
  rg.chunk_right = chunk_right;
  rg.seg_start = RANGED ? seg_start : nullptr;
  rg.seg_i64 = seg_i64;
  rg.bias = bias;
  rg.bias_per_batch = bias_per_batch;
  rg.bias_cols = tk + (CACHED ? app_rows : 0);
  rg.kv_head_start = kv_head_start;
  rg.row_map = row_map;
  rg.row_map_i64 = row_map_i64;
  rg.cache_rows = cache_rows;
  rg.k_app = k_app;
  rg.v_app = v_app;
  rg.app_rows = app_rows;
  rg.app_lens = app_lens;
  rg.app_lens_i64 = app_lens_i64;
  flash_fwd_body<D, NW, CAUSAL, SPLIT, RANGED, BIASED, CACHED, GROUPED, F16>(
      smem, span, rcp_for(span), nqt, rcp_for(nqt), (uint32_t)kv_heads, rcp_for((uint32_t)kv_heads), units,
      (uint32_t)heads | group << 16, key_lens, nullptr, t, (uint32_t)tk | (lens_i64 ? 0x80000000u : 0u), q, k, v, o,
      key_mask, mask_bytes, __builtin_bit_cast(float, scale_bits), sp, q_row_elems > 0 ? q_row_elems : heads * D,
      kv_row_elems > 0 ? kv_row_elems : kv_heads * D, rg);
}
#endif

#define SVODK_FULL_ENTRY(D, T, F16, C, S, R, B, K, G)                                                                 \
  extern "C" __global__ __launch_bounds__(256, ((D) <= 64 && !(B) && !((R) && (K))) ? 3 : ((D) <= 128 ? 2 : 1)) void  \
      svodk_attention_full_d##D##_##T##_c##C##s##S##r##R##b##B##k##K##g##G(SVODK_FULL_PARAMS) {                       \
    __shared__ __attribute__((aligned(1024))) uint8_t smem[Tile<D>::kLds + 4 * kScannedBlocks * 8];                   \
    attention_entry_full<D, C, S, R, B, K, G, F16>(smem, SVODK_FULL_ARGS);                                            \
  }
// The instantiations the library's own dispatch reaches: grouped tiles take neither a causal mask nor
// ranges.
#define SVODK_FULL_SPLITS(D, T, F16, C, R, B, K, G) \
  SVODK_FULL_ENTRY(D, T, F16, C, 0, R, B, K, G) SVODK_FULL_ENTRY(D, T, F16, C, 1, R, B, K, G)
#define SVODK_FULL_TILES(D, T, F16, R, B, K)                                                  \
  SVODK_FULL_SPLITS(D, T, F16, 0, R, B, K, 0) SVODK_FULL_SPLITS(D, T, F16, 1, R, B, K, 0)
#define SVODK_FULL_FAMILY(D, T, F16)                                                          \
  SVODK_FULL_TILES(D, T, F16, 0, 0, 0) SVODK_FULL_SPLITS(D, T, F16, 0, 0, 0, 0, 1)           \
  SVODK_FULL_TILES(D, T, F16, 0, 1, 0) SVODK_FULL_SPLITS(D, T, F16, 0, 0, 1, 0, 1)           \
  SVODK_FULL_TILES(D, T, F16, 1, 0, 0) SVODK_FULL_TILES(D, T, F16, 1, 1, 0)                   \
  SVODK_FULL_TILES(D, T, F16, 0, 0, 1) SVODK_FULL_SPLITS(D, T, F16, 0, 0, 0, 1, 1)           \
  SVODK_FULL_TILES(D, T, F16, 0, 1, 1) SVODK_FULL_SPLITS(D, T, F16, 0, 0, 1, 1, 1)           \
  SVODK_FULL_TILES(D, T, F16, 1, 0, 1) SVODK_FULL_TILES(D, T, F16, 1, 1, 1)

#if defined(SVODK_HEAD)  // one head size's whole family a file
#if SVODK_HEAD == 32
SVODK_FULL_FAMILY(32, bf16, false) SVODK_FULL_FAMILY(32, f16, true)
#elif SVODK_HEAD == 48
SVODK_FULL_FAMILY(48, bf16, false) SVODK_FULL_FAMILY(48, f16, true)
#elif SVODK_HEAD == 64
SVODK_FULL_FAMILY(64, bf16, false) SVODK_FULL_FAMILY(64, f16, true)
#elif SVODK_HEAD == 128
SVODK_FULL_FAMILY(128, bf16, false) SVODK_FULL_FAMILY(128, f16, true)
#elif SVODK_HEAD == 256
SVODK_FULL_FAMILY(256, bf16, false) SVODK_FULL_FAMILY(256, f16, true)
#endif
#else  // the short records: lengths or a key mask, causal or not

#define SVODK_ATTENTION_ENTRY(NAME, D, CAUSAL, F16)                                                                  \
  extern "C" __global__ __launch_bounds__(256, (D) <= 64 ? 3 : ((D) <= 128 ? 2 : 1)) void NAME(                       \
      const uint16_t *__restrict__ q, const uint16_t *__restrict__ k, const uint16_t *__restrict__ v,                 \
      uint16_t *__restrict__ o, const void *__restrict__ key_lens, int32_t batch, int32_t t, int32_t tk, int32_t heads, \
      int32_t kv_heads, int32_t scale_bits) {                                                                         \
    __shared__ __attribute__((aligned(1024))) uint8_t smem[Tile<D>::kLds];                                            \
    attention_entry<D, CAUSAL, F16>(smem, q, k, v, o, key_lens, nullptr, batch, t, tk, heads, kv_heads, scale_bits);  \
  }

// Behind the ring, the words of the scanned key mask row: a copy a wave.
#define SVODK_ATTENTION_MASK_ENTRY(NAME, D, CAUSAL, F16)                                                             \
  extern "C" __global__ __launch_bounds__(256, (D) <= 64 ? 3 : ((D) <= 128 ? 2 : 1)) void NAME(                       \
      const uint16_t *__restrict__ q, const uint16_t *__restrict__ k, const uint16_t *__restrict__ v,                 \
      uint16_t *__restrict__ o, const void *__restrict__ key_mask, int32_t batch, int32_t t, int32_t tk, int32_t heads, \
      int32_t kv_heads, int32_t scale_bits) {                                                                         \
    __shared__ __attribute__((aligned(1024))) uint8_t smem[Tile<D>::kLds + 4 * kScannedBlocks * 8];                   \
    attention_entry<D, CAUSAL, F16>(smem, q, k, v, o, nullptr, key_mask, batch, t, tk, heads, kv_heads, scale_bits);  \
  }

SVODK_ATTENTION_ENTRY(svodk_attention_d32_bf16, 32, false, false)
SVODK_ATTENTION_ENTRY(svodk_attention_d32_bf16_causal, 32, true, false)
SVODK_ATTENTION_ENTRY(svodk_attention_d48_bf16, 48, false, false)
SVODK_ATTENTION_ENTRY(svodk_attention_d48_bf16_causal, 48, true, false)
SVODK_ATTENTION_ENTRY(svodk_attention_d64_bf16, 64, false, false)
SVODK_ATTENTION_ENTRY(svodk_attention_d64_bf16_causal, 64, true, false)
SVODK_ATTENTION_ENTRY(svodk_attention_d128_bf16, 128, false, false)
SVODK_ATTENTION_ENTRY(svodk_attention_d128_bf16_causal, 128, true, false)
SVODK_ATTENTION_ENTRY(svodk_attention_d256_bf16, 256, false, false)
SVODK_ATTENTION_ENTRY(svodk_attention_d256_bf16_causal, 256, true, false)
SVODK_ATTENTION_ENTRY(svodk_attention_d32_f16, 32, false, true)
SVODK_ATTENTION_ENTRY(svodk_attention_d32_f16_causal, 32, true, true)
SVODK_ATTENTION_ENTRY(svodk_attention_d48_f16, 48, false, true)
SVODK_ATTENTION_ENTRY(svodk_attention_d48_f16_causal, 48, true, true)
SVODK_ATTENTION_ENTRY(svodk_attention_d64_f16, 64, false, true)
SVODK_ATTENTION_ENTRY(svodk_attention_d64_f16_causal, 64, true, true)
SVODK_ATTENTION_ENTRY(svodk_attention_d128_f16, 128, false, true)
SVODK_ATTENTION_ENTRY(svodk_attention_d128_f16_causal, 128, true, true)
SVODK_ATTENTION_ENTRY(svodk_attention_d256_f16, 256, false, true)
SVODK_ATTENTION_ENTRY(svodk_attention_d256_f16_causal, 256, true, true)
SVODK_ATTENTION_MASK_ENTRY(svodk_attention_d64_bf16_mask, 64, false, false)
SVODK_ATTENTION_MASK_ENTRY(svodk_attention_d64_bf16_causal_mask, 64, true, false)
SVODK_ATTENTION_MASK_ENTRY(svodk_attention_d128_bf16_mask, 128, false, false)
SVODK_ATTENTION_MASK_ENTRY(svodk_attention_d128_bf16_causal_mask, 128, true, false)
SVODK_ATTENTION_MASK_ENTRY(svodk_attention_d256_bf16_mask, 256, false, false)
SVODK_ATTENTION_MASK_ENTRY(svodk_attention_d256_bf16_causal_mask, 256, true, false)
SVODK_ATTENTION_MASK_ENTRY(svodk_attention_d64_f16_mask, 64, false, true)
SVODK_ATTENTION_MASK_ENTRY(svodk_attention_d64_f16_causal_mask, 64, true, true)
SVODK_ATTENTION_MASK_ENTRY(svodk_attention_d128_f16_mask, 128, false, true)
SVODK_ATTENTION_MASK_ENTRY(svodk_attention_d128_f16_causal_mask, 128, true, true)
SVODK_ATTENTION_MASK_ENTRY(svodk_attention_d256_f16_mask, 256, false, true)
SVODK_ATTENTION_MASK_ENTRY(svodk_attention_d256_f16_causal_mask, 256, true, true)
#undef SVODK_ATTENTION_ENTRY
#undef SVODK_ATTENTION_MASK_ENTRY
#endif  // SVODK_HEAD

}  // namespace
}  // namespace svodk
#endif  // SVODK_CODE_OBJECT

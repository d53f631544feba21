// linear with the rope epilogue for gfx950 (MI355X): y = x . w^T + bias over x [rows, K] and w [N, K]
// (both K-contiguous), the first `heads` heads of `head_dim` output columns turned by the rotary tables'
// row of the token's position before the one rounding at the store.  The algorithm is the reference GEMM
// kernel's epilogue (tk/src/kernels/gemm.rs:604-645 `finish`, :666-716 `turn`): f32 accumulators, the bias
// added in f32, then per turned column  y = fma(partner, +-sin, x * cos)  with the partner half a head
// along and sin negated over a head's first half, then the cast.  A fused projection's queries and keys
// come out rotated and its values plain, so a model without QK norms needs no prologue pass at all
// (tk/src/ops/linear.rs:47-58).
//
// The mapping onto CDNA4 is this file's own.  A workgroup of 8 waves owns a 256 x 256 output tile; a wave
// owns 64 rows x 128 columns as 2 x 4 accumulators of v_mfma_f32_32x32x16.  The product runs transposed,
// C^T = W . X^T, so that a lane owns one output ROW and, per accumulator register quad, four CONSECUTIVE
// columns: the rotation's partner column (32 or 64 columns along) is the same lane's register of another
// accumulator, and the tables (staged through LDS once the ring is done with) are read as 8-byte runs of the
// lane's row.  The finished tile goes through LDS once more, a wave's rows in a stretch of its own, and
// leaves as whole 256-byte row segments, 16 bytes a lane.
// X and W tiles of 64 k-columns stream through a two-stage LDS ring (64 KiB a stage), filled global -> LDS
// by buffer_load_dwordx4 ... lds a stage ahead.  What bounds this kernel is the way from L2 into LDS: the
// part moves about 18 TB/s along it when every fill takes whole 128-byte lines and about 12 TB/s when it
// takes half lines (measured: the fills of this kernel alone, without its products).  Hence tiles this
// large (1 GiB of fills at the projection shape where 256 x 128 tiles move 1.5 GiB) and rows of 128 bytes,
// a whole line each; their eight 16-byte chunks are XOR-swizzled by (row / 2) % 8 through the lanes' source
// addresses so that a ds_read_b128 of 16 rows at one logical chunk touches every bank once.  Rows past the
// operands' ends read as zeros through the buffer descriptors' bounds.  One barrier a stage (32 MFMAs a wave).
#include <hip/hip_runtime.h>

#include <atomic>

#include "kernels.h"

namespace svodk {
namespace {

#if !defined(__HIP_DEVICE_COMPILE__)
#pragma clang diagnostic ignored "-Wunused-function"
#pragma clang diagnostic ignored "-Wunused-const-variable"
#endif

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) int i32x4;

constexpr int kXcds = 8;
constexpr int kBk = 64;                 // k-columns a stage: a row of a tile is one 128-byte line
constexpr int kSteps = kBk / 16;        // k-steps of the matrix instruction a stage
constexpr int kStages = 2;
constexpr int kGroup = 8;               // column tiles an XCD's resident workgroups spread over
constexpr int kRowBytes = kBk * 2;      // a tile row in LDS
constexpr int kOutPitch = 128 * 2 + 16;               // a wave's row of the finished tile in LDS
// The workgroup's output tile in two sizes.  S = 2: 256 x 256 by 8 waves (4 along the rows x 2 along the columns,
// 64 rows x 128 columns a wave), the size for a product with tiles enough to fill the part.  S = 1: 128 x 128 by
// 4 waves (32 rows x 128 columns a wave), two workgroups a compute unit: a product of few rows gets four times the
// workgroups, at twice the fills a flop.  A wave's 128 columns hold whole heads of 64 or 128 either way.
template <int S>
struct Tile {
  static constexpr int kWaves = 4 * S;
  static constexpr int kBm = 128 * S, kBn = 128 * S;
  static constexpr int kTileBytes = kBm * kRowBytes;           // one operand's tile: 32 (16) KiB
  static constexpr int kStageBytes = 2 * kTileBytes;           // W tile, then X tile
  static constexpr int kLds = kStages * kStageBytes;           // 128 (64) KiB
  static constexpr int kFills = kStageBytes / 1024 / kWaves;   // wave instructions of 1 KiB per wave and stage: 8
  static_assert(kWaves * 32 * kOutPitch <= kLds, "32 rows a wave of the finished tile fit where the ring was");
};

template <bool F16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  f32x2 f = {lo, hi};
  if constexpr (F16)
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
  else
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

// One 16-bit element of the operands' type as f32.
template <bool F16>
__device__ __forceinline__ float widen(uint32_t bits16) {
  if constexpr (F16) return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
  return __builtin_bit_cast(float, bits16 << 16);
}

template <bool F16>
__device__ __forceinline__ f32x16 mma(const u32x4 &a, const u32x4 &b, const f32x16 &c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// A raw buffer descriptor over `bytes` bytes at `base`: loads past the end return zero.
__device__ __forceinline__ i32x4 make_rsrc(const void *base, int64_t bytes) {
  const int64_t clamped = bytes < 0 ? 0 : (bytes > 0xffffffffLL ? 0xffffffffLL : bytes);
  const uint64_t addr = (uint64_t)(uintptr_t)base;
  i32x4 r;
  r[0] = (int)(uint32_t)addr;
  r[1] = (int)(uint32_t)((addr >> 32) & 0xffffu);
  r[2] = (int)(uint32_t)clamped;
  r[3] = 0x00020000;
  return r;
}

// Four 16-bit elements at `p` (8-byte aligned) as f32.
template <bool F16>
__device__ __forceinline__ void load4(const uint16_t *p, float (&out)[4]) {
  const u32x2 x = *reinterpret_cast<const u32x2 *>(p);
  out[0] = widen<F16>(x[0] & 0xffffu);
  out[1] = widen<F16>(x[0] >> 16);
  out[2] = widen<F16>(x[1] & 0xffffu);
  out[3] = widen<F16>(x[1] >> 16);
}

#if defined(__HIP_DEVICE_COMPILE__)
// HD: the head size a turning kernel is built for (64 or 128), 0: no turn.
template <bool F16, int HD, int S = 2>
__device__ __forceinline__ void linear_body(uint8_t *smem, const uint16_t *__restrict__ x, const uint16_t *__restrict__ w,
                                            const uint16_t *__restrict__ bias, const uint16_t *__restrict__ cos_t,
                                            const uint16_t *__restrict__ sin_t, uint16_t *__restrict__ y, int64_t y_ld,
                                            int64_t rows, int32_t n, int32_t k, int32_t seq, int32_t heads,
                                            uint32_t tiles_n, uint32_t tiles, uint32_t per_xcd, uint32_t band) {
  constexpr int kWaves = Tile<S>::kWaves, kBm = Tile<S>::kBm, kBn = Tile<S>::kBn, kTileBytes = Tile<S>::kTileBytes;
  constexpr int kStageBytes = Tile<S>::kStageBytes, kLds = Tile<S>::kLds, kFills = Tile<S>::kFills;
  const int tid = __builtin_amdgcn_workitem_id_x();
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, ln = lane & 31;
  // Workgroups are dealt to the 8 XCDs in turn, each XCD with an L2 of its own.  With rows enough
  // (`band` > 0) XCD x owns a band of `band` row tiles and walks it in groups of up to kGroup column
  // tiles, row tile by row tile within a group: the workgroups resident together then share few w tiles
  // (read once per XCD) and few x tiles (read once per group), instead of streaming all of w past every
  // row tile.  With few rows XCD x takes a run of consecutive tiles, column tile fastest.
  const uint32_t wg = __builtin_amdgcn_workgroup_id_x();
  const uint32_t xcd = wg % kXcds, local = wg / kXcds;
  uint32_t tm, tn;
  if (band > 0) {
    const uint32_t full = band * kGroup;            // workgroups of a full-width group
    const uint32_t ng = local / full;               // the group
    const uint32_t first = ng * kGroup;             // its first column tile
    if (first >= tiles_n) return;
    const uint32_t width = min((uint32_t)kGroup, tiles_n - first);
    const uint32_t r = local - ng * full;
    const uint32_t tm_local = r / width;
    if (tm_local >= band) return;
    tm = xcd * band + tm_local;
    tn = first + (r - tm_local * width);
    if ((uint64_t)tm * tiles_n + tn >= tiles) return;  // past the last row tile
  } else {
    const uint32_t tile = xcd * per_xcd + local;
    if (local >= per_xcd || tile >= tiles) return;
    tm = tile / tiles_n;
    tn = tile - tm * tiles_n;
  }
  const int64_t m0 = (int64_t)tm * kBm;
  const int32_t n0 = (int32_t)tn * kBn;
  const int64_t row_bytes = (int64_t)k * 2;

  // ---- this wave's fills of a stage: 8 rows x 8 chunk places an instruction; a stage is 64 of them, the
  // W tile's 32 and then the X tile's 32, and wave v takes instructions v, v + 8, ...  Those are 64 rows
  // apart, a multiple of the swizzle's period of 16, so one lane offset serves all eight; the descriptors'
  // bases differ.
  const int frow = lane >> 3, place = lane & 7;
  const int src = frow * (int)row_bytes + ((place ^ ((4 * (wave & 1) + (frow >> 1)) & 7)) << 4);
  i32x4 rsrc[kFills];
  int lds_at[kFills];
#pragma unroll
  for (int f = 0; f < kFills; f++) {
    const int j = wave + kWaves * f;  // the instruction of the stage
    const bool is_x = f >= kFills / 2;
    const int block_row = 8 * (is_x ? j - kTileBytes / 1024 : j);
    const int64_t first = (is_x ? m0 : (int64_t)n0) + block_row;
    const int64_t limit = is_x ? rows : (int64_t)n;
    const uint16_t *base = is_x ? x : w;
    rsrc[f] = make_rsrc((const uint8_t *)base + first * row_bytes, (limit - first) * row_bytes);
    lds_at[f] = (int)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)(smem) + j * 1024;
  }
  // k is a multiple of 32: a last stage may hold two k-steps only.  The lanes that would fetch the second
  // half of its rows (the next rows' data) then address past every descriptor's bound and land zeros.
  const int nk = (k + kBk - 1) / kBk;
  const bool short_tail = (k % kBk) != 0;
  const bool second_half = ((place ^ ((4 * (wave & 1) + (frow >> 1)) & 7)) & 4) != 0;
  // Stage `s` of the k loop into its ring slot; past the last stage an empty descriptor (zeros land in a
  // slot nothing reads any more) keeps the count of fills in flight the same in every iteration.
  auto fill = [&](int s) {
    const int slot = (s % kStages) * kStageBytes;
    const int voff = (short_tail && s == nk - 1 && second_half) ? (int)0xfffffff0u : src + s * kRowBytes;
#pragma unroll
    for (int f = 0; f < kFills; f++) {
      i32x4 r = rsrc[f];
      if (s >= nk) r[2] = 0;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                   :
                   : "s"(lds_at[f] + slot), "v"(voff), "s"(r)
                   : "memory");
    }
  };
  fill(0);
  fill(1);

  // ---- operand reads: A = W rows (the output's columns), B = X rows (the output's rows); fragment
  // (block of 32 rows, k-step ks): row ln of the block, logical chunk 2 * ks + g.
  const int wave_m = wave & 3, wave_n = wave >> 2;  // 32 S-row and 128-column shares of the tile
  int a_read[4], b_read[S];
#pragma unroll
  for (int cb = 0; cb < 4; cb++) a_read[cb] = (wave_n * 128 + cb * 32 + ln) * kRowBytes;
#pragma unroll
  for (int rb = 0; rb < S; rb++) b_read[rb] = kTileBytes + (wave_m * 32 * S + rb * 32 + ln) * kRowBytes;
  const int swz = (ln >> 1) & 7;  // every block starts on a multiple of 16 rows
  int chunk_at[kSteps];
#pragma unroll
  for (int ks = 0; ks < kSteps; ks++) chunk_at[ks] = ((2 * ks + g) ^ swz) << 4;

  f32x16 acc[S][4];
  const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int rb = 0; rb < S; rb++)
#pragma unroll
    for (int cb = 0; cb < 4; cb++) acc[rb][cb] = zero;

  // One k-step: the 4 S products of the fragment set `set` (four fragments of W: this wave's column blocks; S of
  // X: its row blocks), and beside them the 4 + S fragment reads of k-step `nks` of stage slot `nslot` into the
  // other set (one beside each of the first six of eight products; with four products, two beside the first), so
  // that a product's operands were asked for a k-step earlier.  The fences keep the order: left to itself the
  // scheduler gathers the reads in front of the products that want them.
  constexpr int kReads = 4 + S, kProducts = 4 * S;
  u32x4 af[2][4], bf[2][S];
  auto read_fragment = [&](int slot, int ks, int i, int set) {
    const uint8_t *st = smem + slot * kStageBytes;
    if (i < S)
      bf[set][i] = *reinterpret_cast<const u32x4 *>(st + b_read[i] + chunk_at[ks]);
    else
      af[set][i - S] = *reinterpret_cast<const u32x4 *>(st + a_read[i - S] + chunk_at[ks]);
  };
  auto step = [&](int set, int nslot, int nks, bool reads) {
#pragma unroll
    for (int i = 0; i < kProducts; i++) {
      acc[i % S][i / S] = mma<F16>(af[set][i / S], bf[set][i % S], acc[i % S][i / S]);
      if (reads) {
        if (i < kReads) read_fragment(nslot, nks, i, set ^ 1);
        if (i == 0 && kReads > kProducts) read_fragment(nslot, nks, kProducts, set ^ 1);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // The rotary tables' rows of this tile (16 bytes a lane along the rows, kTables loads a table and lane)
  // are asked for behind the barrier of the last stage but one: they arrive under the last stage's products
  // and are in registers when the epilogue wants them in LDS.
  constexpr int kHalf = (HD > 0 ? HD : 64) / 2, kTChunks = kHalf * 2 / 16, kTables = kBm * kTChunks / (kWaves * 64);
  const bool turning = HD > 0 && n0 < heads * HD;  // the same for the whole workgroup
  u32x4 tc[kTables], ts[kTables];
  bool tables_in = false;
  auto load_tables = [&]() {
    const uint32_t pos0 = (uint32_t)(m0 % seq);
#pragma unroll
    for (int i = 0; i < kTables; i++) {
      const int c = tid + i * kWaves * 64, r = c / kTChunks, ch = c % kTChunks;
      const uint32_t pos = (pos0 + (uint32_t)r) % (uint32_t)seq;  // gemm.rs:685: the table row of the token's position
      tc[i] = *reinterpret_cast<const u32x4 *>(cos_t + (int64_t)pos * kHalf + ch * 8);
      ts[i] = *reinterpret_cast<const u32x4 *>(sin_t + (int64_t)pos * kHalf + ch * 8);
    }
    tables_in = true;
  };

  // A stage is four k-steps.  Before its last one every wave makes sure its own fills of the next stage
  // have landed and its reads of this stage are back, and meets the others: behind that barrier the next
  // stage is whole and this stage's slot is free, so the fills of the stage after next go out and the next
  // stage's first fragments are asked for under this stage's last products.
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kFills) : "memory");  // stage 0 is in
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kReads; i++) read_fragment(0, 0, i, 0);
  for (int s = 0; s < nk; s++) {
    const int slot = s & 1;
    step(0, slot, 1, true);
    step(1, slot, 2, true);
    step(0, slot, 3, true);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // stage s + 1 is in, stage s is read
    __syncthreads();
    fill(s + 2);
    if (HD > 0 && turning && s == nk - 2) load_tables();
    step(1, slot ^ 1, 0, true);
  }
  if (HD > 0 && turning && !tables_in) load_tables();  // a k loop of one stage
  // The empty fills still in flight write LDS: they land before the workgroup's LDS is given away.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- epilogue.  Accumulator (rb, cb) register i: row m0 + 64 wave_m + 32 rb + ln, column
  // n0 + 128 wave_n + 32 cb + 8 (i / 4) + 4 g + i % 4.
  const int col_base = n0 + wave_n * 128 + 4 * g;
  if (bias != nullptr) {
#pragma unroll
    for (int cb = 0; cb < 4; cb++) {
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int col = col_base + 32 * cb + 8 * q;
        if (col >= n) continue;
        float b4[4];
        load4<F16>(bias + col, b4);
#pragma unroll
        for (int rb = 0; rb < S; rb++)
#pragma unroll
          for (int e = 0; e < 4; e++) acc[rb][cb][4 * q + e] += b4[e];
      }
    }
  }
  const int turned = HD > 0 ? heads * HD : 0;
  if (HD > 0 && turning) {
    // The head size is 64 or 128: a head's halves are whole 32-column blocks of a wave's 128 columns, the
    // partner of block cb is block cb +- nb, and a head never straddles two waves.
    constexpr int head_dim = HD > 0 ? HD : 64;
    constexpr int half = head_dim >> 1, nb = half >> 5;
    // The tile's 256 rows of the tables go through LDS (the ring is done with): loaded 16 bytes a lane
    // along the rows, read back 8 bytes a lane down them.  A lane owns a ROW of the output, so reading
    // the tables straight from memory would touch 32 lines an instruction.  Rows of 2 * half + 8 bytes
    // keep the reads off each other's banks.
    constexpr int kPitch = half * 2 + 8, kChunks = half * 2 / 16;
    uint8_t *cos_lds = smem, *sin_lds = smem + kBm * kPitch;
    __syncthreads();  // every wave's last fragments are read and its last fills have landed
    static_assert(2 * kBm * kPitch <= kLds, "the tables fit where the ring was");
    static_assert(kChunks == kTChunks && half == kHalf, "the prefetch's chunks are the tables'");
#pragma unroll
    for (int i = 0; i < kTables; i++) {
      const int c = tid + i * kWaves * 64, r = c / kChunks, ch = c % kChunks;
      const u32x4 vc = tc[i], vs = ts[i];
      u32x2 *cd = reinterpret_cast<u32x2 *>(cos_lds + r * kPitch + ch * 16);
      u32x2 *sd = reinterpret_cast<u32x2 *>(sin_lds + r * kPitch + ch * 16);
      cd[0] = u32x2{vc[0], vc[1]};
      cd[1] = u32x2{vc[2], vc[3]};
      sd[0] = u32x2{vs[0], vs[1]};
      sd[1] = u32x2{vs[2], vs[3]};
    }
    __syncthreads();
    if (n0 + wave_n * 128 < turned) {
#pragma unroll
      for (int rb = 0; rb < S; rb++) {
        const int r = wave_m * 32 * S + rb * 32 + ln;
        const uint16_t *cos_row = reinterpret_cast<const uint16_t *>(cos_lds + r * kPitch);
        const uint16_t *sin_row = reinterpret_cast<const uint16_t *>(sin_lds + r * kPitch);
#pragma unroll
        for (int cb = 0; cb < 4; cb++) {
          constexpr int kBlocks = 4;
          const int in_head = (cb * 32) & (head_dim - 1);  // the block's first column within its head
          if (in_head >= half) continue;                   // second halves are turned with their first
          if (n0 + wave_n * 128 + cb * 32 >= turned) continue;
          const int pb = (cb + nb) % kBlocks;  // the partner block (a head's halves lie in one wave)
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const int at = in_head + 8 * q + 4 * g;  // index into the table row, < half
            float c4[4], s4[4];
            load4<F16>(cos_row + at, c4);
            load4<F16>(sin_row + at, s4);
#pragma unroll
            for (int e = 0; e < 4; e++) {
              const float y1 = acc[rb][cb][4 * q + e], y2 = acc[rb][pb][4 * q + e];
              // gemm.rs:702-705: x cos, then the partner's product joined by one fused multiply-add.
              const float y1c = y1 * c4[e], y2c = y2 * c4[e];
              acc[rb][cb][4 * q + e] = __builtin_fmaf(y2, -s4[e], y1c);
              acc[rb][pb][4 * q + e] = __builtin_fmaf(y1, s4[e], y2c);
            }
          }
        }
      }
    }
  }
  // ---- the store.  A lane owns rows, not runs of columns: written from the registers an instruction would
  // touch 32 rows with 16 bytes each.  The rounded tile goes through LDS instead (every wave is done with the
  // ring, and with the tables), 32 rows of a wave at a time in a stretch of its own, and leaves as whole row
  // segments: an instruction stores 4 rows of 256 bytes, 16 bytes a lane.
  __syncthreads();
  uint8_t *stage = smem + wave * 32 * kOutPitch;
  const int orow = lane >> 4, ochunk = lane & 15;
  const int col = n0 + wave_n * 128 + ochunk * 8;  // n is a multiple of 8: a run of eight lies inside or outside
#pragma unroll
  for (int rb = 0; rb < S; rb++) {
    uint8_t *srow = stage + ln * kOutPitch + 8 * g;
#pragma unroll
    for (int cb = 0; cb < 4; cb++) {
#pragma unroll
      for (int q = 0; q < 4; q++) {
        u32x2 out;
        out[0] = pack2<F16>(acc[rb][cb][4 * q], acc[rb][cb][4 * q + 1]);
        out[1] = pack2<F16>(acc[rb][cb][4 * q + 2], acc[rb][cb][4 * q + 3]);
        *reinterpret_cast<u32x2 *>(srow + (32 * cb + 8 * q) * 2) = out;
      }
    }
#pragma unroll
    for (int it = 0; it < 8; it++) {
      const int r = it * 4 + orow;
      const u32x4 out = *reinterpret_cast<const u32x4 *>(stage + r * kOutPitch + ochunk * 16);
      const int64_t row = m0 + wave_m * 32 * S + rb * 32 + r;
      // Streaming stores: the output is not read again here, and left out of L2 it does not push the operands out.
      if (row < rows && col < n) __builtin_nontemporal_store(out, reinterpret_cast<u32x4 *>(y + row * y_ld + col));
    }
  }
}
#endif  // __HIP_DEVICE_COMPILE__

#if !defined(SVODK_CODE_OBJECT)  // the library's kernel and its launch: not part of a code object build
template <bool F16, int HD, int S>
__global__ __launch_bounds__(Tile<S>::kWaves * 64, 3 - S) void linear_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ w,
                                                                const uint16_t *__restrict__ bias,
                                                                const uint16_t *__restrict__ cos_t,
                                                                const uint16_t *__restrict__ sin_t, uint16_t *__restrict__ y,
                                                                int64_t y_ld, int64_t rows, int32_t n, int32_t k, int32_t seq,
                                                                int32_t heads,
                                                                uint32_t tiles_n, uint32_t tiles, uint32_t per_xcd,
                                                                uint32_t band) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  linear_body<F16, HD, S>(smem, x, w, bias, cos_t, sin_t, y, y_ld, rows, n, k, seq, heads, tiles_n, tiles, per_xcd, band);
#endif
}

template <bool F16, int HD, int S>
hipError_t launch(const LinearArgs &a, hipStream_t stream) {
  constexpr int kBm = Tile<S>::kBm, kBn = Tile<S>::kBn, kLds = Tile<S>::kLds, kWaves = Tile<S>::kWaves;
  const int64_t tiles_m = (a.rows + kBm - 1) / kBm, tiles_n = (a.n + kBn - 1) / kBn;
  const int64_t tiles = tiles_m * tiles_n;
  if (tiles == 0) return hipSuccess;
  // Bands of row tiles per XCD where every XCD gets at least two row tiles; else runs of tiles.
  const int64_t band = tiles_m >= 2 * kXcds ? (tiles_m + kXcds - 1) / kXcds : 0;
  const int64_t per_xcd = band > 0 ? band * tiles_n : (tiles + kXcds - 1) / kXcds;
  if (per_xcd * kXcds > 0x7fffffffLL) return hipErrorInvalidConfiguration;
  auto kernel = linear_kernel<F16, HD, S>;
  static std::atomic<uint64_t> configured{0};  // a bit per device ordinal, devices past 63 always ask
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  const uint64_t bit = device < 64 ? 1ull << device : 0;
  if ((configured.load(std::memory_order_acquire) & bit) == 0) {
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) return e;
    configured.fetch_or(bit, std::memory_order_release);
  }
  hipLaunchKernelGGL(kernel, dim3((uint32_t)(per_xcd * kXcds)), dim3(kWaves * 64), kLds, stream, (const uint16_t *)a.x,
                     (const uint16_t *)a.w, (const uint16_t *)a.bias, (const uint16_t *)a.cos, (const uint16_t *)a.sin,
                     (uint16_t *)a.y, a.y_ld > 0 ? a.y_ld : (int64_t)a.n, a.rows, a.n, a.k, a.seq, a.heads, (uint32_t)tiles_n,
                     (uint32_t)tiles,
                     (uint32_t)per_xcd, (uint32_t)band);
  return hipGetLastError();
}

}  // namespace
#else  // SVODK_CODE_OBJECT
// The same program as kernels for a loader that takes a code object and a flat argument record
// (device/src/amd/program.rs:403-414, 655-675; device/src/hcq.rs:1262-1285): buffers first, then 4-byte
// scalars, nothing hidden, static LDS, no launch geometry from the dispatch packet.
// Parameters follow the reference GEMM's order (tk/src/kernels/gemm.rs:604-645: the operands, the bias, the
// rotary tables, the output): x, w, bias (address 0: none), cos, sin (unread by the kernels that do not turn),
// y, then rows (batch * seq), n, k, seq, heads (the first heads * head size columns are turned).
// Launch: ceil(rows / 256) * ceil(n / 256) workgroups, rounded up to a multiple of 8, of 512 threads
// (`workgroups` in the manifest); rows < 2^31, n a multiple of 8, k a multiple of 32 are the caller's checks.
template <bool F16, int HD>
__device__ __forceinline__ void linear_entry(uint8_t *smem, const uint16_t *x, const uint16_t *w, const uint16_t *bias,
                                             const uint16_t *cos_t, const uint16_t *sin_t, uint16_t *y, int32_t rows,
                                             int32_t n, int32_t k, int32_t seq, int32_t heads) {
  if (rows <= 0 || n <= 0 || k <= 0) return;
  constexpr int kBm = Tile<2>::kBm, kBn = Tile<2>::kBn;  // the code objects hold the 256 x 256 form
  const uint32_t tiles_m = ((uint32_t)rows + kBm - 1) / kBm, tiles_n = ((uint32_t)n + kBn - 1) / kBn;
  const uint32_t tiles = tiles_m * tiles_n;
  // The library's launch geometry (see launch below in the library build): bands of row tiles per XCD
  // where every XCD gets at least two, else runs of tiles.
  const uint32_t band = tiles_m >= 2 * kXcds ? (tiles_m + kXcds - 1) / kXcds : 0;
  const uint32_t per_xcd = band > 0 ? band * tiles_n : (tiles + kXcds - 1) / kXcds;
  linear_body<F16, HD>(smem, x, w, bias, cos_t, sin_t, y, (int64_t)n, (int64_t)rows, n, k, seq > 0 ? seq : 1, heads, tiles_n,
                       tiles, per_xcd, band);
}

#define SVODK_LINEAR_ENTRY(NAME, F16, HD)                                                                             \
  extern "C" __global__ __launch_bounds__(Tile<2>::kWaves * 64, 1) void NAME(                                                  \
      const uint16_t *__restrict__ x, const uint16_t *__restrict__ w, const uint16_t *__restrict__ bias,              \
      const uint16_t *__restrict__ cos_t, const uint16_t *__restrict__ sin_t, uint16_t *__restrict__ y, int32_t rows, \
      int32_t n, int32_t k, int32_t seq, int32_t heads) {                                                             \
    __shared__ __attribute__((aligned(1024))) uint8_t smem[Tile<2>::kLds];                                                   \
    linear_entry<F16, HD>(smem, x, w, bias, cos_t, sin_t, y, rows, n, k, seq, heads);                                 \
  }
SVODK_LINEAR_ENTRY(svodk_linear_bf16, false, 0)
SVODK_LINEAR_ENTRY(svodk_linear_rope64_bf16, false, 64)
SVODK_LINEAR_ENTRY(svodk_linear_rope128_bf16, false, 128)
SVODK_LINEAR_ENTRY(svodk_linear_f16, true, 0)
SVODK_LINEAR_ENTRY(svodk_linear_rope64_f16, true, 64)
SVODK_LINEAR_ENTRY(svodk_linear_rope128_f16, true, 128)
#undef SVODK_LINEAR_ENTRY
}  // namespace
}  // namespace svodk
#endif  // SVODK_CODE_OBJECT

#if !defined(SVODK_CODE_OBJECT)
// A fill's lanes address their rows with 32-bit byte offsets from the descriptor's base: 8 rows of 2 k bytes,
// and the stage's place along them.
bool linear_supports(int64_t n, int64_t k) { return n > 0 && n % 8 == 0 && k >= 32 && k % 32 == 0 && k <= (1 << 25); }

bool linear_turns(int32_t head_dim) { return head_dim == 64 || head_dim == 128; }

// The tile a call's shape takes: 256 x 256 unless that makes fewer workgroups than half the compute units (256 on
// this part; read from the device on a launch), where 128 x 128 makes four times as many.
namespace {
std::atomic<int> g_linear_tile{0};  // 0: by the shape; 128 or 256: every call
}
int linear_tile(int32_t tile) {
  if (tile == 0 || tile == 128 || tile == 256) g_linear_tile.store(tile, std::memory_order_relaxed);
  return g_linear_tile.load(std::memory_order_relaxed);
}
int linear_tile_of(int64_t rows, int64_t n, int units) {
  const int named = g_linear_tile.load(std::memory_order_relaxed);
  if (named != 0) return named;
  const int64_t wide = ((rows + 255) / 256) * ((n + 255) / 256);
  return 2 * wide <= units ? 128 : 256;
}

hipError_t launch_linear(const LinearArgs &a, hipStream_t stream) {
  if (!linear_supports(a.n, a.k)) return hipErrorInvalidValue;
  if (a.cos != nullptr && (!linear_turns(a.head_dim) || a.seq <= 0 || (int64_t)a.heads * a.head_dim > a.n))
    return hipErrorInvalidValue;
  const int hd = a.cos != nullptr ? a.head_dim : 0;
  if (a.tile == 128) {
    if (a.f16) return hd == 0 ? launch<true, 0, 1>(a, stream) : hd == 64 ? launch<true, 64, 1>(a, stream) : launch<true, 128, 1>(a, stream);
    return hd == 0 ? launch<false, 0, 1>(a, stream) : hd == 64 ? launch<false, 64, 1>(a, stream) : launch<false, 128, 1>(a, stream);
  }
  if (a.f16) return hd == 0 ? launch<true, 0, 2>(a, stream) : hd == 64 ? launch<true, 64, 2>(a, stream) : launch<true, 128, 2>(a, stream);
  return hd == 0 ? launch<false, 0, 2>(a, stream) : hd == 64 ? launch<false, 64, 2>(a, stream) : launch<false, 128, 2>(a, stream);
}

}  // namespace svodk
#endif  // !SVODK_CODE_OBJECT

// Grouped (ragged-M) / dense matmul for gfx950: 16-bit or fp8 activations x MXFP4 weights.
//
//   y[dst(r), :] = act(((x[src(r), :] . deq(w[e])) * sx * sw + bias[e, :] * beta[r]) * alpha) * gamma[r]
//
// (matmul_details/_matmul.py:43-669 of the reference; epilogue order :540-559.)
//
// Work decomposition
//   workgroup (4 waves) = one BLOCK_M x 256 output tile of one expert, taken from the ragged
//     block schedule ((block << 16) | expert, -1 = padding);
//   wave w owns the 64 columns [64w, 64w+64) of the tile and ALL its rows;
//   both operands travel HBM -> LDS by 16-byte DMA (buffer_load ... lds): activation rows (gathered)
//     in 128-byte stages, double buffered, chunks XOR-swizzled by row; the weights of a wave's own
//     columns into a wave-private region, 128 K per stage.
//   bf16 / f16 activations: the fp4 codes are expanded in registers with v_cvt_scalef32_pk_*_fp4
//     (scale applied by the instruction) and feed v_mfma_f32_32x32x16, which sustains twice the rate
//     of 16x16x32 on this part (measured 2.45 vs 1.25 PFLOP/s for bf16).
//   fp8 activations: v_mfma_scale_f32_32x32x64_f8f6f4 consumes the fp8 bytes, the fp4 codes and the
//     e8m0 scale bytes directly (no conversion instructions at all).
//
// K order inside a 128-K weight stage: lane half h = lane/32 holds K [64q + 32h, 64q + 32h + 32) of
// its column for q = 0, 1 (two 128-bit LDS reads).  16-bit path: MFMA step s = 4q + u consumes
// elements [8u, 8u+8) of load q in both halves, for A and B alike.  fp8 path: MFMA q consumes load q
// whole; its A operand is, for lane half h, the 16 activations K 64q + 16h.. followed by the 16 at
// K 64q + 32 + 16h.. (the operand layout of the instruction, established by one-hot probing).
#pragma once
#include <type_traits>

#include "common.h"

namespace tamd {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x8_t __attribute__((ext_vector_type(8)));

constexpr bool is_fp8(int dt) { return dt == TAMD_FP8_E4M3 || dt == TAMD_FP8_E5M2; }

constexpr int KB = 128;  // K per weight (super-)stage
constexpr int NF = 2;              // 32-column fragments per wave
constexpr int BLOCK_N = 4 * 32 * NF;

template <int XDT>
struct Mma {  // fp8 activations: operands are raw dwords, no expansion
  typedef i32x8_t frag_t;
};
template <>
struct Mma<TAMD_BF16> {
  typedef bf16x8_t frag_t;
  static TAMD_DEVICE frag_t expand(uint32_t codes, float scale) {
    bf16x2_t p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 0);
    bf16x2_t p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 1);
    bf16x2_t p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 2);
    bf16x2_t p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 3);
    return frag_t{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
  }
  static TAMD_DEVICE f32x16_t mma(frag_t a, frag_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mma<TAMD_F16> {
  typedef f16x8_t frag_t;
  static TAMD_DEVICE frag_t expand(uint32_t codes, float scale) {
    f16x2_t p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, scale, 0);
    f16x2_t p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, scale, 1);
    f16x2_t p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, scale, 2);
    f16x2_t p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, scale, 3);
    return frag_t{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
  }
  static TAMD_DEVICE f32x16_t mma(frag_t a, frag_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

TAMD_DEVICE float load_any_f32(const void *p, int dt, int64_t i) {
  if (dt == TAMD_F32) return ((const float *)p)[i];
  if (dt == TAMD_BF16) return bf16_bits_to_f32(((const uint16_t *)p)[i]);
  return f16_bits_to_f32(((const uint16_t *)p)[i]);
}

TAMD_DEVICE void store_any(void *p, int dt, int64_t i, float v) {
  if (dt == TAMD_F32) ((float *)p)[i] = v;
  else if (dt == TAMD_BF16) ((uint16_t *)p)[i] = (uint16_t)f32_to_bf16_bits(v);
  else ((uint16_t *)p)[i] = (uint16_t)f32_to_f16_bits(v);
}

// Gate for the fused epilogue (swiglu_details/_swiglu.py:55-65): exp and reciprocal on the
// hardware transcendental unit (relative error ~1e-6, far inside the 16-bit output rounding).
TAMD_DEVICE float swiglu_fast(float g, float l, float alpha, float limit, bool has_limit) {
  if (has_limit) {
    g = __builtin_fminf(g, limit);
    l = __builtin_fminf(__builtin_fmaxf(l, -limit), limit);
  }
  float e = __builtin_amdgcn_exp2f(-alpha * 1.4426950408889634f * g);
  float s = g * __builtin_amdgcn_rcpf(1.0f + e);
  return __builtin_fmaf(s, l, s);
}

// Tile coordinates of a workgroup.
struct Tile {
  int expert;   // weight slice
  int z;        // batch index (dense batched) else 0
  int start_m;  // first expert-sorted row of the slice
  int off_m;    // first row of the tile inside the slice
  int rows;     // valid rows in the tile (1..BLOCK_M)
  int n0;       // first column of the tile
};

template <int BLOCK_M, int EXTRA>
TAMD_DEVICE bool locate_tile(const tamd_matmul_args &a, int grid_n, int64_t grid_total, int group_m, Tile &t) {
  // XCD-aware remap: hardware deals workgroups round-robin to the 8 XCDs; give each XCD a
  // contiguous range of tiles so neighbours (same expert, adjacent columns) share one L2.
  // A ragged launch is sized for the worst split of the rows over the experts (grid_total), about twice what a
  // balanced routing needs; the schedule's real entries come first and their number is block_offs[n_experts].  The
  // XCD ranges are cut from that number, read here, so that all eight XCDs share the real tiles; the rest exit.
  // (the launchers keep a grid below 2^31 tiles: 32-bit unsigned arithmetic, whose divisions cost a third of the 64-bit ones)
  uint32_t total = (uint32_t)grid_total;
  const uint32_t gn = (uint32_t)grid_n;
  if (a.block_schedule && a.block_offs) {
    const uint64_t real_total = (uint64_t)(uint32_t)a.block_offs[a.n_experts] * gn;
    total = real_total < total ? (uint32_t)real_total : total;
  }
  const uint32_t per_xcd = (total + 7) / 8;
  const uint32_t bx = blockIdx.x;
  if (bx / 8 >= per_xcd) return false;
  const uint32_t pid = (bx % 8) * per_xcd + bx / 8;
  if (pid >= total) return false;
  // Tiles are walked in groups of `group_m` row blocks: row block fastest inside a group, then the
  // column tile.  With many row blocks per expert the workgroups running together then share one
  // column tile of weights while the group's activation rows stay in L2; group_m = 1 is the plain
  // row-block-major order (right when an expert has only a block or two).
  int pid_m, pid_n;
  if (group_m > 1) {
    const uint32_t gm = (uint32_t)group_m;
    const uint32_t grid_m = total / gn;
    const uint32_t in_group = gm * gn;
    const uint32_t gi = pid / in_group;
    const uint32_t first_m = gi * gm;
    const uint32_t size_m = grid_m - first_m < gm ? grid_m - first_m : gm;
    const uint32_t r = pid - gi * in_group;
    const uint32_t q = r / size_m;
    pid_m = (int)(first_m + (r - q * size_m));
    pid_n = (int)q;
  } else {
    const uint32_t q = pid / gn;
    pid_m = (int)q;
    pid_n = (int)(pid - q * gn);
  }
  t.n0 = pid_n * BLOCK_N;
  t.z = 0;
  int slice_rows;
  if (a.block_schedule) {
    int sched = a.block_schedule[pid_m];
    if (sched == -1) return false;
    t.expert = sched & 0xFFFF;
    int blk = sched >> 16;
    slice_rows = a.slice_sizes[t.expert];
    t.start_m = a.slice_offs[t.expert];
    t.off_m = blk * BLOCK_M;
  } else {
    int bm = (a.M + BLOCK_M - 1) / BLOCK_M;
    int z = pid_m / bm;
    t.expert = z;
    t.z = z;
    slice_rows = a.M;
    t.start_m = 0;
    t.off_m = (pid_m - z * bm) * BLOCK_M;
  }
  // A 128-row block also takes a remainder of up to 32 rows that follows it (one more 32-row
  // fragment), and that remainder's own block does nothing: with about 128 rows per expert this
  // avoids a second, nearly empty pass over the expert's weights.
  const int left = slice_rows - t.off_m;
  if (EXTRA > 0 && t.off_m > 0 && left <= EXTRA) return false;
  t.rows = left > BLOCK_M + EXTRA ? BLOCK_M : left;
  return t.rows > 0;
}

// Tile of a workgroup for ragged problems with few row blocks per expert (at most 1024 row blocks in all), where
// tiles differ in their number of 32-row fragments and a launch is only a handful of rounds of tiles per CU: the row
// blocks are taken in the order (fragments descending, schedule index ascending) and dealt round-robin to the 8
// XCDs, all column tiles of a row block to the same XCD.  Every XCD then gets the same mix of tile sizes (plain
// schedule order gives XCDs sums of fragments that differ by several per cent), and the smallest tiles run last,
// which is what bounds the idle time at the end of the launch.  The order is found by the workgroup itself: every
// thread takes up to four row blocks, their fragment counts are exchanged as ballot masks through LDS, and the thread
// whose block has this workgroup's position publishes it.  The loads (schedule entry, then slice size and offset) are
// issued for all blocks at once: two round trips to memory, one fewer than the plain path's chain of dependent loads.
// When some expert has more than one tile the order is left alone (schedule order, one contiguous range per XCD): the
// tiles of an expert then run next to each other on one XCD and the later ones find the expert's weights in its L2,
// which is worth more than the balance (measured: 64 rows per expert +/- 8, sorted order 14 % slower).
// `lds`: at least 1 KB, free again when the function returns.
template <int BLOCK_M, int EXTRA>
TAMD_DEVICE bool locate_tile_sorted(const tamd_matmul_args &a, int grid_n, int grid_m, Tile &t, uint8_t *lds) {
  constexpr int NB = 4;                              // row blocks per thread
  constexpr int NK = BLOCK_M <= 32 ? 1 : (BLOCK_M + EXTRA) / 32;  // largest fragment count of a tile
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  // (grids stay below 2^31 tiles: 32-bit unsigned arithmetic throughout, whose divisions are the cheap ones)
  const uint32_t gn = (uint32_t)grid_n;
  const int x = blockIdx.x % 8, j = blockIdx.x / 8;
  const int slot = (int)((uint32_t)j / gn), pid_n = j - slot * grid_n;
  const int p = slot * 8 + x;                        // position of this workgroup's row block in the sorted order
  // The schedule entries are requested before anything waits for the number of real ones (entries past it hold -1, and
  // the schedule is grid_m entries wide): one round trip to memory instead of two.
  const int nb = (grid_m + 255) / 256;               // <= NB (checked by the launcher)
  int sched[NB], ssize[NB], soffs[NB], key[NB];
#pragma unroll
  for (int u = 0; u < NB; ++u) {
    const int b = u * 256 + tid;
    sched[u] = (u < nb && b < grid_m) ? a.block_schedule[b] : -1;
  }
  const int n_real = a.block_offs[a.n_experts];
#pragma unroll
  for (int u = 0; u < NB; ++u) sched[u] = u * 256 + tid < n_real ? sched[u] : -1;
  // the same workgroup in schedule order: XCD x owns the tiles [x * per_xcd, (x + 1) * per_xcd)
  const uint32_t real_total = (uint32_t)n_real * gn, per_xcd = (real_total + 7) / 8;
  const uint32_t plain_pid = (uint32_t)x * per_xcd + (uint32_t)j;
  const bool plain_live = (uint32_t)j < per_xcd && plain_pid < real_total;
  if (p >= n_real && !plain_live) return false;
  const int plain_m = plain_live ? (int)(plain_pid / gn) : -1;
#pragma unroll
  for (int u = 0; u < NB; ++u) {
    const int e = sched[u] == -1 ? 0 : (sched[u] & 0xFFFF);
    ssize[u] = u < nb ? a.slice_sizes[e] : 0;
    soffs[u] = u < nb ? a.slice_offs[e] : 0;
  }
  uint64_t *masks = (uint64_t *)lds;                 // [NK][NB][4 waves]
  int *res = (int *)(lds + NK * NB * 4 * 8);         // [0..3] sorted order, [4..7] schedule order, [8..11] second tiles seen
  bool second = false;                               // one of this thread's blocks is an expert's second (or later) tile
#pragma unroll
  for (int u = 0; u < NB; ++u) {
    const int off = (sched[u] >> 16) * BLOCK_M;
    const int left = ssize[u] - off;
    int rows = left > BLOCK_M + EXTRA ? BLOCK_M : left;
    if (sched[u] == -1 || rows < 0 || (EXTRA > 0 && off > 0 && left <= EXTRA)) rows = 0;  // padding / absorbed remainder
    key[u] = (rows + 31) / 32;
    if (BLOCK_M <= 32) key[u] = rows > 0 ? 1 : 0;
    second = second || (key[u] > 0 && off > 0);
    if (u < nb) {
#pragma unroll
      for (int k = 1; k <= NK; ++k) {
        const uint64_t m = __ballot(key[u] == k);
        if (lane == 0) masks[((k - 1) * NB + u) * 4 + wave] = m;
      }
    }
  }
  {
    const uint64_t any_second = __ballot(second);
    if (lane == 0) res[8 + wave] = any_second != 0;
  }
  __syncthreads();
  const bool sorted = (res[8] | res[9] | res[10] | res[11]) == 0;
  // position of each of this thread's blocks: blocks of larger keys first, then those of the same key before it
  int cnt[NK];
#pragma unroll
  for (int k = 1; k <= NK; ++k) {
    cnt[k - 1] = 0;
    for (int i = 0; i < nb * 4; ++i) cnt[k - 1] += __popcll(masks[(k - 1) * NB * 4 + i]);
  }
#pragma unroll
  for (int u = 0; u < NB; ++u) {
    if (u < nb && key[u] > 0) {
      int pos = 0;
#pragma unroll
      for (int k = 1; k <= NK; ++k) pos += k > key[u] ? cnt[k - 1] : 0;
      const uint64_t *mk = masks + (key[u] - 1) * NB * 4;
      for (int i = 0; i < u * 4 + wave; ++i) pos += __popcll(mk[i]);
      pos += __popcll(mk[u * 4 + wave] & ((1ull << lane) - 1ull));
      if (pos == p) {
        res[0] = sched[u];
        res[1] = ssize[u];
        res[2] = soffs[u];
        res[3] = 1;
      }
    }
    if (u * 256 + tid == plain_m) {
      res[4] = sched[u];
      res[5] = ssize[u];
      res[6] = soffs[u];
    }
  }
  if (tid == 0) {
    int total = 0;
#pragma unroll
    for (int k = 1; k <= NK; ++k) total += cnt[k - 1];
    if (p >= total) res[3] = 0;                      // nobody writes: fewer real tiles than schedule entries
  }
  __syncthreads();
  const int found = sorted ? res[3] : (int)plain_live;
  const int sc = res[sorted ? 0 : 4], slice_rows = res[sorted ? 1 : 5], start_m = res[sorted ? 2 : 6];
  __syncthreads();                                   // the scratch may be overwritten from here on
  if (!found || sc == -1) return false;
  t.n0 = (sorted ? pid_n : (int)(plain_pid - (uint32_t)plain_m * gn)) * BLOCK_N;
  t.z = 0;
  t.expert = sc & 0xFFFF;
  t.start_m = start_m;
  t.off_m = (sc >> 16) * BLOCK_M;
  const int left = slice_rows - t.off_m;
  if (EXTRA > 0 && t.off_m > 0 && left <= EXTRA) return false;  // absorbed by the block before it
  t.rows = left > BLOCK_M + EXTRA ? BLOCK_M : left;
  return t.rows > 0;
}

// 128-bit global -> LDS copy that bypasses registers (buffer_load ... lds).  The LDS destination of
// lane L is lds_addr + 16*L; out-of-range offsets (>= num_records of the descriptor) deliver zeros.
// Issued through inline asm so that the compiler does not serialise later LDS reads behind it; the
// kernel waits for these copies itself (wait_dma) before the barrier that publishes a stage.  The
// five wait states cover an SGPR operand written by a v_readfirstlane just before the block (the
// compiler's hazard recognizer does not look inside inline asm) and the write of M0.
typedef int v4i_t __attribute__((ext_vector_type(4)));
TAMD_DEVICE void dma16(v4i_t rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(rsrc),
                 "s"(__builtin_amdgcn_readfirstlane(soff))
               : "memory", "m0");
}
// 1-, 2- and 4-byte global -> LDS copies: lane L's value lands (zero-extended) in the dword at
// lds_addr + 4*L; out-of-range offsets deliver zero.  The five wait states before the load cover an
// SGPR operand that a v_readfirstlane wrote just before the asm block (the compiler's hazard
// recognizer does not look inside inline asm) as well as the write of M0.
TAMD_DEVICE void dma2(v4i_t rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_ushort %1, %2, %3 offen lds"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(rsrc),
                 "s"(__builtin_amdgcn_readfirstlane(soff))
               : "memory", "m0");
}
TAMD_DEVICE void dma1(v4i_t rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_ubyte %1, %2, %3 offen lds"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(rsrc),
                 "s"(__builtin_amdgcn_readfirstlane(soff))
               : "memory", "m0");
}
TAMD_DEVICE void dma4(v4i_t rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 4\n\tbuffer_load_dword %1, %2, %3 offen lds"
               :
               : "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(rsrc),
                 "s"(__builtin_amdgcn_readfirstlane(soff))
               : "memory", "m0");
}
// Four consecutive 1 KB pieces of a linear image with ONE M0 value: the instruction's immediate offset is added to the
// global offset and to the LDS address alike.
TAMD_DEVICE void dma16_x4(v4i_t rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
  asm volatile(
      "s_mov_b32 m0, %0\n\ts_nop 4\n\t"
      "buffer_load_dwordx4 %1, %2, %3 offen lds\n\t"
      "buffer_load_dwordx4 %1, %2, %3 offen offset:1024 lds\n\t"
      "buffer_load_dwordx4 %1, %2, %3 offen offset:2048 lds\n\t"
      "buffer_load_dwordx4 %1, %2, %3 offen offset:3072 lds"
      :
      : "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(rsrc), "s"(__builtin_amdgcn_readfirstlane(soff))
      : "memory", "m0");
}
TAMD_DEVICE void wait_dma() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding).
template <int N>
TAMD_DEVICE void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
  asm volatile("" ::: "memory");
}

TAMD_DEVICE v4i_t make_rsrc(const void *base, uint32_t num_records) {
  uint64_t p = (uint64_t)base;
  return v4i_t{__builtin_amdgcn_readfirstlane((int)(uint32_t)p),
               __builtin_amdgcn_readfirstlane((int)((uint32_t)(p >> 32) & 0xFFFFu)), (int)num_records, 0x00020000};
}

constexpr int A_ROW_BYTES = 128;       // LDS bytes per activation row per stage (64 K of 16-bit, 128 K of fp8)
constexpr int B_BYTES = 4 * 64 * 64;   // 4 waves x 64 columns x 64 bytes (128 K of fp4)
// LDS of the K pipeline.  The usual layout: two activation stages, one weight stage (4 KB per wave), the e8m0 scales
// of the whole tile staged once.  "Ring mode" (fp8 path without the whole-tile scale staging, i.e. pre-shuffled
// scales, or strided scales that do not fit): the scales of a stage travel with its weights (1 KB per wave and
// stage), which leaves room for two weight stages and -- for row blocks of at most 64 rows -- three activation
// stages, so that two stages' copies are in flight instead of one.  The fp8 path needs that: it spends half the
// matrix-core time per weight byte, and with few rows per expert the stream from HBM is all there is to wait for.
struct PipeShape {
  int da, db;        // activation / weight (+ scale) stages
  int as_bytes;      // block scales of MXFP8 activations: da stages x 4 planes x rows x 4 bytes
  int scr_bytes;     // ring-mode scale ring: db stages x 4 waves x 1 KB
  int bytes;
};
// "Deep mode" (16-bit path with the scales staged in LDS, row blocks of at most 64 rows): counted waits with three or
// four activation stages and two weight stages.  With so few rows a stage's MFMAs take less time than a copy needs
// to arrive, and the K loop of the two-stage pipeline runs at the latency of the copies.
// K groups (KS = 2 or 4, row blocks of at most 32 rows): KS groups of four waves share a tile, each taking a
// contiguous part of K through a pipeline of its own; their partial sums meet in LDS.  A problem with fewer tiles than
// the part has CUs is bound by what one wave per SIMD can issue (a copy instruction holds its wave for about a
// hundred cycles); more waves per SIMD fill those gaps.
constexpr bool deep_mode(bool fp8, int lds_rows) { return !fp8 && lds_rows <= 64; }
constexpr PipeShape pipe_shape(bool fp8, bool ring, int lds_rows, bool deep = false, int ks = 1) {
  PipeShape p{};
  p.da = deep ? (ks == 4 ? 3 : (lds_rows <= 32 ? 4 : 3)) : (ring && lds_rows <= 64 ? 3 : 2);
  p.db = (ring || deep) && ks != 4 ? 2 : 1;
  p.as_bytes = fp8 ? p.da * 4 * (lds_rows < 64 ? 64 : lds_rows) * 4 : 0;
  p.scr_bytes = ring ? p.db * 4 * 1024 : 0;
  p.bytes = p.da * lds_rows * 128 + p.db * B_BYTES + p.as_bytes + p.scr_bytes;
  return p;
}

// Copies that a stage of the counted-wait loop (deep mode) may leave in flight.  The requests are made in this order:
// stage j -- the stages before 0 are the loop's prologue -- asks for the activations of stage j + DA - 1 (NA copies)
// and, if j is even, after them for the weights of pair j/2 + DB (NB copies).  A stage needs its own activations and,
// if it is even, its pair's weights; copies complete in the order of their requests, so everything requested after
// the last of those may still be outstanding when the stage begins.
constexpr int ring_outstanding(int DA, int DB, int NA, int NB, bool odd) {
  const int s = 64 + (odd ? 1 : 0);   // any stage in the steady state
  int pos = 0, need_end = 0;
  for (int j = 0; j < s; ++j) {
    pos += NA;
    if (j + DA - 1 == s) need_end = pos;
    if (j % 2 == 0) {
      pos += NB;
      if (!odd && j / 2 + DB == s / 2 && pos > need_end) need_end = pos;
    }
  }
  return pos - need_end;
}
static_assert(ring_outstanding(4, 2, 1, 4, false) == 6 && ring_outstanding(4, 2, 1, 4, true) == 10, "ring bookkeeping");
static_assert(ring_outstanding(3, 2, 2, 4, false) == 6 && ring_outstanding(3, 2, 2, 4, true) == 6, "ring bookkeeping");
static_assert(ring_outstanding(3, 1, 1, 4, false) == 1 && ring_outstanding(3, 1, 1, 4, true) == 5, "ring bookkeeping");

// Epilogue of one output tile (shared by every tiled kernel).  The accumulators hold, for fragment
// (i, f), element j: row 32i + 8(j/4) + 4h + j%4, column t.n0 + wave*64 + c32*NF + f.
//
// YDT: output type fixed at compile time, or -1 to read a.y_dtype; ROWSC: per-row betas / gammas may be
// present; FLEX: flexpoint output (expected / actual scale) may be present; MXO: MXFP8 output (a.y_mx_scale).
// Everything that is false or fixed here is a branch less per output element, and a tile has up to
// 160 x 256 of them.  The element loops must unroll completely (the accumulators are indexed by them and
// would otherwise live in scratch memory), and the compiler gives up on that above a body size that one
// variant holding every feature exceeds: hence MXO and FLEX exclude each other.
// Args: tamd_matmul_args, or the same structure read in place from the kernel-argument segment (see kernel_args_late).
template <int NFR, int ACT, int YDT, bool ROWSC, bool FLEX, bool MXO = false, typename Args = tamd_matmul_args>
TAMD_DEVICE void tile_epilogue_t(const Args &a, const Tile &t, f32x16_t (&acc)[NFR][NF], uint8_t *lds) {
  const int tid = threadIdx.x;
  const int wave = tid / kWave, lane = tid % kWave;
  const int c32 = lane % 32, h = lane / 32;
  const int N = a.N;
  const int col0 = t.n0 + wave * 64 + c32 * NF;
  const int ydt = YDT < 0 ? a.y_dtype : YDT;
  // 16-bit and 8-bit outputs are staged through LDS (the K stages are dead by now) so that the global
  // stores are 16 bytes per lane and whole rows of the tile are contiguous.
  float flex = 1.0f;
  if (a.x_scale) flex *= *a.x_scale;
  if (a.w_scale) flex *= *a.w_scale;
  flex *= a.out_alpha;
  float bias[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f)
    bias[f] = (a.bias && col0 + f < N) ? load_any_f32(a.bias, a.bias_dtype, (int64_t)t.expert * a.bias_stride_e + col0 + f)
                                       : 0.f;
  constexpr int NO = ACT == TAMD_ACT_SWIGLU ? NF / 2 : NF;  // outputs per lane per row
  constexpr int OUT_COLS = 128 * NO;                        // output columns of the tile
  const int n_out = ACT == TAMD_ACT_SWIGLU ? N / 2 : N;
  const int out_col0 = ACT == TAMD_ACT_SWIGLU ? col0 / 2 : col0;
  const int tile_out0 = ACT == TAMD_ACT_SWIGLU ? t.n0 / 2 : t.n0;
  const bool has_limit = a.act_has_limit != 0;
  const int osz = ydt == TAMD_F32 ? 4 : (is_fp8(ydt) ? 1 : 2);  // bytes per output
  const bool staged = osz < 4;
  // flexpoint output: scale by 1 / expected, optionally clamp, and track max|result| for the actual scale
  const float inv_expected = (FLEX && a.y_expected_scale) ? 1.0f / *a.y_expected_scale : 1.0f;
  const bool clamp_out = FLEX && a.y_expected_scale != nullptr && a.y_saturate_inf != 0;
  const float out_max = max_finite_of(ydt);
  const bool track_max = FLEX && a.y_actual_scale != nullptr;
  uint32_t amax = 0;
  auto narrow = [&](float v) -> uint32_t {  // one output value as 8 / 16 bits
    return ydt == TAMD_BF16 ? f32_to_bf16_bits(v) : (ydt == TAMD_F16 ? f32_to_f16_bits(v) : f32_to_fp8_bits(v, ydt));
  };
  auto narrow2 = [&](float lo, float hi) -> uint32_t {  // two 16-bit outputs in one word (one packed conversion)
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    if (ydt == TAMD_BF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, f16x2_t));
  };
  // without per-row factors bias * beta * out_alpha is one value per column
  float bias_a[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) bias_a[f] = bias[f] * a.out_alpha;
  uint8_t *ob = lds;  // [rows][OUT_COLS] outputs of osz bytes
  // per-row factors: lane L fetches those of row L % 32 of every fragment up front (one round trip to memory);
  // an element then takes its row's pair from that lane
  float beta_of[NFR], gamma_of[NFR];
  const bool has_beta = ROWSC && a.betas != nullptr, has_gamma = ROWSC && a.gammas != nullptr;
  if constexpr (ROWSC) {
#pragma unroll
    for (int i = 0; i < NFR; ++i) {
      const int r = i * 32 + c32;
      const int erow = t.start_m + t.off_m + (r < t.rows ? r : t.rows - 1);  // expert-sorted row
      beta_of[i] = has_beta ? a.betas[erow] : 1.0f;
      gamma_of[i] = has_gamma ? a.gammas[erow] : 1.0f;
    }
  }
  // destination rows of the 16-byte chunks this thread copies out at the end (chunk id = tid + 256 u): fetched
  // now, so that the scatter indices arrive while the values are computed
  constexpr bool PRE = YDT >= 0 && YDT != TAMD_F32;
  constexpr int OSZ_C = YDT == TAMD_FP8_E4M3 || YDT == TAMD_FP8_E5M2 ? 1 : 2;
  constexpr int CPR_C = OUT_COLS * OSZ_C / 16;          // chunks per tile row
  constexpr int MAXU = PRE ? NFR * 32 * CPR_C / 256 : 1;  // chunks per thread
  int dst_row[MAXU];
  if constexpr (PRE) {
#pragma unroll
    for (int u = 0; u < MAXU; ++u) {
      const int r = (tid + u * 256) / CPR_C;
      const int erow = t.start_m + t.off_m + (r < t.rows ? r : t.rows - 1);
      dst_row[u] = a.scatter_indx ? a.scatter_indx[erow] : erow;
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < NFR; ++i) {
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int r = i * 32 + (j >> 2) * 8 + h * 4 + (j & 3);
      float v[NF];
      float gamma = 1.0f;
      if constexpr (ROWSC) {
        // the factors of row 32 i + l sit in lane l: lanes of half h need l = 8 (j / 4) + 4 h + j % 4
        const int l0 = (j >> 2) * 8 + (j & 3);
        // (an absent factor was loaded as 1.0: no branch inside the element loop)
        const float b0 = bits_to_f32(__builtin_amdgcn_readlane((int)f32_to_bits(beta_of[i]), l0));
        const float b1 = bits_to_f32(__builtin_amdgcn_readlane((int)f32_to_bits(beta_of[i]), l0 + 4));
        const float beta = h ? b1 : b0;
        const float g0 = bits_to_f32(__builtin_amdgcn_readlane((int)f32_to_bits(gamma_of[i]), l0));
        const float g1 = bits_to_f32(__builtin_amdgcn_readlane((int)f32_to_bits(gamma_of[i]), l0 + 4));
        gamma = h ? g1 : g0;
#pragma unroll
        for (int f = 0; f < NF; ++f) v[f] = __builtin_fmaf(acc[i][f][j], flex, bias_a[f] * beta);
      } else {
#pragma unroll
        for (int f = 0; f < NF; ++f) v[f] = __builtin_fmaf(acc[i][f][j], flex, bias_a[f]);
      }
      float o[NO];
      if constexpr (ACT == TAMD_ACT_SWIGLU) {
        o[0] = swiglu_fast(v[0], v[1], a.act_alpha, a.act_limit, has_limit);
      } else {
#pragma unroll
        for (int p = 0; p < NO; ++p) o[p] = v[p];
      }
      if constexpr (ROWSC) {
#pragma unroll
        for (int p = 0; p < NO; ++p) o[p] *= gamma;
      }
      if constexpr (MXO) {
        {
          // MXFP8 output: a group is 32 consecutive output columns of a row = the outputs of one half wave (of
          // half of it when a lane holds two columns).  max |o| over the group, scale = 2^ceil(log2(max / 448)),
          // o / scale clamped to +-448; the cast below rounds to nearest even (as tamd_downcast_mxfp does).
          float m = 0.f;
#pragma unroll
          for (int p = 0; p < NO; ++p) m = __builtin_fmaxf(m, out_col0 + p < n_out ? __builtin_fabsf(o[p]) : 0.f);
#pragma unroll
          for (int sh = 16 / NO; sh > 0; sh >>= 1) m = __builtin_fmaxf(m, __shfl_xor(m, sh));
          const uint32_t sb = (f32_to_bits(m / 448.0f) + 0x007FFFFFu) & 0x7F800000u;
          const float ds = bits_to_f32(sb);
          const float qs = ds == 0.f ? 0.f : 1.0f / ds;
#pragma unroll
          for (int p = 0; p < NO; ++p) {
            const float q = o[p] * qs;
            o[p] = q != q ? q : __builtin_fminf(__builtin_fmaxf(q, -448.0f), 448.0f);
          }
          // one lane per group leaves the scale byte behind the staged tile; the copy-out below places it
          if ((c32 & (32 / NO - 1)) == 0) ob[NFR * 32 * OUT_COLS + r * (OUT_COLS / 32) + wave * NO + c32 * NO / 32] = (uint8_t)(sb >> 23);
        }
      }
      if constexpr (FLEX) {
        if (track_max && r < t.rows) {
#pragma unroll
          for (int p = 0; p < NO; ++p)
            if (out_col0 + p < n_out) amax = absmax_bits(amax, o[p]);
        }
#pragma unroll
        for (int p = 0; p < NO; ++p) {
          o[p] *= inv_expected;
          if (clamp_out) o[p] = __builtin_fminf(__builtin_fmaxf(o[p], -out_max), out_max);
        }
      }
      if (staged) {
        uint8_t *dstl = ob + (r * OUT_COLS + wave * 32 * NO + c32 * NO) * osz;
        if (osz == 2) {
          if constexpr (NO == 2) *(uint32_t *)dstl = narrow2(o[0], o[NO - 1]);
          else *(uint16_t *)dstl = (uint16_t)narrow(o[0]);
        } else {
          if constexpr (NO == 2) *(uint16_t *)dstl = (uint16_t)(narrow(o[0]) | (narrow(o[NO - 1]) << 8));
          else *dstl = (uint8_t)narrow(o[0]);
        }
      } else if (r < t.rows) {
        int64_t dst = t.start_m + t.off_m + r;
        if (a.scatter_indx) dst = a.scatter_indx[dst];
        if (dst >= 0) {
          const int64_t base = (int64_t)t.z * a.y_stride_z + dst * a.y_stride_m;
#pragma unroll
          for (int p = 0; p < NO; ++p)
            if (out_col0 + p < n_out) ((float *)a.y)[base + out_col0 + p] = o[p];
        }
      }
    }
  }
  if constexpr (FLEX) {
    if (track_max) {
      // wave maximum, then one atomic per wave; positive floats order like their bit patterns
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const uint32_t other = (uint32_t)__shfl_xor((int)amax, o);
        amax = other > amax ? other : amax;
      }
      if (lane == 0) {
        amax = amax < 0x7F800000u ? amax : 0x7F800000u;  // NaN counts as +inf
        const float sc = __builtin_fmaf(bits_to_f32(amax), 1.0f / out_max, 1.0e-30f);
        atomicMax((unsigned int *)a.y_actual_scale, f32_to_bits(sc));
      }
    }
  }
  if (staged) {
    __syncthreads();
    if constexpr (MXO) {
      // scale bytes of the tile: OUT_COLS / 32 per row, to the row's (possibly scattered) place
      constexpr int GPR = OUT_COLS / 32;
      for (int id = tid; id < t.rows * GPR; id += 256) {
        const int r = id / GPR, g = id - r * GPR;
        const int gcol = tile_out0 + g * 32;
        if (gcol >= n_out) continue;
        int64_t dst = t.start_m + t.off_m + r;
        if (a.scatter_indx) dst = a.scatter_indx[dst];
        if (dst >= 0) a.y_mx_scale[(int64_t)t.z * a.y_mx_stride_z + dst * a.y_mx_stride_m + gcol / 32] = ob[NFR * 32 * OUT_COLS + id];
      }
    }
    const int epc = 16 / osz;                 // outputs per 16-byte chunk
    const int cpr = OUT_COLS / epc;           // chunks per tile row
    const int n_chunks = t.rows * cpr;
    if constexpr (PRE) {
      // Usual case -- every chunk of the tile lies wholly inside or wholly outside the output's columns and lands on a
      // 16-byte boundary: the staged chunks are read first, then each is stored under one predicate and no other
      // control flow (the general loop below compiles to a state machine per chunk that takes several times longer).
      constexpr int EPC_C = 16 / OSZ_C;
      const bool whole_chunks =
          n_out % EPC_C == 0 &&
          ((((uintptr_t)a.y) | (uintptr_t)(a.y_stride_m * OSZ_C) | (uintptr_t)(a.y_stride_z * OSZ_C)) & 15) == 0;
      if (whole_chunks) {
        uint4 staged_chunk[MAXU];
#pragma unroll
        for (int u = 0; u < MAXU; ++u) staged_chunk[u] = *(const uint4 *)(ob + (size_t)(tid + u * 256) * 16);
#pragma unroll
        for (int u = 0; u < MAXU; ++u) {
          const int id = tid + u * 256;
          const int r = id / CPR_C, c = (id - r * CPR_C) * EPC_C;
          const int gcol = tile_out0 + c;
          if (id < n_chunks && dst_row[u] >= 0 && gcol < n_out) {
            uint8_t *yp = (uint8_t *)a.y + ((int64_t)t.z * a.y_stride_z + (int64_t)dst_row[u] * a.y_stride_m + gcol) * OSZ_C;
            *(uint4 *)yp = staged_chunk[u];
          }
        }
        return;
      }
#pragma unroll
      for (int u = 0; u < MAXU; ++u) {
        const int id = tid + u * 256;
        if (id >= n_chunks) break;
        const int r = id / CPR_C, c = (id - r * CPR_C) * (16 / OSZ_C);
        const int64_t dst = dst_row[u];
        if (dst < 0) continue;
        const int gcol = tile_out0 + c;
        if (gcol >= n_out) continue;
        uint8_t *yp = (uint8_t *)a.y + ((int64_t)t.z * a.y_stride_z + dst * a.y_stride_m + gcol) * OSZ_C;
        const uint8_t *sp = ob + (r * OUT_COLS + c) * OSZ_C;
        if (gcol + 16 / OSZ_C <= n_out && ((uintptr_t)yp & 15) == 0) {
          *(uint4 *)yp = *(const uint4 *)sp;
        } else {
          const int n_b = (n_out - gcol < 16 / OSZ_C ? n_out - gcol : 16 / OSZ_C) * OSZ_C;
          for (int e = 0; e < n_b; ++e) yp[e] = sp[e];
        }
      }
      return;
    }
    // eight chunks per thread at a time, so that the scatter indices of a batch are fetched together
    for (int id0 = tid; id0 < n_chunks; id0 += 256 * 8) {
      int64_t dsts[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int id = id0 + u * 256;
        const int r = id / cpr;
        dsts[u] = t.start_m + t.off_m + (r < t.rows ? r : t.rows - 1);
        if (a.scatter_indx) dsts[u] = a.scatter_indx[dsts[u]];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int id = id0 + u * 256;
        if (id >= n_chunks) break;
        const int r = id / cpr, c = (id - r * cpr) * epc;
        const int64_t dst = dsts[u];
        if (dst < 0) continue;
        const int gcol = tile_out0 + c;
        if (gcol >= n_out) continue;
        uint8_t *yp = (uint8_t *)a.y + ((int64_t)t.z * a.y_stride_z + dst * a.y_stride_m + gcol) * osz;
        const uint8_t *sp = ob + (r * OUT_COLS + c) * osz;
        if (gcol + epc <= n_out && ((uintptr_t)yp & 15) == 0) {
          *(uint4 *)yp = *(const uint4 *)sp;
        } else {
          const int n_b = (n_out - gcol < epc ? n_out - gcol : epc) * osz;
          for (int e = 0; e < n_b; ++e) yp[e] = sp[e];
        }
      }
    }
  }
}

// FAST_YDT: the 16-bit output type that gets the specialised epilogues (the activations' type; bf16 for fp8
// activations); any other combination takes the general one.
// FP8_ROWS: the kernel's activations are fp8; then a plain float8_e4m3fn output (the rows the next matmul of an
// MoE layer consumes) is specialised as well.
template <int NFR, int ACT, int FAST_YDT, bool FP8_ROWS, typename Args>
TAMD_DEVICE void tile_epilogue(const Args &a, const Tile &t, f32x16_t (&acc)[NFR][NF], uint8_t *lds) {
  const bool flexo = a.y_expected_scale != nullptr || a.y_actual_scale != nullptr;
  if (a.y_mx_scale) {  // always e4m3 values and no flexpoint output (checked by the entry point)
    tile_epilogue_t<NFR, ACT, TAMD_FP8_E4M3, true, false, true, Args>(a, t, acc, lds);
  } else if (FP8_ROWS && a.y_dtype == TAMD_FP8_E4M3 && !flexo) {
    if constexpr (FP8_ROWS) tile_epilogue_t<NFR, ACT, TAMD_FP8_E4M3, true, false, false, Args>(a, t, acc, lds);
  } else if (a.y_dtype == FAST_YDT && !flexo) {
    if (a.betas || a.gammas) tile_epilogue_t<NFR, ACT, FAST_YDT, true, false, false, Args>(a, t, acc, lds);
    else tile_epilogue_t<NFR, ACT, FAST_YDT, false, false, false, Args>(a, t, acc, lds);
  } else {
    tile_epilogue_t<NFR, ACT, -1, true, true, false, Args>(a, t, acc, lds);
  }
}

// The kernel's tamd_matmul_args (its first parameter) read in place from the kernel-argument segment, through a
// pointer the compiler cannot see through.  The compiler loads every field of a by-value kernel argument that is
// used anywhere into scalar registers at the top of the kernel; the few dozen that only the epilogue needs then
// stay live through the K loop, the scalar registers overflow into vector registers, and a kernel that sits at 256
// of those starts spilling accumulators.  Read this way, the epilogue's fields are fetched when it begins.
typedef const __attribute__((address_space(4))) tamd_matmul_args late_args_t;
TAMD_DEVICE late_args_t &kernel_args_late() {
  late_args_t *p = (late_args_t *)__builtin_amdgcn_kernarg_segment_ptr();
  asm volatile("" : "+s"(p));
  return *p;
}

// One output tile with NFR (compile time) active 32-row fragments.
// LDS: [A stages (2 to 4) | B: 4 wave-private regions, one or two stages | (fp8) activation block scales | scale ring or
// the e8m0 scales of the whole tile]; with K groups (KS > 1) one such pipeline per group, the tile's scales behind them.
//
// Both operands reach LDS by DMA.  Activations: 64 K per stage (128 K of fp8); wave w copies rows
// 8w..8w+7 of every 32-row fragment (8 lanes x 16 B per row); chunk c of row r sits at slot
// c ^ ((r>>1)&7), which makes the 32-row MFMA operand reads bank-conflict free.  Weights: every
// second stage (every stage of fp8) each wave copies 128 K of its own 64 columns into its private region: position
// p' = f*32 + c holds global column 2c + f of the wave's strip (so a lane ends up with a gate/linear column pair), the
// four 16-byte parts rotated by ((p'>>2)&3) ^ 2f.  From column-strided weights that is 64 contiguous bytes of each
// column; weights in the block layout (TAMD_W_CDNA4_BLOCKS) hold exactly this image, 4 KB per strip and 128 K, and
// are copied as they lie.  The wave reads the region into registers at the start of the stage and immediately
// requests the next 128 K into it, so weights need no barrier.
// Loops: two stages and full waits (16-bit, row blocks above 64 rows or scales not in LDS); counted waits over a
// deeper ring (deep mode, K groups: 16-bit; ring mode, paired: fp8), see pipe_shape.
template <int XDT, int NFR, int LDS_ROWS, int ACT, bool SC_LDS, int KS = 1>
TAMD_DEVICE void run_tile(const tamd_matmul_args &a, const Tile &t, uint8_t *lds_wg) {
  typedef Mma<XDT> M;
  typedef typename M::frag_t frag_t;
  constexpr bool FP8 = is_fp8(XDT);
  constexpr int ESZ = FP8 ? 1 : 2;            // bytes per activation element
  constexpr int KA = A_ROW_BYTES / ESZ;       // K per activation stage
  constexpr int A_STAGE = LDS_ROWS * A_ROW_BYTES;
  constexpr bool RING = FP8 && !SC_LDS;
  constexpr bool DEEP = SC_LDS && deep_mode(FP8, LDS_ROWS);
  static_assert(KS == 1 || (DEEP && NFR == 1 && (KS == 2 || KS == 4)), "K groups: deep mode, one row fragment");
  constexpr PipeShape PS = pipe_shape(FP8, RING, LDS_ROWS, DEEP, KS);
  constexpr int DA = PS.da, DB = PS.db;
  auto a_slot = [](int it) { return DA == 2 ? (it & 1) : it % DA; };
  constexpr uint32_t kOob = 0x7FFFFFFFu;
  const int tid = threadIdx.x;
  // K group of the wave (0 unless KS > 1) and its place among the group's four waves
  const int grp = KS > 1 ? __builtin_amdgcn_readfirstlane(tid / 256) : 0;
  const int wave = KS > 1 ? __builtin_amdgcn_readfirstlane((tid / kWave) & 3) : tid / kWave, lane = tid % kWave;
  const int c32 = lane % 32, h = lane / 32;
  const int K = a.K, N = a.N, G = K / 32;
  // a wave whose 64 columns lie beyond N (last column tile) copies its share of the activations and keeps the
  // barriers, but neither fetches weights nor runs MFMAs
  const bool wave_live = t.n0 + wave * 64 < N;
  // the pipeline buffers of the wave's K group; the tile's scale image behind the last group's is shared
  constexpr int PIPE_G = PS.bytes;
  uint8_t *lds = lds_wg + grp * PIPE_G;
  // the group's part of K: whole 128-K pairs [sup0, sup0 + n_sup), the same number for every group (a group whose
  // part reaches past K copies zeros there: out-of-range offsets)
  const int n_kb_all = (K + KB - 1) / KB;
  const int n_sup = (n_kb_all + KS - 1) / KS;
  const int sup0 = grp * n_sup;
  const int k0 = sup0 * KB;
  const int k_hi = KS > 1 ? (k0 + n_sup * KB < K ? k0 + n_sup * KB : K) : K;

  const v4i_t rx = make_rsrc((const uint8_t *)a.x + (int64_t)t.z * a.x_stride_z * ESZ, kOob);
  const v4i_t rw = make_rsrc((const uint8_t *)a.w + (int64_t)t.expert * a.w_stride_e, kOob);
  const uint8_t *s_base = a.w_mx_scale + (int64_t)t.expert * a.w_mx_stride_e;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
  const uint32_t lds_b = lds_base + DA * A_STAGE + wave * 4096;
  const uint8_t *bbuf = lds + DA * A_STAGE + wave * 4096;
  // activation block scales (fp8 path): two stages of four planes (one per 32-K group of the stage) of one dword
  // per row; a copy always writes 64 dwords (lanes past the tile's rows write zeros)
  constexpr int AS_ROWS = LDS_ROWS < 64 ? 64 : LDS_ROWS;
  constexpr int AS_BYTES = PS.as_bytes;
  uint8_t *lds_sc = KS > 1 ? lds_wg + KS * PIPE_G : lds + DA * A_STAGE + DB * B_BYTES + AS_BYTES;

  // ---- scales of the whole tile, once.  Strided: 256 columns x G bytes, contiguous in memory.  CDNA4
  // pre-shuffle: the tile's 8 blocks of 32 columns are contiguous too (KSP*32 bytes each); byte
  // 256*(k/8) + 64*(k%4) + 4*(n%16) + 2*((k%8)/4) + (n%32)/16 of a block is the scale of (group k, column n).
  const bool cdna4 = a.w_mx_layout == TAMD_SCALE_CDNA4;
  const int KSP = (G + 7) / 8 * 8;
  const int tile_cols = N - t.n0 < BLOCK_N ? N - t.n0 : BLOCK_N;
  const int64_t sc_tile_off = cdna4 ? (int64_t)(t.n0 / 32) * KSP * 32 : (int64_t)t.n0 * G;
  if constexpr (SC_LDS) {
    const uint8_t *sc_src = s_base + sc_tile_off;
    const int sc_tile_bytes = BLOCK_N * (cdna4 ? KSP : G);
    const int sc_avail = cdna4 ? ((N + 31) / 32 * 32 - t.n0) * KSP : (N - t.n0) * G;  // bytes up to the expert's end
    if (cdna4 || ((((uintptr_t)sc_src) & 15) == 0 && (N * G) % 16 == 0)) {
      // by DMA, 1 KB per instruction: in flight together with the first activation / weight stages and
      // awaited with them at the first barrier of the K loop
      const v4i_t rs = make_rsrc(sc_src, (uint32_t)sc_avail);
      const uint32_t lds_sc_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds_sc;
      for (int i = wave + 4 * grp; i * 1024 < sc_tile_bytes; i += 4 * KS)
        dma16(rs, lds_sc_addr + i * 1024, i * 1024 + lane * 16, 0);
    } else {
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)sc_src, 0, (uint32_t)(tile_cols * G),
                                                                        0x00020000);
      const int n_dw = (BLOCK_N * G + 3) / 4;
      const int avail = tile_cols * G;
      for (int i = tid; i < n_dw; i += 256 * KS) {
        uint32_t v;
        if (i * 4 + 4 <= avail || i * 4 >= avail) {
          v = __builtin_amdgcn_raw_buffer_load_b32(rs, i * 4, 0, 0);  // whole, or wholly outside (zeros)
        } else {
          // the dword that straddles the end of the scales: a dword load that is partly out of range returns
          // zeros for all four bytes, so the bytes inside are fetched one by one
          v = 0;
          for (int b = 0; i * 4 + b < avail; ++b)
            v |= (uint32_t)(uint8_t)__builtin_amdgcn_raw_buffer_load_b8(rs, i * 4 + b, 0, 0) << (8 * b);
        }
        ((uint32_t *)lds_sc)[i] = v;
      }
    }
  }
  // offset of a column's scales inside the tile's image (LDS) or, without staging, from the expert's first scale
  int sc_col_off[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    const int tc = wave * 64 + c32 * NF + f;  // tile column
    if constexpr (SC_LDS) {
      sc_col_off[f] = cdna4 ? (tc / 32) * KSP * 32 + (tc % 16) * 4 + (tc % 32) / 16 : tc * G;
    } else {
      const int col = t.n0 + tc < N ? t.n0 + tc : N - 1;
      sc_col_off[f] = cdna4 ? (col / 32) * KSP * 32 + (col % 16) * 4 + (col % 32) / 16 : 0;  // strided: 64-bit below
    }
  }

  const int sc_lane_off[2] = {h * (cdna4 ? 64 : 1), (2 + h) * (cdna4 ? 64 : 1)};  // the (2q + h) part of a group's offset
  const int sc_clamp = cdna4 ? 0x7FFFFFFF : G - 1;

  // ---- block scales of the activations (MXFP8): the 4 e8m0 bytes of a row's 128-K stage are copied per stage to
  // LDS, one byte-sized copy per group (64 rows per instruction, waves 0 and 1; groups past K/32 are not read at
  // all, so nothing beyond a row's own scales is touched)
  const bool x_mx = FP8 && a.x_mx_scale != nullptr;
  const uint32_t lds_as = lds_base + DA * A_STAGE + DB * B_BYTES;
  const uint32_t *as_buf = (const uint32_t *)(lds + DA * A_STAGE + DB * B_BYTES);
  v4i_t ras = rx;
  uint32_t as_off = kOob;
  if (x_mx) {
    const int64_t xr = a.x_rows > 0 ? a.x_rows : a.M;
    ras = make_rsrc(a.x_mx_scale + (int64_t)t.z * a.x_mx_stride_z, (uint32_t)(xr * a.x_mx_stride_m));
    const int r = wave * 64 + lane;
    if (wave * 64 < LDS_ROWS && r < LDS_ROWS) {
      const int rr = t.off_m + (r < t.rows ? r : t.rows - 1);
      const uint32_t src = a.gather_indx ? (uint32_t)a.gather_indx[t.start_m + rr] : (uint32_t)(t.start_m + rr);
      as_off = src * (uint32_t)a.x_mx_stride_m;
    }
  }
  // Copies per request, as the counted waits of the ring loops below see them (a wave's copies complete in the order
  // of their requests): the loops of the issue_* functions run to these numbers and the waits are written in them.
  constexpr int CP_A = NFR;        // issue_a: one copy per row fragment
  constexpr int CP_AS = 4;         // issue_as: one per 32-K group of the stage (waves that hold rows only)
  constexpr int CP_B = 4;          // issue_b: four 1 KB pieces
  constexpr int CP_BPAIR = 8;      // issue_b_pair: eight
  constexpr int CP_SC_STRIDED = 4; // issue_sc: one per group with strided scales, one in all when pre-shuffled
  auto issue_as = [&](int it) {
    if (x_mx && wave * 64 < LDS_ROWS) {
#pragma unroll
      for (int g4 = 0; g4 < CP_AS; ++g4)
        dma1(ras, lds_as + (a_slot(it) * 4 + g4) * AS_ROWS * 4 + wave * 256, it * 4 + g4 < G ? as_off : kOob,
             (uint32_t)(it * 4 + g4));
    }
  };

  // ---- activation DMA: one instruction per 32-row fragment, lane -> (row 8w + lane/8, slot lane%8)
  const int a_rin = wave * 8 + lane / 8;
  const int a_chunk = (lane % 8) ^ ((a_rin >> 1) & 7);
  uint32_t a_off[NFR];
#pragma unroll
  for (int i = 0; i < NFR; ++i) {
    const int r = i * 32 + a_rin;
    // rows past the end of the slice are never stored: they are copied as zeros (out-of-range offset), which
    // keeps the matrix cores' inputs quiet for the padding of a ragged tile
    const int rr = t.off_m + (r < t.rows ? r : t.rows - 1);
    const uint32_t src = a.gather_indx ? (uint32_t)a.gather_indx[t.start_m + rr] : (uint32_t)(t.start_m + rr);
    a_off[i] = r < t.rows ? src * (uint32_t)(a.x_stride_m * ESZ) + a_chunk * 16 : kOob;
  }
  // ---- weight DMA: instruction j copies LDS positions j*16 + lane/4, part slot lane%4
  // Codes in the block layout (TAMD_W_CDNA4_BLOCKS): a stage of this wave's strip is one 4 KB block that already has
  // the LDS image's order, so the four copies are linear (whole, aligned lines) and the K stage enters through the
  // scalar offset; K and N are padded with zero codes, nothing is masked.
  const bool wnat = a.w_layout == TAMD_W_CDNA4_BLOCKS;
  const int w_stage_shift = wnat ? 12 : 6;   // bytes from one K stage to the next: a 4 KB block, or 64 bytes of a column
  // (the lane's 16-byte part of a column is the same for copies 0, 1 and, two further on, for copies 2, 3:
  // (pos >> 2) & 3 = (lane / 16) & 3 for every j, (pos >> 5) << 1 = 2 (j / 2))
  uint32_t w_off[4];
  const int w_part0 = (lane % 4) ^ ((lane / 16) & 3);
  const int w_kpart0 = wnat ? 0 : w_part0 * 32;   // K offset (codes) of the lane's bytes inside a stage; block layout: padded, 0
  auto w_kpart = [&](int j) { return wnat ? 0 : (w_kpart0 ^ ((j >> 1) << 6)); };
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int pos = j * 16 + lane / 4;  // f*32 + c
    const int col = t.n0 + wave * 64 + 2 * (pos % 32) + pos / 32;
    const int part = w_part0 ^ ((j >> 1) << 1);
    w_off[j] = wnat ? (uint32_t)(((t.n0 >> 6) + wave) * ((K + KB - 1) / KB)) * 4096u + (uint32_t)(j * 1024 + lane * 16)
                    : (uint32_t)(col < N ? col : N - 1) * (uint32_t)a.w_stride_n + part * 16;
  }
  // ---- this lane's MFMA columns
  const int col0 = t.n0 + wave * 64 + c32 * NF;

  f32x16_t acc[NFR][NF];
#pragma unroll
  for (int i = 0; i < NFR; ++i)
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[i][f][j] = 0.f;

  const int n_ka = (K + KA - 1) / KA;      // activation stages
  const int n_kb = (K + KB - 1) / KB;      // weight super-stages (two activation stages each)
  auto issue_a = [&](int it) {             // clamped: past the end the last stage is copied again
    if constexpr (!RING && !DEEP) it = it < n_ka ? it : n_ka - 1;   // (ring / deep mode: chunks past K are not read at all)
    const int kb = k0 + it * KA;
    const uint32_t akill = kb + a_chunk * (16 / ESZ) < k_hi ? 0u : kOob;
    const uint32_t sb = lds_base + a_slot(it) * A_STAGE + wave * 8 * A_ROW_BYTES;
#pragma unroll
    for (int i = 0; i < CP_A; ++i) dma16(rx, sb + i * 32 * A_ROW_BYTES, a_off[i] | akill, kb * ESZ);
  };
  auto issue_b = [&](int sup) {
    const uint32_t region = DB == 2 ? (uint32_t)(sup & 1) * B_BYTES : 0u;
    if constexpr (!RING && !DEEP) sup = sup < n_kb ? sup : n_kb - 1;
    const int kb = k0 + sup * KB;
    static_assert(CP_B == 4, "dma16_x4 makes four copies");
    if (wnat) {   // one 4 KB block, copied as it lies
      dma16_x4(rw, lds_b + region, w_off[0] | ((wave_live && kb < k_hi) ? 0u : kOob), (uint32_t)(sup0 + sup) << 12);
      return;
    }
#pragma unroll
    for (int j = 0; j < CP_B; ++j) {
      const uint32_t bkill = (wave_live && kb + w_kpart(j) < k_hi) ? 0u : kOob;
      dma16(rw, lds_b + region + j * 1024, w_off[j] | bkill, (uint32_t)(sup0 + sup) << w_stage_shift);
    }
  };
  // Paired form (ring mode, row blocks of up to 64 rows): the weights of stages 2p and 2p + 1 are 128 contiguous bytes
  // of every column and are requested as such -- eight lanes per column, so that a column's piece is one 128-byte
  // request where it lies inside a line instead of two of 64 bytes a stage apart.  With few rows per expert these
  // requests are what keeps each CU's address unit and L1 busy.  Instruction j copies positions 8j + lane/8 (128 bytes
  // each, wave-private 8 KB); slot lane%8 of position p holds the column's 16-byte part (lane%8) ^ ((p>>1)&7), which
  // keeps the operand reads of 16 consecutive positions on distinct banks.
  constexpr bool PAIRED = RING && DA == 3;
  const uint32_t lds_b2 = lds_base + DA * A_STAGE + wave * 8192;
  const uint8_t *bbuf2 = lds + DA * A_STAGE + wave * 8192;
  uint32_t w2_off[PAIRED ? 8 : 1];
  int w2_part[PAIRED ? 8 : 1];
  if constexpr (PAIRED) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int pos = j * 8 + lane / 8;
      const int col = t.n0 + wave * 64 + 2 * (pos % 32) + pos / 32;
      w2_part[j] = (lane % 8) ^ ((pos >> 1) & 7);
      w2_off[j] = (uint32_t)(col < N ? col : N - 1) * (uint32_t)a.w_stride_n + w2_part[j] * 16;
    }
  }
  auto issue_b_pair = [&](int pair) {
    if constexpr (PAIRED) {
      const int kb = pair * 256;
      static_assert(CP_BPAIR == 8, "two dma16_x4, or eight copies of 128 bytes per column");
      if (wnat) {
        // block layout: the pair's two stages are two 4 KB blocks, copied as they lie (first stage, then second)
        dma16_x4(rw, lds_b2, w_off[0] | ((wave_live && kb < K) ? 0u : kOob), (uint32_t)(2 * pair) * 4096u);
        dma16_x4(rw, lds_b2 + 4096, w_off[0] | ((wave_live && kb + KB < K) ? 0u : kOob), (uint32_t)(2 * pair + 1) * 4096u);
        return;
      }
#pragma unroll
      for (int j = 0; j < CP_BPAIR; ++j) {
        const uint32_t bkill = (wave_live && kb + w2_part[j] * 32 < K) ? 0u : kOob;
        dma16(rw, lds_b2 + j * 1024, w2_off[j] | bkill, kb >> 1);
      }
    }
  };
  // ring mode: the scales of weight stage `sup` for this wave's 64 columns, into the wave's 1 KB piece of the scale
  // ring.  Pre-shuffled layout: one copy -- the wave's two blocks of 32 columns hold the 8 groups that contain the
  // stage's 4 as 256 contiguous bytes each (lanes 0-15 / 16-31; the other lanes copy nothing).  Strided layout:
  // one byte-sized copy per group, lane L fetching column L of the strip into dword [group][L]; slow (64 lines
  // touched per copy) and only used when the scales of a tile do not fit LDS.
  const uint32_t lds_scr = lds_base + DA * A_STAGE + DB * B_BYTES + AS_BYTES;
  const uint8_t *scr_buf = lds + DA * A_STAGE + DB * B_BYTES + AS_BYTES;
  uint32_t scr_voff = kOob;
  v4i_t rsc = rw;
  if constexpr (RING) {
    rsc = make_rsrc(s_base, kOob);
    if (cdna4) {
      const int blk = (t.n0 + wave * 64) / 32 + lane / 16;
      if (lane < 32 && blk * 32 < N && wave_live) scr_voff = (uint32_t)(blk * KSP * 32 + (lane % 16) * 16);
    } else {
      const int col = t.n0 + wave * 64 + lane;
      if (col < N) scr_voff = (uint32_t)((int64_t)col * a.w_mx_stride_n);
    }
  }
  auto issue_sc = [&](int sup) {
    if constexpr (RING) {
      const uint32_t dst = lds_scr + ((uint32_t)(sup & 1) * 4 + wave) * 1024;
      if (cdna4) {
        dma16(rsc, dst, sup * 4 < G ? scr_voff : kOob, (uint32_t)(256 * (sup >> 1)));
      } else {
#pragma unroll
        for (int g4 = 0; g4 < CP_SC_STRIDED; ++g4) {
          const int kg = sup * 4 + g4;
          dma1(rsc, dst + g4 * 256, kg < G ? scr_voff : kOob, (uint32_t)((int64_t)kg * a.w_mx_stride_k));
        }
      }
    }
  };

  // (two register sets: the ring loop for row blocks of up to 64 rows keeps the weights of two stages)
  uint4 raw[2][NF][2];
  float scf[NF][2];      // 16-bit path: 2^(e-127) as a float
  uint32_t scw[2][NF];   // fp8 path: scale bytes of q = 0, 1 in bytes 0, 1
  // registers (set `set`) <- this wave's weights and scales of super-stage `sup`
  auto load_b = [&](int sup, auto set_c) {
    constexpr int set = decltype(set_c)::value;
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int pos = f * 32 + c32;
        const int rot = ((pos >> 2) & 3) ^ (f << 1);   // slot of part p of position pos: p ^ rot
        if constexpr (PAIRED)
          raw[set][f][q] = wnat ? *(const uint4 *)(bbuf2 + (sup & 1) * 4096 + pos * 64 + (((2 * q + h) ^ rot) * 16))
                                : *(const uint4 *)(bbuf2 + pos * 128 + (((4 * (sup & 1) + 2 * q + h) ^ ((pos >> 1) & 7)) * 16));
        else
          raw[set][f][q] = *(const uint4 *)(bbuf + (DB == 2 ? (sup & 1) * B_BYTES : 0) + pos * 64 +
                                            (((2 * q + h) ^ rot) * 16));
        // group kg = 4*sup + 2q + h of this lane's column.  Strided: byte kg, kept inside the column's G bytes
        // (groups past the end of K meet zero codes and zero activations; their scale only has to be some finite
        // value of this column).  Pre-shuffled: byte 256*(kg/8) + 64*(kg%4) + 2*((kg%8)/4); the padding up to a
        // multiple of 8 groups is stored (zeros), so nothing is clamped.
        // (K groups: a group's pairs past the end of K hold zero codes and meet the last pair's scales)
        const int sg = KS > 1 ? (sup0 + sup < n_kb_all ? sup0 + sup : n_kb_all - 1) : sup;
        const int sup_off = cdna4 ? (sg >> 1) * 256 + (sg & 1) * 2 : sg * 4;  // wave uniform
        int kg_off = sup_off + sc_lane_off[q];
        kg_off = kg_off < sc_clamp ? kg_off : sc_clamp;
        uint32_t sbyte;
        if constexpr (RING) {
          const uint8_t *piece = scr_buf + ((sup & 1) * 4 + wave) * 1024;
          const int n = c32 * NF + f;  // column inside the wave's strip
          sbyte = cdna4 ? piece[(n / 32) * 256 + 64 * (2 * q + h) + 4 * (n % 16) + 2 * (sup & 1) + (n % 32) / 16]
                        : piece[((2 * q + h) * 64 + n) * 4];
        } else if constexpr (SC_LDS) sbyte = lds_sc[sc_col_off[f] + kg_off];
        else if (cdna4) sbyte = s_base[sc_col_off[f] + kg_off];
        else sbyte = s_base[(int64_t)(col0 + f < N ? col0 + f : N - 1) * a.w_mx_stride_n + kg_off];
        if constexpr (FP8) scw[set][f] = q == 0 ? sbyte : (scw[set][f] | (sbyte << 8));
        else scf[f][q] = bits_to_f32(sbyte << 23);
      }
  };

  // fp8 path: A fragments of the two 64-K halves of a stage and the activations' scale operands
  i32x8_t af8[FP8 ? 2 : 1][FP8 ? NFR : 1];
  int sa8[FP8 ? NFR : 1];
  auto fp8_read_frags = [&](const uint8_t *buf, int s, i32x8_t *af) {
    const int swz = (c32 >> 1) & 7;
#pragma unroll
    for (int i = 0; i < NFR; ++i) {
      const uint8_t *row = buf + (i * 32 + c32) * A_ROW_BYTES;
      const uint4 lo = *(const uint4 *)(row + (((4 * s + h) ^ swz) * 16));
      const uint4 hi = *(const uint4 *)(row + (((4 * s + 2 + h) ^ swz) * 16));
      af[i] = i32x8_t{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
    }
  };
  // first-half fragments and scale operands of stage `it`: issued together with the weight reads of the stage, so
  // that their latency passes while the next stage's copies are requested
  auto fp8_read0 = [&](int it) {
    if constexpr (FP8) {
      if (!wave_live) return;
      const uint8_t *buf = lds + a_slot(it) * A_STAGE;
      fp8_read_frags(buf, 0, af8[0]);
      // A scale operand: lane half h supplies K block h of an MFMA; byte 0 is the group of s = 0, byte 2 of s = 1
#pragma unroll
      for (int i = 0; i < NFR; ++i)
        sa8[i] = x_mx ? (int)(as_buf[(a_slot(it) * 4 + h) * AS_ROWS + i * 32 + c32] |
                              (as_buf[(a_slot(it) * 4 + 2 + h) * AS_ROWS + i * 32 + c32] << 16))
                      : 0x7F7F7F7F;
    }
  };

  auto compute = [&](int it, auto qc, auto set_c) {
    constexpr int q = decltype(qc)::value;
    constexpr int set = decltype(set_c)::value;
    if (!wave_live) return;
    const uint8_t *buf = lds + a_slot(it) * A_STAGE;
    if constexpr (FP8) {
      // one stage = 128 K = two scaled MFMAs per (row fragment, column fragment); the fragments of the first half
      // and the activations' scale operands are already in registers (fp8_read0)
      constexpr int CBSZ = XDT == TAMD_FP8_E5M2 ? 1 : 0;
      // (the fragments of the second half are requested one by one behind the last MFMAs that use those of the first:
      // both halves of all fragments at once are 64 registers, which this kernel does not have)
      const int swz = (c32 >> 1) & 7;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
#pragma unroll
        for (int f = 0; f < NF; ++f) {
          const uint4 r = raw[set][f][s];
          const i32x8_t bf = i32x8_t{(int)r.x, (int)r.y, (int)r.z, (int)r.w, 0, 0, 0, 0};
#pragma unroll
          for (int i = 0; i < NFR; ++i) {
            if (s == 0) {
              acc[i][f] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af8[0][i], bf, acc[i][f], CBSZ, 4, 0, sa8[i], 0,
                                                                        (int)scw[set][f]);
              if (f == NF - 1) {
                const uint8_t *row = buf + (i * 32 + c32) * A_ROW_BYTES;
                const uint4 lo = *(const uint4 *)(row + (((4 + h) ^ swz) * 16));
                const uint4 hi = *(const uint4 *)(row + (((6 + h) ^ swz) * 16));
                af8[1][i] = i32x8_t{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
              }
            } else {
              acc[i][f] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af8[1][i], bf, acc[i][f], CBSZ, 4, 2, sa8[i], 1,
                                                                        (int)scw[set][f]);
            }
          }
        }
      }
    } else {
      auto read_frags = [&](int s, frag_t *af) {
        const int slot = (h * 4 + s) ^ ((c32 >> 1) & 7);
#pragma unroll
        for (int i = 0; i < NFR; ++i) af[i] = *(const frag_t *)(buf + (i * 32 + c32) * A_ROW_BYTES + slot * 16);
      };
      frag_t af[2][NFR];
      read_frags(0, af[0]);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        if (s < 3) read_frags(s + 1, af[(s + 1) & 1]);
#pragma unroll
        for (int f = 0; f < NF; ++f) {
          const uint4 r = raw[set][f][q];
          const uint32_t codes = s == 0 ? r.x : (s == 1 ? r.y : (s == 2 ? r.z : r.w));
          const frag_t bf = M::expand(codes, scf[f][q]);
#pragma unroll
          for (int i = 0; i < NFR; ++i) acc[i][f] = M::mma(af[s & 1][i], bf, acc[i][f]);
        }
      }
    }
  };

  typedef std::integral_constant<int, 0> Set0;
  typedef std::integral_constant<int, 1> Set1;
  uint32_t warm = 0;   // (K groups: a byte fetched only to warm the caches, see below)
  if constexpr (RING) {
    // Copies complete in the order of their requests, so a stage waits by count for what it needs and leaves the
    // later requests in flight.
    const bool as_wave = x_mx && wave * 64 < LDS_ROWS;
    constexpr int NSC = CP_SC_STRIDED;  // scale copies of a stage with strided scales (1 when pre-shuffled)
    if constexpr (PAIRED) {
      // Three activation stages; an even stage s moves the weights of s and s + 1 into registers and requests those of
      // s + 2 and s + 3 (one pair), the odd stage requests only activations.
      issue_a(0), issue_as(0);
      issue_b_pair(0), issue_sc(0), issue_sc(1);
      issue_a(1), issue_as(1);
      for (int it = 0; it < n_ka; it += 2) {
        // in flight at most: the activations of stage it + 1
        if (as_wave) wait_vmcnt<CP_A + CP_AS>(); else wait_vmcnt<CP_A>();
        __syncthreads();
        load_b(it, Set0{});
        load_b(it + 1, Set1{});
        fp8_read0(it);
        issue_a(it + 2);
        issue_as(it + 2);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // weights are in registers: their buffer may be refilled
        issue_b_pair((it >> 1) + 1);
        issue_sc(it + 2), issue_sc(it + 3);
        compute(it, Set0{}, Set0{});
        if (it + 1 < n_ka) {
          // in flight at most: everything the even stage requested
          if (cdna4) { if (as_wave) wait_vmcnt<CP_A + CP_AS + CP_BPAIR + 2>(); else wait_vmcnt<CP_A + CP_BPAIR + 2>(); }
          else { if (as_wave) wait_vmcnt<CP_A + CP_AS + CP_BPAIR + 2 * NSC>(); else wait_vmcnt<CP_A + CP_BPAIR + 2 * NSC>(); }
          __syncthreads();
          fp8_read0(it + 1);
          issue_a(it + 3);
          issue_as(it + 3);
          compute(it + 1, Set0{}, Set1{});
        }
      }
    } else {
      // Stage s requests the activations of stage s + 1 and then the weights and scales of stage s + 2 (the weight
      // buffer of stage s is free as soon as its contents are in registers): in flight at the top of a stage are at
      // most the weights and scales the stage before requested (5 copies, or 8 with strided scales).
      issue_b(0), issue_sc(0);
      issue_a(0), issue_as(0), issue_b(1), issue_sc(1);
      for (int it = 0; it < n_ka; ++it) {
        if (cdna4) wait_vmcnt<CP_B + 1>(); else wait_vmcnt<CP_B + NSC>();
        __syncthreads();
        load_b(it, Set0{});
        fp8_read0(it);
        issue_a(it + DA - 1);
        issue_as(it + DA - 1);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // weights are in registers: their buffer may be refilled
        issue_b(it + 2);
        issue_sc(it + 2);
        compute(it, Set0{}, Set0{});
      }
    }
  } else {
  issue_a(0);
  issue_b(0);
  if constexpr (FP8) {
    issue_as(0);
    for (int it = 0; it < n_ka; ++it) {  // activation and weight stages coincide (128 K each)
      wait_dma();
      __syncthreads();
      load_b(it, Set0{});
      fp8_read0(it);
      issue_a(it + 1);
      issue_as(it + 1);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // weights are in registers: the region may be refilled
      issue_b(it + 1);
      compute(it, Set0{}, Set0{});
    }
  } else if constexpr (DEEP) {
    if constexpr (KS > 1) {
      // A K-group tile's fixed costs are a third of its time, so the first thing its epilogue fetches -- the bias of the
      // lane's columns -- is requested here already.  The request is older than every copy (the counted waits cover
      // it) and only warms the caches: the byte is dropped after the loop.
      if (a.bias && grp == 0) {
        const int esz = a.bias_dtype == TAMD_F32 ? 4 : 2;
        const uint8_t *bp = (const uint8_t *)a.bias + (col0 < N ? ((int64_t)t.expert * a.bias_stride_e + col0) * esz : 0);
        asm volatile("global_load_ubyte %0, %1, off" : "=v"(warm) : "v"(bp) : "memory");
      }
    }
    // Stage s requests the activations of stage s + DA - 1, an even stage after them the weights of pair s/2 + DB
    // (a weight region is free once its pair's weights are in registers).  Copies complete in the order of their
    // requests: a stage waits until only the requests made after the ones it needs are outstanding
    // (ring_outstanding).  The requests before the loop are those of the stages before 0, in the same order, so the
    // counts hold from the first stage on.
    constexpr int PRE = DA - 1 > 2 * DB ? DA - 1 : 2 * DB;
#pragma unroll
    for (int j = -PRE; j < 0; ++j) {
      if (j + DA - 1 >= 0) issue_a(j + DA - 1);
      if (j % 2 == 0 && j / 2 + DB >= 0) issue_b(j / 2 + DB);
    }
    const int n_stage = KS > 1 ? 2 * n_sup : n_ka;   // (K groups: the same trip count, and barriers, for every group)
    for (int it = 0; it < n_stage; it += 2) {
      wait_vmcnt<ring_outstanding(DA, DB, CP_A, CP_B, false)>();
      __syncthreads();
      load_b(it >> 1, Set0{});
      issue_a(it + DA - 1);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // weights are in registers: the region may be refilled
      issue_b((it >> 1) + DB);
      compute(it, Set0{}, Set0{});
      if (it + 1 < n_stage) {
        wait_vmcnt<ring_outstanding(DA, DB, CP_A, CP_B, true)>();
        __syncthreads();
        issue_a(it + DA);
        compute(it + 1, Set1{}, Set0{});
      }
    }
  } else {
    for (int it = 0; it < n_ka; it += 2) {
      wait_dma();
      __syncthreads();
      load_b(it >> 1, Set0{});
      issue_a(it + 1);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // weights are in registers: the region may be refilled
      issue_b((it >> 1) + 1);
      compute(it, Set0{}, Set0{});
      if (it + 1 < n_ka) {
        // the weight copies just issued (4, after the activation stage it + 1) are not needed before the next
        // even stage and take the longest (weights stream from HBM, activations mostly hit L2): leave them in flight
        wait_vmcnt<CP_B>();
        __syncthreads();
        issue_a(it + 2);
        compute(it + 1, Set1{}, Set0{});
      }
    }
  }
  }
  wait_dma();
  if constexpr (KS > 1) asm volatile("" ::"v"(warm));

  if constexpr (KS > 1) {
    // The groups' partial sums meet in LDS (the pipelines are dead: after the barrier every copy has landed and every
    // operand has been read): group g > 0 leaves its accumulators in plane g - 1 and ends; group 0 adds the planes in
    // the order of the groups and finishes the tile alone (a barrier waits only for the waves that are still alive).
    // (16 bytes per lane and access: a plane is [4 waves][NF x 4 quads][64 lanes] of four accumulators)
    f32x4_t *red = (f32x4_t *)lds_wg;
    constexpr int PLANE = 4 * NF * 4 * kWave;
    __syncthreads();
    if (grp > 0) {
#pragma unroll
      for (int f = 0; f < NF; ++f)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          red[(grp - 1) * PLANE + ((wave * NF + f) * 4 + j) * kWave + lane] =
              f32x4_t{acc[0][f][4 * j], acc[0][f][4 * j + 1], acc[0][f][4 * j + 2], acc[0][f][4 * j + 3]};
    }
    __syncthreads();
    if (grp > 0) return;
#pragma unroll
    for (int g = 1; g < KS; ++g)
#pragma unroll
      for (int f = 0; f < NF; ++f)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const f32x4_t v = red[(g - 1) * PLANE + ((wave * NF + f) * 4 + j) * kWave + lane];
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[0][f][4 * j + e] += v[e];
        }
    __syncthreads();   // the epilogue stages its output through the same memory
  }
  tile_epilogue<NFR, ACT, FP8 ? TAMD_BF16 : XDT, FP8>(kernel_args_late(), t, acc, lds_wg);
}

// Row fragments a workgroup can hold: a 128-row block of 16-bit activations also takes a remainder of
// up to 32 rows (fifth fragment); the fp8 path keeps four (its A operands are twice as wide).
template <int XDT, int BM>
struct TileShape {
  static constexpr int EXTRA = (BM == 128 && !is_fp8(XDT)) ? 32 : 0;
  static constexpr int MF = BM <= 32 ? 1 : (BM + EXTRA) / 32;
  static constexpr int LDS_ROWS = 32 * MF;
};

// BM: block size of the ragged schedule the kernel consumes (16..128).
template <int XDT, int BM, int ACT, bool SC_LDS, int KS = 1>
TAMD_DEVICE void tile_entry(const tamd_matmul_args &a, int grid_n, int64_t grid_total, int group_m, uint8_t *lds) {
  typedef TileShape<XDT, BM> S;
  Tile t;
  if (KS == 1 && group_m == 0) {  // the workgroup finds its tile's place itself (grid_total = row blocks of the launch)
    if (!locate_tile_sorted<BM, S::EXTRA>(a, grid_n, (int)grid_total, t, lds)) return;
  } else if (!locate_tile<BM, S::EXTRA>(a, grid_n, grid_total, group_m, t)) return;
  const int nfr = (t.rows + 31) / 32;  // active row fragments (workgroup uniform)
#define TAMD_CASE(n)                                                                     \
  case n:                                                                                \
    if constexpr (n <= S::MF) run_tile<XDT, n, S::LDS_ROWS, ACT, SC_LDS, KS>(a, t, lds); \
    break;
  switch (nfr) { TAMD_CASE(1) TAMD_CASE(2) TAMD_CASE(3) TAMD_CASE(4) TAMD_CASE(5) }
#undef TAMD_CASE
}

template <int XDT, int BM, int ACT, bool SC_LDS>
__global__ __launch_bounds__(256, 2) void mm_x16_mxfp4_kernel(tamd_matmul_args a, int grid_n, int64_t grid_total,
                                                                  int group_m) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  tile_entry<XDT, BM, ACT, SC_LDS>(a, grid_n, grid_total, group_m, lds);
}

// K groups: KS x 4 waves per tile of at most 32 rows, scales of the tile in LDS (see pipe_shape).
template <int XDT, int BM, int ACT, int KS>
__global__ __launch_bounds__(256 * KS, 1) void mm_x16_mxfp4_kgroups_kernel(tamd_matmul_args a, int grid_n, int64_t grid_total,
                                                                            int group_m) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  tile_entry<XDT, BM, ACT, true, KS>(a, grid_n, grid_total, group_m, lds);
}

template <int XDT, int BM, int ACT, bool SC_LDS>
__global__ __launch_bounds__(256, 2) void mm_x8_mxfp4_kernel(tamd_matmul_args a, int grid_n, int64_t grid_total,
                                                                 int group_m) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  tile_entry<XDT, BM, ACT, SC_LDS>(a, grid_n, grid_total, group_m, lds);
}

template <int XDT, int BM, int ACT>
int launch_x16_act(const tamd_matmul_args &a, int grid_m, hipStream_t st) {
  constexpr int LDS_ROWS = TileShape<XDT, BM>::LDS_ROWS;
  constexpr bool DEEP = deep_mode(is_fp8(XDT), LDS_ROWS);   // (kernels with the scales in LDS)
  constexpr int PIPE_BYTES = pipe_shape(is_fp8(XDT), false, LDS_ROWS, DEEP).bytes;
  constexpr int RING_BYTES = pipe_shape(is_fp8(XDT), true, LDS_ROWS).bytes;
  constexpr int OUT_BYTES = LDS_ROWS * (ACT == TAMD_ACT_SWIGLU ? 128 : 256) * 2;  // epilogue staging
  int grid_n = (a.N + BLOCK_N - 1) / BLOCK_N;
  int64_t total = (int64_t)grid_m * grid_n;
  if (total <= 0) return 0;
  int64_t launch = ((total + 7) / 8) * 8;
  if (launch > 0x7FFFFFFF) return TAMD_E_UNSUPPORTED;
  // scales of a tile are staged in LDS when they are dense ([N][K/32]) or pre-shuffled and two workgroups still fit a CU;
  // the fp8 path does not stage pre-shuffled scales: they travel with the weight stages (ring mode), as strided ones
  // do when a tile's worth does not fit
  const int64_t G = a.K / 32;
  const bool cdna4 = a.w_mx_layout == TAMD_SCALE_CDNA4;
  const int64_t sc_bytes = (BLOCK_N * (cdna4 ? (G + 7) / 8 * 8 : G) + 1023) / 1024 * 1024;  // whole 1 KB copies
  const bool dense_sc = cdna4 || (a.w_mx_stride_k == 1 && a.w_mx_stride_n == G && a.w_mx_stride_e % 4 == 0 &&
                                  aligned(a.w_mx_scale, 4) && (BLOCK_N * G) % 4 == 0);
  // (deep mode is worth a CU to itself: up to 156 KB; otherwise two workgroups have to fit)
  const int sc_in_lds = dense_sc && PIPE_BYTES + sc_bytes <= (DEEP ? 156 : 80) * 1024 && !(is_fp8(XDT) && cdna4);
  constexpr int PLAIN_BYTES = pipe_shape(is_fp8(XDT), false, LDS_ROWS).bytes;   // 16-bit path, scales read from memory
  size_t lds_bytes = sc_in_lds ? PIPE_BYTES + sc_bytes : (is_fp8(XDT) ? RING_BYTES : PLAIN_BYTES);
  if (lds_bytes < (size_t)OUT_BYTES) lds_bytes = OUT_BYTES;
  void (*kern)(tamd_matmul_args, int, int64_t, int);
  if constexpr (is_fp8(XDT))
    kern = sc_in_lds ? mm_x8_mxfp4_kernel<XDT, BM, ACT, true> : mm_x8_mxfp4_kernel<XDT, BM, ACT, false>;
  else
    kern = sc_in_lds ? mm_x16_mxfp4_kernel<XDT, BM, ACT, true> : mm_x16_mxfp4_kernel<XDT, BM, ACT, false>;
  // row blocks walked together: as many as one expert (or batch entry) has, while their activation
  // rows (BM x K each) fit comfortably in one XCD's 4 MB L2
  const int64_t rows_per_slice = a.block_schedule ? a.M / a.n_experts : a.M;
  int64_t group_m = rows_per_slice / BM;
  const int64_t fit = (int64_t)(2.5 * 1024 * 1024) / ((int64_t)BM * a.K * (is_fp8(XDT) ? 1 : 2));
  group_m = group_m > fit ? fit : group_m;
  group_m = group_m < 1 ? 1 : (group_m > 16 ? 16 : group_m);
  if constexpr (!is_fp8(XDT) && BM == 32) {
    // Fewer tiles than CUs: K groups, so that every SIMD of the CUs that do get a tile holds two to four waves
    // (at least two 128-K pairs per group; the groups' pipelines and the tile's scales have to fit one CU's LDS)
    int cus = 0;
    if (int rc = cu_count(cus)) return rc;
    const int64_t pairs = (a.K + KB - 1) / KB;
    const int ks = total * 2 <= cus && pairs >= 8 ? 4 : (total <= cus && pairs >= 4 ? 2 : 1);
    const size_t pipe = ks == 4 ? 4 * (size_t)pipe_shape(false, false, LDS_ROWS, true, 4).bytes
                                : 2 * (size_t)pipe_shape(false, false, LDS_ROWS, true, 2).bytes;
    if (ks > 1 && dense_sc && pipe + sc_bytes <= 156 * 1024) {
      void (*kk)(tamd_matmul_args, int, int64_t, int) =
          ks == 4 ? mm_x16_mxfp4_kgroups_kernel<XDT, BM, ACT, 4> : mm_x16_mxfp4_kgroups_kernel<XDT, BM, ACT, 2>;
      if (int rc = raise_lds_limit_once((const void *)kk)) return rc;
      kk<<<dim3((unsigned)launch), 256 * ks, pipe + sc_bytes, st>>>(a, grid_n, total, (int)group_m);
      return launch_status();
    }
  }
  if (int rc = raise_lds_limit_once((const void *)kern)) return rc;
  if (a.block_schedule && a.block_offs && group_m == 1 && grid_m <= 1024) {
    // few row blocks per expert: the workgroups take the row blocks largest first, dealt evenly to the XCDs
    const int64_t sorted_launch = (int64_t)((grid_m + 7) / 8) * 8 * grid_n;
    kern<<<dim3((unsigned)sorted_launch), 256, lds_bytes, st>>>(a, grid_n, (int64_t)grid_m, 0);
    return launch_status();
  }
  kern<<<dim3((unsigned)launch), 256, lds_bytes, st>>>(a, grid_n, total, (int)group_m);
  return launch_status();
}

// Row block size of a dense / batched problem (block_m == 0 on entry of a dispatcher): the largest block whose
// tiles still give every CU one, because a tile's K loop is bound by the latency of its stages, not by its
// rows -- 256 x 2048 x 4096 runs 55 us as 2 x 16 tiles of 128 rows and 27 us as 8 x 16 tiles of 32.
inline int dense_block_m(const tamd_matmul_args &a) {
  const int64_t cols = (int64_t)((a.N + BLOCK_N - 1) / BLOCK_N) * a.n_experts;
  const int cand[3] = {128, 64, 32};
  for (int bm : cand)
    if (a.M > bm / 2 && (a.M + bm - 1) / bm * cols >= 256) return bm;
  return 16;  // too few tiles either way: the smallest block gives the most
}
// A dense / batched problem of 161 to 256 rows whose 32-row tiles number at most half the CUs and whose K holds at
// least eight 128-K pairs: faster as 32-row tiles with four K groups each (256 x 2048 x 4096: 13.8 us) than as 16-row
// blocks through the streaming kernel (22 us), which is what problems of fewer rows take.
inline bool dense_prefers_k_groups(const tamd_matmul_args &a) {
  if (is_fp8(a.x_dtype) || a.M <= 160 || a.M > 256 || (a.K + KB - 1) / KB < 8) return false;
  int cus = 0;
  if (cu_count(cus) != 0) return false;
  const int64_t tiles = (int64_t)((a.M + 31) / 32) * a.n_experts * ((a.N + BLOCK_N - 1) / BLOCK_N);
  return tiles * 2 <= cus;
}
inline void dense_grid(const tamd_matmul_args &a, int &block_m, int &grid_m) {
  if (block_m != 0) return;
  block_m = dense_block_m(a);
  grid_m = ((a.M + block_m - 1) / block_m) * a.n_experts;
}

// The tiled kernels of one activation type and one epilogue activation.  The two activations are compiled in
// translation units of their own (moe_matmul_<type>.hip: none, moe_matmul_<type>_swiglu.hip: SwiGLU), which
// is all that separates them: each unit holds 16 kernels of up to 20 unrolled epilogues.
template <int XDT, int ACT>
int dispatch_x16_act(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st) {
  dense_grid(a, block_m, grid_m);
  switch (block_m) {
    case 16: return launch_x16_act<XDT, 16, ACT>(a, grid_m, st);
    case 32: return launch_x16_act<XDT, 32, ACT>(a, grid_m, st);
    case 64: return launch_x16_act<XDT, 64, ACT>(a, grid_m, st);
    case 128: return launch_x16_act<XDT, 128, ACT>(a, grid_m, st);
    default: return TAMD_E_UNSUPPORTED;
  }
}
int tiled_mm_swiglu_bf16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st);
int tiled_mm_swiglu_f16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st);
int tiled_mm_swiglu_fp8e4m3(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st);
int tiled_mm_swiglu_fp8e5m2(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st);

}  // namespace tamd

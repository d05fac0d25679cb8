// Routing kernels for gfx950: top-k (+softmax, bit matrix), expert histogram with a
// stable expert-major ordering of the (token, slot) pairs, and the ragged-tensor
// block metadata.  Integer work only; wave64 ballots / shuffles, no float atomics,
// results independent of scheduling.
#include <atomic>

#include "common.h"

namespace tamd {

// Workspace of tamd_routing_metadata_static: lives in the code object instead of an allocation.  Every GPU that
// loads the library holds its own copy (4 MiB) until the process ends.
constexpr int64_t kStaticWorkspaceInts = 1 << 20;
static __device__ __align__(256) int32_t scratch[kStaticWorkspaceInts];

// ---------------------------------------------------------------------------
// top-k
// ---------------------------------------------------------------------------
// Sort key of a logit: order-preserving map of the float32 bits in the high
// part, (0xFFFF - column) in the low 16 bits so that the lower column wins ties
// (topk_details/_topk_forward.py:15-30).  -0.0 is keyed as +0.0 so that both
// zeros tie, as they do under the reference's stable argsort of -x.
TAMD_DEVICE uint64_t logit_key(float x, int col) {
  uint32_t u = f32_to_bits(x);
  if (u == 0x80000000u) u = 0u;
  u ^= (u >> 31) ? 0xFFFFFFFFu : 0x80000000u;
  return ((uint64_t)u << 16) | (uint64_t)(0xFFFFu - (uint32_t)col);
}

// Inverse of the value part of logit_key (a -0.0 logit comes back as +0.0).
TAMD_DEVICE float logit_of_key(uint64_t key) {
  uint32_t u = (uint32_t)(key >> 16);
  u ^= (u >> 31) ? 0x80000000u : 0xFFFFFFFFu;
  return bits_to_f32(u);
}

// Step O (1, 2, 4, ...) of a butterfly reduction over groups of lanes: the value of a lane of the other aligned block
// of O lanes.  All lanes of a block of O hold the same value by then, so for O = 4 and 8 the partner may be the
// mirrored lane, which, like the swaps inside a quad, the data-parallel move does in the register file; from 16 up it
// is the lane at XOR distance O, through the LDS crossbar.
template <int O>
TAMD_DEVICE uint32_t butterfly_partner(uint32_t v) {
  if constexpr (O == 1) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);        // quad_perm [1,0,3,2]
  else if constexpr (O == 2) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
  else if constexpr (O == 4) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, true);  // row_half_mirror
  else if constexpr (O == 8) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xF, 0xF, true);  // row_mirror
  else return (uint32_t)__shfl_xor((int)v, O);
}

template <int L, int O = 1>
TAMD_DEVICE uint64_t group_max_u64(uint64_t v) {
  if constexpr (O < L) {
    const uint32_t lo = butterfly_partner<O>((uint32_t)v);
    const uint32_t hi = butterfly_partner<O>((uint32_t)(v >> 32));
    const uint64_t w = ((uint64_t)hi << 32) | lo;
    return group_max_u64<L, O * 2>(w > v ? w : v);
  } else {
    return v;
  }
}

template <int L, int O = 1>
TAMD_DEVICE float group_sum_f32(float v) {
  if constexpr (O < L) return group_sum_f32<L, O * 2>(v + bits_to_f32(butterfly_partner<O>(f32_to_bits(v))));
  else return v;
}

template <int L, int O = 1>
TAMD_DEVICE float group_max_f32(float v) {
  if constexpr (O < L) return group_max_f32<L, O * 2>(__builtin_fmaxf(v, bits_to_f32(butterfly_partner<O>(f32_to_bits(v)))));
  else return v;
}

// L lanes cooperate on one row; EPL > 0 keeps ceil(n_cols/L) <= EPL keys in registers.  `row` is the row of this
// thread's group of L lanes (any row >= n_rows: a group that only takes part in the shuffles); lds_indx, when given,
// also receives the picked columns ([row][k] ints) for a kernel that goes on to use them.
template <int DT, int L, int EPL>
TAMD_DEVICE void topk_row(const void *__restrict__ x, int64_t x_stride, int n_rows, int n_cols, int k,
                          int apply_softmax, int use_provided, void *__restrict__ y_vals,
                          int16_t *__restrict__ y_indx, int64_t y_stride, uint32_t *__restrict__ bits,
                          int64_t bits_stride_row, int64_t bits_stride_word, int64_t row, int32_t *lds_indx) {
  const int sub = threadIdx.x % L;
  const bool live = row < n_rows;
  const int64_t rrow = live ? row : 0;
  const int64_t xoff = rrow * x_stride;
  int my_idx = 0;
  uint64_t mine = 0ull;  // key of the column this lane's slot picked
  if (use_provided) {
    if (sub < k) my_idx = y_indx[rrow * y_stride + sub];
  } else {
    uint64_t keys[EPL > 0 ? EPL : 1];
    if constexpr (EPL > 0) {
      // every lane loads (columns past the end re-read the last one) and the values are pinned before they are
      // selected: a load that the compiler may move under the per-lane condition is awaited before the next one is
      // issued, eight round trips to memory instead of one
      float xv[EPL];
#pragma unroll
      for (int j = 0; j < EPL; ++j) {
        const int c = sub + j * L;
        xv[j] = load_as_f32<DT>(x, xoff + (c < n_cols ? c : n_cols - 1));
      }
#pragma unroll
      for (int j = 0; j < EPL; ++j) asm volatile("" : "+v"(xv[j]));
#pragma unroll
      for (int j = 0; j < EPL; ++j) {
        const int c = sub + j * L;
        keys[j] = c < n_cols ? logit_key(xv[j], c) : 0ull;
      }
    }
    uint64_t prev = ~0ull;
    for (int pass = 0; pass < k; ++pass) {
      uint64_t best = 0ull;
      if constexpr (EPL > 0) {
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
          uint64_t q = keys[j];
          best = (q < prev && q > best) ? q : best;
        }
      } else {
        for (int c = sub; c < n_cols; c += L) {
          uint64_t q = logit_key(load_as_f32<DT>(x, xoff + c), c);
          best = (q < prev && q > best) ? q : best;
        }
      }
      best = group_max_u64<L>(best);
      if (sub == pass) mine = best;
      prev = best;
    }
    my_idx = (int)(0xFFFFu - (uint32_t)(mine & 0xFFFFull));
  }
  const bool slot = sub < k;
  float v;
  if (apply_softmax && !use_provided) {
    v = slot ? logit_of_key(mine) : 0.f;  // a zero's sign is lost in the key and makes no difference to the softmax
  } else {
    v = slot ? load_as_f32<DT>(x, xoff + my_idx) : 0.f;
  }
  if (apply_softmax) {
    float mx = group_max_f32<L>(slot ? v : -__builtin_inff());
    float e = slot ? expf(v - mx) : 0.f;
    float s = group_sum_f32<L>(e);
    v = e / s;
  }
  if (live && slot) {
    store_from_f32<DT>(y_vals, rrow * y_stride + sub, v);
    if (!use_provided) y_indx[rrow * y_stride + sub] = (int16_t)my_idx;
    if (lds_indx) lds_indx[rrow * k + sub] = my_idx;
  }
  const int n_words = (n_cols + 31) / 32;
  const int base_lane = (threadIdx.x % kWave) - sub;
  for (int w0 = 0; w0 < n_words; w0 += L) {
    int w = w0 + sub;
    uint32_t word = 0;
    for (int j = 0; j < k; ++j) {
      int ij = __shfl(my_idx, base_lane + j);
      word |= ((ij >> 5) == w) ? (1u << (ij & 31)) : 0u;
    }
    if (live && w < n_words) bits[rrow * bits_stride_row + (int64_t)w * bits_stride_word] = word;
  }
}

template <int DT, int L, int EPL>
__global__ __launch_bounds__(256) void topk_kernel(const void *__restrict__ x, int64_t x_stride, int n_rows,
                                                   int n_cols, int k, int apply_softmax, int use_provided,
                                                   void *__restrict__ y_vals, int16_t *__restrict__ y_indx,
                                                   int64_t y_stride, uint32_t *__restrict__ bits,
                                                   int64_t bits_stride_row, int64_t bits_stride_word) {
  constexpr int ROWS_PER_BLOCK = 256 / L;
  topk_row<DT, L, EPL>(x, x_stride, n_rows, n_cols, k, apply_softmax, use_provided, y_vals, y_indx, y_stride, bits,
                       bits_stride_row, bits_stride_word, (int64_t)blockIdx.x * ROWS_PER_BLOCK + threadIdx.x / L, nullptr);
}

template <int DT>
int launch_topk(const void *x, int64_t xs, int n_rows, int n_cols, int k, int sm, int prov, void *yv, int16_t *yi,
                int64_t ys, uint32_t *bits, int64_t bsr, int64_t bsw, hipStream_t st) {
  int need = (n_cols + 7) / 8;
  if (need < k) need = k;
#define TAMD_TOPK(LL, EE)                                                                                    \
  topk_kernel<DT, LL, EE><<<dim3((unsigned)((n_rows + (256 / LL) - 1) / (256 / LL))), 256, 0, st>>>(          \
      x, xs, n_rows, n_cols, k, sm, prov, yv, yi, ys, bits, bsr, bsw)
  if (need <= 8) TAMD_TOPK(8, 8);
  else if (need <= 16) TAMD_TOPK(16, 8);
  else if (need <= 32) TAMD_TOPK(32, 8);
  else if (n_cols <= 512) TAMD_TOPK(64, 8);
  else TAMD_TOPK(64, 0);
#undef TAMD_TOPK
  return launch_status();
}

// ---------------------------------------------------------------------------
// histogram + stable expert-major ordering
// ---------------------------------------------------------------------------
// Entries are processed in chunks of 64 (one wave, one entry per lane).  Inside a
// chunk the rank of an entry among the entries with the same expert is a popcount
// of the lanes below it that hold the same id; the set of such lanes is built
// from one ballot per bit of the id.  Per-chunk counts are prefix-summed inside a
// block (CH chunks), per-block totals across blocks, expert totals across
// experts; the position of an entry is the sum of those three prefixes and its
// in-chunk rank.  No atomics, so the order is the flat (token, slot) order.

TAMD_DEVICE int load_indx(const void *p, int is16, int64_t i) {
  return is16 ? (int)((const int16_t *)p)[i] : ((const int32_t *)p)[i];
}

TAMD_DEVICE uint64_t same_id_mask(int e, bool valid, int nbits) {
  uint64_t same = __ballot(valid);
  for (int b = 0; b < nbits; ++b) {
    bool bit = (e >> b) & 1;
    uint64_t m = __ballot(valid && bit);
    same &= bit ? m : ~m;
  }
  return same;
}

TAMD_DEVICE uint64_t lanemask_lt() {
  int lane = threadIdx.x % kWave;
  return lane == 0 ? 0ull : (~0ull >> (64 - lane));
}

__global__ __launch_bounds__(1024) void hist_kernel(const void *__restrict__ indx, int is16, int64_t n, int E,
                                                   int CH, int nbits, int32_t *__restrict__ chunk_pref,
                                                   int32_t *__restrict__ block_tot) {
  extern __shared__ int32_t hist[];  // [CH][E]
  const int blk = blockIdx.x;
  for (int i = threadIdx.x; i < CH * E; i += 1024) hist[i] = 0;
  __syncthreads();
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  for (int c = wave; c < CH; c += 16) {  // CH <= 16: one chunk per wave, so a workgroup waits for memory once
    int64_t i = ((int64_t)blk * CH + c) * 64 + lane;
    int e = i < n ? load_indx(indx, is16, i) : -1;
    bool valid = e >= 0 && e < E;
    uint64_t same = same_id_mask(e, valid, nbits);
    if (valid && (same & lanemask_lt()) == 0) hist[c * E + e] = __popcll(same);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 1024) {
    int run = 0;
    for (int c = 0; c < CH; ++c) {
      int t = hist[c * E + e];
      if (chunk_pref) chunk_pref[((int64_t)blk * CH + c) * E + e] = run;  // (not needed by order_scan_kernel)
      run += t;
    }
    block_tot[(int64_t)blk * E + e] = run;
  }
}

// Inclusive prefix sum over the 64 lanes of a wave (all of them active), in the register file: shifts inside the rows
// of 16 lanes, then the last lane of rows 0 and 2 added to rows 1 and 3, then lane 31 added to the upper half.
TAMD_DEVICE int wave_incl_scan(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, false);  // row_shr:1 (a lane without a source adds 0)
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2 and 3
  return v;
}

// Exclusive scan of up to 1024 ints held one per thread; returns the total.
TAMD_DEVICE int block_excl_scan_1024(int v, int &total, int *lds /* >= 17 ints */) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int inc = wave_incl_scan(v);
  __syncthreads();
  if (lane == kWave - 1) lds[wave] = inc;
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int w = 0; w < 16; ++w) {
      int t = lds[w];
      lds[w] = run;
      run += t;
    }
    lds[16] = run;
  }
  __syncthreads();
  total = lds[16];
  return inc - v + lds[wave];
}

// Exclusive prefix over the workgroups' totals of expert e (written to `out` when given; it may be `tot` itself);
// returns the expert's total.  Sixteen totals are loaded before any of them is used or stored, so that a thread
// waits for memory once per sixteen blocks and not once per block.
TAMD_DEVICE int scan_block_totals(const int32_t *tot, int32_t *out, int n_blocks, int E, int e) {
  int run = 0;
  for (int b0 = 0; b0 < n_blocks; b0 += 16) {
    int t[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) t[u] = tot[(int64_t)(b0 + u < n_blocks ? b0 + u : n_blocks - 1) * E + e];
#pragma unroll
    for (int u = 0; u < 16; ++u) asm volatile("" : "+v"(t[u]));
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      if (b0 + u < n_blocks) {
        if (out) out[(int64_t)(b0 + u) * E + e] = run;
        run += t[u];
      }
    }
  }
  return run;
}

__global__ __launch_bounds__(1024) void scan_kernel(int E, int n_blocks, int32_t *__restrict__ block_tot,
                                                    int32_t *__restrict__ col_sum, int32_t *__restrict__ col_offs,
                                                    int32_t *__restrict__ n_valid) {
  __shared__ int lds[17];
  int carry = 0;
  for (int e0 = 0; e0 < E; e0 += 1024) {
    int e = e0 + threadIdx.x;
    int run = 0;
    if (e < E) {
      run = scan_block_totals(block_tot, block_tot, n_blocks, E, e);
      col_sum[e] = run;
    }
    int total;
    int ex = block_excl_scan_1024(run, total, lds);
    if (e < E) col_offs[e] = carry + ex;
    carry += total;
  }
  if (threadIdx.x == 0) *n_valid = carry;
}

__global__ __launch_bounds__(1024) void order_kernel(const void *__restrict__ indx, int is16, int64_t n, int E,
                                                    int CH, int nbits, int k, const int32_t *__restrict__ chunk_pref,
                                                    const int32_t *__restrict__ block_off,
                                                    const int32_t *__restrict__ col_offs,
                                                    const int32_t *__restrict__ n_valid,
                                                    int32_t *__restrict__ col_sorted, int32_t *__restrict__ row_sorted,
                                                    int32_t *__restrict__ gather) {
  const int blk = blockIdx.x;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int nv = *n_valid;
  for (int c = wave; c < CH; c += 16) {
    int64_t chunk = (int64_t)blk * CH + c;
    int64_t i = chunk * 64 + lane;
    int e = i < n ? load_indx(indx, is16, i) : -1;
    bool valid = e >= 0 && e < E;
    uint64_t same = same_id_mask(e, valid, nbits);
    if (valid) {
      int pos = col_offs[e] + block_off[(int64_t)blk * E + e] + chunk_pref[chunk * E + e] +
                __popcll(same & lanemask_lt());
      row_sorted[i] = pos;
      col_sorted[pos] = (int32_t)i;
      if (gather) gather[pos] = (int32_t)(i / k);
    } else if (i < n) {
      row_sorted[i] = -1;
    }
    if (i >= nv && i < n) {
      col_sorted[i] = -1;
      if (gather) gather[i] = 0;  // trunc(-1 / k)
    }
  }
}

struct MetaPlan {
  int CH;
  int nbits;
  int64_t n_chunks, n_blocks;
  int64_t off_chunk_pref, off_block_tot, off_block_off, off_col_offs, off_n_valid, total;
};

inline MetaPlan make_meta_plan(int64_t n_indx, int E) {
  MetaPlan p;
  // LDS histogram of CH*E ints, at most 64 KiB
  int ch = 16;
  while (ch > 1 && (int64_t)ch * E * 4 > 65536) ch >>= 1;
  p.CH = ch;
  p.nbits = 0;
  while ((1 << p.nbits) < E) ++p.nbits;
  p.n_chunks = (n_indx + 63) / 64;
  p.n_blocks = (p.n_chunks + ch - 1) / ch;
  if (p.n_blocks < 1) p.n_blocks = 1;
  p.off_chunk_pref = 0;
  p.off_block_tot = p.n_blocks * ch * (int64_t)E;
  p.off_block_off = p.off_block_tot + p.n_blocks * (int64_t)E;
  p.off_col_offs = p.off_block_off + p.n_blocks * (int64_t)E;
  p.off_n_valid = p.off_col_offs + E;
  p.total = p.off_n_valid + 1;
  return p;
}

inline int launch_bitmatrix_metadata(const void *indx, int is16, int64_t n, int E, int k, int32_t *col_sum,
                                     int32_t *col_sorted, int32_t *row_sorted, int32_t *gather, int32_t *ws,
                                     hipStream_t st, bool before_order(void *), void *ctx) {
  MetaPlan p = make_meta_plan(n, E);
  size_t lds = (size_t)p.CH * E * 4;
  hist_kernel<<<dim3((unsigned)p.n_blocks), 1024, lds, st>>>(indx, is16, n, E, p.CH, p.nbits, ws + p.off_chunk_pref,
                                                           ws + p.off_block_tot);
  scan_kernel<<<1, 1024, 0, st>>>(E, (int)p.n_blocks, ws + p.off_block_tot, col_sum, ws + p.off_col_offs,
                                  ws + p.off_n_valid);
  if (before_order && !before_order(ctx)) return launch_status();
  order_kernel<<<dim3((unsigned)p.n_blocks), 1024, 0, st>>>(indx, is16, n, E, p.CH, p.nbits, k, ws + p.off_chunk_pref,
                                                          ws + p.off_block_tot, ws + p.off_col_offs,
                                                          ws + p.off_n_valid, col_sorted, row_sorted, gather);
  return launch_status();
}

// ---------------------------------------------------------------------------
// ragged tensor metadata
// ---------------------------------------------------------------------------
// Row r of the offsets table: r = 0 slice offsets, r >= 1 block offsets for block size 8 << r.
// Wave r < 6 of a workgroup scans row r (64 slices per step with a running carry) into `tab`
// (pitch S + 1) and, when `offs` is given, into global memory.
TAMD_DEVICE void ragged_scan_rows(const int32_t *sizes, int S, int32_t *tab, int32_t *offs, int64_t offs_pitch) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (wave >= 6) return;
  const int sh = wave == 0 ? 0 : wave + 3;
  int32_t *trow = tab + (int64_t)wave * (S + 1);
  int32_t *grow = offs ? offs + (int64_t)wave * offs_pitch : nullptr;
  int carry = 0;
  for (int s0 = 0; s0 < S; s0 += kWave) {
    const int s = s0 + lane;
    const int v = s < S ? ((sizes[s] + ((1 << sh) - 1)) >> sh) : 0;
    const int inc = wave_incl_scan(v);
    if (s < S) {
      trow[s] = carry + inc - v;
      if (grow) grow[s] = carry + inc - v;
    }
    carry += __shfl(inc, kWave - 1);
  }
  if (lane == 0) {
    trow[S] = carry;
    if (grow) grow[S] = carry;
  }
}

// Schedule entry j of block size index b is ((j - block_offs[s]) << 16) | s for the slice s whose block
// range holds j (binary search in the scanned row; empty slices are skipped by the search), -1 past
// the last block.  Entries [first, first + count) of the flattened [5][max_blocks] table.
TAMD_DEVICE void ragged_fill_schedule(const int32_t *tab, int S, int32_t *sched, int64_t sched_pitch, int max_blocks,
                                      int64_t first, int64_t count) {
  const bool narrow = first + count <= 0x7FFFFFFF;  // then the table index is found with a 32-bit division
  for (int64_t idx = first + threadIdx.x; idx < first + count; idx += blockDim.x) {
    const int b = narrow ? (int)((uint32_t)idx / (uint32_t)max_blocks) : (int)(idx / max_blocks);
    const int j = (int)(idx - (int64_t)b * max_blocks);
    const int32_t *row = tab + (int64_t)(b + 1) * (S + 1);
    int val = -1;
    if (j < row[S]) {
      int lo = 0, hi = S - 1;
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (row[mid + 1] <= j) lo = mid + 1;
        else hi = mid;
      }
      val = ((j - row[lo]) << 16) + lo;
    }
    sched[(int64_t)b * sched_pitch + j] = val;
  }
}

// Every workgroup scans the (small) size vector into its own LDS copy of the table, workgroup 0 also
// writes it out, and the schedule entries are split evenly over the workgroups.
__global__ __launch_bounds__(1024) void ragged_kernel(const int32_t *__restrict__ sizes, int S,
                                                      int32_t *__restrict__ offs, int64_t offs_pitch,
                                                      int32_t *__restrict__ sched, int64_t sched_pitch, int max_blocks) {
  extern __shared__ int32_t tab[];  // [6][S + 1]
  ragged_scan_rows(sizes, S, tab, blockIdx.x == 0 ? offs : nullptr, offs_pitch);
  __syncthreads();
  const int64_t total = 5 * (int64_t)max_blocks;
  const int64_t per = (total + gridDim.x - 1) / gridDim.x;
  const int64_t first = per * blockIdx.x;
  if (first < total) ragged_fill_schedule(tab, S, sched, sched_pitch, max_blocks, first, per < total - first ? per : total - first);
}

// Second of three launches for larger index arrays: the prefix sums over the per-workgroup histograms
// (as scan_kernel) merged with the ragged tables.  Every workgroup repeats the small scans into its own
// LDS and fills its share of the schedule; workgroup 0 alone writes the scan results.  The prefix over
// workgroups goes to `block_off` (not in place: the other workgroups still read `block_tot`).
__global__ __launch_bounds__(1024) void scan_ragged_kernel(int E, int n_blocks, const int32_t *__restrict__ block_tot,
                                                           int32_t *__restrict__ block_off, int32_t *__restrict__ col_sum,
                                                           int32_t *__restrict__ col_offs, int32_t *__restrict__ n_valid,
                                                           int32_t *__restrict__ offs, int64_t offs_pitch,
                                                           int32_t *__restrict__ sched, int64_t sched_pitch, int max_blocks) {
  extern __shared__ int32_t sm[];
  int32_t *csum = sm;             // [E]
  int32_t *tab = csum + E;        // [6][E + 1]
  int32_t *scr = tab + 6 * (E + 1);
  const bool lead = blockIdx.x == 0;
  int carry = 0;
  for (int e0 = 0; e0 < E; e0 += 1024) {
    const int e = e0 + threadIdx.x;
    int run = 0;
    if (e < E) {
      run = scan_block_totals(block_tot, lead ? block_off : nullptr, n_blocks, E, e);
      csum[e] = run;
      if (lead) col_sum[e] = run;
    }
    int total;
    const int ex = block_excl_scan_1024(run, total, scr);
    if (lead && e < E) col_offs[e] = carry + ex;
    carry += total;
    __syncthreads();
  }
  if (lead && threadIdx.x == 0) *n_valid = carry;
  ragged_scan_rows(csum, E, tab, lead ? offs : nullptr, offs_pitch);
  __syncthreads();
  const int64_t total_e = 5 * (int64_t)max_blocks;
  const int64_t per = (total_e + gridDim.x - 1) / gridDim.x;
  const int64_t first = per * blockIdx.x;
  if (first < total_e)
    ragged_fill_schedule(tab, E, sched, sched_pitch, max_blocks, first, per < total_e - first ? per : total_e - first);
}

// ---------------------------------------------------------------------------
// metadata in two launches (up to kMaxTableBlocks blocks of chunks)
// ---------------------------------------------------------------------------
// The first launch leaves one histogram per block of CH chunks (hist_kernel, or topk_hist_kernel straight from the
// logits).  In the second, every workgroup reduces that small table by itself -- the experts' totals, their prefix and,
// for the workgroup that orders block `blk`, the counts of the blocks before it -- instead of waiting for a scan kernel
// in between: workgroups 0..nb-1 recount their own chunks and place their entries, the remaining ones build the ragged
// tables and fill the block schedule.
constexpr int kMaxTableBlocks = 128;

// Sums of tot[b][e] over the blocks b of [b_lo, b_hi): all of them, and those before block `blk`.  Sixteen loads are
// in flight together.
TAMD_DEVICE void sum_block_range(const int32_t *__restrict__ tot, int E, int e, int b_lo, int b_hi, int blk, int &all,
                                 int &below) {
  all = 0;
  below = 0;
  for (int b0 = b_lo; b0 < b_hi; b0 += 16) {
    int t[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) t[u] = tot[(int64_t)(b0 + u < b_hi ? b0 + u : b_hi - 1) * E + e];
#pragma unroll
    for (int u = 0; u < 16; ++u) asm volatile("" : "+v"(t[u]));
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      all += b0 + u < b_hi ? t[u] : 0;
      below += b0 + u < b_hi && b0 + u < blk ? t[u] : 0;
    }
  }
}

__global__ __launch_bounds__(1024) void order_scan_kernel(const void *__restrict__ indx, int is16, int n, int E, int CH,
                                                          int nbits, int k, const int32_t *__restrict__ block_tot, int nb,
                                                          int P, int32_t *__restrict__ col_sum,
                                                          int32_t *__restrict__ col_sorted, int32_t *__restrict__ row_sorted,
                                                          int32_t *__restrict__ gather, int32_t *__restrict__ offs,
                                                          int64_t offs_pitch, int32_t *__restrict__ sched,
                                                          int64_t sched_pitch, int max_blocks) {
  extern __shared__ int32_t sm[];
  int32_t *hist = sm;                          // [CH][E]  counts of this block's chunks, then their exclusive prefix
  int32_t *tot = hist + (int64_t)CH * E;       // [E]      entries per expert
  int32_t *boff = tot + E;                     // [E]      entries per expert in the blocks before this one
  int32_t *psum = boff + E;                    // [P][E]   partial sums over ranges of blocks
  int32_t *pbel = psum + (int64_t)P * E;       // [P][E]
  int32_t *tab = pbel + (int64_t)P * E;        // [6][E + 1]
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int blk = blockIdx.x;
  const bool orders = blk < nb;
  // this wave's chunk of the index array: requested first, used after the table has been reduced
  const int i = (blk * CH + wave) * 64 + lane;
  const bool has = orders && wave < CH && i < n;
  int ev = 0;
  if (n > 0) ev = load_indx(indx, is16, has ? i : 0);
  if (orders)
    for (int j = tid; j < CH * E; j += 1024) hist[j] = 0;
  // 1. partial sums of the table: thread (part, e) takes the blocks [part * per, (part + 1) * per)
  {
    const int part = tid / E, e = tid - part * E;
    if (part < P) {
      const int per = (nb + P - 1) / P;
      const int b_hi = (part + 1) * per < nb ? (part + 1) * per : nb;
      int all, below;
      sum_block_range(block_tot, E, e, part * per, b_hi, blk, all, below);
      psum[part * E + e] = all;
      pbel[part * E + e] = below;
    }
  }
  asm volatile("" : "+v"(ev));
  ev = has ? ev : -1;
  __syncthreads();
  // 2. totals per expert; counts of this wave's chunk
  for (int e = tid; e < E; e += 1024) {
    int all = 0, below = 0;
    for (int q = 0; q < P; ++q) {
      all += psum[q * E + e];
      below += pbel[q * E + e];
    }
    tot[e] = all;
    boff[e] = below;
    if (blk == 0) col_sum[e] = all;
  }
  const bool valid = ev >= 0 && ev < E;
  const uint64_t same = same_id_mask(ev, valid, nbits);
  if (valid && (same & lanemask_lt()) == 0) hist[wave * E + ev] = __popcll(same);
  __syncthreads();
  // 3. exclusive prefix over this block's chunks; the ragged tables (row 0: exclusive prefix over the experts)
  if (orders) {
    for (int e = tid; e < E; e += 1024) {
      int run = 0;
      for (int c = 0; c < CH; ++c) {
        const int v = hist[c * E + e];
        hist[c * E + e] = run;
        run += v;
      }
    }
  }
  ragged_scan_rows(tot, E, tab, blk == nb ? offs : nullptr, offs_pitch);
  __syncthreads();
  if (orders) {
    // 4. placement
    const int nv = tab[E];
    if (valid) {
      const int pos = tab[ev] + boff[ev] + hist[wave * E + ev] + __popcll(same & lanemask_lt());
      row_sorted[i] = pos;
      col_sorted[pos] = i;
      if (gather) gather[pos] = i / k;
    } else if (wave < CH && i < n) {
      row_sorted[i] = -1;
    }
    if (wave < CH && i >= nv && i < n) {
      col_sorted[i] = -1;
      if (gather) gather[i] = 0;  // trunc(-1 / k)
    }
  } else {
    // 4'. this workgroup's share of the block schedule
    const int64_t total = 5 * (int64_t)max_blocks;
    const int64_t shares = (int64_t)gridDim.x - nb;
    const int64_t per = (total + shares - 1) / shares;
    const int64_t first = per * (blk - nb);
    if (first < total) ragged_fill_schedule(tab, E, sched, sched_pitch, max_blocks, first, per < total - first ? per : total - first);
  }
}

// Second launch of the two: the grid, the LDS size and the limits of order_scan_kernel.
inline bool order_scan_applicable(int64_t n, int E, int CH, int64_t nb) {
  if (E > 1024 || nb < 1 || nb > kMaxTableBlocks || n > 0x7FFFFFFF - 64 * 1024) return false;
  int P = 1024 / E;
  P = P > 16 ? 16 : P;
  const int64_t ints = (int64_t)CH * E + 2 * (int64_t)E + 2 * (int64_t)P * E + 6 * ((int64_t)E + 1);
  return ints * 4 <= 150 * 1024;
}

inline int launch_order_scan(const void *indx, int is16, int64_t n, int E, int CH, int nbits, int k, const int32_t *block_tot,
                             int64_t nb, int32_t *col_sum, int32_t *col_sorted, int32_t *row_sorted, int32_t *gather,
                             int32_t *offs, int64_t offs_pitch, int32_t *sched, int64_t sched_pitch, int max_blocks,
                             hipStream_t st) {
  int P = 1024 / E;
  P = P > 16 ? 16 : P;
  P = P > nb ? (int)nb : P;
  const int64_t ints = (int64_t)CH * E + 2 * (int64_t)E + 2 * (int64_t)P * E + 6 * ((int64_t)E + 1);
  int64_t shares = (5 * (int64_t)max_blocks + 4095) / 4096;  // about four schedule entries per thread
  shares = shares < 1 ? 1 : (shares > 64 ? 64 : shares);
  if (int rc = raise_lds_limit_once((const void *)order_scan_kernel)) return rc;
  order_scan_kernel<<<dim3((unsigned)(nb + shares)), 1024, (size_t)ints * 4, st>>>(
      indx, is16, (int)n, E, CH, nbits, k, block_tot, (int)nb, P, col_sum, col_sorted, row_sorted, gather, offs, offs_pitch,
      sched, sched_pitch, max_blocks);
  return launch_status();
}

// First launch of the two, from the logits: the experts of 1024 / L rows per workgroup (their picked columns also go to
// LDS) and the histogram of that block of (1024 / L) * k / 64 whole chunks.
template <int DT, int L, int EPL>
__global__ __launch_bounds__(1024) void topk_hist_kernel(const void *__restrict__ x, int64_t x_stride, int n_rows, int E,
                                                         int k, void *__restrict__ y_vals, int16_t *__restrict__ y_indx,
                                                         uint32_t *__restrict__ bits, int64_t bits_stride_row,
                                                         int64_t bits_stride_word, int nbits, int CH,
                                                         int32_t *__restrict__ block_tot) {
  extern __shared__ int32_t sm[];
  constexpr int ROWS = 1024 / L;
  int32_t *lidx = sm;            // [CH * 64] picked columns of this block's rows
  int32_t *hist = sm + CH * 64;  // [CH][E]
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int64_t row0 = (int64_t)blockIdx.x * ROWS;
  for (int j = tid; j < CH * E; j += 1024) hist[j] = 0;  // (the barrier below covers them)
  topk_row<DT, L, EPL>(x, x_stride, n_rows, E, k, 1, 0, y_vals, y_indx, k, bits, bits_stride_row, bits_stride_word,
                       row0 + tid / L, lidx - row0 * k);
  __syncthreads();
  if (wave < CH) {
    const int j = wave * 64 + lane;  // entry of the block; its row exists or not
    const bool valid = row0 + j / k < n_rows;
    const int e = valid ? lidx[j] : -1;
    const uint64_t same = same_id_mask(e, valid, nbits);
    if (valid && (same & lanemask_lt()) == 0) hist[wave * E + e] = __popcll(same);
  }
  __syncthreads();
  for (int e = tid; e < E; e += 1024) {
    int run = 0;
    for (int c = 0; c < CH; ++c) run += hist[c * E + e];
    block_tot[(int64_t)blockIdx.x * E + e] = run;
  }
}

template <int DT>
int launch_topk_hist(const void *x, int64_t xs, int n_rows, int E, int k, void *yv, int16_t *yi, uint32_t *bits, int64_t bsr,
                     int64_t bsw, int nbits, int L, int CH, int32_t *block_tot, hipStream_t st) {
  const size_t lds = ((size_t)CH * 64 + (size_t)CH * E) * 4;
  const unsigned grid = (unsigned)((n_rows + 1024 / L - 1) / (1024 / L));
#define TAMD_TH(LL, EE) \
  topk_hist_kernel<DT, LL, EE><<<grid, 1024, lds, st>>>(x, xs, n_rows, E, k, yv, yi, bits, bsr, bsw, nbits, CH, block_tot)
  if (L == 8) TAMD_TH(8, 8);
  else if (L == 16) TAMD_TH(16, 8);
  else if (L == 32) TAMD_TH(32, 8);
  else TAMD_TH(64, 8);
#undef TAMD_TH
  return launch_status();
}

// ---------------------------------------------------------------------------
// all routing metadata in one workgroup
// ---------------------------------------------------------------------------
// For index arrays small enough that the per-chunk histogram fits LDS (n/64 * E ints): histogram,
// the three prefix sums, the ordering and the ragged tables without leaving the workgroup --
// one launch instead of four, which is what the cost of routing is made of at these sizes.
// lidx: the index array in LDS (a kernel that has just computed it), or null to read `indx` from memory.
TAMD_DEVICE void meta_fused_body(int32_t *sm, bool zeroed, const int32_t *lidx, const void *__restrict__ indx, int is16,
                                 int n, int E, int k, int nbits, int NC, int P, int32_t *__restrict__ col_sum,
                                 int32_t *__restrict__ col_sorted, int32_t *__restrict__ row_sorted,
                                 int32_t *__restrict__ gather, int32_t *__restrict__ offs, int64_t offs_pitch,
                                 int32_t *__restrict__ sched, int64_t sched_pitch, int max_blocks) {
  int32_t *hist = sm;                         // [NC][E]  counts, then exclusive prefix over chunks
  int32_t *csum = hist + (int64_t)NC * E;     // [E]
  int32_t *psum = csum + E;                   // [P][E]   partial sums of chunk ranges
  int32_t *tab = psum + (int64_t)P * E;       // [6][E + 1]
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  if (!zeroed) {
    for (int i = tid; i < NC * E; i += 1024) hist[i] = 0;
    __syncthreads();
  }
  // 1. per-chunk histogram.  A wave takes its chunks eight at a time so that eight index loads are in
  // flight together (one workgroup has nothing else to hide their latency with).
  for (int c0 = wave; c0 < NC && n > 0; c0 += 16 * 8) {
    int ev[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {  // unconditional loads (entries past the end re-read entry 0), so all eight are in flight
      const int i = (c0 + 16 * u) * 64 + lane;
      const bool ok = c0 + 16 * u < NC && i < n;
      ev[u] = lidx ? lidx[ok ? i : 0] : load_indx(indx, is16, ok ? i : 0);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) asm volatile("" : "+v"(ev[u]));  // pinned: the loads stay outside the selection below
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = (c0 + 16 * u) * 64 + lane;
      ev[u] = (c0 + 16 * u < NC && i < n) ? ev[u] : -1;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = c0 + 16 * u;
      if (c >= NC) break;
      const int e = ev[u];
      const bool valid = e >= 0 && e < E;
      const uint64_t same = same_id_mask(e, valid, nbits);
      if (valid && (same & lanemask_lt()) == 0) hist[c * E + e] = __popcll(same);
    }
  }
  __syncthreads();
  // 2. exclusive prefix over chunks for every expert: a few chunks in one go, else P chunk ranges per expert in two passes
  const int per = (NC + P - 1) / P;
  if (NC <= 8) {
    for (int e = tid; e < E; e += 1024) {
      int run = 0;
      for (int c = 0; c < NC; ++c) {
        const int v = hist[c * E + e];
        hist[c * E + e] = run;
        run += v;
      }
      csum[e] = run;
      col_sum[e] = run;
    }
  } else {
  for (int t = tid; t < P * E; t += 1024) {
    const int part = t / E, e = t - part * E;
    int run = 0;
    for (int c = part * per; c < NC && c < (part + 1) * per; ++c) run += hist[c * E + e];
    psum[part * E + e] = run;
  }
  __syncthreads();
  for (int t = tid; t < P * E; t += 1024) {
    const int part = t / E, e = t - part * E;
    int run = 0;
    for (int q = 0; q < part; ++q) run += psum[q * E + e];
    for (int c = part * per; c < NC && c < (part + 1) * per; ++c) {
      const int v = hist[c * E + e];
      hist[c * E + e] = run;
      run += v;
    }
    if (part == P - 1) {
      csum[e] = run;
      col_sum[e] = run;
    }
  }
  }
  __syncthreads();
  // 3. ragged tables of the histogram; the first one is the exclusive prefix over experts that places the entries
  ragged_scan_rows(csum, E, tab, offs, offs_pitch);
  __syncthreads();
  const int32_t *coff = tab;
  const int nv = tab[E];
  // 4. placement
  for (int c0 = wave; c0 < NC && n > 0; c0 += 16 * 8) {
    int ev[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {  // unconditional loads (entries past the end re-read entry 0), so all eight are in flight
      const int i = (c0 + 16 * u) * 64 + lane;
      const bool ok = c0 + 16 * u < NC && i < n;
      ev[u] = lidx ? lidx[ok ? i : 0] : load_indx(indx, is16, ok ? i : 0);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) asm volatile("" : "+v"(ev[u]));  // pinned: the loads stay outside the selection below
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = (c0 + 16 * u) * 64 + lane;
      ev[u] = (c0 + 16 * u < NC && i < n) ? ev[u] : -1;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = c0 + 16 * u;
      if (c >= NC) break;
      const int i = c * 64 + lane;
      const int e = ev[u];
      const bool valid = e >= 0 && e < E;
      const uint64_t same = same_id_mask(e, valid, nbits);
      if (valid) {
        const int pos = coff[e] + hist[c * E + e] + __popcll(same & lanemask_lt());
        row_sorted[i] = pos;
        col_sorted[pos] = i;
        if (gather) gather[pos] = i / k;
      } else if (i < n) {
        row_sorted[i] = -1;
      }
      if (i >= nv && i < n) {
        col_sorted[i] = -1;
        if (gather) gather[i] = 0;  // trunc(-1 / k)
      }
    }
  }
  // 5. block schedule (reads the tables only: no barrier after the placement)
  ragged_fill_schedule(tab, E, sched, sched_pitch, max_blocks, 0, 5 * (int64_t)max_blocks);
}

__global__ __launch_bounds__(1024) void meta_fused_kernel(const void *__restrict__ indx, int is16, int n, int E, int k,
                                                          int nbits, int NC, int P, int32_t *__restrict__ col_sum,
                                                          int32_t *__restrict__ col_sorted, int32_t *__restrict__ row_sorted,
                                                          int32_t *__restrict__ gather, int32_t *__restrict__ offs,
                                                          int64_t offs_pitch, int32_t *__restrict__ sched,
                                                          int64_t sched_pitch, int max_blocks) {
  extern __shared__ int32_t sm[];
  meta_fused_body(sm, false, nullptr, indx, is16, n, E, k, nbits, NC, P, col_sum, col_sorted, row_sorted, gather, offs,
                  offs_pitch, sched, sched_pitch, max_blocks);
}

// ---------------------------------------------------------------------------
// top-k and all routing metadata in one workgroup (decode sizes)
// ---------------------------------------------------------------------------
// With a few dozen tokens the two launches of routing cost more than their work.  Here the 1024 threads first pick
// the experts of 1024 / L rows at a time (the picked columns also go to LDS), then run the metadata phases of
// meta_fused_kernel on the index array in LDS.
template <int DT, int L, int EPL>
__global__ __launch_bounds__(1024) void routing_fused_kernel(const void *__restrict__ x, int64_t x_stride, int n_rows,
                                                             int E, int k, void *__restrict__ y_vals,
                                                             int16_t *__restrict__ y_indx, uint32_t *__restrict__ bits,
                                                             int64_t bits_stride_row, int64_t bits_stride_word, int nbits,
                                                             int NC, int P, int32_t *__restrict__ col_sum,
                                                             int32_t *__restrict__ col_sorted,
                                                             int32_t *__restrict__ row_sorted, int32_t *__restrict__ gather,
                                                             int32_t *__restrict__ offs, int64_t offs_pitch,
                                                             int32_t *__restrict__ sched, int64_t sched_pitch,
                                                             int max_blocks) {
  extern __shared__ int32_t sm[];
  const int n = n_rows * k;
  int32_t *lidx = sm;                        // [n] picked columns
  int32_t *meta = sm + (n + 3) / 4 * 4;
  constexpr int ROWS = 1024 / L;
  for (int i = threadIdx.x; i < NC * E; i += 1024) meta[i] = 0;  // the histograms (the barrier below covers them)
  for (int row0 = 0; row0 < n_rows; row0 += ROWS)
    topk_row<DT, L, EPL>(x, x_stride, n_rows, E, k, 1, 0, y_vals, y_indx, k, bits, bits_stride_row, bits_stride_word,
                         (int64_t)row0 + threadIdx.x / L, lidx);
  __syncthreads();
  meta_fused_body(meta, true, lidx, nullptr, 0, n, E, k, nbits, NC, P, col_sum, col_sorted, row_sorted, gather, offs,
                  offs_pitch, sched, sched_pitch, max_blocks);
}

template <int DT>
int launch_routing_fused(const void *x, int64_t xs, int n_rows, int E, int k, void *yv, int16_t *yi, uint32_t *bits,
                         int64_t bsr, int64_t bsw, int nbits, int NC, int P, size_t lds, int32_t *col_sum,
                         int32_t *col_sorted, int32_t *row_sorted, int32_t *gather, int32_t *offs, int64_t offs_pitch,
                         int32_t *sched, int64_t sched_pitch, int max_blocks, hipStream_t st) {
  int need = (E + 7) / 8;
  if (need < k) need = k;
#define TAMD_RF(LL, EE)                                                                                              \
  do {                                                                                                               \
    auto kern = routing_fused_kernel<DT, LL, EE>;                                                                    \
    if (int rc = raise_lds_limit_once((const void *)kern)) return rc;                                                \
    kern<<<1, 1024, lds, st>>>(x, xs, n_rows, E, k, yv, yi, bits, bsr, bsw, nbits, NC, P, col_sum, col_sorted,        \
                               row_sorted, gather, offs, offs_pitch, sched, sched_pitch, max_blocks);                \
  } while (0)
  if (need <= 8) TAMD_RF(8, 8);
  else if (need <= 16) TAMD_RF(16, 8);
  else if (need <= 32) TAMD_RF(32, 8);
  else TAMD_RF(64, 8);
#undef TAMD_RF
  return launch_status();
}

}  // namespace tamd

using namespace tamd;

extern "C" int tamd_topk_forward(const void *x, int x_dtype, int64_t x_stride, int n_rows, int n_cols, int k,
                                 int apply_softmax, int use_provided_indx, void *y_vals, int16_t *y_indx,
                                 int64_t y_stride, uint32_t *bits, int64_t bits_stride_row,
                                 int64_t bits_stride_word, void *stream) {
  if (n_rows < 0 || n_cols <= 0 || n_cols >= 32768 || k < 1 || k > 64 || k > n_cols) return TAMD_E_INVALID;
  if (n_rows == 0) return 0;
  if (!x || !y_vals || !y_indx || !bits) return TAMD_E_INVALID;
  hipStream_t st = (hipStream_t)stream;
  switch (x_dtype) {
    case TAMD_F32:
      return launch_topk<TAMD_F32>(x, x_stride, n_rows, n_cols, k, apply_softmax, use_provided_indx, y_vals, y_indx,
                                   y_stride, bits, bits_stride_row, bits_stride_word, st);
    case TAMD_BF16:
      return launch_topk<TAMD_BF16>(x, x_stride, n_rows, n_cols, k, apply_softmax, use_provided_indx, y_vals, y_indx,
                                    y_stride, bits, bits_stride_row, bits_stride_word, st);
    case TAMD_F16:
      return launch_topk<TAMD_F16>(x, x_stride, n_rows, n_cols, k, apply_softmax, use_provided_indx, y_vals, y_indx,
                                   y_stride, bits, bits_stride_row, bits_stride_word, st);
    default:
      return TAMD_E_INVALID;
  }
}

extern "C" int64_t tamd_bitmatrix_metadata_workspace(int64_t n_indx, int n_cols) {
  if (n_indx < 0 || n_cols <= 0) return 0;
  return make_meta_plan(n_indx, n_cols).total;
}

extern "C" int tamd_bitmatrix_metadata(const void *indx, int indx_is_int16, int64_t n_indx, int n_cols,
                                       int32_t *col_sum, int32_t *col_sorted_indx, int32_t *row_sorted_indx,
                                       int32_t *workspace, void *stream) {
  if (n_indx < 0 || n_cols <= 0 || n_cols > 16384 || n_indx > 0x7FFFFFFF) return TAMD_E_INVALID;
  if (!col_sum || !workspace || (n_indx > 0 && (!indx || !col_sorted_indx || !row_sorted_indx))) return TAMD_E_INVALID;
  return launch_bitmatrix_metadata(indx, indx_is_int16, n_indx, n_cols, 1, col_sum, col_sorted_indx, row_sorted_indx,
                                   nullptr, workspace, (hipStream_t)stream, nullptr, nullptr);
}

static int ragged_launch(const int32_t *slice_sizes, int n_slices, int32_t *offs, int64_t offs_pitch,
                         int32_t *schedule, int64_t sched_pitch, int max_n_blocks, hipStream_t st) {
  const size_t lds = 6 * (size_t)(n_slices + 1) * 4;
  if (lds > 150 * 1024) return TAMD_E_UNSUPPORTED;  // more than ~6000 slices
  if (int rc = raise_lds_limit_once((const void *)ragged_kernel)) return rc;
  int64_t wgs = (5 * (int64_t)max_n_blocks + 4095) / 4096;  // about four entries per thread
  wgs = wgs < 1 ? 1 : (wgs > 256 ? 256 : wgs);
  ragged_kernel<<<dim3((unsigned)wgs), 1024, lds, st>>>(slice_sizes, n_slices, offs, offs_pitch, schedule, sched_pitch,
                                                      max_n_blocks);
  return launch_status();
}

extern "C" int tamd_ragged_metadata(const int32_t *slice_sizes, int n_slices, int32_t *offs, int64_t offs_pitch,
                                    int32_t *schedule, int64_t sched_pitch, int max_n_blocks, void *stream) {
  if (n_slices < 0 || n_slices > 65535 || max_n_blocks < 0 || offs_pitch < n_slices + 1 ||
      sched_pitch < max_n_blocks)
    return TAMD_E_INVALID;
  if (!offs || (n_slices > 0 && !slice_sizes) || (max_n_blocks > 0 && !schedule)) return TAMD_E_INVALID;
  return ragged_launch(slice_sizes, n_slices, offs, offs_pitch, schedule, sched_pitch, max_n_blocks,
                       (hipStream_t)stream);
}

namespace {
struct RaggedCtx {
  const int32_t *sizes;
  int n_slices;
  int32_t *offs;
  int64_t offs_pitch;
  int32_t *sched;
  int64_t sched_pitch;
  int max_blocks;
  hipStream_t st;
};
bool ragged_between(void *p) {
  RaggedCtx *c = (RaggedCtx *)p;
  return ragged_launch(c->sizes, c->n_slices, c->offs, c->offs_pitch, c->sched, c->sched_pitch, c->max_blocks,
                       c->st) == 0;
}
}  // namespace

static int routing_metadata_impl(const void *indx, int indx_is_int16, int64_t n_indx, int n_cols, int k,
                                 int32_t *col_sum, int32_t *col_sorted_indx, int32_t *row_sorted_indx,
                                 int32_t *gather_indx, int32_t *offs, int64_t offs_pitch, int32_t *schedule,
                                 int64_t sched_pitch, int max_n_blocks, int32_t *workspace, void *stream) {
  if (n_indx < 0 || n_cols <= 0 || n_cols > 16384 || n_indx > 0x7FFFFFFF || k < 1) return TAMD_E_INVALID;
  if (max_n_blocks < 0 || offs_pitch < n_cols + 1 || sched_pitch < max_n_blocks) return TAMD_E_INVALID;
  if (!col_sum || !workspace || !offs || (max_n_blocks > 0 && !schedule)) return TAMD_E_INVALID;
  if (n_indx > 0 && (!indx || !col_sorted_indx || !row_sorted_indx)) return TAMD_E_INVALID;
  {
    // one workgroup does it all when the per-chunk histogram fits its LDS
    const int64_t NC = (n_indx + 63) / 64 > 0 ? (n_indx + 63) / 64 : 1;
    int64_t P = 1024 / n_cols;
    P = P < 1 ? 1 : (P > NC ? NC : P);
    const int64_t ints = NC * n_cols + (int64_t)n_cols + P * n_cols + 6 * (int64_t)(n_cols + 1);
    if (NC <= 64 && ints * 4 <= 156 * 1024) {  // beyond ~4096 entries one CU is slower than three launches
      int nbits = 0;
      while ((1 << nbits) < n_cols) ++nbits;
      if (int rc = raise_lds_limit_once((const void *)meta_fused_kernel)) return rc;
      meta_fused_kernel<<<1, 1024, (size_t)ints * 4, (hipStream_t)stream>>>(
          indx, indx_is_int16, (int)n_indx, n_cols, k, nbits, (int)NC, (int)P, col_sum, col_sorted_indx, row_sorted_indx,
          gather_indx, offs, offs_pitch, schedule, sched_pitch, max_n_blocks);
      return launch_status();
    }
  }
  {
    // two launches while the table of block histograms is small enough for every workgroup to reduce by itself
    const MetaPlan p = make_meta_plan(n_indx, n_cols);
    if (order_scan_applicable(n_indx, n_cols, p.CH, p.n_blocks)) {
      hipStream_t st = (hipStream_t)stream;
      hist_kernel<<<dim3((unsigned)p.n_blocks), 1024, (size_t)p.CH * n_cols * 4, st>>>(
          indx, indx_is_int16, n_indx, n_cols, p.CH, p.nbits, nullptr, workspace + p.off_block_tot);
      return launch_order_scan(indx, indx_is_int16, n_indx, n_cols, p.CH, p.nbits, k, workspace + p.off_block_tot, p.n_blocks,
                               col_sum, col_sorted_indx, row_sorted_indx, gather_indx, offs, offs_pitch, schedule, sched_pitch,
                               max_n_blocks, st);
    }
  }
  const size_t sr_lds = ((size_t)n_cols + 6 * ((size_t)n_cols + 1) + 17) * 4;
  if (sr_lds <= 150 * 1024) {
    // three launches: histograms per workgroup, scans + ragged tables, placement
    hipStream_t st = (hipStream_t)stream;
    MetaPlan p = make_meta_plan(n_indx, n_cols);
    hist_kernel<<<dim3((unsigned)p.n_blocks), 1024, (size_t)p.CH * n_cols * 4, st>>>(
        indx, indx_is_int16, n_indx, n_cols, p.CH, p.nbits, workspace + p.off_chunk_pref, workspace + p.off_block_tot);
    if (int rc = raise_lds_limit_once((const void *)scan_ragged_kernel)) return rc;
    int64_t wgs = (5 * (int64_t)max_n_blocks + 4095) / 4096;
    wgs = wgs < 1 ? 1 : (wgs > 64 ? 64 : wgs);
    scan_ragged_kernel<<<dim3((unsigned)wgs), 1024, sr_lds, st>>>(
        n_cols, (int)p.n_blocks, workspace + p.off_block_tot, workspace + p.off_block_off, col_sum,
        workspace + p.off_col_offs, workspace + p.off_n_valid, offs, offs_pitch, schedule, sched_pitch, max_n_blocks);
    order_kernel<<<dim3((unsigned)p.n_blocks), 1024, 0, st>>>(
        indx, indx_is_int16, n_indx, n_cols, p.CH, p.nbits, k, workspace + p.off_chunk_pref, workspace + p.off_block_off,
        workspace + p.off_col_offs, workspace + p.off_n_valid, col_sorted_indx, row_sorted_indx, gather_indx);
    return launch_status();
  }
  RaggedCtx ctx{col_sum, n_cols, offs, offs_pitch, schedule, sched_pitch, max_n_blocks, (hipStream_t)stream};
  return launch_bitmatrix_metadata(indx, indx_is_int16, n_indx, n_cols, k, col_sum, col_sorted_indx,
                                   row_sorted_indx, gather_indx, workspace, (hipStream_t)stream, ragged_between, &ctx);
}

extern "C" int tamd_routing_metadata(const void *indx, int indx_is_int16, int64_t n_indx, int n_cols, int k,
                                     int32_t *col_sum, int32_t *col_sorted_indx, int32_t *row_sorted_indx,
                                     int32_t *gather_indx, int32_t *offs, int64_t offs_pitch, int32_t *schedule,
                                     int64_t sched_pitch, int max_n_blocks, int32_t *workspace, void *stream) {
  return routing_metadata_impl(indx, indx_is_int16, n_indx, n_cols, k, col_sum, col_sorted_indx, row_sorted_indx,
                               gather_indx, offs, offs_pitch, schedule, sched_pitch, max_n_blocks, workspace, stream);
}

extern "C" int tamd_routing(const void *logits, int dtype, int64_t stride, int n_rows, int n_cols, int k, void *y_vals,
                            int16_t *y_indx, uint32_t *bits, int64_t bits_stride_row, int64_t bits_stride_word,
                            int32_t *col_sum, int32_t *col_sorted_indx, int32_t *row_sorted_indx, int32_t *gather_indx,
                            int32_t *offs, int64_t offs_pitch, int32_t *schedule, int64_t sched_pitch, int max_n_blocks,
                            int32_t *workspace, void *stream) {
  // a few rows (at most two passes of the workgroup's 1024 threads over them), at most 512 columns, and the
  // metadata workspace of one workgroup fits LDS: one launch for everything
  if (n_rows > 0 && n_cols > 0 && n_cols <= 512 && k >= 1 && k <= 64 && k <= n_cols && logits && y_vals && y_indx && bits &&
      (dtype == TAMD_F32 || dtype == TAMD_BF16 || dtype == TAMD_F16) && col_sum && offs && col_sorted_indx &&
      row_sorted_indx && max_n_blocks >= 0 && offs_pitch >= n_cols + 1 && sched_pitch >= max_n_blocks &&
      (max_n_blocks == 0 || schedule)) {
    int need = (n_cols + 7) / 8;
    if (need < k) need = k;
    const int L = need <= 8 ? 8 : (need <= 16 ? 16 : (need <= 32 ? 32 : 64));
    const int64_t n = (int64_t)n_rows * k;
    const int64_t NC = (n + 63) / 64;
    int64_t P = 1024 / n_cols;
    P = P < 1 ? 1 : (P > NC ? NC : P);
    const int64_t ints = (n + 3) / 4 * 4 + NC * n_cols + (int64_t)n_cols + P * n_cols + 6 * (int64_t)(n_cols + 1);
    if (n_rows <= 2 * (1024 / L) && NC <= 64 && ints * 4 <= 156 * 1024) {
      int nbits = 0;
      while ((1 << nbits) < n_cols) ++nbits;
      hipStream_t st = (hipStream_t)stream;
#define TAMD_RFD(DT)                                                                                                  \
  return launch_routing_fused<DT>(logits, stride, n_rows, n_cols, k, y_vals, y_indx, bits, bits_stride_row,            \
                                  bits_stride_word, nbits, (int)NC, (int)P, (size_t)ints * 4, col_sum, col_sorted_indx,  \
                                  row_sorted_indx, gather_indx, offs, offs_pitch, schedule, sched_pitch, max_n_blocks, st)
      if (dtype == TAMD_F32) TAMD_RFD(TAMD_F32);
      if (dtype == TAMD_BF16) TAMD_RFD(TAMD_BF16);
      TAMD_RFD(TAMD_F16);
#undef TAMD_RFD
    }
    // two launches: top-k with the histogram of each workgroup's rows, then ordering and tables.  The rows of a
    // workgroup (1024 / L) must make whole chunks of 64 entries.
    const int CH = 16 * k / L;
    const int64_t nb = ((int64_t)n_rows + 1024 / L - 1) / (1024 / L);
    if ((16 * k) % L == 0 && CH >= 1 && CH <= 16 && workspace && order_scan_applicable(n, n_cols, CH, nb) &&
        nb * n_cols <= tamd_bitmatrix_metadata_workspace(n, n_cols)) {
      int nbits = 0;
      while ((1 << nbits) < n_cols) ++nbits;
      hipStream_t st = (hipStream_t)stream;
      int rc;
      if (dtype == TAMD_F32)
        rc = launch_topk_hist<TAMD_F32>(logits, stride, n_rows, n_cols, k, y_vals, y_indx, bits, bits_stride_row,
                                        bits_stride_word, nbits, L, CH, workspace, st);
      else if (dtype == TAMD_BF16)
        rc = launch_topk_hist<TAMD_BF16>(logits, stride, n_rows, n_cols, k, y_vals, y_indx, bits, bits_stride_row,
                                         bits_stride_word, nbits, L, CH, workspace, st);
      else
        rc = launch_topk_hist<TAMD_F16>(logits, stride, n_rows, n_cols, k, y_vals, y_indx, bits, bits_stride_row,
                                        bits_stride_word, nbits, L, CH, workspace, st);
      if (rc != 0) return rc;
      return launch_order_scan(y_indx, 1, n, n_cols, CH, nbits, k, workspace, nb, col_sum, col_sorted_indx, row_sorted_indx,
                               gather_indx, offs, offs_pitch, schedule, sched_pitch, max_n_blocks, st);
    }
  }
  const int rc = tamd_topk_forward(logits, dtype, stride, n_rows, n_cols, k, 1, 0, y_vals, y_indx, k, bits, bits_stride_row,
                                   bits_stride_word, stream);
  if (rc != 0) return rc;
  return routing_metadata_impl(y_indx, 1, (int64_t)n_rows * k, n_cols, k, col_sum, col_sorted_indx, row_sorted_indx,
                               gather_indx, offs, offs_pitch, schedule, sched_pitch, max_n_blocks, workspace, stream);
}

// Device address of `scratch` on the current device.  In host code the array's name only stands for the symbol: its
// memory is reached through the address the runtime reports, which differs from GPU to GPU and is looked up once
// per device (with that device current) and kept.
static int static_workspace(int32_t **out) {
  constexpr int kMaxDevices = 64;
  static std::atomic<int32_t *> ptr_of_device[kMaxDevices];
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return TAMD_E_UNSUPPORTED;
  int32_t *p = ptr_of_device[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return TAMD_E_INVALID;
    ptr_of_device[dev].store(p, std::memory_order_release);  // two racing first calls store the same address
  }
  *out = p;
  return 0;
}

extern "C" int64_t tamd_routing_metadata_static_max_workspace(void) { return kStaticWorkspaceInts; }

// Everything tamd_routing_metadata_static does once per device on the host side -- the address of the static array
// and the raised LDS limits of the kernels the metadata path launches -- so that callers under graph capture can have
// it done beforehand.  (tamd_routing_metadata_static does the same by itself on a device's first call.)
extern "C" int tamd_routing_metadata_static_init(void) {
  int32_t *ws = nullptr;
  if (int rc = static_workspace(&ws)) return rc;
  if (int rc = raise_lds_limit_once((const void *)meta_fused_kernel)) return rc;
  if (int rc = raise_lds_limit_once((const void *)order_scan_kernel)) return rc;
  if (int rc = raise_lds_limit_once((const void *)scan_ragged_kernel)) return rc;
  return 0;
}

extern "C" int tamd_routing_metadata_static(const void *indx, int indx_is_int16, int64_t n_indx, int n_cols, int k,
                                            int32_t *col_sum, int32_t *col_sorted_indx, int32_t *row_sorted_indx,
                                            int32_t *gather_indx, int32_t *offs, int64_t offs_pitch,
                                            int32_t *schedule, int64_t sched_pitch, int max_n_blocks, void *stream) {
  if (n_indx < 0 || n_cols <= 0) return TAMD_E_INVALID;
  if (make_meta_plan(n_indx, n_cols).total > kStaticWorkspaceInts) return TAMD_E_TOO_LARGE;
  int32_t *ws = nullptr;
  const int rc = static_workspace(&ws);
  if (rc != 0) return rc;
  // every entry of the workspace that a launch reads is written earlier by the same call (per-chunk prefixes and
  // per-workgroup totals by the histogram kernel, the prefix tables by the scan kernel): nothing has to start at zero
  return routing_metadata_impl(indx, indx_is_int16, n_indx, n_cols, k, col_sum, col_sorted_indx, row_sorted_indx,
                               gather_indx, offs, offs_pitch, schedule, sched_pitch, max_n_blocks, ws, stream);
}

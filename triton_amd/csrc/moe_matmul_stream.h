// Weight-streaming grouped matmul for row blocks of at most 16 rows (decode): 16-bit activations x
// MXFP4 weights.  Same arithmetic as the tiled kernel of moe_matmul_impl.h; the design goal here is
// HBM bandwidth, since with a handful of rows per expert every weight byte is used exactly once.
//
// Measured on this part: reading 128 bytes of every column per K step (columns 1440 bytes apart)
// tops out near 3.4 TB/s, a linear read reaches 6.2 TB/s.  So the kernel reads the weights in
// memory order:
//   * a unit of work is (row block, group of 16 consecutive columns).  With K contiguous per column
//     the 16 columns are one contiguous run of 16*K/2 bytes (plus 16*K/32 scale bytes);
//   * one workgroup per CU walks a contiguous range of units, cut from the number of real row blocks
//     read on the device (block_offs[n_experts]), so consecutive units continue the same linear
//     stream and the padding of the block schedule costs nothing;
//   * two or four waves copy, four compute, two finish.  The copying waves send the runs HBM -> LDS by DMA
//     (buffer_load ... lds) as they lie in memory, through a ring of stages filled several units
//     ahead (about 100 KB in flight per CU); every per-unit operand, bias included, travels in that
//     stream so that no other load ever drains it;
//   * the K range is split over the four compute waves (split-K inside the workgroup): wave w keeps
//     its quarter of the up-to-16 activation rows in registers for as long as the row block lasts,
//     so activations never occupy LDS; partial 16x16 results go through LDS to the finishing waves,
//     which apply bias / activation / gate weight and store one unit later;
//   * v_mfma_f32_16x16x32: lane (c = lane%16, g = lane/16) is row c of A and column c of B; in super
//     step j of wave w it owns e8m0 group 4*SS*w + 4j + g (32 K), consumed 8 K at a time by 4 MFMAs.
#pragma once
#include "moe_matmul_impl.h"


namespace tamd {

template <int XDT>
struct Mma16;
template <>
struct Mma16<TAMD_BF16> {
  static TAMD_DEVICE f32x4_t mma(bf16x8_t a, bf16x8_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mma16<TAMD_F16> {
  static TAMD_DEVICE f32x4_t mma(f16x8_t a, f16x8_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

// 16-byte copies with an instruction offset: OFF is added to the global offset and to the LDS address
// alike, so one M0 value serves up to four consecutive 1 KB pieces of a linear image.  Every weight byte is
// read once, so the copies are non-temporal (nt): measured 11 % faster than cached reads on the decode shape.
// SETM0: also loads M0 with lds_addr first (with the wait states an SGPR operand written by a
// preceding v_readfirstlane needs; pieces that follow reuse the same registers).
template <int OFF, bool SETM0>
TAMD_DEVICE void dma16_at(v4i_t rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
  if constexpr (SETM0)
    asm volatile("s_mov_b32 m0, %4\n\ts_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2 offen offset:%3 nt lds"
                 :
                 : "v"(voff), "s"(rsrc), "s"(__builtin_amdgcn_readfirstlane(soff)), "n"(OFF),
                   "s"(__builtin_amdgcn_readfirstlane(lds_addr))
                 : "memory", "m0");
  else
    asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:%3 nt lds"
                 :
                 : "v"(voff), "s"(rsrc), "s"(__builtin_amdgcn_readfirstlane(soff)), "n"(OFF)
                 : "memory");
}

// byte SEL of a dword as float32 (the selector of the conversion is an immediate)
template <int A8, int SEL>
TAMD_DEVICE float fp8_byte(uint32_t word) {
  if constexpr (A8 == 2) return __builtin_amdgcn_cvt_f32_bf8((int)word, SEL);
  else return __builtin_amdgcn_cvt_f32_fp8((int)word, SEL);
}

template <int SS, int RING_, int NCW = 4>
struct StreamShape {
  static constexpr int TS = NCW * SS;               // super steps (128 K) of the whole K range: NCW compute waves x SS
  static constexpr int CODE_BYTES = TS * 1024;      // image of 16 columns' codes, padded to whole 1 KB copies
  static constexpr int NSC = (TS + 7) / 8;          // 1 KB pieces of the scale image: 16 * K/32 bytes, or the whole
  static constexpr int SC_BYTES = NSC * 1024;       // pre-shuffled block of 32 columns (ceil(K/256)*8 * 32 bytes)
  static constexpr int BIAS_BYTES = 256;            // 16 bias values, one dword each
  static constexpr int STAGE = CODE_BYTES + SC_BYTES + BIAS_BYTES;
  static constexpr int RED_BYTES = 2 * NCW * 1024;  // partial sums: 2 buffers x NCW waves x 16x16 floats
  static constexpr int RING = RING_;
  static constexpr int DMA_PER_STAGE = TS / 2 + NSC;  // most copies one wave has per stage
  static constexpr int LDS = RING * STAGE + RED_BYTES;
  static_assert(RING >= 2 && (RING - 1) * DMA_PER_STAGE < 64, "ring does not fit the vmcnt counter");
};

// SS: super steps (4 e8m0 groups = 128 K each) per compute wave; covers K <= 128 * NCW * SS.  N is a multiple of 16.
//
// Three roles: waves 0 .. NCW-1 compute (LDS -> convert -> MFMA -> partial sums), the next NC waves issue and await
// the copies, the last two finish and store the previous unit.  A wave that issues copies
// stalls whenever the memory pipeline is full; with nothing else to do it refills the pipeline the
// moment there is room, and the stalls never delay MFMA work or stores.
// NCW: compute waves (4 or 8) that split K between them.  The same kernel without its conversions and MFMAs runs the
// decode shape in 144 instead of 159 us; eight waves halve each wave's part of a unit but were slower in all (171 us:
// fourteen waves at the unit's barrier, eight partial sums to add), and the launcher uses four.
// A8 (1: float8_e4m3fn, 2: float8_e5m2; 0: rows of XDT): the activations are stored as fp8 (optionally with e8m0 block
// scales per 32 K) and are expanded to
// XDT when a row block's slice is loaded into registers -- exact, so the K loop is the same as for 16-bit rows.
// NC: copying waves (2 or 4).  A 1 KB copy holds the wave that issues it for about 110 cycles, so two copying waves
// move at most 18 bytes per cycle and CU and, with the K of the decode shape (24 pieces of codes per unit), spend
// most of a unit issuing; four take a quarter of a unit's pieces each (decode shape: 161 -> 158 us).
template <int XDT, int ACT, int SS, int RING, int A8, int NC, int NCW>
__global__ __launch_bounds__((NCW + NC + 2) * 64, 1) void mm_stream16_kernel(tamd_matmul_args a, int n_cg, int dense_blocks) {
  typedef Mma<XDT> M;
  typedef typename M::frag_t frag_t;
  typedef StreamShape<SS, RING, NCW> S;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr uint32_t kOob = 0x7FFFFFFFu;
  constexpr bool SW = ACT == TAMD_ACT_SWIGLU;
  const int tid = threadIdx.x;
  const int wave8 = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
  const int wave = wave8;      // (compute waves: which part of K)
  const int K = a.K, N = a.N, G = K / 32;
  const uint32_t col_bytes = (uint32_t)(K / 2);

  // ---- this workgroup's range of units
  const int n_blocks = a.block_schedule ? a.block_offs[a.n_experts] : dense_blocks;
  const int64_t total = (int64_t)n_blocks * n_cg;
  const int64_t first = (int64_t)blockIdx.x * total / gridDim.x;
  const int64_t last = (int64_t)(blockIdx.x + 1) * total / gridDim.x;
  if (first >= last) return;
  const int total_stages = (int)(last - first);
  const int blk0 = (int)(first / n_cg), cg0 = (int)(first - (int64_t)blk0 * n_cg);

  struct Block {  // a row block of at most 16 rows
    int expert, z, row0, rows;
  };
  auto get_block = [&](int blk, Block &b) {
    b.z = 0;
    int slice_rows, off_m;
    if (a.block_schedule) {
      const int sched = a.block_schedule[blk];
      if (sched == -1) {  // cannot happen below block_offs[n_experts]; an empty block keeps the ring in step
        b.expert = 0, b.row0 = 0, b.rows = 0;
        return;
      }
      b.expert = sched & 0xFFFF;
      slice_rows = a.slice_sizes[b.expert];
      off_m = (sched >> 16) * 16;
      b.row0 = a.slice_offs[b.expert] + off_m;
    } else {
      const int bm = (a.M + 15) / 16;
      const int z = blk / bm;
      b.expert = z, b.z = z;
      slice_rows = a.M;
      off_m = (blk - z * bm) * 16;
      b.row0 = off_m;
    }
    const int left = slice_rows - off_m;
    b.rows = left > 16 ? 16 : (left < 0 ? 0 : left);
  };
  float *red = (float *)(lds + S::RING * S::STAGE);

  if (wave8 >= NCW + NC) {
    // =========================================================================== finishing waves
    // 128 threads: thread -> (row er, column pair pc) of the 16x16 result of a unit; they read the four
    // partial sums one stage late, apply scale / bias / activation / gate weight and store.  These
    // waves never issue copies, so their loads and stores do not interfere with the copy counters.
    const int ft = tid - (NCW + NC) * 64;
    const int er = ft / 8, pc = ft % 8;
    float flex = 1.0f;
    if (a.x_scale) flex *= *a.x_scale;
    if (a.w_scale) flex *= *a.w_scale;
    const bool has_limit = a.act_has_limit != 0;
    const int n_out = SW ? N / 2 : N;
    const int red_idx = ((er >> 2) * 16 + 2 * pc) * 4 + (er & 3);  // column 2*pc; column 2*pc + 1 is 4 floats on
    int c_blk = blk0 - 1, c_cg = cg0;
    float row_beta = 1.f, row_gamma = 1.f, p_bias0 = 0.f, p_bias1 = 0.f, p_beta = 1.f, p_gamma = 1.f;
    int64_t row_dst = -1, p_dst = -1;
    int p_col0 = 0;
    auto load_rows = [&](int blk) {
      Block cb;
      get_block(blk, cb);
      const bool rv = er < cb.rows;
      const int erow = cb.row0 + (rv ? er : 0);
      row_beta = (a.betas && rv) ? a.betas[erow] : 1.0f;
      row_gamma = (a.gammas && rv) ? a.gammas[erow] : 1.0f;
      row_dst = rv ? (a.scatter_indx ? (int64_t)a.scatter_indx[erow] : (int64_t)erow) : -1;
      row_dst = row_dst < 0 ? -1 : (int64_t)cb.z * a.y_stride_z + row_dst * a.y_stride_m;
    };
    auto to_f32 = [&](uint32_t raw) {
      return a.bias == nullptr ? 0.f
                               : (a.bias_dtype == TAMD_F32 ? bits_to_f32(raw)
                                                           : (a.bias_dtype == TAMD_BF16 ? bits_to_f32(raw << 16)
                                                                                        : f16_bits_to_f32((uint16_t)raw)));
    };
    const int osz = a.y_dtype == TAMD_F32 ? 4 : (is_fp8(a.y_dtype) ? 1 : 2);
    auto narrow = [&](float v) -> uint32_t {  // one output value as 8 / 16 bits
      return a.y_dtype == TAMD_BF16 ? f32_to_bf16_bits(v) & 0xFFFFu
                                    : (a.y_dtype == TAMD_F16 ? f32_to_f16_bits(v) & 0xFFFFu : f32_to_fp8_bits(v, a.y_dtype));
    };
    // flexpoint output: scale by 1 / expected, optionally clamp, and track max|result| for the actual scale
    const float inv_expected = a.y_expected_scale ? 1.0f / *a.y_expected_scale : 1.0f;
    const bool clamp_out = a.y_expected_scale != nullptr && a.y_saturate_inf != 0;
    const float out_max = max_finite_of(a.y_dtype);
    uint32_t amax = 0;
    auto flex_out = [&](float v) {
      if (a.y_actual_scale) amax = absmax_bits(amax, v);
      v *= inv_expected;
      return clamp_out ? __builtin_fminf(__builtin_fmaxf(v, -out_max), out_max) : v;
    };
    auto finish = [&](int buf) {
      const float *rbuf = red + buf * (NCW * 256) + red_idx;
      float s0 = (rbuf[0] + rbuf[256]) + (rbuf[512] + rbuf[768]);
      float s1 = (rbuf[4] + rbuf[260]) + (rbuf[516] + rbuf[772]);
      if constexpr (NCW == 8) {
        s0 += (rbuf[1024] + rbuf[1280]) + (rbuf[1536] + rbuf[1792]);
        s1 += (rbuf[1028] + rbuf[1284]) + (rbuf[1540] + rbuf[1796]);
      }
      const float v0 = (s0 * flex + p_bias0 * p_beta) * a.out_alpha;
      const float v1 = (s1 * flex + p_bias1 * p_beta) * a.out_alpha;
      if (p_dst < 0) return;
      if constexpr (SW) {
        const int col = (p_col0 >> 1) + pc;
        if (col >= n_out) return;
        const float o = flex_out(swiglu_fast(v0, v1, a.act_alpha, a.act_limit, has_limit) * p_gamma);
        if (osz == 4) ((float *)a.y)[p_dst + col] = o;
        else if (osz == 2) ((uint16_t *)a.y)[p_dst + col] = (uint16_t)narrow(o);
        else ((uint8_t *)a.y)[p_dst + col] = (uint8_t)narrow(o);
      } else {
        const int col = p_col0 + 2 * pc;
        if (col >= n_out) return;  // N is a multiple of 16: the pair is inside or outside together
        const float o0 = flex_out(v0 * p_gamma), o1 = flex_out(v1 * p_gamma);
        if (osz == 4) {
          ((float *)a.y)[p_dst + col] = o0;
          ((float *)a.y)[p_dst + col + 1] = o1;
        } else if (osz == 2) {
          uint16_t *yp = (uint16_t *)a.y + p_dst + col;
          if (((uintptr_t)yp & 3) == 0) *(uint32_t *)yp = narrow(o0) | (narrow(o1) << 16);
          else yp[0] = (uint16_t)narrow(o0), yp[1] = (uint16_t)narrow(o1);
        } else {
          uint8_t *yp = (uint8_t *)a.y + p_dst + col;
          if (((uintptr_t)yp & 1) == 0) *(uint16_t *)yp = (uint16_t)(narrow(o0) | (narrow(o1) << 8));
          else yp[0] = (uint8_t)narrow(o0), yp[1] = (uint8_t)narrow(o1);
        }
      }
    };
    int slot = 0;
#pragma unroll 1
    for (int s = 0; s < total_stages; ++s) {
      __syncthreads();  // the partial sums of stage s - 1 and the bias of stage s are visible
      if (s > 0) finish((s - 1) & 1);
      if (c_blk < blk0 || c_cg == n_cg) {
        if (c_cg == n_cg) c_cg = 0;
        load_rows(++c_blk);
      }
      // this unit's bias and row data travel to the next iteration
      const uint2 braw = *(const uint2 *)(lds + slot * S::STAGE + S::CODE_BYTES + S::SC_BYTES + pc * 8);
      p_bias0 = to_f32(braw.x), p_bias1 = to_f32(braw.y);
      p_beta = row_beta, p_gamma = row_gamma, p_dst = row_dst;
      p_col0 = c_cg * 16;
      ++c_cg;
      slot = slot + 1 == S::RING ? 0 : slot + 1;
    }
    __syncthreads();
    finish((total_stages - 1) & 1);
    if (a.y_actual_scale) {
      // wave maximum, then one atomic per wave; positive floats order like their bit patterns
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const uint32_t other = (uint32_t)__shfl_xor((int)amax, o);
        amax = other > amax ? other : amax;
      }
      if (lane == 0) {
        amax = amax < 0x7F800000u ? amax : 0x7F800000u;  // NaN counts as +inf
        atomicMax((unsigned int *)a.y_actual_scale, f32_to_bits(__builtin_fmaf(bits_to_f32(amax), 1.0f / out_max, 1.0e-30f)));
      }
    }
  } else if (wave8 >= NCW) {
    // =========================================================================== copying waves
    // Wave 4 requests the first half of a unit's code image and its scale image, wave 5 the second half
    // and the bias.  A wave that issues copies stalls whenever the memory pipeline is full, which is
    // exactly how these two keep it full; nothing else runs on them.
    const int half = wave8 - NCW;   // which part of a unit's code image this wave copies (0 .. NC - 1)
    const v4i_t rw = make_rsrc(a.w, kOob), rs = make_rsrc(a.w_mx_scale, kOob), rb = make_rsrc(a.bias, kOob);
    // empty descriptors (no records: every lane out of range) for copies past the end of the range,
    // issued so that the count of outstanding copies per stage never changes
    const v4i_t rw0 = make_rsrc(a.w, 0), rs0 = make_rsrc(a.w_mx_scale, 0), rb0 = make_rsrc(a.bias, 0);
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
    const int bias_esz = a.bias_dtype == TAMD_F32 ? 4 : 2;
    constexpr int NP = S::TS / NC;  // code pieces (1 KB) per copying wave
    static_assert(S::TS % NC == 0, "the copying waves take equal parts of a unit's code image");
    // per-lane source offsets never change: a unit's codes, scales and bias are linear images
    uint32_t w_voff[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const uint32_t lin = (uint32_t)(half * NP + i) * 1024u + lane * 16u;
      w_voff[i] = lin < 16u * col_bytes ? (uint32_t)(half * NP) * 1024u + lane * 16u : kOob;  // piece i adds i*1024 itself
    }
    // scale image of a unit: its 16 * G bytes, or (pre-shuffled scales) the block of 32 columns it lies in
    const bool cdna4 = a.w_mx_layout == TAMD_SCALE_CDNA4;
    const uint32_t sc_unit_bytes = cdna4 ? (uint32_t)((G + 7) / 8 * 8 * 32) : (uint32_t)(16 * G);
    uint32_t x_voff[S::NSC];
    if (half == 0) {
#pragma unroll
      for (int q = 0; q < S::NSC; ++q) x_voff[q] = q * 1024u + lane * 16u < sc_unit_bytes ? q * 1024u + lane * 16u : kOob;
    } else {
      x_voff[0] = (half == 1 && a.bias != nullptr && lane < 16) ? (uint32_t)(lane * bias_esz) : kOob;
#pragma unroll
      for (int q = 1; q < S::NSC; ++q) x_voff[q] = kOob;
    }
    // codes in the block layout (TAMD_W_CDNA4_BLOCKS): the unit's 16 columns are, in every K stage's 4 KB block of
    // their strip, two runs of 512 bytes (positions 8u.. and 32 + 8u.., u = unit inside the strip): piece i of the
    // image is K stage i, lanes 0-31 copy the first run and lanes 32-63 the second
    const bool wnat = a.w_layout == TAMD_W_CDNA4_BLOCKS;
    const int n_kstage = (K + 127) / 128;
    const uint32_t nat_voff = (uint32_t)((lane / 32) * 2048 + (lane % 32) * 16);
    int i_blk = blk0 - 1, i_cg = cg0, i_left = total_stages;
    uint32_t i_wbase = 0, i_sbase = 0, i_bbase = 0, i_ebase = 0;
    auto issue = [&](int slot) {
      const bool live = i_left > 0;
      if (live && (i_blk < blk0 || i_cg == n_cg)) {
        if (i_cg == n_cg) i_cg = 0;
        ++i_blk;
        Block b;
        get_block(i_blk, b);
        const int e = __builtin_amdgcn_readfirstlane(b.expert);  // keeps the running offsets in scalar registers
        i_ebase = (uint32_t)((int64_t)e * a.w_stride_e);
        i_wbase = i_ebase + (uint32_t)i_cg * 16u * col_bytes;
        i_sbase = (uint32_t)((int64_t)e * a.w_mx_stride_e);
        i_bbase = (uint32_t)(((int64_t)e * a.bias_stride_e + i_cg * 16) * bias_esz);
      }
      const uint32_t sb = lds_base + slot * S::STAGE;
      const v4i_t dw = live ? rw : rw0;
      if (wnat) {
        const uint32_t ub = i_ebase + (uint32_t)((i_cg >> 2) * n_kstage) * 4096u + (uint32_t)(i_cg & 3) * 512u;
#pragma unroll
        for (int i = 0; i < NP; ++i) {
          const int ks = half * NP + i;
          dma16_at<0, true>(ks < n_kstage ? dw : rw0, sb + ks * 1024, nat_voff, ub + (uint32_t)ks * 4096u);
        }
      } else
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const uint32_t m0v = sb + (half * NP + i / 4 * 4) * 1024;
        const uint32_t so = i_wbase + (uint32_t)(i / 4) * 4096u;
        if (i % 4 == 0) dma16_at<0, true>(dw, m0v, w_voff[i], so);
        if (i % 4 == 1) dma16_at<1024, false>(dw, m0v, w_voff[i], so);
        if (i % 4 == 2) dma16_at<2048, false>(dw, m0v, w_voff[i], so);
        if (i % 4 == 3) dma16_at<3072, false>(dw, m0v, w_voff[i], so);
      }
      if (half == 0) {
        const uint32_t so = i_sbase + (cdna4 ? (uint32_t)(i_cg >> 1) : (uint32_t)i_cg) * sc_unit_bytes;
#pragma unroll
        for (int q = 0; q < S::NSC; ++q) dma16(live ? rs : rs0, sb + S::CODE_BYTES + q * 1024, x_voff[q], so);
      } else if (half == 1) {
        const uint32_t dst = sb + S::CODE_BYTES + S::SC_BYTES;
        if (bias_esz == 4) dma4(live ? rb : rb0, dst, x_voff[0], i_bbase);
        else dma2(live ? rb : rb0, dst, x_voff[0], i_bbase);
      }
      ++i_cg, --i_left;
      i_wbase += 16u * col_bytes, i_bbase += (uint32_t)(16 * bias_esz);
    };
    // stage s lives in slot s % RING and is requested RING - 1 stages ahead
    int i_slot = 0;
#pragma unroll 1
    for (int s = 0; s < S::RING - 1; ++s) {
      issue(i_slot);
      i_slot = i_slot + 1 == S::RING ? 0 : i_slot + 1;
    }
#pragma unroll 1
    for (int s = 0; s < total_stages; ++s) {
      // copies complete in order: once at most RING - 2 stages' worth are outstanding, stage s has landed
      if (half == 0) wait_vmcnt<(S::RING - 2) * (NP + S::NSC)>();
      else if (half == 1) wait_vmcnt<(S::RING - 2) * (NP + 1)>();
      else wait_vmcnt<(S::RING - 2) * NP>();
      __syncthreads();  // publishes stage s; every wave is done with stage s - 1, whose slot is refilled now
      issue(i_slot);
      i_slot = i_slot + 1 == S::RING ? 0 : i_slot + 1;
    }
    __syncthreads();
    wait_vmcnt<0>();  // the empty copies issued past the end still write (zeros) to LDS
  } else {
    // =========================================================================== compute waves
    const int c16 = lane % 16, g = lane / 16;
    const bool cdna4 = a.w_mx_layout == TAMD_SCALE_CDNA4;
    const int kb = 4 * SS * wave;  // first e8m0 group of this wave's K slice
    frag_t areg[SS * 4];           // this wave's K slice of the block's rows, row c16
    int c_blk = blk0 - 1, c_cg = cg0;
    auto load_block = [&](int blk) {
      Block cb;
      get_block(blk, cb);
      int rc = c16 < cb.rows ? c16 : cb.rows - 1;
      rc = cb.row0 + (rc < 0 ? 0 : rc);
      const int64_t src = a.gather_indx ? (int64_t)a.gather_indx[rc] : (int64_t)rc;
      if constexpr (A8) {
        const uint8_t *xr = (const uint8_t *)a.x + (int64_t)cb.z * a.x_stride_z + src * a.x_stride_m;
        const uint8_t *xs = a.x_mx_scale ? a.x_mx_scale + (int64_t)cb.z * a.x_mx_stride_z + src * a.x_mx_stride_m : nullptr;
#pragma unroll
        for (int j = 0; j < SS; ++j) {
          const int kg = kb + 4 * j + g;
          const bool live = kg < G && cb.rows > 0;
          const float mult = (live && xs) ? bits_to_f32((uint32_t)xs[kg] << 23) : 1.0f;  // 2^(e - 127); 0xFF gives +inf
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            uint2 v = make_uint2(0, 0);
            if (live) v = *(const uint2 *)(xr + 32 * kg + 8 * u);
            float f[8];
            f[0] = fp8_byte<A8, 0>(v.x) * mult;
            f[1] = fp8_byte<A8, 1>(v.x) * mult;
            f[2] = fp8_byte<A8, 2>(v.x) * mult;
            f[3] = fp8_byte<A8, 3>(v.x) * mult;
            f[4] = fp8_byte<A8, 0>(v.y) * mult;
            f[5] = fp8_byte<A8, 1>(v.y) * mult;
            f[6] = fp8_byte<A8, 2>(v.y) * mult;
            f[7] = fp8_byte<A8, 3>(v.y) * mult;
            // packed by hand, two values per register: an fp8 value times a power of two has at most four significant
            // bits, so the upper half of its float32 pattern is its bf16 pattern
            uint32_t w[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
              if constexpr (XDT == TAMD_BF16) w[p] = (f32_to_bits(f[2 * p + 1]) & 0xFFFF0000u) | (f32_to_bits(f[2 * p]) >> 16);
              else w[p] = (f32_to_f16_bits(f[2 * p]) & 0xFFFFu) | (f32_to_f16_bits(f[2 * p + 1]) << 16);
            }
            areg[j * 4 + u] = __builtin_bit_cast(frag_t, make_uint4(w[0], w[1], w[2], w[3]));
          }
        }
      } else {
        const uint16_t *xr = (const uint16_t *)a.x + (int64_t)cb.z * a.x_stride_z + src * a.x_stride_m;
#pragma unroll
        for (int j = 0; j < SS; ++j) {
          const int kg = kb + 4 * j + g;
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (kg < G && cb.rows > 0) v = *(const uint4 *)(xr + 32 * kg + 8 * u);
            areg[j * 4 + u] = __builtin_bit_cast(frag_t, v);
          }
        }
      }
    };
    // per-lane LDS offsets of this wave's K slice inside a stage (beyond K: group 0 with scale 1.0 --
    // the activations there are zero, the weight operand only has to stay finite)
    const bool wnat = a.w_layout == TAMD_W_CDNA4_BLOCKS;
    uint32_t b_loff[SS], s_loff[SS];
    bool kvalid[SS];
#pragma unroll
    for (int j = 0; j < SS; ++j) {
      const int kg = kb + 4 * j + g;
      kvalid[j] = kg < G;
      // block layout: stage kg / 4 of the image, run f = column parity, position c' = column / 2, the group's part
      // in slot part ^ (c' >> 2) ^ 2 f (^ 2 for the odd units of a strip, applied per unit below)
      const int kgv0 = kvalid[j] ? kg : 0, cf = c16 & 1, cp = c16 >> 1;
      b_loff[j] = wnat ? (uint32_t)((kgv0 >> 2) * 1024 + cf * 512 + cp * 64 + (((kgv0 & 3) ^ (cp >> 2) ^ (cf << 1)) * 16))
                       : (uint32_t)c16 * col_bytes + kgv0 * 16;
      const int kgv = kvalid[j] ? kg : 0;
      s_loff[j] = (uint32_t)(S::CODE_BYTES +
                             (cdna4 ? (kgv / 8) * 256 + (kgv % 4) * 64 + c16 * 4 + ((kgv % 8) / 4) * 2 : c16 * G + kgv));
    }
    int slot = 0;
#pragma unroll 1
    for (int s = 0; s < total_stages; ++s) {
      __syncthreads();
      if (c_blk < blk0 || c_cg == n_cg) {
        if (c_cg == n_cg) c_cg = 0;
        load_block(++c_blk);
      }
      const uint32_t sc_par = cdna4 ? (uint32_t)(c_cg & 1) : 0u;  // which 16 of the block's 32 columns
      const uint32_t b_flip = wnat ? (uint32_t)(c_cg & 1) << 5 : 0u;  // odd unit of a strip: slots rotated by 2
      ++c_cg;
      const uint8_t *img = lds + slot * S::STAGE;
      uint4 raw[SS];
      uint32_t sby[SS];
#pragma unroll
      for (int j = 0; j < SS; ++j) {
        raw[j] = *(const uint4 *)(img + (b_loff[j] ^ b_flip));
        sby[j] = img[s_loff[j] + sc_par];
      }
      // four independent accumulation chains keep dependent MFMAs apart
      f32x4_t acc0 = f32x4_t{0.f, 0.f, 0.f, 0.f}, acc1 = acc0, acc2 = acc0, acc3 = acc0;
#pragma unroll
      for (int j = 0; j < SS; ++j) {
        const float sc = bits_to_f32((kvalid[j] ? sby[j] : 127u) << 23);
        acc0 = Mma16<XDT>::mma(areg[j * 4 + 0], M::expand(raw[j].x, sc), acc0);
        acc1 = Mma16<XDT>::mma(areg[j * 4 + 1], M::expand(raw[j].y, sc), acc1);
        acc2 = Mma16<XDT>::mma(areg[j * 4 + 2], M::expand(raw[j].z, sc), acc2);
        acc3 = Mma16<XDT>::mma(areg[j * 4 + 3], M::expand(raw[j].w, sc), acc3);
      }
      *(f32x4_t *)(red + (s & 1) * (NCW * 256) + wave * 256 + lane * 4) = (acc0 + acc1) + (acc2 + acc3);
      slot = slot + 1 == S::RING ? 0 : slot + 1;
    }
    __syncthreads();
  }
}

// Whether the streaming kernel covers the problem: K contiguous and dense per column for codes and
// scales, 16-byte aligned column groups, N a multiple of 16, K <= 4096, whole tensors addressable
// with 32-bit offsets.
inline bool stream16_applicable(const tamd_matmul_args &a) {
  const int64_t lim = 0x7FFFFF00;
  const int64_t G = a.K / 32;
  if (a.K > 4096 || a.K % 32 != 0) return false;
  const bool cdna4 = a.w_mx_layout == TAMD_SCALE_CDNA4;
  const bool wnat = a.w_layout == TAMD_W_CDNA4_BLOCKS;
  if (!wnat && (a.w_stride_k != 1 || a.w_stride_n != a.K / 2)) return false;
  if (!cdna4 && (a.w_mx_stride_k != 1 || a.w_mx_stride_n != G)) return false;
  if (!aligned(a.w, 16) || a.w_stride_e % 16 != 0 || !aligned(a.w_mx_scale, 16) || a.w_mx_stride_e % 16 != 0) return false;
  if ((int64_t)a.n_experts * a.w_stride_e + (wnat ? (int64_t)0 : (int64_t)a.N * a.w_stride_n) >= lim) return false;
  if ((int64_t)a.n_experts * a.w_mx_stride_e + (int64_t)(a.N + 32) * (G + 8) >= lim) return false;
  if (a.bias && ((int64_t)a.n_experts * a.bias_stride_e + a.N) * 4 >= lim) return false;
  if (a.bias && !aligned(a.bias, a.bias_dtype == TAMD_F32 ? 4 : 2)) return false;
  if (a.N % 16 != 0) return false;  // whole 16-column groups only (their scale run is then a multiple of 16 bytes)
  if (a.block_schedule && !a.block_offs) return false;
  if (a.y_mx_scale) return false;  // a unit is 16 columns, an output scale group 32
  return true;
}

template <int XDT, int ACT, int SS, int A8, int NCW>
int launch_stream16_ss(const tamd_matmul_args &a, int grid_m, hipStream_t st) {
  constexpr int TS = NCW * SS;
  // four copying waves where the registers allow three or four waves per SIMD (the kernels that expand fp8 rows keep a
  // wave's whole slice of the rows in registers twice over while they convert it)
  constexpr int NC = NCW * 64 + 6 * 64 <= 640 && (A8 == 0 ? SS <= 6 : SS <= 4) ? 4 : 2;
  constexpr int RING_FIT = (156 * 1024 - 2 * NCW * 1024) / (TS * 1024 + (TS + 7) / 8 * 1024 + 256);
  constexpr int RING = RING_FIT > 6 ? 6 : RING_FIT;
  const int n_cg = (a.N + 15) / 16;
  const int64_t upper = (int64_t)grid_m * n_cg;
  if (upper <= 0) return 0;
  int cus = 0;
  if (int rc = cu_count(cus)) return rc;
  const int wgs = (int)(upper < cus ? upper : cus);
  auto kern = mm_stream16_kernel<XDT, ACT, SS, RING, A8, NC, NCW>;
  if (int rc = raise_lds_limit_once((const void *)kern)) return rc;
  kern<<<dim3((unsigned)wgs), (NCW + NC + 2) * 64, StreamShape<SS, RING, NCW>::LDS, st>>>(a, n_cg, a.block_schedule ? 0 : grid_m);
  return launch_status();
}

template <int XDT, int ACT, int A8 = 0>
int launch_stream16(const tamd_matmul_args &a, int grid_m, hipStream_t st) {
  // four compute waves: with eight (each wave half the conversions and MFMAs of a unit, fourteen waves at the unit's
  // barrier, eight partial sums to add) the decode shape ran 171 us instead of 159
  const int ss = (a.K / 32 + 15) / 16;  // super steps per wave
  if (ss <= 2) return launch_stream16_ss<XDT, ACT, 2, A8, 4>(a, grid_m, st);
  if (ss <= 4) return launch_stream16_ss<XDT, ACT, 4, A8, 4>(a, grid_m, st);
  if (ss <= 6) return launch_stream16_ss<XDT, ACT, 6, A8, 4>(a, grid_m, st);
  return launch_stream16_ss<XDT, ACT, 8, A8, 4>(a, grid_m, st);
}

// The streaming kernels of one activation type live in a translation unit of their own (moe_matmul_stream_*.hip).
int stream_mm_bf16(const tamd_matmul_args &a, int grid_m, hipStream_t st);
int stream_mm_f16(const tamd_matmul_args &a, int grid_m, hipStream_t st);
int stream_mm_fp8e4m3(const tamd_matmul_args &a, int grid_m, hipStream_t st);  // fp8 rows expanded to bf16
int stream_mm_fp8e5m2(const tamd_matmul_args &a, int grid_m, hipStream_t st);

}  // namespace tamd

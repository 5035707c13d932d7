// W4A16 tile GEMM with the weights dequantised in registers (large M): the int4 words go from global memory into
// registers, become MFMA operands there, and never pass through LDS; only the activations are staged.
//
// 256 x 256 output tile, four wavefronts side by side along N (one per SIMD), each 256 rows x 64 columns:
// 8 x 2 accumulator blocks of v_mfma_f32_32x32x16 = 256 accumulation registers per lane.
//
//  * Weights.  A wavefront owns four native 16-column tiles.  Two neighbouring tiles X, Y give one 32-column MFMA
//    operand: lane 16 o + r of a native word holds 8 codes of rows 32 j + 8 o .. + 7, column r, and one
//    v_permlane16_swap turns (X, Y) into X' = [X o0 | Y o0 | X o2 | Y o2], Y' = [X o1 | Y o1 | X o3 | Y o3]: lane l of X'
//    holds column l & 31 of the 32-column block at k-octet 2 (l >> 5), of Y' at k-octet 2 (l >> 5) + 1 -- two A operands
//    (rows = n) of the 32x32x16 MFMA, each word dequantised exactly like the LDS-staged kernel does
//    (fma(code, s, -z s) rounded once to the 16-bit type = the reference's (q - z).to(dtype) * s).
//    The 16-bit operand of a k-slice is dequantised while the MFMAs of the slice before it run.
//  * Activations.  256 rows x 64 k per K step, global -> LDS by direct-to-LDS loads, four stages, requested four steps
//    ahead; the LDS image is the one of the LDS-staged kernel (128-byte rows, two to a 256-byte line, 16-byte chunks
//    XOR-ed with the line number).  A slice's B operands (columns = m) are 8 reads of 16 bytes per lane, each register
//    quad refilled in place for the next slice once its two MFMAs are issued.  Every wavefront reads the whole tile:
//    4 x 32 KiB per K step and compute unit, against 12 x 8 KiB + the weight writes of the 8-wavefront kernel.
//  * One workgroup barrier per K step (64 k), placed after the reads of the step's last slice: behind it the next
//    step's stage may be read and the stage just finished may be requested again.
//  * Scales / zero points: one (n, group) value per lane and 32-column block, requested two groups ahead.
#pragma once
#include "w4a16_prefill_kernel.h"

namespace vaq {

template <bool BF16, bool HAS_ZP>
__global__ __launch_bounds__(256) void w4a16_prefill3_kernel(const PrefillParams p) {
  using T = F16Traits<BF16>;
  constexpr int BM = 256, BN = 256, NW = 4, TM = 256, TN = 64;
  constexpr int WMB = TM / 32, WNB = TN / 32;      // 8 x 2 accumulator blocks
  constexpr int NST = 4;                           // activation stages
  constexpr int A_ST = BM * 128;                   // bytes per stage
  constexpr int A_LD = BM / (8 * NW);              // direct-to-LDS instructions per wavefront and K step (1 KiB each)
  constexpr int KW = 4 + 2 * (HAS_ZP ? 2 : 1);     // vector-memory instructions of one load_w
  constexpr bool HP = !BF16;                       // packed fp16 dequantisation
  extern __shared__ __attribute__((aligned(16))) uint8_t lds8[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n;
  const TileSlot sl = tile_slot(total, p.SK, p.tail_first);          // one contiguous range of tile positions per XCD
  const int t = sl.pos;
  constexpr int GM = 4;                                              // bands of 4 tile rows (see the LDS-staged kernel)
  const int band = t / (GM * tiles_n);
  const int first_m = band * GM;
  const int gsz = min(tiles_m - first_m, GM);
  const int tin = t - band * GM * tiles_n;
  const int tm = first_m + tin % gsz, tn = tin / gsz;
  const int m0 = tm * BM, n0 = tn * BN, nt0 = n0 / 16;

  // ---- activation tile: direct-to-LDS loads (same image as w4a16_prefill2_kernel) ----
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(p.a), 0, (int)((uint32_t)p.M * (uint32_t)p.lda * 2u), 0x00020000);
  uint32_t voff_a[A_LD];
#pragma unroll
  for (int i = 0; i < A_LD; ++i) {
    const int j = (wave * A_LD + i) * 4 + (lane >> 4);
    const int c16 = (lane & 15) ^ (j & 15);
    const int lrow = 2 * (lane >> 4) + (c16 >> 3);
    voff_a[i] = ((uint32_t)lrow * (uint32_t)p.lda) * 2u + (uint32_t)(c16 & 7) * 16u;
  }
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  auto issue_a = [&](int step, int buf) {
    uint8_t* Ab = lds8 + (size_t)buf * A_ST;
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
      const int r0 = (wave * A_LD + i) * 8;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(Ab + r0 * 128), 16, (int)voff_a[i],
                                               (int)(((uint32_t)(m0 + r0) * (uint32_t)p.lda + (uint32_t)step * 64u) * 2u), 0, 0);
    }
  };

  // ---- weights: raw words of the groups in flight (n1 = next, n2 = the one after), the current group already swapped ----
  // this lane's column inside 32-column block nb: tile 2 nb + ((lane >> 4) & 1), column lane & 15 of it
  int ntile[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) ntile[i] = min(nt0 + wave * 4 + i, p.NT - 1);     // clamped: columns past N are never stored
  int ncol[WNB];
#pragma unroll
  for (int nb = 0; nb < WNB; ++nb) ncol[nb] = (((lane >> 4) & 1) ? ntile[2 * nb + 1] : ntile[2 * nb]) * 16 + (lane & 15);

  struct WSet {
    v4u w[4];
    uint16_t s[WNB];
    uint32_t z[WNB];
  };
  WSet n1, n2;
  auto load_w = [&](WSet& d, int g) {
#pragma unroll
    for (int i = 0; i < 4; ++i) d.w[i] = p.b[((int64_t)ntile[i] * p.G + g) * 64 + lane];
#pragma unroll
    for (int nb = 0; nb < WNB; ++nb) {
      d.s[nb] = p.scales[(int64_t)g * p.s_stride + ncol[nb]];
      if constexpr (HAS_ZP) d.z[nb] = p.zeros[(int64_t)g * p.z_stride + (ncol[nb] >> 3)];
      else d.z[nb] = 0u;
    }
  };
  // current group: swapped words [nb][j][X' / Y'], scale and -(zero * scale) per block
  uint32_t wsw[WNB][4][2];
  float scur[WNB], zcur[WNB];
  uint32_t s2cur[HP ? WNB : 1], nzb2cur[HP ? WNB : 1];
  auto advance_w = [&]() {      // n1 becomes current, n2 becomes n1
#pragma unroll
    for (int nb = 0; nb < WNB; ++nb) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const auto sw = __builtin_amdgcn_permlane16_swap(n1.w[2 * nb][j], n1.w[2 * nb + 1][j], false, false);
        wsw[nb][j][0] = sw[0];
        wsw[nb][j][1] = sw[1];
      }
      const float sv = T::to_float(n1.s[nb]);
      uint32_t zc = 8u;
      if constexpr (HAS_ZP) zc = (n1.z[nb] >> ((lane & 7) * 4)) & 0xFu;      // column 16 * tile + (lane & 15)
      scur[nb] = sv;
      zcur[nb] = -((float)zc * sv);                                          // exact: <= 4 + 11 significant bits
      if constexpr (HP) {
        const uint32_t sb = n1.s[nb], zb = 0xE400u | zc;                     // -(1024 + zero) as fp16 bits
        s2cur[nb] = sb | (sb << 16);
        nzb2cur[nb] = zb | (zb << 16);
      }
    }
    n1 = n2;
  };
  // the 16-bit A operand of slice (j, xy) for block nb
  auto dequant = [&](int nb, int j, int xy) -> v4u {
    if constexpr (HP) return dequant_scaled_h(wsw[nb][j][xy], s2cur[nb], nzb2cur[nb]);
    else return dequant_scaled<BF16>(wsw[nb][j][xy], scur[nb], zcur[nb]);
  };

  v16f acc[WMB][WNB];
#pragma unroll
  for (int i = 0; i < WMB; ++i)
#pragma unroll
    for (int j = 0; j < WNB; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // operand reads of slice sl = 2 jj + xy (jj = word of the step, xy = X' / Y'): row lane & 31 of a 32-row block,
  // 16-byte chunk 4 jj + 2 (lane >> 5) + xy of its 128-byte row
  uint32_t coff[4];
#pragma unroll
  for (int sl = 0; sl < 4; ++sl) {
    const int chunk = 4 * (sl >> 1) + 2 * (lane >> 5) + (sl & 1);
    coff[sl] = (uint32_t)(((lane & 31) >> 1) * 256 + ((((lane & 1) * 8 + chunk) ^ ((lane >> 1) & 15)) * 16));
  }

  // K may be split over workgroups: this one covers the groups [g_lo, g_hi)
  const int g_lo = (int)(((int64_t)p.G * sl.split) / sl.nsplit), g_hi = (int)(((int64_t)p.G * (sl.split + 1)) / sl.nsplit);
  const int s_lo = 2 * g_lo, s_last = 2 * g_hi - 1;      // K steps of 64

  v4u af[WMB];        // B operands (activations) of the current slice, refilled in place
  v4u wf[2][WNB];     // A operands (weights) of the current and of the next slice

  // One k-slice: its 16 MFMAs, with the reads of the next slice's activation fragments (from `next_a`, offset
  // coff[next_sl]) and the dequantisation of the next slice's weights (word next_j, half next_sl & 1, into the other
  // operand buffer) in their shadow.
  auto slice = [&](auto cbuf_c, const uint8_t* next_a, auto next_sl_c, auto next_j_c, auto tail_c) {
    constexpr bool tail = decltype(tail_c)::value;
    constexpr int cbuf = decltype(cbuf_c)::value, nbuf = cbuf ^ 1;
    constexpr int next_sl = decltype(next_sl_c)::value, next_j = decltype(next_j_c)::value;
#pragma unroll
    for (int mb = 0; mb < WMB; ++mb) {
#pragma unroll
      for (int nb = 0; nb < WNB; ++nb) acc[mb][nb] = T::mfma32(wf[cbuf][nb], af[mb], acc[mb][nb]);      // rows = n, columns = m
      if constexpr (!tail) {
        af[mb] = *reinterpret_cast<const v4u*>(next_a + mb * 4096 + coff[next_sl]);
        // a quarter of a weight operand per m-block: 2 blocks x 4 registers over 8 m-blocks
        const int nb = mb >> 2, q = mb & 3;
        if constexpr (HP) wf[nbuf][nb][q] = dequant_pair_h(wsw[nb][next_j][next_sl & 1], s2cur[nb], nzb2cur[nb], q);
        else wf[nbuf][nb][q] = dequant_part<BF16>(wsw[nb][next_j][next_sl & 1], scur[nb], zcur[nb], q);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  using C2 = std::integral_constant<int, 2>;
  using C3 = std::integral_constant<int, 3>;
  using TT = std::true_type;
  using FF = std::false_type;

  // ---- prologue.  Request order (vector-memory operations retire in order): tile 0, weights g_lo, tile 1, weights
  // g_lo + 1, tiles 2 and 3; every later request repeats the pattern of the main loop. ----
  auto clamp_s = [&](int s) { return min(s, s_last); };
  auto clamp_g = [&](int g) { return min(g, g_hi - 1); };
  issue_a(s_lo, 0);
  load_w(n1, g_lo);
  issue_a(clamp_s(s_lo + 1), 1);
  load_w(n2, clamp_g(g_lo + 1));
  issue_a(clamp_s(s_lo + 2), 2);
  issue_a(clamp_s(s_lo + 3), 3);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * A_LD + KW) : "memory");      // tile 0 and the weights of g_lo have landed
  advance_w();                                                              // (its copy n1 = n2 waits for g_lo + 1 as well)
#pragma unroll
  for (int nb = 0; nb < WNB; ++nb) wf[0][nb] = dequant(nb, 0, 0);
  asm volatile("s_barrier" ::: "memory");
#pragma unroll
  for (int mb = 0; mb < WMB; ++mb) af[mb] = *reinterpret_cast<const v4u*>(lds8 + mb * 4096 + coff[0]);

  // ---- main loop: two K steps per group.  In a step, slices 0..2 run, then the wait + barrier, then slice 3, in whose
  // shadow the first fragments of the next step are read and the stage this step used is requested again. ----
  int cur = 0;      // stage of the current step
  for (int g = g_lo; g < g_hi; ++g) {
    // even step 2g: words 0, 1 of the group
    {
      const uint8_t* Acur = lds8 + (size_t)cur * A_ST;
      const uint8_t* Anext = lds8 + (size_t)((cur + 1) & (NST - 1)) * A_ST;
      load_w(n2, clamp_g(g + 2));
      slice(C0{}, Acur, C1{}, C0{}, FF{});      // slice (word 0, X'); in its shadow: (word 0, Y')
      slice(C1{}, Acur, C2{}, C1{}, FF{});      // slice (0, Y'); next (1, X')
      slice(C0{}, Acur, C3{}, C1{}, FF{});      // slice (1, X'); next (1, Y')
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(2 * A_LD + 2 * KW) : "memory");
      issue_a(clamp_s(2 * g + 4), cur);
      slice(C1{}, Anext, C0{}, C2{}, FF{});     // slice (1, Y'); next: step 2g + 1, (word 2, X')
      cur = (cur + 1) & (NST - 1);
    }
    // odd step 2g + 1: words 2, 3
    {
      const uint8_t* Acur = lds8 + (size_t)cur * A_ST;
      const uint8_t* Anext = lds8 + (size_t)((cur + 1) & (NST - 1)) * A_ST;
      slice(C0{}, Acur, C1{}, C2{}, FF{});
      slice(C1{}, Acur, C2{}, C3{}, FF{});
      slice(C0{}, Acur, C3{}, C3{}, FF{});
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(2 * A_LD + KW) : "memory");
      issue_a(clamp_s(2 * g + 5), cur);
      // The operands of the group's last slice are in wf[1] already: the next group's words become current in front of
      // it, and its first slice is prepared in the shadow of these MFMAs like any other.  Behind the last group the same
      // code runs on the repeated (clamped) requests and its results are dropped: one path through the loop body keeps
      // the 256 accumulation registers where they are (with a branch here the compiler moved accumulators between the
      // two register files and spilled).
      advance_w();
      slice(C1{}, Anext, C0{}, C0{}, FF{});
      cur = (cur + 1) & (NST - 1);
    }
  }
  // every wavefront is done with the stages (the requests beyond the last step repeat it: drain them), then the
  // epilogue reuses the LDS
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  static_assert(NST * A_ST >= NW * 32 * (TN * 2 + 16), "stages too small for the epilogue staging");
  tile_epilogue<BF16, WMB, WNB, NW, TM, TN>(p, acc, lds8, sl, wave, lane, m0, n0, 0, wave);
}

template <bool BF16, bool HAS_ZP>
static int launch_prefill3(const PrefillParams& p, hipStream_t s) {
  const size_t lds = (size_t)4 * 256 * 128;
  auto kern = w4a16_prefill3_kernel<BF16, HAS_ZP>;
  static size_t reserved[VAQ_MAX_DEVICES];
  if (const int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), lds, reserved, "w4a16_gemm(prefill)"); rc != VAQ_OK) return rc;
  const int tiles = ((p.M + 255) / 256) * ((p.N + 255) / 256);
  const dim3 grid = p.tail_first > 0 ? dim3(p.tail_first + (tiles - p.tail_first) * p.SK) : dim3(tiles, p.SK);
  hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, p);
  return VAQ_OK;
}

}  // namespace vaq

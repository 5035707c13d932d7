// Host side of the LDS-staged decode kernel (w4a16_decode2_kernel.h): configuration choice, workspace sizes, launch
// of the instances for quantisation groups of 128 rows and channelwise scales.
#include "w4a16_decode2_kernel.h"

namespace vaq {

// ----------------------------------------------------------------------------- host side

struct Decode2Config {
  int gs, wks, wn, sk, mr;
  int rc;      // ring variant of long streams (see the kernel): 0 two slots refilled early, 1 / 2 four / three slots refilled late
};

static inline bool exp_off(const VaqTuning& tn, int i) { return tn.exp[i] != 1; }      // development switch i not set to "off"

static int round_gs(int x, int sub, bool w8) {
  const int opts[] = {1, 2, 4, 7, 8, 14, 16};
  for (int o : opts) {
    if (sub > 1 && (o & (o - 1)) != 0) continue;     // sub-group instances exist for powers of two only
    if (w8 && (o & 1)) continue;                     // 8-bit codes: two tiles (nibble planes) per group
    if (o >= x) return o;
  }
  return 16;
}

// Groups per slab are limited by LDS (128 KiB of activations, 256 bytes per group and staged row): 512 / rows.
// G, gslab, gs and slab_max below count weight tiles: one per 128 rows of K, two (nibble planes) for 8-bit codes.
// `nt_mult`: copies of every n-tile's stream that run side by side (rows split over workgroups, see the kernel).
static Decode2Config pick_decode2_config(int M, int N, int K, int sub, bool w8, int nt_mult = 1, bool allow8 = true) {
  const int TPG = w8 ? 2 : 1;
  const int G = K / 128 * TPG, NT = N / 16 * nt_mult;
  const int MB = (M + 15) / 16;
  Decode2Config c;
  c.mr = M == 1 ? 1 : (M <= 4 ? 4 : (M <= 8 && sub == 1 && !w8 && allow8 && tuning().exp[3] != 1 ? 8 : 16));      // rows staged (8: 4-bit codes in groups of 128 rows only)
  const int slab_max = 512 / (c.mr * MB) * TPG;
  c.sk = (G + slab_max - 1) / slab_max;
  const int gslab = (G + c.sk - 1) / c.sk;            // groups per slab
  const int cus = num_cus_current_device();
  // K slices wanted: about 16 wavefronts per compute unit, 8 when few rows are staged (measured: with little LDS to
  // fill, longer per-wavefront tile streams beat more wavefronts on layers with few n-tiles)
  // (also with 16 staged rows when there is at most one workgroup per compute unit: 4096 x 4096 at M = 16, 6.60 -> 6.34 us)
  // (and with 16 staged rows on up to two (n-tile, K slab) pairs per compute unit: four K slices of 8 tiles with the
  // three-slot ring below, 4096 x 6144 at M = 16 6.9 -> 6.5 us, 8192 x 6144 10.9 -> 9.5 us, 4096 x 8192 7.5 -> 7.0 us)
  int want = (cus * ((NT * c.sk <= 2 * cus && MB == 1) || NT * c.sk <= cus ? 8 : D2_WAVES)) / (NT * c.sk);
  int wks = 1;
  while (wks * 2 <= want && wks < 16) wks *= 2;
  while (wks > 1 && wks > gslab) wks /= 2;
  // A single row: as many K slices as it takes to cover K with streams of at most 16 tiles, rather than a split over
  // workgroups and its hand-over (28672 x 8192 at M = 1: 30.2 -> 24.5 us, 28672 x 4096 17.7 -> 14.8 us; from two rows on
  // the split wins or ties) -- where those workgroups, one per n-tile, make full rounds (20480 x 5120, 320 n-tiles:
  // 16.7 -> 19.4 us).
  if (c.mr == 1 && (NT <= cus || NT % cus == 0 || (NT % cus) * 5 >= cus * 4))
    while (wks < 16 && wks * 16 < gslab) wks *= 2;
  const VaqTuning& tn = tuning();
  // Two m-blocks of a long K on a layer of at most one n-tile per compute unit: slabs of one 14-tile stream per
  // wavefront with the four-slot ring (14336 x 4096 at M = 17 / 32: 13.8 / 14.7 -> 12.9 / 13.2 us; 11008 x 4096 14.1 -> 12.4 us;
  // 16-tile streams, two slices of 7 or 8, and the same on 8192 x 8192 or a 28672-wide layer are slower).
  // n-tiles per workgroup (at most 16 / wks).  A compute unit holds 16 of these wavefronts and as many workgroups as
  // its LDS allows.  First the fewest rounds of workgroups per compute unit, then the fewest wavefronts on the busiest
  // compute unit (i.e. spread over the device), then the smaller workgroup.
  auto pick_wn = [&](int wks_, int gs_, int sk_, long* rounds_out) {
    int best_wn = 1;
    long best_rounds = -1, best_waves = -1;
    const size_t lds_wg = decode2_lds_bytes(wks_, gs_ / TPG, c.mr, MB);
    for (int wn = 1; wn <= D2_WAVES / wks_; ++wn) {
      long slots = D2_WAVES / (wks_ * wn);
      const long lds_slots = (long)((size_t)(160 * 1024) / lds_wg);
      if (slots > lds_slots) slots = lds_slots;
      if (slots < 1) slots = 1;
      const long wgs = (long)((NT + wn - 1) / wn) * sk_;
      const long per_cu = (wgs + cus - 1) / cus;
      const long rounds = (per_cu + slots - 1) / slots;
      const long waves = (per_cu < slots ? per_cu : slots) * wn * wks_;
      if (best_rounds < 0 || rounds < best_rounds || (rounds == best_rounds && waves < best_waves)) {
        best_rounds = rounds;
        best_waves = waves;
        best_wn = wn;
      }
    }
    if (rounds_out) *rounds_out = best_rounds;
    return best_wn;
  };
  bool long_k_two_blocks = MB == 2 && NT <= cus && G >= 80 && sub == 1 && !w8 && nt_mult == 1;
  if (long_k_two_blocks) {
    // ... and only as one round of workgroups of 7 to 10 wavefronts that fill 85 % of the device (measured slower with
    // 4, 11 and 15 wavefronts: 14336 x 2048 10.3 -> 12.2 us, 16384 x 4096 14.2 -> 15.5 us, 24576 x 4096 18.9 -> 20.3 us)
    const int sk_b = (G + 13) / 14;
    long rounds_b = 0;
    const int wn_b = pick_wn(1, 14, sk_b, &rounds_b);
    const long wgs_b = (long)((NT + wn_b - 1) / wn_b) * sk_b;
    long_k_two_blocks = rounds_b == 1 && wn_b >= 7 && wn_b <= 10 && wgs_b * 100 >= (long)cus * 85;
  }
  if (long_k_two_blocks) wks = 1;
  if (tn.decode2_wks > 0) wks = tn.decode2_wks;
  int gs = long_k_two_blocks ? 14 : round_gs((gslab + wks - 1) / wks, sub, w8);
  if (tn.decode2_gs > 0) gs = tn.decode2_gs;
  while (wks * gs > slab_max && wks > 1) wks /= 2;     // respect the LDS limit
  if (gs > slab_max) {                                 // rounding up went past it: largest instantiated size below
    const int opts[] = {8, 7, 4, 2, 1};
    for (int o : opts)
      if (o <= slab_max && !(w8 && (o & 1)) && !(sub > 1 && (o & (o - 1)) != 0)) {
        gs = o;
        break;
      }
  }
  // Two slabs that twice the K slices would cover as one (at most 15 % of their tiles beyond K): one slab, no hand-over
  // between workgroups.  Cold, M = 1 / 4 / 16: 3584 x 37888 (16 + 12 groups) 20.3 / 27.8 / 23.2 -> 17.7 / 17.7 / 19.6 us,
  // 13824 x 5120 (64 + 44) 12.1 / 12.9 -> 11.0 / 11.9 us.
  if (MB == 1 && sub == 1 && !w8 && !long_k_two_blocks && tn.decode2_gs <= 0 && tn.decode2_wks <= 0 && exp_off(tn, 5) &&
      (G + wks * gs - 1) / (wks * gs) == 2 && wks * 2 <= 16) {
    const int g2 = round_gs((G + 2 * wks - 1) / (2 * wks), sub, w8);
    const int cover = 2 * wks * g2;
    if (cover >= G && cover <= slab_max && (cover - G) * 100 <= G * 15) {
      wks *= 2;
      gs = g2;
    }
  }
  // A last slab of less than 35 % of the others on a layer of at most two n-tiles per compute unit: the stream length
  // (same K slices) that leaves the fewest tiles beyond K, a further slab counted as 3 %.  Cold, M = 1 / 4: 9216 x 4608
  // (64 + 8 groups -> 3 x 28) 11.0 / 12.1 -> 8.9 / 9.3 us, 18944 x 3584 at M = 4 (64 + 64 + 20 -> 3 x 56) 13.5 -> 12.0 us; on
  // a wide layer the further slab costs more than it brings (5120 x 27648, 32 + 8 -> 3 x 14: +3 .. +13 %).
  if (MB == 1 && sub == 1 && !w8 && !long_k_two_blocks && tn.decode2_gs <= 0 && tn.decode2_wks <= 0 && exp_off(tn, 5) &&
      NT <= 2 * cus) {
    auto slabs = [&](int g) { return (G + wks * g - 1) / (wks * g); };
    const int sk0 = slabs(gs), last = G - (sk0 - 1) * wks * gs;
    if (sk0 >= 2 && last * 20 < wks * gs * 7) {
      auto score = [&](int g) { return (double)(slabs(g) * wks * g - G) / G + 0.03 * slabs(g); };
      int bg = gs;
      double best = score(gs);
      for (int g : {16, 14, 8, 7}) {
        if (wks * g > slab_max || slabs(g) > 10) continue;
        if (score(g) < best - 1e-9) { best = score(g); bg = g; }
      }
      gs = bg;
    }
  }
  // One slab whose streams reach 35 % and more beyond K (wavefronts without tiles) on a layer of at most 1.25 n-tiles per
  // compute unit: two or three slabs of streams of 7 tiles and more (the K slices as planned or half of them) that fit K
  // better.  Cold, M = 2 / 4 / 16: 5120 x 5120 (4 x 14 for 40 groups -> 3 slabs of 2 x 7) 7.9 / 7.9 / 8.6 -> 6.9 / 6.9 / 7.4 us,
  // 10240 x 2560 (8 x 14 for 80 -> 3 slabs of 4 x 7) 8.0 / 8.0 -> 6.8 / 6.9 us, 9216 x 2304 8.0 -> 6.8 us; wider layers lose with
  // it (2560 x 10240, 5120 x 15360: +20 .. +60 %), so do a single row (10240 x 4096: +18 %) and a K of 2560 (+11 .. +14 %);
  // 10240 x 4096 at M = 2 / 4 is 3 % slower with it.
  if (MB == 1 && sub == 1 && !w8 && !long_k_two_blocks && tn.decode2_gs <= 0 && tn.decode2_wks <= 0 && exp_off(tn, 5) &&
      c.mr >= 4 && G >= 32 && NT * 4 <= cus * 5 && wks <= 8 && wks * gs >= G && (wks * gs - G) * 100 >= G * 35) {
    auto slabs = [&](int w, int g) { return (G + w * g - 1) / (w * g); };
    auto score = [&](int w, int g) { return (double)(slabs(w, g) * w * g - G) / G + 0.03 * slabs(w, g); };
    int bw = wks, bg = gs;
    double best = score(wks, gs);
    for (int w : {wks, wks / 2}) {
      if (w < 1) continue;
      for (int g : {14, 8, 7}) {
        if (w * g > slab_max || slabs(w, g) > 3) continue;
        if (score(w, g) < best - 1e-9) { best = score(w, g); bw = w; bg = g; }
      }
    }
    wks = bw;
    gs = bg;
  }
  // the slab is now wks*gs groups; recompute the number of slabs
  c.sk = (G + wks * gs - 1) / (wks * gs);
  c.gs = gs;
  c.wks = wks;
  const size_t lds_wg = decode2_lds_bytes(wks, gs / TPG, c.mr, MB);
  const int best_wn = pick_wn(wks, gs, c.sk, nullptr);
  c.wn = tn.decode2_wn > 0 ? tn.decode2_wn : best_wn;
  if (c.wn * wks > D2_WAVES) c.wn = D2_WAVES / wks;
  // ring variant of long streams (instances exist for 4-bit codes in groups of 128 rows / channelwise, up to two
  // m-blocks): by the wavefronts that share a compute unit
  c.rc = 0;
  if (sub == 1 && !w8 && MB <= 2 && gs >= 7) {
    long slots = D2_WAVES / (wks * c.wn);
    const long lds_slots = (long)((size_t)(160 * 1024) / lds_wg);
    if (slots > lds_slots) slots = lds_slots;
    if (slots < 1) slots = 1;
    const long per_cu = ((long)((NT + c.wn - 1) / c.wn) * c.sk + cus - 1) / cus;
    const long waves_cu = (per_cu < slots ? per_cu : slots) * wks * c.wn;
    if (long_k_two_blocks && wks == 1 && gs == 14) c.rc = 1;
    else if (c.mr >= 8 && (gs >= 8 || waves_cu <= 8)) c.rc = 2;      // (7 tiles per wavefront, 16 wavefronts, 14336 x 4096 at M = 16: three slots 11.5 us, two 11.2 us)
    else if (waves_cu <= 8) c.rc = 1;
  }
  if (tn.exp[1] > 0) c.rc = tn.exp[1] - 1;      // (development switch: forced ring variant + 1)
  // 8 staged rows allow slabs twice as long, and a slab is a whole number of instantiated stream lengths: where that
  // leaves a last slab of less than 60 % of the others the workgroups of the full slabs set the pace, and the plan for
  // 16 staged rows (shorter, evener slabs) is taken instead (M = 8, cold: 10240 x 2560, slabs of 56 + 24 groups, 9.7 us
  // against 7.5 us; 5120 x 27648, 32 + 8, 23.2 against 20.8 us; 17920 x 6656, 4 x 32 + 12, 20.0 against 16.9 us)
  if (c.mr == 8 && c.sk > 1 && tn.decode2_gs <= 0 && tn.decode2_wks <= 0) {
    const int slab = c.wks * c.gs, last = G - (c.sk - 1) * slab;
    if (last * 10 < slab * 6) return pick_decode2_config(M, N, K, sub, w8, nt_mult, false);
  }
  return c;
}

template <bool BF16, int MB, bool HAS_ZP, int MR, int GS>
static int dispatch_rc2(const Decode2Params& p, int rc, hipStream_t s) {
  if (rc == 1) return launch_decode2<BF16, GS, MB, HAS_ZP, MR, 1, 0, 1>(p, s);
  if (rc == 2) return launch_decode2<BF16, GS, MB, HAS_ZP, MR, 1, 0, 2>(p, s);
  if (rc == 3) return launch_decode2<BF16, GS, MB, HAS_ZP, MR, 1, 0, 3>(p, s);
  return launch_decode2<BF16, GS, MB, HAS_ZP, MR, 1>(p, s);
}

template <bool BF16, int MB, bool HAS_ZP, int MR>
static int dispatch_gs2(const Decode2Params& p, int gs, int rc, hipStream_t s) {
  switch (gs) {
    case 1: return launch_decode2<BF16, 1, MB, HAS_ZP, MR, 1>(p, s);
    case 2: return launch_decode2<BF16, 2, MB, HAS_ZP, MR, 1>(p, s);
    case 4: return launch_decode2<BF16, 4, MB, HAS_ZP, MR, 1>(p, s);
    case 7: return dispatch_rc2<BF16, MB, HAS_ZP, MR, 7>(p, rc, s);
    case 8: return dispatch_rc2<BF16, MB, HAS_ZP, MR, 8>(p, rc, s);
    case 14: return dispatch_rc2<BF16, MB, HAS_ZP, MR, 14>(p, rc, s);
    case 16: return dispatch_rc2<BF16, MB, HAS_ZP, MR, 16>(p, rc, s);
    default: break;
  }
  set_error("w4a16_gemm(decode): unsupported groups per wavefront %d", gs);
  return VAQ_ERR_UNSUPPORTED;
}

template <int MB, int MR>
static int dispatch_types2(const Decode2Params& p, int gs, int rc, bool bf16, bool zp, hipStream_t s) {
  if (bf16) return zp ? dispatch_gs2<true, MB, true, MR>(p, gs, rc, s) : dispatch_gs2<true, MB, false, MR>(p, gs, rc, s);
  return zp ? dispatch_gs2<false, MB, true, MR>(p, gs, rc, s) : dispatch_gs2<false, MB, false, MR>(p, gs, rc, s);
}

template <int MB>
static int dispatch_mr2(const Decode2Params& p, const Decode2Config& c, bool bf16, bool zp, hipStream_t s) {
  switch (c.mr) {
    case 1: return dispatch_types2<MB, 1>(p, c.gs, c.rc, bf16, zp, s);
    case 4: return dispatch_types2<MB, 4>(p, c.gs, c.rc, bf16, zp, s);
    case 8:
      if constexpr (MB == 1) return dispatch_types2<MB, 8>(p, c.gs, c.rc, bf16, zp, s);
      [[fallthrough]];
    default: return dispatch_types2<MB, 16>(p, c.gs, c.rc, bf16, zp, s);
  }
}

// Rows split over workgroups (one m-block each, see the kernel) instead of several m-blocks per workgroup: 4-bit codes
// in groups of 128 rows / channelwise, no act_order, and only where a single m-block needs no split of K.  On success
// `out` is the configuration of the one-m-block kernel that every workgroup runs.
// (development switch exp[2]: 1 forces it off, 2 on wherever it is built)
static bool row_split_config(int M, int N, int K, int sub, int wt, bool has_perm, Decode2Config* out) {
  if (M <= 16 || sub != 1 || wt != 0 || has_perm || tuning().exp[2] == 1) return false;
  const int MB = (M + 15) / 16, NT = N / 16;
  Decode2Config c = pick_decode2_config(16, N, K, sub, false, MB);
  if (c.sk != 1) return false;
  *out = c;
  if (tuning().exp[2] == 2) return true;
  const long cus = num_cus_current_device();
  if (M <= DECODE2_MAX_M) {
    // Against two to four m-blocks in one workgroup: one round of full workgroups.  Measured: 4096 x 4096 at M = 32 / 64:
    // 8.5 / 10.5 -> 6.6 / 9.2 us, 4096 x 6144: 8.8 / 11.4 -> 8.7 / 10.6 us; with three m-blocks the grids of those layers spill
    // into a second round (15 us) or leave ten wavefronts per workgroup (9.9 -> 11.7 us).  A 28672-wide layer would need
    // streams of 32 tiles (measured 20.4 -> 21.7 us).
    // (Two m-blocks also as eight wavefronts of 8-tile streams with the three-slot ring: 4096 x 4096 at M = 32 6.3 us.)
    const long wgs = (long)((NT + c.wn - 1) / c.wn) * MB;
    return wgs <= cus && c.wks * c.wn >= (M <= 32 ? 8 : 12);
  }
  // Five to sixteen m-blocks, against the tile kernel (whose K step is a latency chain of half a microsecond at these
  // sizes): the fewest n-tiles per workgroup whose grid -- counted exactly -- is one round of workgroups with at least 12
  // wavefronts on a compute unit.  Cold: 4096 x 4096 at M = 128 16.2 -> 13.4 us, 4096 x 6144 at M = 80 18.8 -> 13.5 us,
  // 4096 x 2048 at M = 128 / 256 14.8 / 16.0 -> 8.8 / 13.2 us, 2048 x 2048 at M = 128 / 256 11.5 / 12.5 -> 6.3 / 8.3 us; grids
  // of a second round lose (4096 x 4096 at M = 96 with 258 workgroups: 16.1 -> 22.3 us), ten wavefronts too (M = 80: 20.2 us).
  // (An odd number of n-tiles gives way to the next even one where that grid passes too: seven n-tiles -- 14 wavefronts and
  // a ragged last workgroup -- measured 15-20 % behind eight, 4096 x 4096 at M = 96 15.6 against 13.3 us, 4096 x 2048 at
  // M = 192 / 208 15.4 / 15.7 against 13.1 us, and five behind six, 2048 x 2048 at M = 144 9.0 against 7.6 us.)
  const long lds_slots = (long)((size_t)(160 * 1024) / decode2_lds_bytes(c.wks, c.gs, c.mr, 1));
  auto passes = [&](int wn) {
    if (wn * c.wks > D2_WAVES) return false;
    long slots = D2_WAVES / (c.wks * wn);
    if (slots > lds_slots) slots = lds_slots;
    if (slots < 1) slots = 1;
    const long wgs = (long)((NT + wn - 1) / wn) * MB;
    const long per_cu = (wgs + cus - 1) / cus;
    return per_cu <= slots && per_cu * c.wks * wn >= 12;
  };
  for (int wn = 1; wn * c.wks <= D2_WAVES; ++wn) {
    if (tuning().decode2_wn > 0 && wn != tuning().decode2_wn) continue;
    if (!passes(wn)) continue;
    if (tuning().decode2_wn <= 0 && wn >= 3 && (wn & 1) && passes(wn + 1)) continue;
    out->wn = wn;
    return true;
  }
  return false;
}

bool w4a16_decode2_takes_rows(int M, int N, int K, int sub, int wt, bool has_perm) {
  Decode2Config c;
  return M > DECODE2_MAX_M && M <= DECODE2_MAX_M_ROWS && row_split_config(M, N, K, sub, wt, has_perm, &c);
}

int decode2_launch_msp(const Decode2Params& p, int gs, int rc, bool bf16, bool zp, hipStream_t s);      // w4a16_decode2_msp.hip

int w4a16_decode2_workspace(int M, int N, int K, int sub, bool w8, size_t* c_tmp_bytes, size_t* counter_ints) {
  const Decode2Config c = pick_decode2_config(M, N, K, sub, w8);
  const int MB = (M + 15) / 16;
  const int NT = N / 16;
  *c_tmp_bytes = c.sk > 1 ? (size_t)c.sk * NT * MB * 64 * sizeof(v4f) : 0;
  *counter_ints = c.sk > 1 ? (size_t)NT * MB : 0;
  return VAQ_OK;
}

int w4a16_decode2_launch(const void* a, int64_t lda, const int32_t* b, const void* scales, const int32_t* zeros,
                         const int32_t* perm, const void* bias, void* c, float* c_tmp, int64_t c_tmp_bytes,
                         int32_t* counters, int64_t counter_ints, int M, int N, int K, int sub, bool channelwise,
                         int wt, int dtype, hipStream_t s) {
  const bool w8 = wt != 0;      // 8-bit weights of either kind (1: nibble planes, 2: FP8 bytes): two blocks per 128 rows
  Decode2Params p;
  p.a = (const uint16_t*)a;
  p.lda = lda;
  p.b = (const v4u*)b;
  p.scales = (const uint16_t*)scales;
  p.zeros = (const uint32_t*)zeros;
  p.perm = perm;
  p.bias = (const uint16_t*)bias;
  p.c = (uint16_t*)c;
  p.c_tmp = c_tmp;
  p.counters = counters;
  p.M = M; p.N = N; p.K = K;
  p.G = K / 128 * (w8 ? 2 : 1);
  p.NT = N / 16;
  p.GR = channelwise ? 1 : K / 128 * sub;
  p.s_stride = channelwise ? 0 : N;
  p.z_stride = channelwise ? 0 : N / 8;
  p.k_mask = 0x000f000fu;
  p.k_ex = dtype == VAQ_BF16 ? 0x43004300u : 0x64006400u;
  Decode2Config cfg;
  const bool row_split = row_split_config(M, N, K, sub, wt, perm != nullptr, &cfg);
  if (!row_split) {
    VAQ_CHECK_ARG(M <= DECODE2_MAX_M, "w4a16_gemm(decode): %d rows without the split of the rows over workgroups", M);
    cfg = pick_decode2_config(M, N, K, sub, w8);
  }
  p.SK = cfg.sk;
  p.WKS = cfg.wks;
  p.WN = cfg.wn;
  // private activation fill (see the kernel): measured ahead only on short streams with few staged rows (4096 x 4096 at
  // M = 1 / 4: 4.53 / 4.83 -> 4.38 / 4.52 us; 14336 x 4096 at M = 4: 9.1 -> 9.3 us; with 16 staged rows, where every
  // wavefront would fetch 16 rows of its own slice: 4096 x 4096 at M = 16 5.39 -> 5.47 us, 14336 x 4096 11.08 -> 11.07 us)
  p.PRIV = (cfg.wn == 1 && perm == nullptr && cfg.mr <= 4 && cfg.gs <= 8 && tuning().exp[0] != 1) ? 1 : 0;
  const int MB = (M + 15) / 16;
  if (cfg.sk > 1) {
    VAQ_CHECK_ARG(c_tmp != nullptr && counters != nullptr, "w4a16_gemm: split-K needs c_tmp and counters");
    VAQ_CHECK_ARG(((uintptr_t)c_tmp % 16) == 0, "w4a16_gemm: c_tmp must be 16-byte aligned");
    VAQ_CHECK_ARG((uint64_t)cfg.sk * (uint64_t)p.NT * MB * 1024u < (1ull << 31), "w4a16_gemm: split-K scratch too large");
    VAQ_CHECK_ARG(counter_ints >= (int64_t)p.NT * MB,
                  "w4a16_gemm: workspace.numel = %lld is below min_workspace_size = %lld", (long long)counter_ints,
                  (long long)p.NT * MB);
    VAQ_CHECK_ARG(c_tmp_bytes >= (int64_t)cfg.sk * p.NT * MB * 1024, "w4a16_gemm: c_tmp holds %lld bytes, the K split needs %lld",
                  (long long)c_tmp_bytes, (long long)cfg.sk * p.NT * MB * 1024);
  }
  const bool bf16 = dtype == VAQ_BF16, zp = zeros != nullptr;
  int rc;
  if (row_split) rc = decode2_launch_msp(p, cfg.gs, cfg.rc, bf16, zp, s);
  else if (wt == 2) rc = decode2_launch_f8(p, cfg.gs, MB, cfg.mr, bf16, s);
  else if (w8 && sub > 1) rc = decode2_launch_w8sub(p, sub, cfg.gs, MB, cfg.mr, bf16, s);
  else if (w8) rc = decode2_launch_w8(p, cfg.gs, MB, cfg.mr, bf16, s);
  else if (sub == 2) rc = decode2_launch_sub2(p, cfg.gs, MB, cfg.mr, bf16, zp, s);
  else if (sub == 4) rc = decode2_launch_sub4(p, cfg.gs, MB, cfg.mr, bf16, zp, s);
  else if (MB > 2) rc = decode2_launch_mb34(p, cfg.gs, MB, bf16, zp, s);
  else if (MB == 1) rc = dispatch_mr2<1>(p, cfg, bf16, zp, s);
  else rc = dispatch_types2<2, 16>(p, cfg.gs, cfg.rc, bf16, zp, s);
  if (rc != VAQ_OK) return rc;
  VAQ_CHECK_LAUNCH("w4a16_gemm(decode)");
  return VAQ_OK;
}

}  // namespace vaq

// Host side of the prefill kernels (w4a16_prefill_kernel.h): tile and K-split choice, workspace sizes, launch of the
// instances for quantisation groups of 128 rows and channelwise scales.
#include "w4a16_prefill_kernel.h"

namespace vaq {

// ----------------------------------------------------------------------------- host side

// tile ids: 0..2 = register-staged kernel (256x256, 128x128, 64x128); 10.. = direct-to-LDS kernel (BM x BN);
// 30 = 256 x 256 with the weights dequantised in registers (w4a16_prefill3_kernel.h)
int prefill_launch_reg(const PrefillParams& p, bool bf16, bool zp, hipStream_t s);      // w4a16_prefill3.hip

template <bool BF16, bool HAS_ZP>
static int dispatch_tile(const PrefillParams& p, int tile, hipStream_t s) {
  switch (tile) {
    case 10: return launch_prefill2<BF16, 256, 256, 2, 4, HAS_ZP, 1>(p, s);   // 8 wavefronts, 128 x 64 each
    case 20: return launch_prefill2<BF16, 256, 256, 2, 4, HAS_ZP, 1, false, true>(p, s);   // the same, alternating phases
    case 30: return prefill_launch_reg(p, BF16, HAS_ZP, s);                                // 4 wavefronts, 256 x 64 each
    case 11: return launch_prefill2<BF16, 256, 256, 2, 2, HAS_ZP, 1>(p, s);   // 4 wavefronts, 128 x 128 each
    case 12: return launch_prefill2<BF16, 128, 128, 2, 2, HAS_ZP, 1>(p, s);   // 4 wavefronts, 64 x 64 each
    case 13: return launch_prefill2<BF16, 128, 256, 2, 4, HAS_ZP, 1>(p, s);   // 8 wavefronts, 64 x 64 each
    case 14: return launch_prefill2<BF16, 64, 128, 2, 2, HAS_ZP, 1>(p, s);    // 4 wavefronts, 32 x 64 each
    case 15: return launch_prefill2<BF16, 128, 64, 2, 2, HAS_ZP, 1>(p, s);    // 4 wavefronts, 64 x 32 each
    case 0: return launch_prefill<BF16, 4, 4, HAS_ZP, 1>(p, s);   // 256 x 256
    case 1: return launch_prefill<BF16, 2, 2, HAS_ZP, 1>(p, s);   // 128 x 128
    case 2: return launch_prefill<BF16, 1, 2, HAS_ZP, 1>(p, s);   //  64 x 128
    default: break;
  }
  set_error("w4a16_gemm(prefill): unknown tile id %d", tile);
  return VAQ_ERR_UNSUPPORTED;
}

// Splits of K for the 256 x 256 tile (one workgroup per compute unit): as many as bring the workgroup count to one per
// compute unit, every split at least 28 groups (3584 rows) long -- 16 groups on a K of up to 4096, so that it can run in
// two parts (72 .. 127 tiles: 4096 x 6144 at M = 768 / 1024 73.8 / 75.2 -> 62.8 / 68.8 us, 4096 x 4096 at M = 1280 / 1536
// 73.9 / 76.1 -> 64.7 / 68.8 us, against the 128 x 128 tiles that ran there).
static int splits_256(int64_t tiles256, int K, int cus) {
  const int G = K / 128, min_groups = G <= 32 ? 16 : 28;
  int sk = (int)(cus / (tiles256 > 0 ? tiles256 : 1));
  if (sk > G / min_groups) sk = G / min_groups;
  return sk < 1 ? 1 : (sk > 8 ? 8 : sk);
}

static int pick_tile(int M, int N, int K, bool direct_ok, bool reg_ok) {
  if (tuning().prefill_tile > 0) return tuning().prefill_tile - 1;
  const int cus = num_cus_current_device();
  auto tiles = [&](int bm, int bn) { return (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  if (direct_ok) {
    // measured: the 256x256 / 8-wavefront tile wins as soon as it fills ~55 % of the compute units, also when it
    // takes a split of a long K to get there (14336 x 4096 at M = 1024 / 2048: 4 % / 21 % faster than 128 x 128)
    // (from 55 % on: 4096 x 6144 at M = 1536, 144 tiles, 112 -> 85 us; at 50 %, 4096 x 4096 at M = 2048, 76 against 85 us)
    // (not for a single tile row that M fills at most half: 8192 x 28672 at M = 128, 104 against 85 us with 128 x 128)
    // (... nor when M fills less than 70 % of the 256-row tiles and the 128 x 128 tiles fit the device in one round of two
    // workgroups per compute unit: 3584 x 18944 at M = 288 / 320, 444 tiles, 78 -> 63 us; on 4096 x 28672, 672 tiles, the
    // 256 x 256 tiles stay ahead, 90 against 108 us)
    const bool rows_poorly_filled = (int64_t)M * 10 < (int64_t)((M + 255) / 256) * 256 * 7 && tiles(128, 128) <= 2 * (int64_t)cus &&
                                    tuning().exp[9] != 1;
    // 128 x 256 tiles (8 wavefronts of 64 x 64) where they fill 85-100 % of the compute units in one round on a short K:
    // no K split and so no hand-over (4096 x 4096 at M = 1792 / 2048: 75.3 / 82.0 us for 256 x 256 tiles in two parts,
    // 73.6 / 78.5 us for these; 4096 x 6144 at M = 1280: 79.9 against 76.2 us; on K = 14336 they lose, 232 against 200 us)
    // (built for 4-bit codes in groups of 128 rows / channelwise, like the register-dequantising kernel: `reg_ok`)
    if (reg_ok && M > 128 && K <= 4096 && tiles(128, 256) <= cus && tiles(128, 256) * 20 >= (int64_t)cus * 17 && tuning().exp[11] != 1) return 13;
    if (M > 128 && !rows_poorly_filled && tiles(256, 256) * splits_256(tiles(256, 256), K, cus) * 20 >= cus * 11) {
      // 256 x 256.  With at least one tile per compute unit and K unsplit, the kernel that dequantises in registers (four
      // wavefronts of 256 x 64) is 1-4 % ahead at M = 4096 on the four Llama-3-8B layers (206 / 123 / 807 / 400 -> 205 / 121 /
      // 792 / 384 us); with fewer tiles or a split K the 8-wavefront kernel with alternating phases is (its second
      // wavefront per SIMD covers the waits of the first: 14336 x 4096 at M = 512, 95.8 against 102.5 us).  `reg_ok`: 4-bit
      // codes in groups of 128 rows or channelwise -- what the register kernel is built for.
      return (reg_ok && tiles(256, 256) >= cus) ? 30 : 20;
    }
    // An odd number of 64-row blocks on a short K: 64 x 128 tiles (the last 128-row tile would be half empty) where they
    // come to 80-100 % of one or of two workgroups per compute unit (cold: 3584 x 18944 at M = 136 .. 192, 444 tiles, 60 ->
    // 45 us; 2560 x 10240, 240 tiles, 30.8 -> 22.6 us; 4096 x 11008 at M = 288 / 320, 430 tiles, 67 -> 50 us; with 258 or
    // 324 tiles they lose 15-20 %, and on K = 8192 as well)
    // (three or five blocks; with seven or nine the half-empty tile is a tenth of the rows and these tiles lose 6-9 %)
    if (M > 64 && M <= 320 && ((M + 63) / 64) % 2 == 1 && K <= 4096) {
      const int64_t t = tiles(64, 128);
      if ((t * 5 >= (int64_t)cus * 4 && t <= cus) || (t * 5 >= (int64_t)cus * 8 && t <= 2 * (int64_t)cus)) return 14;
    }
    if (tiles(128, 128) >= cus) return 12;
    // Few tiles: 64 x 128, or 128 x 64 once M fills more than one 64-row tile (the dequantisation of a weight tile is
    // then shared by twice as many rows: 7-15 % faster at M = 128 .. 768 on the narrow layers); K is split over
    // workgroups when the tiles leave units idle.  Measured on the Llama shapes, M = 80 .. 1280, cold weights:
    //  * 128 x 128 where the 128 x 64 tiles fill the device or need a second round and these fill half of it (4096 x 6144 at
    //    M = 384: 44.5 -> 33.7 us; 4096 x 4096 at M = 640: 44.3 -> 34.9 us), and on a long K from 3/8 of the device on
    //    (14336 x 4096 at M = 320 .. 512: 79 .. 88 -> 61 .. 79 us);
    //  * 64 x 128 where an odd number of 64-row blocks would leave the last 128-row tile half empty (4096 x 6144 at
    //    M = 192: 28.2 -> 23.4 us; 4096 x 4096 at M = 320: 28.1 -> 23.5 us).
    // (M beyond one 64-row block: with 64 rows or fewer the 128-row tiles are half empty -- 4096 x 28672 at M = 64, 224 tiles
    // of either size: 48.1 us against 36.6 us for 64 x 128 tiles in two K parts)
    if (M > 64 && ((tiles(128, 64) >= cus && tiles(128, 128) * 2 >= cus) || (K >= 8192 && tiles(128, 128) * 8 >= (int64_t)cus * 3))) return 12;
    if (M > 64 && ((M + 63) / 64) % 2 == 1 && tiles(64, 128) <= cus) return 14;
    if (M > 64 && tuning().exp[8] != 1) {
      // 128 x 64 tiles whose K parts (two workgroups per compute unit, at most 8 parts of at least 8 groups) would still
      // run 24 groups and more: 128 x 128 tiles, half as many, in twice the parts, where that is at least 80 % as many
      // workgroups (cold: 28672 x 8192 at M = 80 .. 128 92 -> 81 us, 22016 x 4096 at M = 256 74 -> 67 us, 12288 x 3072 at
      // M = 384 50.6 -> 46.5 us, 13824 x 5120, 18944 x 3584, 6656 x 6656, 7168 x 7168 at M = 256 -5 .. -7 %; 12288 x 3072 at
      // M = 640 +4 %)
      auto parts = [&](int64_t t) {
        int sk = (int)((2 * (int64_t)cus) / t);
        if (sk > 8) sk = 8;
        if (sk > K / 128 / 8) sk = K / 128 / 8;
        return sk < 1 ? 1 : sk;
      };
      const int64_t t15 = tiles(128, 64), t12 = tiles(128, 128);
      if (t15 < cus && K / 128 / parts(t15) >= 24 && t12 * parts(t12) * 10 >= t15 * parts(t15) * 8) return 12;
    }
    return M > 64 ? 15 : 14;
  }
  if (tiles(256, 256) >= cus) return 0;
  if (tiles(128, 128) >= cus) return 1;
  return 2;
}

struct PrefillPlan {
  int tile, sk, bm, bn, nw;
  int64_t tiles;
  int64_t tail_first;      // > 0: only the tiles from this position on are split (tile_handover.h)
  // scratch of the K split: partial tiles and arrival counters of the tiles that are split
  int64_t split_tiles() const { return sk > 1 ? tiles - tail_first : 0; }
  int64_t tmp_bytes() const { return (int64_t)sk * split_tiles() * bm * bn * 4; }
  int64_t counter_ints() const { return split_tiles() * nw; }
};

// Tile shape and K split for a problem.  K is split (direct-to-LDS tiles only) when the output tiles alone leave
// compute units idle: as many splits as bring the workgroup count to about two per compute unit, at most 8, every
// split at least 8 groups (16 K steps) long, 32 groups when the tiles already fill the device -- measured on the Llama
// shapes for M = 48 .. 512.
static PrefillPlan plan_prefill(int M, int N, int K, bool direct_ok, bool reg_ok = false) {
  PrefillPlan pl;
  pl.tile = pick_tile(M, N, K, direct_ok, reg_ok);
  switch (pl.tile) {
    case 10: case 20: pl.bm = 256; pl.bn = 256; pl.nw = 8; break;
    case 11: case 30: pl.bm = 256; pl.bn = 256; pl.nw = 4; break;
    case 12: pl.bm = 128; pl.bn = 128; pl.nw = 4; break;
    case 13: pl.bm = 128; pl.bn = 256; pl.nw = 8; break;
    case 14: pl.bm = 64; pl.bn = 128; pl.nw = 4; break;
    case 15: pl.bm = 128; pl.bn = 64; pl.nw = 4; break;
    default: pl.bm = 0; pl.bn = 0; pl.nw = 0; break;
  }
  pl.sk = 1;
  pl.tiles = 0;
  pl.tail_first = 0;
  if (pl.bm == 0) return pl;
  pl.tiles = (int64_t)((M + pl.bm - 1) / pl.bm) * ((N + pl.bn - 1) / pl.bn);
  const int cus = num_cus_current_device();
  const int G = K / 128;
  int sk = 1;
  if (pl.bm == 256 && pl.bn == 256 && (pl.nw == 8 || pl.tile == 30)) {
    sk = splits_256(pl.tiles, K, cus);
  } else if (pl.tiles < 2 * (int64_t)cus) {
    sk = (int)((2 * (int64_t)cus) / pl.tiles);
    if (sk > 8) sk = 8;
    const int min_groups = pl.tiles < cus ? 8 : 32;     // a device already full of tiles only splits a very long K
    if (sk > G / min_groups) sk = G / min_groups;
    if (sk < 1) sk = 1;
    // A short K on few tiles (what the 8-group minimum leaves unsplit or nearly so): parts of at least 3 groups, up to
    // one workgroup per compute unit.  Cold weights, M = 96 .. 512: 1536 x 1536 15.4 -> 10.4 .. 12.7 us, 2048 x 2048 at
    // M = 128 / 256 13.7 / 14.1 -> 11.3 / 12.4 us, 2560 x 2560 15.8 / 16.2 / 20.7 -> 12.5 / 14.0 / 18.2 us, 1024 x 4096 at
    // M = 128 11.6 -> 10.6 us (finer parts than these lose again: 1536 x 1536 at M = 256 in 6 parts 13.1 us).
    if (pl.tiles * 2 < (int64_t)cus) {
      int fine = (int)((int64_t)cus / pl.tiles);
      if (fine > 8) fine = 8;
      if (fine > G / 3) fine = G / 3;
      if (fine > sk) sk = fine;
    }
    // 128 x 256 tiles that fill a round of workgroups on their own (what the automatic choice takes them for) stay whole
    if (pl.tile == 13 && pl.tiles <= cus && pl.tiles * 20 >= (int64_t)cus * 17) sk = 1;
  }
  // 256 x 256 tiles (one workgroup per compute unit) whose count ends in a round of workgroups that is at most half full:
  // the tiles of that round are split over K so that their parts fill it, the others stay whole (4096 x 6144 at M = 4096:
  // 384 tiles = 256 whole + 128 in two parts each, 205 -> 189 us; M = 3072, 256 + 32 in four parts, 196 -> 156 us;
  // 14336 x 4096 at M = 5120: 662 -> 509 us; 4096 x 28672 at M = 2560, 1024 + 96 in two parts: 542 -> 516 us).  The gain is
  // less than the rounds saved: a half-empty round runs faster per workgroup than a full one (the device is
  // power-limited), and the parts' hand-over costs 15 us.  Parts of at least 8 groups.
  if (sk == 1 && pl.bm == 256 && pl.bn == 256 && pl.tiles > cus && tuning().exp[10] != 1 && tuning().prefill_split <= 0) {
    const int64_t rest = pl.tiles % cus;
    if (rest > 0 && rest * 2 <= cus && G >= 16) {
      int parts = (int)(cus / rest);
      if (parts > 4) parts = 4;
      if (parts > G / 8) parts = G / 8;
      if (parts >= 2) {
        sk = parts;
        pl.tail_first = pl.tiles - rest;
        // (the parts run on the 8-wavefront kernel: short K ranges suit the register-dequantising one badly -- 4096 x 6144
        // at M = 4096: 205 -> 189 us against 207 -> 210 us; 4096 x 4096 at M = 4352: 195 -> 154 against 206 -> 176 us)
        if (pl.tile == 30 && tuning().prefill_tile <= 0) {
          pl.tile = 20;
          pl.nw = 8;
        }
      }
    }
  }
  if (tuning().prefill_split > 0) sk = tuning().prefill_split <= G ? tuning().prefill_split : G;
  while (sk > 1 && (uint64_t)sk * (uint64_t)(pl.tiles - pl.tail_first) * pl.bm * pl.bn * 4 >= (1ull << 32)) --sk;   // 32-bit buffer offsets
  pl.sk = sk;
  if (sk == 1) pl.tail_first = 0;
  return pl;
}

int w4a16_prefill_workspace(int M, int N, int K, size_t* c_tmp_bytes, size_t* counter_ints) {
  const PrefillPlan pl = plan_prefill(M, N, K, true);
  *c_tmp_bytes = (size_t)pl.tmp_bytes();
  *counter_ints = (size_t)pl.counter_ints();
  return VAQ_OK;
}

int w4a16_prefill_launch(const void* a, int64_t lda, const int32_t* b, const void* scales, const int32_t* zeros,
                         const void* bias, void* c, float* c_tmp, int64_t c_tmp_bytes, int32_t* counters,
                         int64_t counter_ints, int M, int N, int K, int sub, bool channelwise, int wt, int dtype,
                         hipStream_t s) {
  const bool w8 = wt != 0;      // 8-bit weights of either kind: two 1 KiB blocks per tile
  PrefillParams p;
  p.a = (const uint16_t*)a;
  p.lda = lda;
  p.b = (const v4u*)b;
  p.scales = (const uint16_t*)scales;
  p.zeros = (const uint32_t*)zeros;
  p.bias = (const uint16_t*)bias;
  p.c = (uint16_t*)c;
  p.c_tmp = c_tmp;
  p.counters = counters;
  p.M = M; p.N = N; p.K = K;
  p.G = K / 128;
  p.NT = N / 16;
  p.s_stride = channelwise ? 0 : N;
  p.z_stride = channelwise ? 0 : N / 8;
  const bool direct_ok = (uint64_t)M * (uint64_t)lda * 2 < (1ull << 32);
  if (w8 && !direct_ok) {
    set_error("w4a16_gemm(prefill): 8-bit weights with an A of 4 GiB or more are not built");
    return VAQ_ERR_UNSUPPORTED;
  }
  PrefillPlan pl = plan_prefill(M, N, K, direct_ok, !w8 && sub == 1);
  // A caller that passes no scratch at all gets the unsplit kernel (same result, no K split); scratch that is there but
  // too small is the caller's mistake and is reported, not worked around.
  if (pl.sk > 1 && c_tmp == nullptr && counters == nullptr) pl.sk = 1;
  // Splitting only the tiles of a half-empty last round is an optimisation that whole tiles replace at no other cost than
  // time: scratch that does not hold it (the library-owned scratch of the no-allocation entry point, say) switches it off.
  if (pl.sk > 1 && pl.tail_first > 0 && (c_tmp_bytes < pl.tmp_bytes() || counter_ints < pl.counter_ints())) pl.sk = 1;
  if (pl.sk == 1) pl.tail_first = 0;
  if (pl.sk > 1) {
    const int64_t need_tmp = pl.tmp_bytes(), need_cnt = pl.counter_ints();
    VAQ_CHECK_ARG(c_tmp != nullptr && counters != nullptr, "w4a16_gemm: split-K needs both c_tmp and counters");
    VAQ_CHECK_ARG(counter_ints >= need_cnt, "w4a16_gemm: workspace.numel = %lld is below min_workspace_size = %lld",
                  (long long)counter_ints, (long long)need_cnt);
    VAQ_CHECK_ARG(c_tmp_bytes >= need_tmp, "w4a16_gemm: c_tmp holds %lld bytes, the K split needs %lld",
                  (long long)c_tmp_bytes, (long long)need_tmp);
  }
  p.SK = pl.sk;
  p.tail_first = (int)pl.tail_first;
  const bool bf16 = dtype == VAQ_BF16, zp = zeros != nullptr;
  int rc;
  // the alternating-phase and the register-dequantising variants exist for 4-bit codes in groups of 128 rows / channelwise
  const int tile_other = (pl.tile == 20 || pl.tile == 30) ? 10 : pl.tile;
  if (wt == 2) rc = prefill_launch_f8(p, tile_other, bf16, s);
  else if (w8) rc = prefill_launch_w8(p, sub, tile_other, bf16, s);
  else if (sub > 1) rc = prefill_launch_sub(p, sub, tile_other, bf16, zp, s);
  else if (bf16) rc = zp ? dispatch_tile<true, true>(p, pl.tile, s) : dispatch_tile<true, false>(p, pl.tile, s);
  else rc = zp ? dispatch_tile<false, true>(p, pl.tile, s) : dispatch_tile<false, false>(p, pl.tile, s);
  if (rc != VAQ_OK) return rc;
  VAQ_CHECK_LAUNCH("w4a16_gemm(prefill)");
  return VAQ_OK;
}

}  // namespace vaq

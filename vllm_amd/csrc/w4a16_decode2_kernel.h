// W4A16 decode-shaped GEMM (M <= 32), barrier-free variant: activations staged in LDS, one independent task per
// wavefront.  C[M,N] = A[M,K] . dequant(B[K,N]) (+bias), same arithmetic as w4a16_decode.hip.
//
//  * A workgroup is WKS slices of K  x  WN n-tiles (16 columns each) = up to 16 wavefronts.  Wavefront (wks, wn)
//    streams the GS consecutive 1 KiB weight tiles (= quantisation groups) of its slice for its n-tile through a
//    register ring of min(GS, 2) slots; no wavefront ever waits for another one inside the K loop.
//  * The activations of the workgroup's K slab (WKS*GS groups) are staged once in LDS by direct-to-LDS loads, row-major
//    with the 16-byte chunks XOR-swizzled inside aligned 256-byte blocks (rows m >= M zero; both the 1 KiB fill
//    pieces and the operand reads are bank-conflict free) and read back with one ds_read_b128 per MFMA.  The activation
//    loads are issued before the first weight loads (see step 1).  Only MR rows per m-block are staged
//    (MR = 1, 4 or 16, the smallest that holds M): MFMA columns are independent, so lanes of the columns m >= MR read
//    the slot of row m mod MR and their results are never stored.  With few rows a whole K = 14336 slab fits LDS and
//    K need not be split over workgroups.
//  * Per tile: 4 x { dequantise one word to 8 biased 16-bit numbers (7 VALU ops), MFMA with the activations, MFMA of
//    the constant operand -(BIAS + zero) with the same activations }, then acc += scale * P (fp32).  The second MFMA
//    removes the bias and the zero point exactly as `P - (BIAS+z)*S` would, without keeping S anywhere.
//  * Quantisation groups of 64 or 32 rows (SUBG = 2 or 4 groups per tile): the same, per sub-group of 2 or 1 MFMA pairs.
//    Channelwise scales are one row read with a row stride of 0.
//  * 8-bit codes (W8, symmetric, bias 128): the weights come as two 4-bit planes per tile (high nibbles, then low
//    nibbles), code - 128 = 16 * (hi - 8) + lo.  Each plane is one tile of the stream, multiplied with the same
//    activations; the high plane uses the constant operand -(BIAS + 8) and 16 * scale, the low plane -(BIAS + 0).
//  * FP8 e4m3 weights (WT = 2, 16-bit activations): whole bytes, two 1 KiB blocks per tile (MFMAs 0,1 and 2,3), each byte
//    pair turned into two 16-bit numbers by one packed conversion; no bias or zero point, so one MFMA per operand.
//  * WKS > 1: one LDS reduction at the end (wavefronts wks == 0 sum their column's slices).  K slabs that do not fit
//    LDS (SK > 1 workgroups per n-tile) hand partial tiles over through device-scope write-through stores and an
//    arrival counter, summed in fixed order by the last arriver.
#pragma once
#include "vaq_common.h"

#include <type_traits>

namespace vaq {

struct Decode2Params {
  const uint16_t* a;
  int64_t lda;
  const v4u* b;
  const uint16_t* scales;
  const uint32_t* zeros;
  const int32_t* perm;
  const uint16_t* bias;
  uint16_t* c;
  float* c_tmp;
  int32_t* counters;
  int M, N, K, G, NT, SK, WKS, WN, PRIV;   // PRIV: private activation fill (see the kernel; needs WN == 1, no perm); G: weight tiles along K per 16-column strip (K/128, twice that for 8-bit codes)
  int GR;                  // rows of the scale / zero-point tensors (G * SUBG, or 1 for channelwise scales)
  int s_stride, z_stride;  // elements between consecutive rows of scales (N) / zeros (N/8); 0 for channelwise
  uint32_t k_mask, k_ex;   // 0x000f000f and the exponent pattern, passed as run-time values (see and_or)
  // Set by the launcher (it knows the template arguments): the divisions of the kernel's first instructions, done on
  // the host.  x / WN = (x * wn_magic) >> 16 for a wavefront index, x / KO = umulhi(x, ko_magic) for a thread index (KO =
  // k-octets of the staged slab; both exact in those ranges); step_m, step_ko = (threads / KO, threads % KO).
  uint32_t wn_magic, ko_magic;
  int step_m, step_ko;
  int gx8;                 // see the kernel's n-tile order
  uint32_t b_bytes, s_bytes, z_bytes, a_bytes;   // extents of the buffer descriptors (saturated to 4 GiB - 1)
};

// (x & mask) | ex.  mask and ex reach the kernel as run-time arguments: with literal constants the compiler emits two
// instructions (a VOP3 op of this architecture cannot carry two literals); with register operands it selects the
// single v_and_or_b32, and unlike inline assembly the instruction stays visible to the MFMA hazard recogniser.
static __device__ inline uint32_t d2_and_or(uint32_t x, uint32_t mask, uint32_t ex) { return (x & mask) | ex; }

static __device__ inline __amdgpu_buffer_rsrc_t d2_rsrc(const void* base, uint64_t bytes) {
  const uint32_t n = bytes > 0xffffffffull ? 0xffffffffu : (uint32_t)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)n, 0x00020000);
}
static __device__ inline __amdgpu_buffer_rsrc_t d2_rsrc32(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
static inline uint32_t d2_sat32(uint64_t bytes) { return bytes > 0xffffffffull ? 0xffffffffu : (uint32_t)bytes; }

constexpr int D2_WAVES = 16;
constexpr int DECODE2_MAX_M = 64;           // rows of one workgroup: up to four m-blocks of 16
constexpr int DECODE2_MAX_M_ROWS = 256;     // rows when every m-block has workgroups of its own (see MSP)

template <bool BF16, int GS, int MB, bool HAS_ZP, int MR, int SUBG, int WT = 0, int RC = 0, bool MSP = false>
__global__ __launch_bounds__(D2_WAVES * 64) void w4a16_decode2_kernel(const Decode2Params p) {
  using T = F16Traits<BF16>;
  static_assert(!MSP || (MB == 1 && MR == 16), "rows split over workgroups: one full m-block each");
  // MSP: more than 16 rows handled as independent m-blocks, one per blockIdx.z -- every workgroup is the single-m-block
  // kernel on rows 16z .. 16z+15 (the weights are read once per m-block; the workgroups of one n-tile run side by side
  // and the later ones find the tiles in L2).  Against two m-blocks in one workgroup this halves the staged activations
  // per workgroup: a K of 4096 fits LDS again and needs no split over workgroups.
  const int mz = MSP ? (int)blockIdx.z : 0;
  const int M_loc = MSP ? min(16, p.M - 16 * mz) : p.M;
  const uint16_t* const a_loc = MSP ? p.a + (int64_t)mz * 16 * p.lda : p.a;
  const uint32_t a_bytes_loc = MSP ? p.a_bytes - (uint32_t)mz * 32u * (uint32_t)p.lda : p.a_bytes;
  uint16_t* const c_loc = MSP ? p.c + (int64_t)mz * 16 * p.N : p.c;
  static_assert(SUBG == 1 || SUBG == 2 || SUBG == 4, "quantisation groups per 128-row tile");
  constexpr bool W8 = WT == 1, F8 = WT == 2;           // 8-bit codes as two nibble planes / FP8 e4m3 bytes (see the head comment)
  constexpr int TPG = WT != 0 ? 2 : 1;                 // 1 KiB weight blocks per 128 rows of K
  static_assert(WT == 0 || (!HAS_ZP && GS % 2 == 0), "8-bit weights: two blocks per 128 rows, no zero points");
  static_assert(!F8 || SUBG == 1, "FP8 weights: channelwise scales or groups of 128 rows");
  static_assert(MR == 16 || MB == 1, "compact row staging is for a single m-block");
  // Ring of weight tiles in flight per wavefront.
  //  * Short streams with few staged rows (up to 8 tiles per wavefront, M <= 4) request everything up front: the whole
  //    layer is then in flight within the first microsecond, which is what a layer of a few megabytes needs to come near
  //    the memory system's rate (4096 x 6144 at M = 1: 5.9 -> 5.4 us; with 16 staged rows the same depth competes with
  //    the activation fill and loses 0.2-1 us).
  //  * Long streams, RC = 0: two slots, each refilled as soon as its tile's registers have been copied.  The wavefront
  //    then waits for both tiles at the top of every trip, so it overlaps little by itself: right when 14-16 wavefronts
  //    share a compute unit and overlap each other (about 28 KiB in flight per unit; deeper rings measured 2-6 % slower
  //    on 4096 x 28672).  (Four slots with 16 staged rows: the activation fill takes 2 us during which nothing else is
  //    requested, and four tiles in flight fill that gap.)
  //  * Long streams, RC = 1 / 2: four / three slots, each refilled only after its tile's arithmetic has been issued: no
  //    register copies, and the wait in front of a tile leaves the other R - 1 tiles in flight.  For launches with at
  //    most 8 wavefronts per compute unit, which are latency-bound with two slots (14336 x 4096 at M = 1: 9.2 -> 8.0 us
  //    with four slots; six slots 8.7 us; 16 wavefronts of two slots 10.3 us), and, with three slots, for 16 staged rows
  //    (4096 x 28672 at M = 16: 15.2 -> 14.8 us).
  // Two or more m-blocks: the second MFMA of every pair would be the same for all n-tiles of a k-tile, and with 16
  // MFMAs per tile the matrix core, not memory, sets the pace (4096 x 28672 at M = 32: the wavefronts of a compute unit
  // finished 10 us apart).  The row sums S[m] of every staged 128-row tile are then computed once per workgroup, right
  // after the fill, kept in LDS, and the correction is  P - (BIAS + z) * S  in fp32.
  constexpr bool SPRE = MB >= 2 && WT == 0 && SUBG == 1;
  constexpr int LPT = 1 + SUBG * (HAS_ZP ? 2 : 1);              // vector-memory instructions per tile request
  constexpr int R_SHORT = (GS < 63 / LPT ? GS : 63 / LPT) & (WT != 0 ? ~1 : ~0);      // (8-bit weights: whole block pairs)
  constexpr bool SHORT = MR <= 4 && GS <= 8 && GS >= 2;
  constexpr bool LATE = RC != 0 && !SHORT;
  constexpr int R_LATE = RC == 1 ? 4 : (RC == 2 ? 3 : 2);
  static_assert(!(WT != 0 && RC != 0), "8-bit weights take the block of a tile from the slot parity: even rings only");
  constexpr int R = SHORT ? R_SHORT : (LATE ? (GS < R_LATE ? GS : R_LATE) : ((MR >= 8 && MB == 1 && GS >= 7) ? 4 : (GS < 2 ? GS : 2)));
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const int lane = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.y);
  const int o = lane >> 4, r16 = lane & 15;
  const int WKS = p.WKS, WN = p.WN;
  const int wks = (int)(((uint32_t)w * p.wn_magic) >> 16), wn = w - wks * WN;
  const int sk = blockIdx.y;
  const int slab_groups = WKS * GS;                 // tiles in this workgroup's K slab
  const int slab_g0 = sk * slab_groups;             // first tile of the slab
  // Workgroups go to the XCDs round robin, and an n-tile's scales, zero points and output are 32-byte pieces of lines that
  // it shares with its neighbours: workgroups of one XCD take neighbouring n-tiles, so that an L2 fetches those lines once
  // instead of once per XCD (gx8 = workgroups along N / 8 where that is a whole number, else 0).
  const int bx = p.gx8 > 0 ? (int)(blockIdx.x & 7u) * p.gx8 + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
  const int nt_raw = bx * WN + wn;
  const bool nt_ok = nt_raw < p.NT;
  const int nt = nt_ok ? nt_raw : p.NT - 1;
  const int g_first = slab_g0 + wks * GS;           // this wavefront's first group

  // ---- 1. activations of the K slab -> LDS, then the first R weight tiles requested ----
  // Loads retire in issue order as far as the wait counter is concerned, so the activation loads go out FIRST: the
  // wait before the barrier then leaves the weight tiles in flight instead of draining them.
  const __amdgpu_buffer_rsrc_t rb = d2_rsrc32(p.b, p.b_bytes);
  const __amdgpu_buffer_rsrc_t rs = d2_rsrc32(p.scales, p.s_bytes);
  const __amdgpu_buffer_rsrc_t rz = d2_rsrc32(HAS_ZP ? (const void*)p.zeros : (const void*)p.scales, p.z_bytes);
  // zero points: as an MFMA operand a lane needs the one of column r16, in the output layout those of columns 4o .. 4o+3
  const int vo_b = lane * 16, vo_s = o * 8, vo_z = ((SPRE ? (o >> 1) : (r16 >> 3))) * 4;
  v4u wq[R];
  v2u sc[R][SUBG];
  uint32_t zq[R][SUBG];
  auto issue_load = [&](int slot, int gi) {
    const uint32_t g = (uint32_t)min(g_first + gi, p.G - 1);     // clamped: activations past K are zero
    wq[slot] = __builtin_amdgcn_raw_buffer_load_b128(rb, vo_b, (int)(((uint32_t)nt * (uint32_t)p.G + g) * 1024u), 2);
#pragma unroll
    for (int sj = 0; sj < SUBG; ++sj) {
      const uint32_t row = (g / (uint32_t)TPG) * (uint32_t)SUBG + (uint32_t)sj;
      sc[slot][sj] = __builtin_amdgcn_raw_buffer_load_b64(rs, vo_s, (int)((row * (uint32_t)p.s_stride + (uint32_t)nt * 16u) * 2u), 0);
      if constexpr (HAS_ZP)
        zq[slot][sj] = __builtin_amdgcn_raw_buffer_load_b32(rz, vo_z, (int)((row * (uint32_t)p.z_stride + (uint32_t)nt * 2u) * 4u), 0);
      else
        zq[slot][sj] = 0u;
    }
  };

  const int KO = slab_groups / TPG * 16;             // k-octets in the slab
  // LDS image of the slab's activations: row-major, slot (16 bytes) of (row m, k-octet ko) = m*KO + (ko ^ (m & (MR-1))).
  // A row is contiguous like in global memory, so 64 consecutive slots are one coalesced 1 KiB piece of a row (the XOR
  // permutes 16-byte chunks inside aligned 256-byte blocks) and a direct-to-LDS load can fill them; the operand reads
  // of 16 lanes (16 rows, one k-octet) hit 16 different bank groups because the row pitch is a multiple of 256 bytes.
  {
    const int tid = w * 64 + lane;
    const int chunks = KO * MR * MB;
    const int k_slab0 = (slab_g0 / TPG) * 128;          // 32-bit arithmetic: the launcher checks that A ends below 2 GiB
    const int lda32 = (int)p.lda;
    const int NTHR = WKS * WN * 64;
    const int step_m = p.step_m, step_ko = p.step_ko;               // NTHR / KO, NTHR % KO
    // chunk c = m * KO + ko' (LDS slot c); thread tid handles c = tid, tid + NTHR, ...  The (m, ko') pair is advanced
    // incrementally: one scalar division per kernel instead of one vector division per chunk.
    int m = (int)__umulhi((uint32_t)tid, p.ko_magic), ko = tid - m * KO;
    if (p.PRIV != 0) {
      // Private fill (one n-tile per workgroup, so no two wavefronts read the same k-octets): every wavefront fetches the
      // k-octets of its own K slice, row by row, and waits for nobody -- the same bytes travel as in the shared fill, but
      // a wavefront starts on its first tile as soon as ITS activations and ITS first weight tile are there instead of
      // when the slowest wavefront's activations are.  An instruction whose 64 slots reach past the slice covers part of
      // the next wavefront's slice (or of the next row) and writes there exactly what its owner writes.  The first
      // weight tile is requested before the activations, the others after them: the wait below then leaves R - 1 tiles
      // in flight.
      const __amdgpu_buffer_rsrc_t ra = d2_rsrc32(a_loc, a_bytes_loc);
      typedef __attribute__((address_space(3))) void* lds_ptr_t;
      issue_load(0, 0);
      const int own = (GS / TPG) * 16;                         // k-octets of this wavefront's slice
      for (int mrow = 0; mrow < MR * MB; ++mrow) {
        for (int q0 = 0; q0 < own; q0 += 64) {
          const int c0 = mrow * KO + wks * own + q0;           // first slot of this instruction (wave-uniform)
          const int sl = c0 + lane;
          const int m2 = (int)__umulhi((uint32_t)sl, p.ko_magic), ko2 = sl - m2 * KO;
          const int k = k_slab0 + (ko2 ^ (m2 & (MR - 1))) * 8;
          const bool ok = m2 < MR * MB && m2 < M_loc && k < p.K;
          const uint32_t off = ok ? (uint32_t)(m2 * lda32 + k) * 2u : 0x80000000u;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(lds + (size_t)c0 * 16), 16, (int)off, 0, 0, 0);
        }
      }
#pragma unroll
      for (int s = 1; s < R; ++s) issue_load(s, s);
      constexpr int W_LATER = (R - 1) * LPT;      // vector-memory instructions requested after the activations
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(W_LATER) : "memory");
    } else if (p.perm == nullptr) {
      // Direct-to-LDS loads (no registers, no LDS write instructions): wavefront instruction q fills slots 64q .. 64q+63,
      // lane l fetching the chunk that belongs in slot 64q + l.  Rows past M, k past K and slots past the image get an
      // out-of-range offset of the buffer descriptor (which ends with the last valid element) and arrive as zeros; the
      // image is padded to a multiple of 1 KiB for the last instruction.  The weight tiles are requested after these
      // loads (loads retire in order as far as the wait counter is concerned) and stay in flight across the barrier.
      const __amdgpu_buffer_rsrc_t ra = d2_rsrc32(a_loc, a_bytes_loc);
      typedef __attribute__((address_space(3))) void* lds_ptr_t;
      for (int c0 = w * 64; c0 < chunks; c0 += NTHR) {
        const int k = k_slab0 + (ko ^ (m & (MR - 1))) * 8;
        const bool ok = m < MR * MB && m < M_loc && k < p.K;
        const uint32_t off = ok ? (uint32_t)(m * lda32 + k) * 2u : 0x80000000u;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(lds + (size_t)c0 * 16), 16, (int)off, 0, 0, 0);
        m += step_m;
        ko += step_ko;
        if (ko >= KO) {
          ko -= KO;
          m += 1;
        }
      }
#pragma unroll
      for (int s = 0; s < R; ++s) issue_load(s, s);
      constexpr int W_LOADS = R * LPT;      // vector-memory instructions of the weight requests
      static_assert(W_LOADS < 64, "the wait counter holds 6 bits");
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(W_LOADS) : "memory");
    } else {
      // act_order: the columns of A are gathered through `perm`; two dependent levels of loads, weights requested first
#pragma unroll
      for (int s = 0; s < R; ++s) issue_load(s, s);
      for (int c0 = 0; c0 < chunks; c0 += NTHR * 4) {
        v4u v[4];
        int mm[4], kk[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          mm[i] = m;
          kk[i] = ko;
          const int64_t k = (int64_t)k_slab0 + (int64_t)(ko ^ (m & (MR - 1))) * 8;
          v[i] = v4u{0u, 0u, 0u, 0u};
          if (m < MR * MB && m < M_loc && k < p.K) {
            const uint16_t* row = a_loc + (int64_t)m * p.lda;
            const v4i p0 = *reinterpret_cast<const v4i*>(p.perm + k);
            const v4i p1 = *reinterpret_cast<const v4i*>(p.perm + k + 4);
            v[i].x = (uint32_t)row[p0.x] | ((uint32_t)row[p0.y] << 16);
            v[i].y = (uint32_t)row[p0.z] | ((uint32_t)row[p0.w] << 16);
            v[i].z = (uint32_t)row[p1.x] | ((uint32_t)row[p1.y] << 16);
            v[i].w = (uint32_t)row[p1.z] | ((uint32_t)row[p1.w] << 16);
          }
          m += step_m;
          ko += step_ko;
          if (ko >= KO) {
            ko -= KO;
            m += 1;
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (mm[i] < MR * MB) *reinterpret_cast<v4u*>(lds + ((size_t)mm[i] * KO + kk[i]) * 16) = v[i];
        }
      }
      __syncthreads();
    }
  }

  // ---- 2. row sums of the staged tiles (two or more m-blocks) ----
  constexpr bool RED_ALIAS = MB > 2;
  // LDS behind the activation image (padded to 1 KiB): the reduction buffer of the K slices (see step 4; three and four
  // m-blocks: on top of the activations), then the row sums.  With two m-blocks the buffer is compact -- the
  // wavefronts of slice 0 write nothing, so it holds the tiles of the wavefronts WN .. WKS*WN - 1 only -- which is what
  // lets 128 KiB of activations, the buffer and the sums fit the 160 KiB.
  constexpr bool RED_COMPACT = MB == 2;
  float* rowsum = nullptr;
  if constexpr (SPRE) {
    const size_t act_b = ((size_t)KO * MR * MB * 16 + 1023) & ~(size_t)1023;
    const size_t red_b = WKS > 1 ? (size_t)(RED_COMPACT ? D2_WAVES - D2_WAVES / WKS : D2_WAVES) * MB * 1024 : 0;
    rowsum = reinterpret_cast<float*>(lds + (RED_ALIAS ? (act_b > red_b ? act_b : red_b) : act_b + red_b));
    constexpr uint32_t ONE2 = BF16 ? 0x3f803f80u : 0x3c003c00u;
    const v4u ones = {ONE2, ONE2, ONE2, ONE2};
    const int NW = WKS * WN;
    for (int t = w; t < slab_groups; t += NW) {          // tile t of the slab: its 128 k of every staged row
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        v4f q = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const v4u bop = *reinterpret_cast<const v4u*>(lds + (uint32_t)((r16 * KO + t * 16 + ((jj * 4 + o) ^ r16)) * 16) + (uint32_t)(mb * KO * MR * 16));
          q = T::mfma16(ones, bop, q);
        }
        if (o == 0) rowsum[(t * MB + mb) * 16 + r16] = q[0];      // every register of column r16 holds the sum of row r16
      }
    }
    // the LDS writes only: the weight tiles requested above stay in flight across this barrier
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  }

  // ---- 3. the K loop of this wavefront: GS tiles, fully unrolled ----
  // operand read of MFMA jj of local group gl: k-octet = gl*16 + jj*4 + o  ->  (ko & 15) = jj*4 + o
  uint32_t abase[4];
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) {
    const int kol = jj * 4 + o;
    const int ml = r16 & (MR - 1);
    abase[jj] = (uint32_t)((ml * KO + wks * (GS / TPG) * 16 + (kol ^ ml)) * 16);
  }
  uint32_t ex;     // kept in a vector register so that (x & MSK) | ex is a legal single VOP3 instruction (one scalar operand)
  asm volatile("v_mov_b32 %0, %1" : "=v"(ex) : "s"(p.k_ex));
  const uint32_t MSK = p.k_mask;
  constexpr uint32_t NEG_BIAS_BITS = BF16 ? 0xC300u : 0xE400u;     // -(BIAS) as a 16-bit pattern; "| z" adds the zero point
  v4f acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = v4f{0.f, 0.f, 0.f, 0.f};

  // One tile: `slot` is a compile-time constant wherever this is expanded; `reissue` refills the slot R tiles ahead.
  auto do_tile = [&](int gi, int slot, bool reissue) {
    const uint32_t wj[4] = {wq[slot].x, wq[slot].y, wq[slot].z, wq[slot].w};
    v2u sct[SUBG];
    uint32_t zqt[SUBG];
#pragma unroll
    for (int sj = 0; sj < SUBG; ++sj) {
      sct[sj] = sc[slot][sj];
      zqt[sj] = zq[slot][sj];
    }
    if constexpr (!LATE) {
      if (reissue) issue_load(slot, gi + R);
    }

#pragma unroll
    for (int sj = 0; sj < SUBG; ++sj) {
      uint32_t zbits;
      if constexpr (HAS_ZP) zbits = NEG_BIAS_BITS | ((zqt[sj] >> ((r16 & 7) * 4)) & 0xFu);
      else if constexpr (W8) zbits = NEG_BIAS_BITS | ((slot & 1) ? 0u : 8u);     // slot parity == plane (ring of 2, GS even)
      else zbits = NEG_BIAS_BITS | 8u;
      const uint32_t z2 = zbits | (zbits << 16);
      const v4u zop = {z2, z2, z2, z2};
      // (row sums kept in LDS: the factor -(BIAS + z) of output column 4o + r, and the sums of this lane's row)
      float zf[4], rs_m[MB];
      if constexpr (SPRE) {
        constexpr float BIASF = BF16 ? 128.0f : 1024.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if constexpr (HAS_ZP) zf[r] = -(BIASF + (float)((zqt[sj] >> ((((o & 1) * 4 + r)) * 4)) & 0xFu));
          else zf[r] = -(BIASF + 8.0f);
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) rs_m[mb] = rowsum[((wks * GS + gi) * MB + mb) * 16 + r16];
      }

      // Two accumulation chains per m-block -- the products with the codes in P, the bias / zero-point correction in Q --
      // issued alternately: an MFMA that accumulates on the previous one's result waits for it, and one chain of eight
      // left the matrix core idle most of the time when few wavefronts share a SIMD.
      v4f P[MB], Q[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) P[mb] = Q[mb] = v4f{0.f, 0.f, 0.f, 0.f};
      if constexpr (F8) {
        // FP8 bytes: block h = slot parity holds the 8-byte operands of MFMAs 2h and 2h + 1 (words 0,1 and 2,3); a packed
        // conversion turns two bytes into two 16-bit numbers exactly (every e4m3 value is a bf16 and an fp16 value; the
        // instruction's scale operand only contributes its power of two, 1.0 here).  No bias, no zero point: P and Q are
        // the two MFMAs' own chains.
#pragma unroll
        for (int j2 = 0; j2 < 2; ++j2) {
          const uint32_t wa = wj[2 * j2], wb = wj[2 * j2 + 1];
          v4u aop;
          if constexpr (BF16) {
            aop.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wa, 1.0f, false));
            aop.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wa, 1.0f, true));
            aop.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wb, 1.0f, false));
            aop.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(wb, 1.0f, true));
          } else {
            aop.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(wa, 1.0f, false));
            aop.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(wa, 1.0f, true));
            aop.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(wb, 1.0f, false));
            aop.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(wb, 1.0f, true));
          }
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            const v4u bop = *reinterpret_cast<const v4u*>(lds + abase[2 * (slot & 1) + j2] + (uint32_t)(mb * KO * MR * 16) + (uint32_t)((gi / TPG) * 256));
            if (j2 == 0) P[mb] = T::mfma16(aop, bop, P[mb]);
            else Q[mb] = T::mfma16(aop, bop, Q[mb]);
          }
        }
      } else {
#pragma unroll
      for (int jj = sj * (4 / SUBG); jj < (sj + 1) * (4 / SUBG); ++jj) {
        v4u aop;
        aop.x = d2_and_or(wj[jj], MSK, ex);
        aop.y = d2_and_or(wj[jj] >> 4, MSK, ex);
        aop.z = d2_and_or(wj[jj] >> 8, MSK, ex);
        aop.w = d2_and_or(wj[jj] >> 12, MSK, ex);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const v4u bop = *reinterpret_cast<const v4u*>(lds + abase[jj] + (uint32_t)(mb * KO * MR * 16) + (uint32_t)((gi / TPG) * 256));
          P[mb] = T::mfma16(aop, bop, P[mb]);
          if constexpr (!SPRE) Q[mb] = T::mfma16(zop, bop, Q[mb]);
        }
      }
      }
      if constexpr (SPRE) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int r = 0; r < 4; ++r) Q[mb][r] = zf[r] * rs_m[mb];
      }
      float s[4];
      if constexpr (BF16) {
        s[0] = __uint_as_float(sct[sj].x << 16);
        s[1] = __uint_as_float(sct[sj].x & 0xffff0000u);
        s[2] = __uint_as_float(sct[sj].y << 16);
        s[3] = __uint_as_float(sct[sj].y & 0xffff0000u);
      } else {
        s[0] = T::to_float((uint16_t)(sct[sj].x & 0xffffu));
        s[1] = T::to_float((uint16_t)(sct[sj].x >> 16));
        s[2] = T::to_float((uint16_t)(sct[sj].y & 0xffffu));
        s[3] = T::to_float((uint16_t)(sct[sj].y >> 16));
      }
      if constexpr (W8) {
        if ((slot & 1) == 0) {
#pragma unroll
          for (int r = 0; r < 4; ++r) s[r] *= 16.0f;        // high-nibble plane
        }
      }
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[mb][r] = fmaf(s[r], P[mb][r] + Q[mb][r], acc[mb][r]);
    }
    if constexpr (LATE) {
      if (reissue) issue_load(slot, gi + R);
    }
  };
  if constexpr (GS <= 4) {
#pragma unroll
    for (int gi = 0; gi < GS; ++gi) do_tile(gi, gi % R, gi + R < GS);
  } else {
    // Long streams run as a rolled loop of R tiles per trip (short code: these kernels alternate with others and
    // start with a cold instruction cache).  Every trip of the loop refills its slots unconditionally -- a branch
    // around a load would make the compiler's wait counts drain the ring -- and the last tiles are peeled.
    constexpr int MAIN = ((GS - R) / R) * R;      // tiles consumed inside the loop
#pragma unroll 1
    for (int g0 = 0; g0 < MAIN; g0 += R) {
#pragma unroll
      for (int u = 0; u < R; ++u) do_tile(g0 + u, u, true);
    }
#pragma unroll
    for (int gi = MAIN; gi < GS; ++gi) do_tile(gi, gi % R, gi + R < GS);
  }

  // ---- 4. reduce the K slices of the workgroup ----
  // [16 waves][MB][64] partial tiles: behind the activations, or -- with three or four m-blocks, where both would not
  // fit -- on top of them once every wavefront is through its K loop
  // (one m-block: the unused tile of wavefront 0 doubles as the padding that the last instruction of a private fill
  // may write zeros into)
  v4f* red = reinterpret_cast<v4f*>(RED_ALIAS ? lds : lds + (((size_t)KO * MR * MB * 16 + 1023) & ~(size_t)1023)) - (RED_COMPACT ? WN * MB * 64 : 0);
  if (WKS > 1) {
    if constexpr (RED_ALIAS) __syncthreads();
    if (!RED_COMPACT || wks != 0) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) red[(w * MB + mb) * 64 + lane] = acc[mb];
    }
    __syncthreads();
    if (wks != 0) return;
    // the partial tiles of the other slices, added in slice order; with many slices, seven reads in flight at a time
    // (one by one, each read waits out the LDS latency: 0.3 us for eight slices)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      v4f t = acc[mb];
      if (WKS <= 4) {
        for (int s2 = 1; s2 < WKS; ++s2) t += red[((s2 * WN + wn) * MB + mb) * 64 + lane];
      } else {
        for (int s0 = 1; s0 < WKS; s0 += 7) {
          v4f part[7];
#pragma unroll
          for (int i = 0; i < 7; ++i) part[i] = red[((min(s0 + i, WKS - 1) * WN + wn) * MB + mb) * 64 + lane];
#pragma unroll
          for (int i = 0; i < 7; ++i)
            if (s0 + i < WKS) t += part[i];
        }
      }
      acc[mb] = t;
    }
  }
  if (!nt_ok) return;

  // ---- 5. hand over across workgroups if K is split, then write the 16-bit outputs ----
  // Partial tiles cross workgroups (and XCDs, whose L2 caches are not coherent with each other) through 16-byte buffer
  // stores / loads with the sc1 cache-policy bit (device scope): one wait for the stores to be acknowledged, one arrival
  // counter per n-tile; the last of the SK workgroups to arrive sums the partials in split order (deterministic).
  if (p.SK > 1) {
    constexpr int SC1 = 16;
    const uint32_t sk_stride = (uint32_t)p.NT * (uint32_t)MB * 1024u;            // bytes per split
    const __amdgpu_buffer_rsrc_t rt = d2_rsrc(p.c_tmp, (uint64_t)sk_stride * (uint64_t)p.SK);
    const uint32_t unit = (uint32_t)nt * (uint32_t)MB * 1024u;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, acc[mb]), rt, lane * 16,
                                             (int)((uint32_t)sk * sk_stride + unit + (uint32_t)mb * 1024u), SC1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // partial tiles acknowledged before the counter moves
    int old = 0;
    if (lane == 0) old = __hip_atomic_fetch_add(&p.counters[nt * MB], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    old = __builtin_amdgcn_readfirstlane(old);      // lane 0 holds it; a scalar keeps what depends on it scalar
    if (old != p.SK - 1) return;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < p.SK; s0 += 4) {               // four splits in flight, added in split order
      v4u part[4][MB];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t s2 = (uint32_t)min(s0 + i, p.SK - 1);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          part[i][mb] = __builtin_amdgcn_raw_buffer_load_b128(rt, lane * 16, (int)(s2 * sk_stride + unit + (uint32_t)mb * 1024u), SC1);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (s0 + i < p.SK) {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) acc[mb] += __builtin_bit_cast(v4f, part[i][mb]);
        }
      }
    }
    if (lane == 0) __hip_atomic_store(&p.counters[nt * MB], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    v4f val = acc[mb];
    const bool write_out = true;
    const int m = mb * 16 + r16;
    if (write_out && m < M_loc) {
      const int n = nt * 16 + o * 4;
      if (p.bias) {
        const v2u bb = *reinterpret_cast<const v2u*>(p.bias + n);
        val[0] += T::to_float((uint16_t)(bb.x & 0xffffu));
        val[1] += T::to_float((uint16_t)(bb.x >> 16));
        val[2] += T::to_float((uint16_t)(bb.y & 0xffffu));
        val[3] += T::to_float((uint16_t)(bb.y >> 16));
      }
      v2u outv;
      outv.x = (uint32_t)T::from_float(val[0]) | ((uint32_t)T::from_float(val[1]) << 16);
      outv.y = (uint32_t)T::from_float(val[2]) | ((uint32_t)T::from_float(val[3]) << 16);
      *reinterpret_cast<v2u*>(c_loc + (int64_t)m * p.N + n) = outv;
    }
  }
}

// LDS of a workgroup: activations of `groups` = WKS * (groups per wavefront) quantisation groups for MR x MB rows, the
// reduction buffer of the K slices (on top of the activations for MB > 2, see the kernel), and with two or more
// m-blocks the row sums of the staged tiles.
static inline size_t decode2_lds_bytes(int wks, int groups_per_wave, int mr, int mb) {
  // padded to 1 KiB (see the fill).  With one K slice per workgroup nothing else follows the image, and the last
  // instruction of the private fill may write (zeros) up to 63 slots past it: one more KiB.
  const size_t act = (((size_t)wks * groups_per_wave * 256 * mr * mb + 1023) & ~(size_t)1023) + (wks == 1 ? 1024 : 0);
  const size_t red = wks > 1 ? (size_t)(mb == 2 ? D2_WAVES - D2_WAVES / wks : D2_WAVES) * mb * 1024 : 0;
  const size_t sums = mb >= 2 ? (size_t)wks * groups_per_wave * mb * 64 : 0;      // row sums of the staged tiles (see SPRE)
  if (mb > 2) return (act > red ? act : red) + sums;
  return act + red + sums;
}

template <bool BF16, int GS, int MB, bool HAS_ZP, int MR, int SUBG, int WT = 0, int RC = 0, bool MSP = false>
static int launch_decode2(const Decode2Params& p_in, hipStream_t s) {
  Decode2Params p = p_in;
  const int WN = p.WN;
  {
    const int ko = p.WKS * GS / (WT != 0 ? 2 : 1) * 16, nthr = p.WKS * WN * 64;
    p.wn_magic = (uint32_t)((65536 + WN - 1) / WN);
    if (WN != 1 || p.perm != nullptr) p.PRIV = 0;
    p.ko_magic = (uint32_t)(((1ull << 32) + (uint64_t)ko - 1) / (uint64_t)ko);
    p.step_m = nthr / ko;
    p.step_ko = nthr - p.step_m * ko;
    p.b_bytes = d2_sat32((uint64_t)p.K * p.N / 2 * (WT != 0 ? 2 : 1));
    p.s_bytes = d2_sat32((uint64_t)p.GR * p.N * 2);
    p.z_bytes = d2_sat32((uint64_t)p.GR * (p.N / 8) * 4);
    p.a_bytes = d2_sat32(((uint64_t)(p.M - 1) * (uint64_t)p.lda + (uint64_t)p.K) * 2);
    if (p.a_bytes >= 0x80000000u) {
      set_error("w4a16_gemm(decode): activations beyond 2 GiB (M = %d, row stride %lld)", p.M, (long long)p.lda);
      return VAQ_ERR_UNSUPPORTED;
    }
  }
  const size_t lds = decode2_lds_bytes(p.WKS, GS / (WT != 0 ? 2 : 1), MR, MB);
  if (p.PRIV != 0) {
    // the private fill writes whole 64-slot instructions: the last one (last row, last K slice) must end inside the
    // allocation, whatever the planner chose; otherwise the shared fill, which stays inside the padded image, is taken
    const int own = GS / (WT != 0 ? 2 : 1) * 16, ko = p.WKS * own;
    const size_t last_c0 = (size_t)(MR * MB - 1) * ko + (size_t)(p.WKS - 1) * own + (size_t)((own - 1) / 64) * 64;
    if ((last_c0 + 64) * 16 > lds) p.PRIV = 0;
  }
  auto kern = w4a16_decode2_kernel<BF16, GS, MB, HAS_ZP, MR, SUBG, WT, RC, MSP>;
  static size_t reserved[VAQ_MAX_DEVICES];
  if (const int rc = reserve_dynamic_lds(reinterpret_cast<const void*>(kern), lds, reserved, "w4a16_gemm(decode)"); rc != VAQ_OK) return rc;
  const int gx = (p.NT + WN - 1) / WN;
  // n-tiles grouped by XCD (see the kernel) on layers of up to 1.5 n-tiles per compute unit whose K is not split over
  // workgroups.  Cold, M = 1 / 4 / 16: 4096 x 6144 5.35 / 5.75 / 6.59 -> 5.16 / 5.55 / 6.32 us, 4096 x 4096 4.44 / 4.55 / 5.42 -> 4.23 /
  // 4.42 / 5.27 us, 14336 x 4096 at M = 1 / 4 8.16 / 9.09 -> 7.78 / 8.76 us; with K parts and their hand-over it costs 4 % (14336 x
  // 4096 at M = 16 / 32), wider layers show nothing either way (4096 x 28672, 4096 x 14336) or lose (8192 x 8192 at M = 1 +9 %).
  p.gx8 = (gx % 8 == 0 && p.SK == 1 && p.NT * 2 <= num_cus_current_device() * 3 && tuning().exp[7] != 1) ? gx / 8 : 0;
  hipLaunchKernelGGL(kern, dim3(gx, p.SK, MSP ? (p.M + 15) / 16 : 1), dim3(64, p.WKS * WN), lds, s, p);
  return VAQ_OK;
}

// Groups of 64 / 32 rows (2 / 4 per tile); defined in w4a16_decode2_sub2.hip / w4a16_decode2_sub4.hip: groups per
// wavefront gs in {1, 2, 4, 8, 16}, staged rows mr in {1, 4, 16} (16 when MB == 2).
int decode2_launch_sub2(const Decode2Params& p, int gs, int MB, int mr, bool bf16, bool zp, hipStream_t s);
int decode2_launch_sub4(const Decode2Params& p, int gs, int MB, int mr, bool bf16, bool zp, hipStream_t s);
// Three and four m-blocks (32 < M <= 64), groups of 128 rows / channelwise; defined in w4a16_decode2_mb34.hip.
int decode2_launch_mb34(const Decode2Params& p, int gs, int MB, bool bf16, bool zp, hipStream_t s);
// 8-bit codes; defined in w4a16_decode2_w8.hip (groups of 128 rows / channelwise: gs in {2, 4, 8, 14, 16}) and
// w4a16_decode2_w8sub.hip (sub = 2 / 4 groups per 128 rows: gs in {2, 4, 8, 16}); staged rows mr in {1, 4, 16} (16 when MB == 2).
int decode2_launch_w8(const Decode2Params& p, int gs, int MB, int mr, bool bf16, hipStream_t s);
int decode2_launch_w8sub(const Decode2Params& p, int sub, int gs, int MB, int mr, bool bf16, hipStream_t s);
// FP8 e4m3 weights (bytes), channelwise scales or groups of 128 rows; defined in w4a16_decode2_f8.hip: gs in {2, 4, 8, 14, 16},
// staged rows mr in {1, 4, 16} (16 when MB == 2).
int decode2_launch_f8(const Decode2Params& p, int gs, int MB, int mr, bool bf16, hipStream_t s);

}  // namespace vaq

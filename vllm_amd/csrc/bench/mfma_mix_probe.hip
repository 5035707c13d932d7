// Measurement aid, not part of the quantized-linear library (built into libvaq_bench_probe.so, which only the
// benchmark loads): what the matrix core sustains when a wavefront's instruction stream mixes MFMAs with the other
// instructions a GEMM main loop needs -- LDS fragment reads and the VALU work of a dequantisation.  One workgroup per
// compute unit, 4 wavefronts (one per SIMD) or 8 (two per SIMD); per iteration each wavefront issues NM MFMAs on NA
// accumulators (in the accumulation registers), NV independent VALU instructions and NR 16-byte LDS reads spread
// evenly between them; a fragment read is consumed one iteration after it was requested (counted wait), as in a
// software-pipelined main loop.  Operands vary from lane to lane and from read to read (a matrix core fed with constant
// operands draws less power and runs at a higher clock than any real GEMM).
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef unsigned v8u __attribute__((ext_vector_type(8)));

// KIND: 0 v_mfma_f32_32x32x16_bf16, 1 v_mfma_f32_16x16x32_bf16, 2 v_mfma_f32_32x32x64_f8f6f4 (fp8), 3 v_mfma_f32_16x16x128_f8f6f4
template <int KIND>
constexpr double flops_per_mfma() { return KIND == 0 ? 32768.0 : KIND == 1 ? 16384.0 : KIND == 2 ? 131072.0 : 65536.0; }

template <int NWV, int KIND, int NM, int NA, int NV, int NR>
__global__ __launch_bounds__(NWV * 64) void mix_kernel(unsigned long long* ticks, unsigned* sink, int iters) {
  constexpr bool BIG = KIND == 0 || KIND == 2;      // 32 x 32 output block: 16 accumulation registers
  constexpr bool F8 = KIND >= 2;                    // 32-byte operands: a fragment is two reads
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  // finite, moderately sized values in either format: bf16 1.0 .. 2.0 with random mantissas / e4m3 bytes 0x30 .. 0x3f
  for (int i = threadIdx.x; i < 16384; i += blockDim.x)
    ((unsigned*)lds)[i] = F8 ? (((i * 2654435761u) & 0x0f0f0f0fu) | 0x30303030u) : (((i * 2654435761u) & 0x007f007fu) | 0x3f803f80u);
  __syncthreads();
  v4u a = {F8 ? 0x38343230u + threadIdx.x * 0x01000100u % 0x08080808u : 0x3f803f80u + threadIdx.x * 0x00010001u % 0x00400040u,
           F8 ? 0x31353933u : 0x3fa03fc0u, F8 ? 0x3a3c3e30u : 0x3f903f70u, F8 ? 0x32363a3eu : 0x3fb03f88u};
  v16f acc16[BIG ? NA : 1];
  v4f acc4[BIG ? 1 : NA];
  for (int j = 0; j < (BIG ? NA : 1); ++j) for (int e = 0; e < 16; ++e) acc16[j][e] = 0.f;
  for (int j = 0; j < (BIG ? 1 : NA); ++j) for (int e = 0; e < 4; ++e) acc4[j][e] = 0.f;
  unsigned r[4] = {threadIdx.x, threadIdx.x + 1u, threadIdx.x + 2u, threadIdx.x + 3u};
  const unsigned ca = 0x3f800001u, cb = 0x40000003u;
  constexpr int NRR = NR > 0 ? NR : 1;
  v4u rd[NRR];
  for (int q = 0; q < NRR; ++q) rd[q] = a;
  const unsigned base = (threadIdx.x & 63) * 16 + (threadIdx.x >> 6) * 4096;
  const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
  for (int i = 0; i < iters; ++i) {
    int vdone = 0, rdone = 0;
#pragma unroll
    for (int j = 0; j < NM; ++j) {
      const int ri = NR > 0 ? (j * NR / NM) % NR : 0;
      // rd[ri] was requested NR reads ago
      if (!F8 && NR > 0 && (j * NR) % NM == 0) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(NR - 1 < 15 ? NR - 1 : 15) : "memory");      // (the counter has four bits)
      a.x ^= rd[ri].y & (F8 ? 0x07070707u : 0x003f003fu);
      if constexpr (KIND == 0) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc16[j % NA]) : "v"(a), "v"(rd[ri]));
      } else if constexpr (KIND == 1) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc4[j % NA]) : "v"(a), "v"(rd[ri]));
      } else {
        // 32-byte operands: two reads make one fragment (the compiler keeps these accumulators where it likes: at most
        // 128 registers here)
        typedef int v8i __attribute__((ext_vector_type(8)));
        const v4u o = rd[(ri + 1) % NRR];
        const v8i a8 = {(int)a.x, (int)a.y, (int)a.z, (int)a.w, (int)a.y, (int)a.x, (int)a.w, (int)a.z};
        const v8i b8 = {(int)rd[ri].x, (int)rd[ri].y, (int)rd[ri].z, (int)rd[ri].w, (int)o.x, (int)o.y, (int)o.z, (int)o.w};
        if constexpr (KIND == 2) acc16[j % NA] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, acc16[j % NA], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
        else acc4[j % NA] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, acc4[j % NA], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
      }
      const int vt = (j + 1) * NV / NM;
#pragma unroll
      for (; vdone < vt; ++vdone) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(r[vdone & 3]) : "v"(ca), "v"(cb));
      const int rt = (j + 1) * NR / NM;
#pragma unroll
      for (; rdone < rt; ++rdone) {
        if constexpr (F8) rd[rdone] = *reinterpret_cast<const v4u*>(lds + ((base + rdone * 1024 + i * 64) & 65535));
        else asm volatile("ds_read_b128 %0, %1" : "=v"(rd[rdone]) : "v"((base + rdone * 1024 + i * 64) & 65535));
      }
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  const unsigned long long t1 = __builtin_amdgcn_s_memrealtime();
  float s = 0;
  if constexpr (F8) {
    for (int j = 0; j < (BIG ? NA : 1); ++j) s += acc16[j][0];
    for (int j = 0; j < (BIG ? 1 : NA); ++j) s += acc4[j][0];
  } else {
    for (int j = 0; j < (BIG ? NA : 1); ++j) { float t; asm volatile("s_nop 15\n\ts_nop 15\n\tv_accvgpr_read_b32 %0, %1" : "=v"(t) : "a"(acc16[j][0])); s += t; }
    for (int j = 0; j < (BIG ? 1 : NA); ++j) { float t; asm volatile("s_nop 15\n\ts_nop 15\n\tv_accvgpr_read_b32 %0, %1" : "=v"(t) : "a"(acc4[j][0])); s += t; }
  }
  if (s == 1.2345f || (r[0] ^ r[1] ^ r[2] ^ r[3]) == 0x12345678u) sink[0] = 1;      // practically never
  if ((threadIdx.x & 63) == 0) ticks[blockIdx.x * 8 + (threadIdx.x >> 6)] = t1 - t0;
}

struct MixConfig {
  const char* what;
  int waves, kind, nm, na, nv, nr;
  void (*launch)(unsigned long long*, unsigned*, int, hipStream_t);
};

template <int NWV, int KIND, int NM, int NA, int NV, int NR>
void launch_mix(unsigned long long* ticks, unsigned* sink, int iters, hipStream_t s) {
  auto kern = mix_kernel<NWV, KIND, NM, NA, NV, NR>;
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
  hipLaunchKernelGGL(kern, dim3(256), dim3(NWV * 64), 65536, s, ticks, sink, iters);
}
#define MIX(what, w, kind, nm, na, nv, nr) {what, w, kind, nm, na, nv, nr, launch_mix<w, kind, nm, na, nv, nr>}

// Per 32 k (16-bit) / 128 k (fp8) of a wavefront tile.  (FP8 only as bare MFMAs: with 32-byte operands the fragment
// reads of an 8-wavefront GEMM cannot be expressed in this one-size-fits-all loop without register copies that the real
// kernels do not have, and the figures it gave were far below what those kernels reach.)
const MixConfig kConfigs[] = {
    MIX("bf16 32x32x16: MFMAs only, two wavefronts per SIMD", 8, 0, 8, 8, 0, 0),
    MIX("bf16 32x32x16: MFMAs only, one wavefront per SIMD", 4, 0, 16, 16, 0, 0),
    MIX("bf16 16x16x32: MFMAs only, two wavefronts per SIMD", 8, 1, 32, 32, 0, 0),
    MIX("bf16 16x16x32: MFMAs only, one wavefront per SIMD", 4, 1, 64, 64, 0, 0),
    MIX("bf16 plain GEMM, 8 wavefronts of 128 x 64: 12 fragment reads per 16 MFMAs", 8, 0, 16, 8, 0, 12),
    MIX("bf16 plain GEMM, 8 wavefronts of 128 x 64, 16x16x32", 8, 1, 32, 32, 0, 12),
    MIX("bf16 plain GEMM, 4 wavefronts of 128 x 128: 16 reads per 32 MFMAs", 4, 0, 32, 16, 0, 16),
    MIX("bf16 plain GEMM, 4 wavefronts of 128 x 128, 16x16x32", 4, 1, 64, 64, 0, 16),
    MIX("W4A16, weights dequantised into LDS (8 wavefronts of 128 x 64): 46 VALU, 12 reads + 2 for the writes", 8, 0, 16, 8, 46, 14),
    MIX("W4A16, the same with 16x16x32", 8, 1, 32, 32, 46, 14),
    MIX("W4A16, weights dequantised in registers, 8 wavefronts of 128 x 64: 92 VALU, 8 reads", 8, 0, 16, 8, 92, 8),
    MIX("W4A16, the same with 16x16x32", 8, 1, 32, 32, 92, 8),
    MIX("W4A16, weights dequantised in registers, 4 wavefronts of 256 x 64: 92 VALU, 16 reads per 32 MFMAs", 4, 0, 32, 16, 92, 16),
    MIX("fp8 32x32x64: MFMAs only, two wavefronts per SIMD", 8, 2, 8, 8, 0, 0),
    MIX("fp8 16x16x128: MFMAs only, two wavefronts per SIMD", 8, 3, 32, 32, 0, 0),
    MIX("fp8 32x32x64: MFMAs only, one wavefront per SIMD", 4, 2, 16, 16, 0, 0),
};
constexpr int kNumConfigs = sizeof(kConfigs) / sizeof(kConfigs[0]);

}  // namespace

// Number of configurations; description / shape of configuration `i` (NULL / 0 beyond the end).
extern "C" __attribute__((visibility("default"))) int vaq_mfma_mix_probe_count(void) { return kNumConfigs; }
extern "C" __attribute__((visibility("default"))) const char* vaq_mfma_mix_probe_name(int i) {
  return i >= 0 && i < kNumConfigs ? kConfigs[i].what : nullptr;
}
// FLOPs of one launch of configuration `i` with `iters` iterations (256 workgroups).
extern "C" __attribute__((visibility("default"))) double vaq_mfma_mix_probe_flops(int i, int iters) {
  if (i < 0 || i >= kNumConfigs) return 0.0;
  const MixConfig& c = kConfigs[i];
  const double per = c.kind == 0 ? 32768.0 : c.kind == 1 ? 16384.0 : c.kind == 2 ? 131072.0 : 65536.0;
  return 256.0 * c.waves * (double)iters * c.nm * per;
}
// Launches configuration `i` on `stream`: `ticks` = 2048 device words (per workgroup and wavefront: 100 MHz ticks spent in
// the loop), `sink` = a device word that is practically never written.  Returns 0, or -1 for an unknown configuration.
extern "C" __attribute__((visibility("default"))) int vaq_mfma_mix_probe(int i, int iters, void* ticks, void* sink, void* stream) {
  if (i < 0 || i >= kNumConfigs || iters < 1 || !ticks || !sink) return -1;
  kConfigs[i].launch((unsigned long long*)ticks, (unsigned*)sink, iters, (hipStream_t)stream);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

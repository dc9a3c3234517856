// Shared device helpers for the gfx950 (CDNA4) kernels: bf16 / fp8 conversion with the
// rounding the reference's torch emulations use (round to nearest even, one rounding per
// output), 128-bit vector types, wavefront (64-lane) reductions and the status codes the
// C-ABI returns.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define TFB_OK 0
#define TFB_ERR_SHAPE 1     // a dimension the kernels do not take (caller falls back or raises)
#define TFB_ERR_ARG 2       // null pointer / bad enum
#define TFB_ERR_LAUNCH 3    // hipGetLastError() after the launch was not hipSuccess
#define TFB_ERR_WORKSPACE 4 // workspace too small

#define TFB_WAVE 64

typedef uint16_t bf16_t;  // raw bf16 bits; arithmetic is always done in fp32

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf2f(bf16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// Two fp32 -> packed bf16 pair (lo in bits 0..15), round to nearest even. Written as a vector conversion so that the
// compiler selects gfx950's v_cvt_pk_bf16_f32 itself: as inline assembly the instruction is opaque to the hazard
// recognizer, and a conversion scheduled right behind the MFMA / transcendental that feeds it read stale lanes.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack2bf(float lo, float hi) {
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ float bflo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bfhi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// fp32 -> bf16, round to nearest even (torch's .to(torch.bfloat16)); NaN stays NaN. One hardware conversion: the
// integer form of this rounding (add 0x7fff + lsb, shift, a NaN test) costs seven vector instructions per value, and
// epilogues that round every element twice spent more cycles on it than their GEMM's k-loop on MFMAs.
__device__ __forceinline__ bf16_t f2bf(float f) { return (bf16_t)pack2bf(f, 0.f); }

// acc + lo + hi of a packed bf16 pair in one instruction (v_dot2c_f32_bf16 against the pair (1, 1)).
__device__ __forceinline__ float sum2bf(uint32_t w, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), acc,
                                         false);
}

// Round an fp32 value to the nearest bf16 and return it as fp32 (a rounding point of the
// reference arithmetic that stays in registers).
__device__ __forceinline__ float round_bf(float f) { return bflo(pack2bf(f, 0.f)); }
// The same for a pair, in place (one conversion for the two): returns the packed bf16 pair as well.
__device__ __forceinline__ uint32_t round2_bf(float& a, float& b) {
  const uint32_t w = pack2bf(a, b);
  a = bflo(w);
  b = bfhi(w);
  return w;
}

// 8 fp32 values <-> 8 bf16 in four 32-bit words (one 128-bit access)
__device__ __forceinline__ u32x4 pack8bf(const float (&v)[8]) {
  u32x4 o = {pack2bf(v[0], v[1]), pack2bf(v[2], v[3]), pack2bf(v[4], v[5]), pack2bf(v[6], v[7])};
  return o;
}
__device__ __forceinline__ void unpack8bf(u32x4 u, float (&v)[8]) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    v[2 * k] = bflo(u[k]);
    v[2 * k + 1] = bfhi(u[k]);
  }
}

// fp32 -> OCP fp8 bytes (gfx950's v_cvt_pk_*_f32 are OCP e4m3fn / e5m2, round to nearest
// even). Inputs are clamped to the format's finite range first, so a value beyond it
// saturates instead of becoming NaN/Inf (a NaN input stays NaN, as in torch's cast); inside the range the bytes are torch's
// .to(float8_e4m3fn) / .to(float8_e5m2).
#define TFB_E4M3_MAX 448.0f
#define TFB_E5M2_MAX 57344.0f
#define TFB_FMT_E4M3 0
#define TFB_FMT_E5M2 1

// CLAMP = false: for values the caller has already bounded inside the format's range.
template <int FMT, bool CLAMP = true>
__device__ __forceinline__ uint32_t cvt4_fp8(float a, float b, float c, float d) {
  if (CLAMP) {  // saturate the finite values; a NaN stays a NaN (fminf / fmaxf alone would turn it into -max)
    const float mx = FMT == TFB_FMT_E4M3 ? TFB_E4M3_MAX : TFB_E5M2_MAX;
    a = a != a ? a : fminf(fmaxf(a, -mx), mx);
    b = b != b ? b : fminf(fmaxf(b, -mx), mx);
    c = c != c ? c : fminf(fmaxf(c, -mx), mx);
    d = d != d ? d : fminf(fmaxf(d, -mx), mx);
  }
  int w = 0;
  if (FMT == TFB_FMT_E4M3) {
    w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  } else {
    w = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, w, false);
    w = __builtin_amdgcn_cvt_pk_bf8_f32(c, d, w, true);
  }
  return (uint32_t)w;
}

// Streaming accesses: a tensor written now and read again much later (or read once) goes past the L2's retention with the
// non-temporal hint, so that it does not push out the tiles other workgroups re-read. Only for accesses that cover whole
// 128-byte lines between the lanes of one instruction: on partial lines the hint bypasses the L2's write merging.
// Each use is switched by a macro (default on) so that it can be measured alone.
template <class T>
__device__ __forceinline__ void tfb_store_nt(T* p, T v, bool on = true) {
  if (on) __builtin_nontemporal_store(v, p);
  else *p = v;
}
template <class T>
__device__ __forceinline__ T tfb_load_nt(const T* p, bool on = true) {
  return on ? __builtin_nontemporal_load(p) : *p;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Workgroups that are resident at once when `per_cu` of them fit a compute unit: per_cu x the device's CU count (read
// once per device). Kernels use it for what concerns the FIRST round of workgroups only (the start offset between the
// workgroups that share a CU, the split-K cost model); 256 CUs are assumed if the query fails.
static inline int tfb_resident_slots(int per_cu) {
  static int cus[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return per_cu * 256;
  if (cus[dev] == 0) {
    int n = 0;
    cus[dev] = (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) ? n : 256;
  }
  return per_cu * cus[dev];
}

#define TFB_LAUNCH_CHECK()                                  \
  do {                                                      \
    if (hipGetLastError() != hipSuccess) return TFB_ERR_LAUNCH; \
  } while (0)

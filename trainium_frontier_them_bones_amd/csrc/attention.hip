// Causal flash attention forward / backward for gfx950, bf16 with fp32 accumulation.
//
// Replaces _attn_fwd_kernel / _attn_bwd_kernel (round1/source/train.py:7536, 7591; the same
// pair in round2/source/kernels/nki_attn_bandpro.py) behind nki_causal_attention
// (round1/source/train.py:8069). Arithmetic follows the reference emulation
// (nki_attn_bandpro.py:1510-1551): scores in fp32, P = exp(scale*S - shift) rounded to bf16
// before every product it enters, the row sum taken over those rounded values, O = acc / sum
// rounded once, lse = log(sum) + shift, D = sum(dO * O) in fp32, dS = (dP - D) * P rounded to
// bf16, dQ and dK scaled in fp32 and rounded once. The shift is a running row maximum (the
// reference's fixed shift assumes QK-normed inputs), which changes results only by fp32
// rescaling error.
//
// The kernels live in attention64.hip (D = 64) and attention128.hip (D = 128): a wavefront owns 32 queries (forward, dQ)
// or 32 keys (dK/dV) as the MFMA *column* index (32x32x16 bf16, 64-lane wavefronts), so every row statistic (max, sum,
// lse, D) is one scalar per lane, and the score tile's accumulator registers, packed to bf16, are directly the B operand
// of the next product (P never touches LDS). This file holds the C-ABI entry points and their argument checks.
//
// Tensors are addressed by (batch, head, token) element strides with the head dimension
// contiguous, so q/k/v may be thirds of a fused qkv [B,T,3C] buffer and o / dO are [B,T,H,D].
#include <cstdlib>
#include "common.hpp"

namespace {
bool strides_ok(const long* s) { return s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0; }
}  // namespace

// D = 64 runs the kernels of attention64.hip (direct-to-LDS tile loads, transposed LDS fragment reads).
int tfb_attn64_fwd_impl(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs, void* o,
                        const long* os, float* lse, int B, int H, int T, float scale, int nw, hipStream_t s);
int tfb_attn64_bwd_impl(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs,
                        const void* o, const long* os, const void* go, const long* gos, void* dq, const long* dqs, void* dk,
                        const long* dks, void* dv, const long* dvs, const float* lse, float* stats, int B, int H, int T,
                        float scale, const void* cos_t, const void* sin_t, int nw, hipStream_t s);

// D = 128 runs the kernels of attention128.hip (the same data movement at the other head dimension).
int tfb_attn128_fwd_impl(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs,
                       void* o, const long* os, float* lse, int B, int H, int T, float scale, int nw, hipStream_t s);
int tfb_attn128_bwd_impl(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs,
                       const void* o, const long* os, const void* go, const long* gos, void* dq, const long* dqs, void* dk,
                       const long* dks, void* dv, const long* dvs, const float* lse, float* stats, int B, int H, int T,
                       float scale, int nw, hipStream_t s);
// Every tensor argument comes with long[3] element strides (batch, head, token); the head dimension is contiguous.
// lse: fp32 [B*H][T].
// nw > 0: the tile band of the reference's windowed layers (band_mask, round2/source/kernels/nki_attn_bandpro.py:1654):
// a query of 128-token tile i sees the keys k <= q of tiles i - nw + 1 .. i; nw = 0: all keys k <= q.
extern "C" int tfb_attn_fwd_band(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs,
                                 void* o, const long* os, void* lse, int B, int H, int T, int D, float scale, int nw,
                                 void* stream) {
  if (!q || !k || !v || !o || !lse || !qs || !ks || !vs || !os) return TFB_ERR_ARG;
  if (B <= 0 || H <= 0 || T <= 0 || T % 128 || (D != 64 && D != 128) || nw < 0) return TFB_ERR_SHAPE;
  if (!strides_ok(qs) || !strides_ok(ks) || !strides_ok(vs) || !strides_ok(os)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (D == 64) return tfb_attn64_fwd_impl(q, qs, k, ks, v, vs, o, os, (float*)lse, B, H, T, scale, nw, s);
  return tfb_attn128_fwd_impl(q, qs, k, ks, v, vs, o, os, (float*)lse, B, H, T, scale, nw, s);
}
extern "C" int tfb_attn_fwd(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs, void* o,
                            const long* os, void* lse, int B, int H, int T, int D, float scale, void* stream) {
  return tfb_attn_fwd_band(q, qs, k, ks, v, vs, o, os, lse, B, H, T, D, scale, 0, stream);
}

// delta: fp32 [2][B*H][T] scratch (the rows' -sum(dO O), then their -lse / scale: the dQ kernel writes both, dK/dV reads them). dq, dk, dv may alias thirds of one dqkv buffer.
// cos_t / sin_t (bf16 [T][D/2], both or neither): dq and dk come out with the inverse RoPE rotation applied, i.e. as
// gradients of the projections the rotation was applied to (D = 64 only; otherwise TFB_ERR_SHAPE and the caller runs
// tfb_rope itself).
extern "C" int tfb_attn_bwd_band(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs,
                                 const void* o, const long* os, const void* go, const long* gos, void* dq, const long* dqs,
                                 void* dk, const long* dks, void* dv, const long* dvs, const void* lse, void* delta,
                                 const void* cos_t, const void* sin_t, int B, int H, int T, int D, float scale, int nw,
                                 void* stream) {
  if (!q || !k || !v || !o || !go || !dq || !dk || !dv || !lse || !delta) return TFB_ERR_ARG;
  if (!qs || !ks || !vs || !os || !gos || !dqs || !dks || !dvs) return TFB_ERR_ARG;
  if ((cos_t == nullptr) != (sin_t == nullptr)) return TFB_ERR_ARG;
  if (B <= 0 || H <= 0 || T <= 0 || T % 128 || (D != 64 && D != 128) || nw < 0) return TFB_ERR_SHAPE;
  if (cos_t && D != 64) return TFB_ERR_SHAPE;
  if (!strides_ok(qs) || !strides_ok(ks) || !strides_ok(vs) || !strides_ok(os) || !strides_ok(gos) || !strides_ok(dqs) ||
      !strides_ok(dks) || !strides_ok(dvs))
    return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (D == 64)
    return tfb_attn64_bwd_impl(q, qs, k, ks, v, vs, o, os, go, gos, dq, dqs, dk, dks, dv, dvs, (const float*)lse, (float*)delta,
                               B, H, T, scale, cos_t, sin_t, nw, s);
  return tfb_attn128_bwd_impl(q, qs, k, ks, v, vs, o, os, go, gos, dq, dqs, dk, dks, dv, dvs, (const float*)lse, (float*)delta,
                              B, H, T, scale, nw, s);
}
extern "C" int tfb_attn_bwd_rope(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs,
                                 const void* o, const long* os, const void* go, const long* gos, void* dq, const long* dqs,
                                 void* dk, const long* dks, void* dv, const long* dvs, const void* lse, void* delta,
                                 const void* cos_t, const void* sin_t, int B, int H, int T, int D, float scale, void* stream) {
  return tfb_attn_bwd_band(q, qs, k, ks, v, vs, o, os, go, gos, dq, dqs, dk, dks, dv, dvs, lse, delta, cos_t, sin_t, B, H, T, D,
                           scale, 0, stream);
}

extern "C" int tfb_attn_bwd(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs,
                            const void* o, const long* os, const void* go, const long* gos, void* dq, const long* dqs, void* dk,
                            const long* dks, void* dv, const long* dvs, const void* lse, void* delta, int B, int H, int T, int D,
                            float scale, void* stream) {
  return tfb_attn_bwd_rope(q, qs, k, ks, v, vs, o, os, go, gos, dq, dqs, dk, dks, dv, dvs, lse, delta, nullptr, nullptr, B, H, T,
                           D, scale, stream);
}

// ---- attention backward for callers that cannot allocate --------------------------------------------------------------
// tfb_attn_bwd needs fp32 [2][B*H][T] of device scratch (the row statistics its first kernel, dQ, leaves for
// the second) and takes it from the caller. Code under HIP graph capture, tight serving loops and harnesses that forbid
// hipMalloc cannot provide one, so this variant keeps that scratch in the library's own image: a file-scope device
// array of TFB_ATTN_STATIC_ROWS * 2 floats (8 MiB, held by every GPU the library runs on until the process ends).
// In host code the array's name is only a stand-in for the symbol: its per-device address comes from
// hipGetSymbolAddress, once per device, and that pointer - never the name - is what the kernels receive.
// Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams) race on it. The first
// kernel writes every element the later ones read, so nothing has to be cleared between calls.
#define TFB_ATTN_STATIC_ROWS (1L << 20)
#define TFB_MAX_DEVICES 64
static __device__ __align__(256) float scratch[2 * TFB_ATTN_STATIC_ROWS];
static float* volatile scratch_ptr[TFB_MAX_DEVICES];

static int attn_static_scratch(float** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= TFB_MAX_DEVICES) return TFB_ERR_ARG;
  float* p = scratch_ptr[dev];
  if (!p) {
    // (two threads racing here both ask for the same address: the second store is the first one again)
    if (hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return TFB_ERR_LAUNCH;
    scratch_ptr[dev] = p;
  }
  *out = p;
  return TFB_OK;
}

extern "C" long tfb_attn_bwd_static_max_rows(void) { return TFB_ATTN_STATIC_ROWS; }

extern "C" int tfb_attn_bwd_static(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs,
                                   const void* o, const long* os, const void* go, const long* gos, void* dq, const long* dqs,
                                   void* dk, const long* dks, void* dv, const long* dvs, const void* lse, int B, int H, int T,
                                   int D, float scale, void* stream) {
  if (B <= 0 || H <= 0 || T <= 0) return TFB_ERR_SHAPE;
  if ((long)B * H * T > TFB_ATTN_STATIC_ROWS) return TFB_ERR_WORKSPACE;  // beyond the static scratch: use tfb_attn_bwd
  float* delta = nullptr;
  const int st = attn_static_scratch(&delta);
  if (st != TFB_OK) return st;
  return tfb_attn_bwd(q, qs, k, ks, v, vs, o, os, go, gos, dq, dqs, dk, dks, dv, dvs, lse, delta, B, H, T, D, scale, stream);
}

// bf16 GEMM primitive behind the C-ABI: C[M,N] = op(A) @ op(B), fp32 accumulation, one
// rounding to bf16 (or fp32 output), optional accumulate into C (the in-place weight-gradient
// sum) and split-K through an fp32 workspace for small outputs with a long contraction.
// Replaces the reference's nki_matmul(a, b, trans_a, trans_b) (round1/source/train.py:1137)
// and the torch matmuls its Linear glue issues (round1/source/train.py:8419-8711).
#include "gemm_pp.hpp"

namespace {

template <int LAYP, int LAYQ>
int run(GemmOperand P, GemmOperand Q, int N, int M, int K, void* C, int out_f32, int accumulate, float* ws, long ws_bytes,
        const float* alpha, hipStream_t stream) {
  using Cfg = GemmCfg<128, 128, 2, 2, 2, LAYP, LAYQ>;
  // Long contractions (at least 128 k-tiles) in any operand layout: the persistent 256 x 256 kernel, partial tiles through
  // the fp32 workspace. With 64 or more output tiles the k range is cut into the fewest parts that fill whole rounds of
  // the CUs to 90 % (the LM head's two gradient GEMMs: 384 tiles x 2 = 3 per CU). With fewer (the layers' weight
  // gradients: 9 to 27 tiles of 512 k-tiles) every workgroup gets one work item: as many k ranges per XCD as its 32 CUs
  // have room for tiles, so that an XCD's workgroups read one k range of the operands together (27 tiles: 8 ranges,
  // 9 tiles: 24), or, from 33 tiles, the number of ranges that fills the CUs.
#ifndef TFB_PP_LONGK
#define TFB_PP_LONGK 1
#endif
#ifndef TFB_PP_FEWTILE
#define TFB_PP_FEWTILE 1
#endif
  if (TFB_PP && TFB_PP_LONGK && N % 256 == 0 && M % 256 == 0 && K % 64 == 0 && K / 64 >= 128) {
    const long t256 = (long)(N / 256) * (M / 256), nkt = K / 64, cus = tfb_resident_slots(1);
    int sp = 0;
    if (t256 >= 64) {
      for (int c = 1; c <= 8 && !sp; ++c) {
        if (nkt / c < 32) continue;
        if (c > 1 && (!ws || (long)c * M * N * 4 > ws_bytes)) continue;
        const long items = t256 * c, rounds = (items + cus - 1) / cus;
        if ((double)items >= 0.9 * (double)(rounds * cus)) sp = c;
      }
    } else if (ws && TFB_PP_FEWTILE) {
      sp = gemm_pp_fewtile_splits(t256, nkt, (long)M * N, ws_bytes);
    }
    if (sp == 1 && !out_f32 && !accumulate) {
      EpiStore e{C, (long)N, out_f32, accumulate, alpha};
      return gemm_pp_launch_lay<2, 0, 0, LAYP, LAYQ>(P, Q, N, M, (long)K * 2, 1, e, stream);
    }
    if (sp > 1) {
      EpiSplit e{ws, (long)N, (long)M * N};
      int st = gemm_pp_launch_lay<2, 0, 0, LAYP, LAYQ>(P, Q, N, M, (long)K * 2, sp, e, stream);
      if (st != TFB_OK) return st;
      return splitk_reduce(ws, C, (long)M * N, sp, out_f32, accumulate, stream, nullptr, nullptr, 1.0f, alpha);
    }
  }
  const long tiles = (long)(N / 128) * (M / 128);
  const int splits = ws ? choose_splits(tiles, K / 64, (long)M * N, ws_bytes) : 1;
  if (splits == 1) {
    EpiStore e{C, (long)N, out_f32, accumulate, alpha};
    // large outputs: the persistent 256 x 256 kernel (same sums in the same order), in any operand layout (the input
    // gradient of the QKV projection, whose weight is read k-strided: 123.6 -> 117.7 us inside the step)
    if (!out_f32 && !accumulate && gemm_pp_applies(N, M, (long)K * 2))
      return gemm_pp_launch_lay<2, 0, 0, LAYP, LAYQ>(P, Q, N, M, (long)K * 2, 1, e, stream);
    return gemm_launch<Cfg>(P, Q, N, M, (long)K * 2, 1, LoadIdentity{}, LoadIdentity{}, e, stream);
  }
  EpiSplit e{ws, (long)N, (long)M * N};
  int st = gemm_launch<Cfg>(P, Q, N, M, (long)K * 2, splits, LoadIdentity{}, LoadIdentity{}, e, stream);
  if (st != TFB_OK) return st;
  return splitk_reduce(ws, C, (long)M * N, splits, out_f32, accumulate, stream, nullptr, nullptr, 1.0f, alpha);
}

// out [q][ld] = bf16(D) with the rotary embedding applied to the first rot_cols columns (heads of 64: y1 = x1 c + x2 s,
// y2 = x2 c - x1 s on the bf16-rounded products, rounded again - what tfb_rope computes from the stored projection).
struct EpiStoreRope {
  static constexpr bool kPartner32 = true;
  bf16_t* out;
  long ld;
  const bf16_t* cs;  // [T][32]
  const bf16_t* sn;
  int T, rot_cols;
  struct pre_t {  // the chunk's cos / sin values, requested before the k-loop
    u32x4 c, s;
  };
  __device__ __forceinline__ pre_t prefetch(int p, int q) const {
    pre_t r = {};
    if (p < rot_cols) {
      const int t = q % T, idx = p & 31;
      r.c = *(const u32x4*)(cs + (long)t * 32 + idx);
      r.s = *(const u32x4*)(sn + (long)t * 32 + idx);
    }
    return r;
  }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], const float (&vp)[8], const pre_t& tab,
                                             int) const {
    u32x4 x = pack8bf(v);
    if (p < rot_cols) {
      const u32x4 y = pack8bf(vp);
      const bool low = (p & 32) == 0;
      const u32x4 c = tab.c, s = tab.s;
      u32x4 o;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float x0 = bflo(x[k]), x1 = bfhi(x[k]), y0 = bflo(y[k]), y1 = bfhi(y[k]);
        const float c0 = bflo(c[k]), c1 = bfhi(c[k]), s0 = bflo(s[k]), s1 = bfhi(s[k]);
        o[k] = low ? pack2bf(x0 * c0 + y0 * s0, x1 * c1 + y1 * s1) : pack2bf(x0 * c0 - y0 * s0, x1 * c1 - y1 * s1);
      }
      x = o;
    }
    *(u32x4*)(out + (long)q * ld + p) = x;
  }
  // the 256 x 256 kernel's protocol: the same from the rounded products
  __device__ __forceinline__ float pre(float x) const { return x; }
  __device__ __forceinline__ void chunk(int p, int q, const u32x4& xin, const u32x4& y, const pre_t& tab) const {
    u32x4 x = xin;
    if (p < rot_cols) {
      const bool low = (p & 32) == 0;
      const u32x4 c = tab.c, s = tab.s;
      u32x4 o;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float x0 = bflo(x[k]), x1 = bfhi(x[k]), y0 = bflo(y[k]), y1 = bfhi(y[k]);
        const float c0 = bflo(c[k]), c1 = bfhi(c[k]), s0 = bflo(s[k]), s1 = bfhi(s[k]);
        o[k] = low ? pack2bf(x0 * c0 + y0 * s0, x1 * c1 + y1 * s1) : pack2bf(x0 * c0 - y0 * s0, x1 * c1 - y1 * s1);
      }
      x = o;
    }
    *(u32x4*)(out + (long)q * ld + p) = x;
  }
};

}  // namespace

// tfb_gemm_bf16 with the product multiplied by the device fp32 scalar *alpha (NULL = 1) before its one rounding:
// C (+)= alpha op(A) @ op(B). For gradient GEMMs whose upstream scalar lives on the device.
extern "C" int tfb_gemm_bf16_scaled(const void* A, const void* B, void* C, int M, int N, int K, int trans_a, int trans_b,
                                    int out_f32, int accumulate, void* workspace, long workspace_bytes, const void* alpha,
                                    void* stream) {
  if (!A || !B || !C) return TFB_ERR_ARG;
  if (M <= 0 || N <= 0 || K <= 0 || M % 128 || N % 128 || K % 64) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  // The output's contiguous dimension (n) rides the P side of the core.
  GemmOperand P, Q;
  P.base = (const uint8_t*)B;
  Q.base = (const uint8_t*)A;
  P.ld = trans_b ? (long)K * 2 : (long)N * 2;
  Q.ld = trans_a ? (long)M * 2 : (long)K * 2;
  float* ws = (float*)workspace;
  const float* al = (const float*)alpha;
  if (trans_b && !trans_a) return run<TFB_K_CONTIG, TFB_K_CONTIG>(P, Q, N, M, K, C, out_f32, accumulate, ws, workspace_bytes, al, s);
  if (!trans_b && !trans_a) return run<TFB_K_STRIDED, TFB_K_CONTIG>(P, Q, N, M, K, C, out_f32, accumulate, ws, workspace_bytes, al, s);
  if (!trans_b && trans_a) return run<TFB_K_STRIDED, TFB_K_STRIDED>(P, Q, N, M, K, C, out_f32, accumulate, ws, workspace_bytes, al, s);
  return run<TFB_K_CONTIG, TFB_K_STRIDED>(P, Q, N, M, K, C, out_f32, accumulate, ws, workspace_bytes, al, s);
}

extern "C" int tfb_gemm_bf16(const void* A, const void* B, void* C, int M, int N, int K, int trans_a, int trans_b,
                             int out_f32, int accumulate, void* workspace, long workspace_bytes, void* stream) {
  return tfb_gemm_bf16_scaled(A, B, C, M, N, K, trans_a, trans_b, out_f32, accumulate, workspace, workspace_bytes, nullptr, stream);
}

// C [M][N] = bf16(res + bf16(A [M][K] @ op(B))), B [N][K] (trans_b) or [K][N]: a projection with the residual add that
// follows it made in the store. Equal to tfb_gemm_bf16 followed by a bf16 add, bit for bit. The bf16 form of the
// reference's projection-with-residual forward (round2/source/kernels/nki_attn_nr8.py:1003).
extern "C" int tfb_gemm_bf16_res(const void* A, const void* B, const void* res, void* C, int M, int N, int K, int trans_b,
                                 void* stream) {
  if (!A || !B || !res || !C) return TFB_ERR_ARG;
  if (M <= 0 || N <= 0 || K <= 0 || M % 128 || N % 128 || K % 64) return TFB_ERR_SHAPE;
  GemmOperand P{(const uint8_t*)B, trans_b ? (long)K * 2 : (long)N * 2}, Q{(const uint8_t*)A, (long)K * 2};
  EpiStoreRes e{(bf16_t*)C, (const bf16_t*)res, (long)N};
  if (trans_b && gemm_pp_applies(N, M, (long)K * 2)) return gemm_pp_launch<2, 0, 0>(P, Q, N, M, (long)K * 2, e, (hipStream_t)stream);
  if (trans_b)
    return gemm_launch<GemmCfg<128, 128, 2, 2, 2, TFB_K_CONTIG, TFB_K_CONTIG>>(P, Q, N, M, (long)K * 2, 1, LoadIdentity{},
                                                                               LoadIdentity{}, e, (hipStream_t)stream);
  return gemm_launch<GemmCfg<128, 128, 2, 2, 2, TFB_K_STRIDED, TFB_K_CONTIG>>(P, Q, N, M, (long)K * 2, 1, LoadIdentity{},
                                                                              LoadIdentity{}, e, (hipStream_t)stream);
}

// qkv [M][N] = rope(x [M][K] @ w [N][K]^T): the fused attention projection with the rotary embedding of the q and k
// thirds (the first rot_cols columns, heads of 64 elements) applied in the GEMM epilogue; row m is token m % T.
// cos_t, sin_t: bf16 [T][32]. The output equals tfb_gemm_bf16 followed by tfb_rope bit for bit.
extern "C" int tfb_qkv_rope_fwd(const void* x, const void* w, const void* cos_t, const void* sin_t, void* out, int M, int N,
                                int K, int T, int rot_cols, void* stream) {
  if (!x || !w || !cos_t || !sin_t || !out) return TFB_ERR_ARG;
  if (M <= 0 || N <= 0 || K <= 0 || M % 128 || N % 128 || K % 64 || T <= 0 || rot_cols < 0 || rot_cols > N || rot_cols % 64)
    return TFB_ERR_SHAPE;
  using Cfg = GemmCfg<128, 128, 2, 2, 2, TFB_K_CONTIG, TFB_K_CONTIG>;
  GemmOperand P{(const uint8_t*)w, (long)K * 2}, Q{(const uint8_t*)x, (long)K * 2};
  EpiStoreRope e{(bf16_t*)out, (long)N, (const bf16_t*)cos_t, (const bf16_t*)sin_t, T, rot_cols};
  if (gemm_pp_applies(N, M, (long)K * 2)) return gemm_pp_launch<2, 0, 0>(P, Q, N, M, (long)K * 2, e, (hipStream_t)stream);
  return gemm_launch<Cfg>(P, Q, N, M, (long)K * 2, 1, LoadIdentity{}, LoadIdentity{}, e, (hipStream_t)stream);
}

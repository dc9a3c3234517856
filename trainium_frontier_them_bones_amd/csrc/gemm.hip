// bf16 GEMM primitive behind the C-ABI: C[M,N] = op(A) @ op(B), fp32 accumulation, one
// rounding to bf16 (or fp32 output), optional accumulate into C (the in-place weight-gradient
// sum) and split-K through an fp32 workspace for small outputs with a long contraction.
// Replaces the reference's nki_matmul(a, b, trans_a, trans_b) (round1/source/train.py:1137)
// and the torch matmuls its Linear glue issues (round1/source/train.py:8419-8711).
#include "gemm_core.hpp"

namespace {

struct EpiStore {
  void* out;   // bf16 or fp32 [nq][ld]
  long ld;     // elements
  int f32;
  int accumulate;
  __device__ __forceinline__ void operator()(int p, int q, f32x4 v, int) const {
    if (f32) {
      float* o = (float*)out + (long)q * ld + p;
      if (accumulate) {
        f32x4 c = *(const f32x4*)o;
        v += c;
      }
      *(f32x4*)o = v;
    } else {
      bf16_t* o = (bf16_t*)out + (long)q * ld + p;
      if (accumulate) {
        u32x2 c = *(const u32x2*)o;
        v[0] += bflo(c.x);
        v[1] += bfhi(c.x);
        v[2] += bflo(c.y);
        v[3] += bfhi(c.y);
      }
      u32x2 r = {pack2bf(v[0], v[1]), pack2bf(v[2], v[3])};
      *(u32x2*)o = r;
    }
  }
};

struct EpiSplit {
  float* ws;      // [splits][nq][ld]
  long ld, slab;  // slab = nq * ld
  __device__ __forceinline__ void operator()(int p, int q, f32x4 v, int split) const {
    *(f32x4*)(ws + (long)split * slab + (long)q * ld + p) = v;
  }
};

__global__ void splitk_reduce_kernel(const float* __restrict__ ws, void* out, long n, int splits, int f32, int accumulate) {
  long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= n) return;
  f32x4 s = *(const f32x4*)(ws + i);
  for (int k = 1; k < splits; ++k) s += *(const f32x4*)(ws + (long)k * n + i);
  if (f32) {
    float* o = (float*)out + i;
    if (accumulate) s += *(const f32x4*)o;
    *(f32x4*)o = s;
  } else {
    bf16_t* o = (bf16_t*)out + i;
    if (accumulate) {
      u32x2 c = *(const u32x2*)o;
      s[0] += bflo(c.x);
      s[1] += bfhi(c.x);
      s[2] += bflo(c.y);
      s[3] += bfhi(c.y);
    }
    u32x2 r = {pack2bf(s[0], s[1]), pack2bf(s[2], s[3])};
    *(u32x2*)o = r;
  }
}

template <int LAYP, int LAYQ>
int run(GemmOperand P, GemmOperand Q, int N, int M, int K, void* C, int out_f32, int accumulate, float* ws, long ws_bytes,
        hipStream_t stream) {
  using Cfg = GemmCfg<128, 128, 2, 2, 2, LAYP, LAYQ>;
  const long tiles = (long)(N / 128) * (M / 128);
  const int nkt = K / 64;
  int splits = 1;
  if (ws && tiles < 512 && nkt >= 32) {
    splits = (int)((768 + tiles - 1) / tiles);
    while (splits > 1 && (nkt % splits != 0 || nkt / splits < 8)) --splits;
    if ((long)splits * M * N * 4 > ws_bytes) splits = 1;
  }
  if (splits == 1) {
    EpiStore e{C, (long)N, out_f32, accumulate};
    return gemm_launch<Cfg>(P, Q, N, M, (long)K * 2, 1, LoadIdentity{}, LoadIdentity{}, e, stream);
  }
  EpiSplit e{ws, (long)N, (long)M * N};
  int st = gemm_launch<Cfg>(P, Q, N, M, (long)K * 2, splits, LoadIdentity{}, LoadIdentity{}, e, stream);
  if (st != TFB_OK) return st;
  long n = (long)M * N;
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, stream, ws, C, n, splits,
                     out_f32, accumulate);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

}  // namespace

extern "C" int tfb_gemm_bf16(const void* A, const void* B, void* C, int M, int N, int K, int trans_a, int trans_b,
                             int out_f32, int accumulate, void* workspace, long workspace_bytes, void* stream) {
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
  if (trans_b && !trans_a) return run<TFB_K_CONTIG, TFB_K_CONTIG>(P, Q, N, M, K, C, out_f32, accumulate, ws, workspace_bytes, s);
  if (!trans_b && !trans_a) return run<TFB_K_STRIDED, TFB_K_CONTIG>(P, Q, N, M, K, C, out_f32, accumulate, ws, workspace_bytes, s);
  if (!trans_b && trans_a) return run<TFB_K_STRIDED, TFB_K_STRIDED>(P, Q, N, M, K, C, out_f32, accumulate, ws, workspace_bytes, s);
  return run<TFB_K_CONTIG, TFB_K_STRIDED>(P, Q, N, M, K, C, out_f32, accumulate, ws, workspace_bytes, s);
}

// bf16 GEMM primitive behind the C-ABI: C[M,N] = op(A) @ op(B), fp32 accumulation, one
// rounding to bf16 (or fp32 output), optional accumulate into C (the in-place weight-gradient
// sum) and split-K through an fp32 workspace for small outputs with a long contraction.
// Replaces the reference's nki_matmul(a, b, trans_a, trans_b) (round1/source/train.py:1137)
// and the torch matmuls its Linear glue issues (round1/source/train.py:8419-8711).
#include "gemm_core.hpp"

namespace {

template <int LAYP, int LAYQ>
int run(GemmOperand P, GemmOperand Q, int N, int M, int K, void* C, int out_f32, int accumulate, float* ws, long ws_bytes,
        hipStream_t stream) {
  using Cfg = GemmCfg<128, 128, 2, 2, 2, LAYP, LAYQ>;
  const long tiles = (long)(N / 128) * (M / 128);
  const int splits = ws ? choose_splits(tiles, K / 64, (long)M * N, ws_bytes) : 1;
  if (splits == 1) {
    EpiStore e{C, (long)N, out_f32, accumulate};
    return gemm_launch<Cfg>(P, Q, N, M, (long)K * 2, 1, LoadIdentity{}, LoadIdentity{}, e, stream);
  }
  EpiSplit e{ws, (long)N, (long)M * N};
  int st = gemm_launch<Cfg>(P, Q, N, M, (long)K * 2, splits, LoadIdentity{}, LoadIdentity{}, e, stream);
  if (st != TFB_OK) return st;
  return splitk_reduce(ws, C, (long)M * N, splits, out_f32, accumulate, stream);
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

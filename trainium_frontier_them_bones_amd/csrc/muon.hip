// Muon's Newton-Schulz ("Polar Express") orthogonalisation of a stack of gradient matrices, five iterations, bf16 with
// fp32 accumulation. Replaces _nsk_kernel (round2/source/kernels/nki_nsk.py:370; arithmetic: emulate_nsk 452, _ns_tall 426)
// and the loop of muon_math_body it restates (reference_ns, nki_nsk.py:471).
//
// Per matrix, held tall X [M][N] (M >= N; a wide input [N][M] is transposed on the way in and out):
//   X0 = bf16(bf16(g) * (1 / d))
//   G  = bf16(X^T X)                          [N][N]   contraction over the M rows
//   B  = bf16(fp32(G G * c) + fp32(b * G))    [N][N]   one rounding
//   X' = bf16(fp32(X B) + fp32(a * X))        [M][N]   one rounding
// with the five (a, b, c) of the caller, then v[m] = sum_n X5[m][n]^2 in fp32 from the bf16 X5.
//
// The whole stack runs in three grouped GEMM launches per iteration (not three per matrix): the matrices are stacked
// along the rows, G's contraction is segmented per matrix (k_seg), and the two products against the per-matrix [N][N]
// operand pick it by the row tile's matrix (q_group). G and G G are symmetric bit for bit (the same products summed in
// the same order on either side of the diagonal), so B^T = B and both products run in the k-contiguous "x @ w^T" form
// with the [N][N] matrix as the weight; the reference's mirror fill of the lower blocks is therefore not needed.
#include "gemm_core.hpp"

namespace {

// out = bf16(fp32(alpha * D) + fp32(beta * z)), z and out [rows][ld] bf16; the z chunk is requested before the k-loop
struct EpiAxpby {
  bf16_t* out;
  const bf16_t* z;
  long ld;
  float alpha, beta;
  using pre_t = u32x4;
  __device__ __forceinline__ pre_t prefetch(int p, int q) const { return *(const u32x4*)(z + (long)q * ld + p); }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], const pre_t& zv, int) const {
    float zf[8], r[8];
    unpack8bf(zv, zf);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float t1 = v[k] * alpha, t2 = beta * zf[k];
      r[k] = t1 + t2;
    }
    *(u32x4*)(out + (long)q * ld + p) = pack8bf(r);
  }
};

// k_seg[i] = i * M (i <= K); gq[t] = t / (N / 128) for the K N / 128 row tiles of the stacked G; xq[t] = t / (M / 128)
__global__ void ns_tables_kernel(int* k_seg, int* gq, int* xq, int K, int M, int N) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i <= K) k_seg[i] = i * M;
  if (i < K * (N / 128)) gq[i] = i / (N / 128);
  if (i < K * (M / 128)) xq[i] = i / (M / 128);
}

// X0 [K][M][N] bf16 = bf16(bf16(g) * inv_d[k]); g fp32 [K][M][N], or with WIDE [K][N][M] (32 x 32 tiles through LDS)
template <bool WIDE>
__global__ __launch_bounds__(256) void ns_load_kernel(const float* __restrict__ g, const float* __restrict__ inv_d,
                                                     bf16_t* __restrict__ x, int M, int N) {
  const int k = blockIdx.z;
  const float r = inv_d[k];
  const long mat = (long)k * M * N;
  if (!WIDE) {
    const long n = (long)M * N;
    for (long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4; i < n; i += (long)gridDim.x * 256 * 4) {
      const f32x4 v = *(const f32x4*)(g + mat + i);
      u32x2 o = {pack2bf(round_bf(v[0]) * r, round_bf(v[1]) * r), pack2bf(round_bf(v[2]) * r, round_bf(v[3]) * r)};
      *(u32x2*)(x + mat + i) = o;
    }
  } else {
    __shared__ float t[32][33];
    const int m0 = blockIdx.x * 32, n0 = blockIdx.y * 32;  // tile of the tall X: rows m0.., columns n0..
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
    for (int j = 0; j < 32; j += 8) t[ty + j][tx] = g[mat + (long)(n0 + ty + j) * M + m0 + tx];  // g[n][m]
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 32; j += 8) x[mat + (long)(m0 + ty + j) * N + n0 + tx] = f2bf(round_bf(t[tx][ty + j]) * r);
  }
}

// v[k][m] = sum_n X[k][m][n]^2 (fp32, from the bf16 values): one wavefront per row
__global__ __launch_bounds__(256) void ns_rowsq_kernel(const bf16_t* __restrict__ x, float* __restrict__ v, long rows, int N) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  float s = 0.f;
  for (int c = lane * 8; c < N; c += 512) {
    float f[8];
    unpack8bf(*(const u32x4*)(x + row * N + c), f);
#pragma unroll
    for (int k = 0; k < 8; ++k) s += f[k] * f[k];
  }
  s = wave_sum(s);
  if (lane == 0) v[row] = s;
}

// y [K][N][M] = X [K][M][N]^T (bf16), 32 x 32 tiles through LDS
__global__ __launch_bounds__(256) void ns_transpose_out_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ y, int M, int N) {
  __shared__ bf16_t t[32][34];
  const long mat = (long)blockIdx.z * M * N;
  const int m0 = blockIdx.x * 32, n0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
  for (int j = 0; j < 32; j += 8) t[ty + j][tx] = x[mat + (long)(m0 + ty + j) * N + n0 + tx];
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 32; j += 8) y[mat + (long)(n0 + ty + j) * M + m0 + tx] = t[tx][ty + j];
}

inline long align256(long b) { return (b + 255) & ~255L; }

}  // namespace

// Bytes of device workspace tfb_ns5 needs for a stack of K matrices with long side M and short side N.
extern "C" long tfb_ns5_workspace_bytes(int K, int M, int N) {
  if (K <= 0 || M <= 0 || N <= 0) return 0;
  const long xb = align256((long)K * M * N * 2), gb = align256((long)K * N * N * 2);
  return 2 * xb + 2 * gb + align256(((long)K + 1 + (long)K * (N / 128) + (long)K * (M / 128)) * 4);
}

// g: fp32 [K][M][N] (wide = 0) or [K][N][M] (wide = 1: each matrix is handled as its transpose), M >= N; inv_d: fp32 [K]
// device (1 / d of each matrix, d as the caller's optimizer computes it); coeffs: 15 HOST floats, (a, b, c) of the five
// iterations; y: bf16, the layout of g; v: fp32 [K][M]. M, N multiples of 128. The call enqueues 3 + 15 (+1) launches
// on `stream` and returns; the workspace must stay untouched until they have run.
extern "C" int tfb_ns5(const void* g, const void* inv_d, const float* coeffs, void* y, void* v, int K, int M, int N, int wide,
                       void* workspace, long workspace_bytes, void* stream) {
  if (!g || !inv_d || !coeffs || !y || !v || !workspace) return TFB_ERR_ARG;
  if (K <= 0 || M <= 0 || N <= 0 || M % 128 || N % 128 || M < N || (long)K * M > 0x7fffffffL / 2 || K > 65535)
    return TFB_ERR_SHAPE;
  if (workspace_bytes < tfb_ns5_workspace_bytes(K, M, N)) return TFB_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  uint8_t* w = (uint8_t*)workspace;
  const long xb = align256((long)K * M * N * 2), gb = align256((long)K * N * N * 2);
  bf16_t* X[2] = {(bf16_t*)w, (bf16_t*)(w + xb)};
  bf16_t* G = (bf16_t*)(w + 2 * xb);
  bf16_t* Bm = (bf16_t*)(w + 2 * xb + gb);
  int* k_seg = (int*)(w + 2 * xb + 2 * gb);
  int* gq = k_seg + K + 1;
  int* xq = gq + (long)K * (N / 128);

  const int ntab = K * (M / 128) + 1;
  hipLaunchKernelGGL(ns_tables_kernel, dim3((ntab + 255) / 256), dim3(256), 0, s, k_seg, gq, xq, K, M, N);
  TFB_LAUNCH_CHECK();
  if (wide)
    hipLaunchKernelGGL(ns_load_kernel<true>, dim3(M / 32, N / 32, K), dim3(256), 0, s, (const float*)g, (const float*)inv_d, X[0],
                       M, N);
  else
    hipLaunchKernelGGL(ns_load_kernel<false>, dim3(256, 1, K), dim3(256), 0, s, (const float*)g, (const float*)inv_d, X[0], M, N);
  TFB_LAUNCH_CHECK();

  using CfgT = GemmCfg<128, 128, 2, 2, 2, TFB_K_STRIDED, TFB_K_STRIDED>;
  using CfgN = GemmCfg<128, 128, 2, 2, 2, TFB_K_CONTIG, TFB_K_CONTIG>;
  int cur = 0;
  for (int it = 0; it < 5; ++it) {
    const float a = coeffs[3 * it], b = coeffs[3 * it + 1], c = coeffs[3 * it + 2];
    bf16_t* xin = X[cur];
    // the tall stack's last iteration writes y itself
    bf16_t* xout = (it == 4 && !wide) ? (bf16_t*)y : X[cur ^ 1];
    GemmArgs ga;
    // G[k] = X[k]^T X[k]: both operands k-strided (rows of the stacked X), the contraction segmented per matrix
    ga.P = GemmOperand{(const uint8_t*)xin, (long)N * 2};
    ga.Q = ga.P;
    ga.np = N;
    ga.nq = N;
    ga.nkt = 0;
    ga.ntp = N / 128;
    ga.q_group = nullptr;
    ga.p_group_stride = 0;
    ga.k_seg = k_seg;
    EpiStoreGrouped eg{EpiStore{G, (long)N, 0, 0}, (long)N * N};
    int st = gemm_launch_args<CfgT>(ga, K, 1, LoadIdentity{}, LoadIdentity{}, eg, s);
    if (st != TFB_OK) return st;
    // B = c G G + b G on the stacked G: rows of G[k] against G[k] as the weight (G G^T = G G)
    GemmArgs gb2;
    gb2.P = GemmOperand{(const uint8_t*)G, (long)N * 2};
    gb2.Q = gb2.P;
    gb2.np = N;
    gb2.nq = K * N;
    gb2.nkt = N * 2 / 128;
    gb2.ntp = N / 128;
    gb2.q_group = gq;
    gb2.p_group_stride = (long)N * N * 2;
    gb2.k_seg = nullptr;
    EpiAxpby eb{Bm, G, (long)N, c, b};
    st = gemm_launch_args<CfgN>(gb2, 1, 1, LoadIdentity{}, LoadIdentity{}, eb, s);
    if (st != TFB_OK) return st;
    // X' = X B + a X on the stacked X: rows of X[k] against B[k] as the weight (X B^T = X B)
    GemmArgs gx;
    gx.P = GemmOperand{(const uint8_t*)Bm, (long)N * 2};
    gx.Q = GemmOperand{(const uint8_t*)xin, (long)N * 2};
    gx.np = N;
    gx.nq = K * M;
    gx.nkt = N * 2 / 128;
    gx.ntp = N / 128;
    gx.q_group = xq;
    gx.p_group_stride = (long)N * N * 2;
    gx.k_seg = nullptr;
    EpiAxpby ex{xout, xin, (long)N, 1.0f, a};
    st = gemm_launch_args<CfgN>(gx, 1, 1, LoadIdentity{}, LoadIdentity{}, ex, s);
    if (st != TFB_OK) return st;
    cur ^= 1;
  }
  const bf16_t* x5 = wide ? X[cur] : (const bf16_t*)y;
  const long rows = (long)K * M;
  hipLaunchKernelGGL(ns_rowsq_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, x5, (float*)v, rows, N);
  TFB_LAUNCH_CHECK();
  if (wide) {
    hipLaunchKernelGGL(ns_transpose_out_kernel, dim3(M / 32, N / 32, K), dim3(256), 0, s, x5, (bf16_t*)y, M, N);
    TFB_LAUNCH_CHECK();
  }
  return TFB_OK;
}

// fp8 fused MLP (up-projection -> ReLU^2 -> down-projection) for gfx950.
//
// Replaces _mlp8_fwd_kernel / _mlp8_bwd_kernel and their host helpers
// (round2/source/kernels/nki_mlp_fused8.py:509, 571, 742-858) and the per-step weight pre-cast
// (round2/source/kernels/nki_mlp_l4t.py:392, 948-970).
//
// MI355X design: the hidden activation of a 128-token block (128 x 3072 fp8 = 384 KB) does not
// fit a CU's 160 KB LDS, so the two GEMMs are two launches and h lives in HBM as e4m3 bytes
// (50 MB at 16384 x 3072: inside the 256 MB Infinity Cache between producer and consumer);
// everything elementwise (descale, ReLU, the saved r, clamp, square, fp8 casts, the ReLU^2
// backward) is fused into the GEMM epilogues, and weights are cast once per optimizer step into a
// pack of four k-contiguous byte layouts so that all four activation GEMMs are NT fp8 GEMMs on
// v_mfma_scale_f32_32x32x64_f8f6f4. Rounding points are the reference emulation's:
//   x8 = e4m3(x * s_x); r = bf16(max(acc * dq_fc, 0)); rc = bf16(min(r * c_h, 15.375));
//   h8 = e4m3(rc^2); y = bf16(acc * dq_proj); dy8 = e5m2(dy * s_dy);
//   dpre = bf16((acc * dq_dh2) * r); dp8 = e5m2(dpre * s_dp); dx = bf16(acc * dq_dx).
#include "gemm_ws8.hpp"

// scale-row columns (nki_mlp_fused8.py:111-114)
#define SC_S_WFC 0
#define SC_DQ_FC 1
#define SC_C_H 2
#define SC_S_WPROJ 3
#define SC_DQ_PROJ 4
#define SC_S_DY 5
#define SC_DQ_DH2 6
#define SC_S_DP 7
#define SC_DQ_DX 8
#define SC_RHO2 9
#define SC_KAPPA2 10
#define SC_I_WFC 11
#define SC_I_WPROJ 12
#define SC_S_H 13
#define SC_AMAX_WFC 14
#define SC_AMAX_WPROJ 15
#define NSC 16

namespace {

constexpr float H_CLAMP = 15.375f;

// ------------------------------------------------------------------------------------ scale search
// s = 2^e, largest e in [e_lo, e_hi] with v * s <= limit; comparisons and power-of-two products
// only (nki_mlp_fused8.py:742-758), so s and 1/s are exact.
__device__ void pow2_le(float v, float limit, int e_lo, int e_hi, float* s_out, float* inv_out) {
  float s = ldexpf(1.0f, e_lo), inv = ldexpf(1.0f, -e_lo);
  const float top = ldexpf(1.0f, e_hi);
  const int span = e_hi - e_lo;
  for (int b = 64; b >= 1; b >>= 1) {
    if (b > span) continue;
    float cand = s * ldexpf(1.0f, b);
    bool ok = (v * cand <= limit) && (cand <= top);
    if (ok) {
      s = cand;
      inv = inv * ldexpf(1.0f, -b);
    }
  }
  *s_out = s;
  *inv_out = inv;
}

// s = 4^e (nki_mlp_fused8.py:761-779); c = 2^e.
__device__ void pow4_le(float v, float limit, int e_lo, int e_hi, float* s_out, float* inv_out, float* c_out) {
  float s = ldexpf(1.0f, 2 * e_lo), inv = ldexpf(1.0f, -2 * e_lo), c = ldexpf(1.0f, e_lo);
  const float top = ldexpf(1.0f, 2 * e_hi);
  const int span = e_hi - e_lo;
  for (int b = 32; b >= 1; b >>= 1) {
    if (b > span) continue;
    float cand = s * ldexpf(1.0f, 2 * b);
    bool ok = (v * cand <= limit) && (cand <= top);
    if (ok) {
      s = cand;
      inv = inv * ldexpf(1.0f, -2 * b);
      c = c * ldexpf(1.0f, b);
    }
  }
  *s_out = s;
  *inv_out = inv;
  *c_out = c;
}

__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float m = red[0];
  for (int i = 1; i < (int)(blockDim.x >> 6); ++i) m = fmaxf(m, red[i]);
  return m;
}

// ------------------------------------------------------------------------------------ statistics
// amax over a bf16 tensor: per-workgroup partials.
__global__ __launch_bounds__(256) void amax_partial_kernel(const bf16_t* __restrict__ x, long n, float* __restrict__ part) {
  __shared__ float red[4];
  float m = 0.f;
  for (long i = ((long)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += (long)gridDim.x * 256 * 8) {
    u32x4 u = *(const u32x4*)(x + i);
#pragma unroll
    for (int k = 0; k < 4; ++k) m = fmaxf(m, fmaxf(fabsf(bflo(u[k])), fabsf(bfhi(u[k]))));
  }
  m = block_max(m, red);
  if (threadIdx.x == 0) part[blockIdx.x] = m;
}

// One wavefront per row of w [rows][cols]: sum of squares per row; amax partial per workgroup.
// blockIdx.z = layer of a batched refresh: w advances by wz elements, the outputs by their per-layer sizes (oz floats).
// (bx of gx workgroups; the job of weight_stats_kernel's first gx workgroups)
__device__ __forceinline__ void row_stats_job(const bf16_t* __restrict__ w, int rows, int cols, float* __restrict__ rowss,
                                              float* __restrict__ amax_part, int bx, int gx, float* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float m = 0.f;
  for (int r = bx * 4 + wave; r < rows; r += gx * 4) {
    float ss = 0.f;
    for (int c = lane * 8; c < cols; c += 512) {
      u32x4 u = *(const u32x4*)(w + (long)r * cols + c);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float a = bflo(u[k]), b = bfhi(u[k]);
        ss += a * a;
        ss += b * b;
        m = fmaxf(m, fmaxf(fabsf(a), fabsf(b)));
      }
    }
    ss = wave_sum(ss);
    if (lane == 0) rowss[r] = ss;
  }
  m = block_max(m, red);
  if (threadIdx.x == 0) amax_part[bx] = m;
}

// Column sums of squares of w [rows][cols]: a workgroup owns 512 columns (64 lanes x 8) of one slice of the rows
// (blockIdx.y of COL_SLICES), its 4 wavefronts take interleaved rows; the slices' partial sums go to
// colss_part [COL_SLICES][cols] and are added in slice order by the scale kernel; amax partial per workgroup.
constexpr int COL_SLICES = 32;
__device__ __forceinline__ void col_stats_job(const bf16_t* __restrict__ w, int rows, int cols, float* __restrict__ colss_part,
                                              float* __restrict__ amax_part, int bx, int by, int gx, int gy, float* red,
                                              float (*acc)[512]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = bx * 512 + lane * 8;
  const int per = (rows + gy - 1) / gy;
  const int r0 = by * per, r1 = min(rows, r0 + per);
  float ss[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  float m = 0.f;
  if (c < cols) {
    for (int r = r0 + wave; r < r1; r += 4) {
      u32x4 u = *(const u32x4*)(w + (long)r * cols + c);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float a = bflo(u[k]), b = bfhi(u[k]);
        ss[2 * k] += a * a;
        ss[2 * k + 1] += b * b;
        m = fmaxf(m, fmaxf(fabsf(a), fabsf(b)));
      }
    }
  }
#pragma unroll
  for (int k = 0; k < 8; ++k) acc[wave][lane * 8 + k] = ss[k];
  m = block_max(m, red);  // contains the barriers that publish acc
  for (int i = threadIdx.x; i < 512; i += 256) {
    int cc = bx * 512 + i;
    if (cc < cols) colss_part[(long)by * cols + cc] = acc[0][i] + acc[1][i] + acc[2][i] + acc[3][i];
  }
  if (threadIdx.x == 0) amax_part[by * gx + bx] = m;
}

// Both weights' statistics in one launch: workgroups [0, nfc) take the rows of w_fc [F][d], the other npj x slices the
// column slices of w_proj [d][F] (the two jobs share nothing, so one launch instead of two costs neither anything).
__global__ __launch_bounds__(256) void weight_stats_kernel(const bf16_t* __restrict__ w_fc, const bf16_t* __restrict__ w_proj,
                                                          int F, int d, float* __restrict__ rowss,
                                                          float* __restrict__ amax_fc_part, float* __restrict__ colss_part,
                                                          float* __restrict__ amax_pj_part, int nfc, int npj, int slices,
                                                          long wz, long oz) {
  __shared__ float red[4];
  __shared__ float acc[4][512];
  const long wo = blockIdx.z * wz, oo = blockIdx.z * oz;
  const int b = blockIdx.x;
  if (b < nfc) {
    row_stats_job(w_fc + wo, F, d, rowss + oo, amax_fc_part + oo, b, nfc, red);
  } else {
    const int bb = b - nfc;
    col_stats_job(w_proj + wo, d, F, colss_part + oo, amax_pj_part + oo, bb % npj, bb / npj, npj, slices, red, acc);
  }
}

// colss[c] = sum over the row slices, in slice order (eight loads in flight, the additions in that order all the same)
__global__ __launch_bounds__(256) void col_finish_kernel(const float* __restrict__ part, int n, int slices,
                                                        float* __restrict__ colss, long oz) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  part += blockIdx.z * oz;
  colss += blockIdx.z * oz;
  float t = 0.f;
  int sl = 0;
  for (; sl + 8 <= slices; sl += 8) {
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = part[(long)(sl + k) * n + i];
#pragma unroll
    for (int k = 0; k < 8; ++k) t += v[k];
  }
  for (; sl < slices; ++sl) t += part[(long)sl * n + i];
  colss[i] = t;
}

__device__ float reduce_max_array(const float* a, int n, float* red) {
  float m = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) m = fmaxf(m, a[i]);
  return block_max(m, red);
}

// One workgroup: the forward scale row (nki_mlp_fused8.py:782-800).
__global__ __launch_bounds__(256) void forward_scales_kernel(const float* rowss, int F, const float* amax_fc_part, int nfc,
                                                            const float* colss, const float* amax_pj_part, int npj,
                                                            float e4m3_limit, float h_bound, float inv_x_scale,
                                                            const float* __restrict__ x_scale_dev, float* row_out, long oz) {
  rowss += blockIdx.z * oz;
  amax_fc_part += blockIdx.z * oz;
  colss += blockIdx.z * oz;
  amax_pj_part += blockIdx.z * oz;
  row_out += blockIdx.z * NSC;
  // the four maxima: a thread's loads of all four arrays are in flight together, then ONE reduction over the workgroup
  // (a maximum does not depend on the order, so the values equal four reduce_max_array calls')
  __shared__ float red4[4][4];
  float mx[4] = {0.f, 0.f, 0.f, 0.f};
  for (int i = threadIdx.x; i < F; i += 1024) {
    float a[4], b[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int j = i + 256 * k;
      a[k] = j < F ? rowss[j] : 0.f;
      b[k] = j < F ? colss[j] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) mx[0] = fmaxf(mx[0], a[k]), mx[1] = fmaxf(mx[1], b[k]);
  }
  for (int i = threadIdx.x; i < nfc; i += 256) mx[2] = fmaxf(mx[2], amax_fc_part[i]);
  for (int i = threadIdx.x; i < npj; i += 256) mx[3] = fmaxf(mx[3], amax_pj_part[i]);
#pragma unroll
  for (int k = 0; k < 4; ++k) mx[k] = wave_max(mx[k]);
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int k = 0; k < 4; ++k) red4[threadIdx.x >> 6][k] = mx[k];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int k = 0; k < 4; ++k) mx[k] = fmaxf(fmaxf(red4[0][k], red4[1][k]), fmaxf(red4[2][k], red4[3][k]));
    const float rho2 = mx[0], kappa2 = mx[1], amax_fc = mx[2], amax_pj = mx[3];
    float s_wfc, i_wfc, s_wpj, i_wpj, s_h, i_h, c_h;
    pow2_le(amax_fc, e4m3_limit, -24, 40, &s_wfc, &i_wfc);
    pow2_le(amax_pj, e4m3_limit, -24, 40, &s_wpj, &i_wpj);
    pow4_le(rho2 * h_bound, e4m3_limit, -16, 8, &s_h, &i_h, &c_h);
    row_out[SC_S_WFC] = s_wfc;
    row_out[SC_DQ_FC] = i_wfc * (x_scale_dev ? 1.0f / *x_scale_dev : inv_x_scale);   // (a power of two: exact either way)
    row_out[SC_C_H] = c_h;
    row_out[SC_S_WPROJ] = s_wpj;
    row_out[SC_DQ_PROJ] = i_h * i_wpj;
    row_out[SC_S_DY] = 0.f;
    row_out[SC_DQ_DH2] = 0.f;
    row_out[SC_S_DP] = 0.f;
    row_out[SC_DQ_DX] = 0.f;
    row_out[SC_RHO2] = rho2;
    row_out[SC_KAPPA2] = kappa2;
    row_out[SC_I_WFC] = i_wfc;
    row_out[SC_I_WPROJ] = i_wpj;
    row_out[SC_S_H] = s_h;
    row_out[SC_AMAX_WFC] = amax_fc;
    row_out[SC_AMAX_WPROJ] = amax_pj;
  }
}

// One workgroup: the backward call's row from amax(dy) (nki_mlp_fused8.py:803-813).
__global__ __launch_bounds__(256) void backward_scales_kernel(const float* amax_part, int npart, const float* row_in,
                                                             float dp_factor, float* row_out) {
  __shared__ float red[4];
  float amax_dy = reduce_max_array(amax_part, npart, red);
  if (threadIdx.x < NSC) row_out[threadIdx.x] = row_in[threadIdx.x];
  __syncthreads();
  if (threadIdx.x == 0) {
    float s_dy, i_dy, s_dp, i_dp;
    pow2_le(amax_dy, TFB_E5M2_MAX / 2.0f, -40, 60, &s_dy, &i_dy);
    float bound = sqrtf(row_in[SC_RHO2] * row_in[SC_KAPPA2]) * amax_dy * dp_factor;
    pow2_le(bound, TFB_E5M2_MAX, -40, 60, &s_dp, &i_dp);
    row_out[SC_S_DY] = s_dy;
    row_out[SC_DQ_DH2] = i_dy * row_in[SC_I_WPROJ] * 2.0f;
    row_out[SC_S_DP] = s_dp;
    row_out[SC_DQ_DX] = i_dp * row_in[SC_I_WFC];
  }
}

// One workgroup: out[0] = s = 2^e (largest with amax * s <= limit), out[1] = 1/s.
__global__ __launch_bounds__(256) void amax_scale_kernel(const float* amax_part, int npart, float limit, int e_lo, int e_hi,
                                                        float* out) {
  __shared__ float red[4];
  float amax = reduce_max_array(amax_part, npart, red);
  if (threadIdx.x == 0) {
    float s, inv;
    pow2_le(amax, limit, e_lo, e_hi, &s, &inv);
    out[0] = s;
    out[1] = inv;
    out[2] = amax;
  }
}

// ------------------------------------------------------------------------------------ casts
template <int FMT>
__global__ __launch_bounds__(256) void quant_kernel(const bf16_t* __restrict__ x, const float* __restrict__ scale_ptr,
                                                   float scale_imm, uint8_t* __restrict__ out, long n) {
  const float s = scale_ptr ? *scale_ptr : scale_imm;
  for (long i = ((long)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += (long)gridDim.x * 256 * 8) {
    u32x4 u = *(const u32x4*)(x + i);
    u32x2 o;
    o.x = cvt4_fp8<FMT>(bflo(u[0]) * s, bfhi(u[0]) * s, bflo(u[1]) * s, bfhi(u[1]) * s);
    o.y = cvt4_fp8<FMT>(bflo(u[2]) * s, bfhi(u[2]) * s, bflo(u[3]) * s, bfhi(u[3]) * s);
    *(u32x2*)(out + i) = o;
  }
}

// w [R][C] bf16 -> out [R][C] e4m3 and outT [C][R] e4m3, 64 x 64 tiles through LDS.
__device__ __forceinline__ void precast_tile(const bf16_t* __restrict__ w, const float s, uint8_t* __restrict__ out,
                                             uint8_t* __restrict__ outT, int R, int C, int r0, int c0, uint8_t (*t)[80]) {
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    int ch = threadIdx.x + i * 256;  // 512 chunks of 8 elements
    int r = ch >> 3, cc = (ch & 7) * 8;
    u32x4 u = *(const u32x4*)(w + (long)(r0 + r) * C + c0 + cc);
    u32x2 o;
    o.x = cvt4_fp8<TFB_FMT_E4M3>(bflo(u[0]) * s, bfhi(u[0]) * s, bflo(u[1]) * s, bfhi(u[1]) * s);
    o.y = cvt4_fp8<TFB_FMT_E4M3>(bflo(u[2]) * s, bfhi(u[2]) * s, bflo(u[3]) * s, bfhi(u[3]) * s);
    *(u32x2*)(out + (long)(r0 + r) * C + c0 + cc) = o;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      t[cc + k][r] = (uint8_t)(o.x >> (8 * k));
      t[cc + 4 + k][r] = (uint8_t)(o.y >> (8 * k));
    }
  }
  __syncthreads();
  {
    int c = threadIdx.x >> 2, j = (threadIdx.x & 3) * 16;
    u32x4 v = *(const u32x4*)(&t[c][j]);
    *(u32x4*)(outT + (long)(c0 + c) * R + r0 + j) = v;
  }
}

__global__ __launch_bounds__(256) void precast_kernel(const bf16_t* __restrict__ w, const float* __restrict__ scale_ptr,
                                                     uint8_t* __restrict__ out, uint8_t* __restrict__ outT, int R, int C,
                                                     long wz, long sz, long bz) {
  __shared__ uint8_t t[64][80];
  const long z = blockIdx.z;
  precast_tile(w + z * wz, scale_ptr[z * sz], out + z * bz, outT + z * bz, R, C, blockIdx.y * 64, blockIdx.x * 64, t);
}

// An MLP's two weights in one launch: workgroups [0, T) take the tiles of w_fc [F][d], [T, 2T) those of w_proj [d][F],
// T = (F / 64)(d / 64); the pack b8 [4][F d] gets w_fc8, its transpose, w_proj8, its transpose. row: the layer's scale row.
__global__ __launch_bounds__(256) void precast_mlp_kernel(const bf16_t* __restrict__ w_fc, const bf16_t* __restrict__ w_proj,
                                                         const float* __restrict__ row, uint8_t* __restrict__ b8, int F, int d,
                                                         long wz, long sz, long bz) {
  __shared__ uint8_t t[64][80];
  const long z = blockIdx.z;
  const long n = (long)F * d;
  const int T = (F >> 6) * (d >> 6);
  row += z * sz;
  b8 += z * bz;
  int b = blockIdx.x;
  if (b < T) {
    const int nc = d >> 6;
    precast_tile(w_fc + z * wz, row[SC_S_WFC], b8, b8 + n, F, d, (b / nc) * 64, (b % nc) * 64, t);
  } else {
    b -= T;
    const int nc = F >> 6;
    precast_tile(w_proj + z * wz, row[SC_S_WPROJ], b8 + 2 * n, b8 + 3 * n, d, F, (b / nc) * 64, (b % nc) * 64, t);
  }
}

// ------------------------------------------------------------------------------------ GEMM epilogues
// All activation GEMMs: P side = the weight pack layout whose rows are the output's contiguous
// dimension, Q side = the token-major fp8 activation. p = output column (4 consecutive), q = token.

struct EpiUp {  // pre = x8 @ wf8^T: r, h8
  const float* sc;
  bf16_t* r;     // [M][F]
  uint8_t* h8;   // [M][F]
  long F;
  float dq = 0.f, c = 0.f;  // sc[SC_DQ_FC], sc[SC_C_H], read once by prepare()
  __device__ __forceinline__ EpiUp for_group(int g) const {
    EpiUp e = *this;
    e.sc = sc + g * NSC;
    return e;
  }
  __device__ __forceinline__ EpiUp prepare() const {
    EpiUp e = *this;
    e.dq = sc[SC_DQ_FC];
    e.c = sc[SC_C_H];
    return e;
  }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], int) const {
    float hh[8];
    u32x4 rbits;
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      float a = fmaxf(v[i] * dq, 0.f), b = fmaxf(v[i + 1] * dq, 0.f);
      rbits[i >> 1] = round2_bf(a, b);                       // r = bf16(max(acc dq, 0)): saved before the clamp
      float ca = fminf(a * c, H_CLAMP), cb = fminf(b * c, H_CLAMP);
      round2_bf(ca, cb);                                     // rc = bf16(min(r c_h, 15.375))
      hh[i] = ca * ca;
      hh[i + 1] = cb * cb;
    }
    const long off = (long)q * F + p;
    // r is read again only by the backward: a non-temporal store keeps its 201 MB per layer from pushing the operand
    // tiles the other workgroups re-read out of the L2 (forward 2.69 -> 2.29 ms per step); full lines only: the same hint
    // on stores of part of a line (the LM head's logits, 16 bytes a row) bypasses the L2's merging and costs 2x
    __builtin_nontemporal_store(rbits, (u32x4*)(r + off));
    // 0 <= rc^2 <= 15.375^2 < 240: inside the e4m3 range, no saturation clamp needed
    u32x2 o = {cvt4_fp8<TFB_FMT_E4M3, false>(hh[0], hh[1], hh[2], hh[3]),
               cvt4_fp8<TFB_FMT_E4M3, false>(hh[4], hh[5], hh[6], hh[7])};
    *(u32x2*)(h8 + off) = o;   // (read by the next GEMM: a non-temporal store here costs 0.2 ms per step)
  }
  // the 256 x 256 kernel's protocol (pre() before the rounding to bf16, chunk() on the 8 rounded values): the same values
  __device__ __forceinline__ float pre(float x) const { return fmaxf(x * dq, 0.f); }
  __device__ __forceinline__ void chunk(int p, int q, const u32x4& rbits) const {
    float a[8], hh[8];
    unpack8bf(rbits, a);
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      float ca = fminf(a[i] * c, H_CLAMP), cb = fminf(a[i + 1] * c, H_CLAMP);
      round2_bf(ca, cb);
      hh[i] = ca * ca;
      hh[i + 1] = cb * cb;
    }
    const long off = (long)q * F + p;
    __builtin_nontemporal_store(rbits, (u32x4*)(r + off));
    u32x2 o = {cvt4_fp8<TFB_FMT_E4M3, false>(hh[0], hh[1], hh[2], hh[3]),
               cvt4_fp8<TFB_FMT_E4M3, false>(hh[4], hh[5], hh[6], hh[7])};
    *(u32x2*)(h8 + off) = o;
  }
};

struct EpiScaleStore {  // out = bf16(acc * sc[col])
  const float* sc;
  int col;
  bf16_t* out;
  long ld;
  float dq = 0.f;  // sc[col], read once by prepare()
  __device__ __forceinline__ EpiScaleStore for_group(int g) const {
    EpiScaleStore e = *this;
    e.sc = sc + g * NSC;
    return e;
  }
  __device__ __forceinline__ EpiScaleStore prepare() const {
    EpiScaleStore e = *this;
    e.dq = sc[col];
    return e;
  }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], int) const {
    float r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = v[i] * dq;
    *(u32x4*)(out + (long)q * ld + p) = pack8bf(r);
  }
  __device__ __forceinline__ float pre(float x) const { return x * dq; }
  __device__ __forceinline__ void chunk(int p, int q, const u32x4& v) const { *(u32x4*)(out + (long)q * ld + p) = v; }
};

// out = bf16(res + bf16(acc * dq)): EpiScaleStore / EpiDescale with the residual add that follows the projection made in
// the same store (the reference's projection-with-residual forward, K/nki_attn_nr8.py:1003, and the residual half of
// K/nki_mlp_nr8.py:1032); dq = sc[col] when sc is given, else dq_imm * *dq_a * *dq_b. Two roundings, as the separate add.
struct EpiDescaleRes {
  const float* sc;
  int col;
  const float* dq_a;
  const float* dq_b;
  float dq_imm;
  const bf16_t* res;
  bf16_t* out;
  long ld;
  float dq = 0.f;  // the descale factor, read once by prepare()
  using pre_t = u32x4;
  __device__ __forceinline__ EpiDescaleRes prepare() const {
    EpiDescaleRes e = *this;
    if (sc) {
      e.dq = sc[col];
    } else {
      e.dq = dq_imm;
      if (dq_a) e.dq *= *dq_a;
      if (dq_b) e.dq *= *dq_b;
    }
    return e;
  }
  __device__ __forceinline__ pre_t prefetch(int p, int q) const { return tfb_load_nt((const u32x4*)(res + (long)q * ld + p), TFB_NT_RES); }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], const pre_t& rv, int) const {
    float r[8], a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = v[i] * dq;
    unpack8bf(pack8bf(r), a);
    unpack8bf(rv, b);
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] += b[i];
    *(u32x4*)(out + (long)q * ld + p) = pack8bf(a);
  }
  __device__ __forceinline__ float pre(float x) const { return x * dq; }
  __device__ __forceinline__ void chunk(int p, int q, const u32x4& v, const pre_t& rv) const {
    float a[8], b[8];
    unpack8bf(v, a);
    unpack8bf(rv, b);
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] += b[i];
    *(u32x4*)(out + (long)q * ld + p) = pack8bf(a);
  }
};

struct EpiDescale {  // out = bf16(acc * dq), dq = dq_imm * *dq_a * *dq_b (absent factors are 1)
  const float* dq_a;
  const float* dq_b;
  float dq_imm;
  bf16_t* out;
  long ld;
  float dq = 0.f;  // dq_imm * *dq_a * *dq_b, read once by prepare()
  __device__ __forceinline__ EpiDescale prepare() const {
    EpiDescale e = *this;
    e.dq = dq_imm;
    if (dq_a) e.dq *= *dq_a;
    if (dq_b) e.dq *= *dq_b;
    return e;
  }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], int) const {
    float r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = v[i] * dq;
    *(u32x4*)(out + (long)q * ld + p) = pack8bf(r);
  }
  __device__ __forceinline__ float pre(float x) const { return x * dq; }
  __device__ __forceinline__ void chunk(int p, int q, const u32x4& v) const { *(u32x4*)(out + (long)q * ld + p) = v; }
};

struct EpiDh {  // dh = dy8 @ wp8: dpre = bf16((acc*dq_dh2)*r), dp8 = e5m2(dpre*s_dp), optional h = bf16(r^2) and
                // hq8 = e4m3(min(h*s_h, limit)) (the fp8 weight gradient's operand)
  const float* sc;
  const bf16_t* r;  // [M][F]
  bf16_t* dpre;     // [M][F] or null (the fp8 weight gradients read dp8, not dpre)
  uint8_t* dp8;     // [M][F]
  bf16_t* h;        // [M][F] or null
  uint8_t* hq8;     // [M][F] or null
  float hq_limit;
  long F;
  float dq = 0.f, sdp = 0.f, sh = 0.f;  // sc[SC_DQ_DH2], sc[SC_S_DP], sc[SC_S_H], read once by prepare()
  // With a power-of-two scale (what the scale search produces) the cast of a rounded bf16 value times the scale is one
  // instruction per pair, v_cvt_scalef32_pk_{bf8,fp8}_bf16 on the packed pair and 1 / scale: the same bytes as unpacking,
  // multiplying and converting for every value inside the format's range (all 65536 bf16 patterns compared on the GPU
  // for six scales); beyond the range the instruction does not saturate, so the saturation is applied to the fp32 value
  // before its rounding, at limit / scale (a bf16 number: rounding is monotonic, so clamping before or after it is the same).
  float inv_sdp = 0.f, lim_dp = 0.f, inv_sh = 0.f, lim_h = 0.f;
  bool fast_dp = false, fast_h = false;
  static __device__ __forceinline__ bool pow2(float x) {
    const uint32_t b = __float_as_uint(x);
    return (b & 0x807fffffu) == 0 && (b >> 23) > 16 && (b >> 23) < 238;
  }
  __device__ __forceinline__ EpiDh for_group(int g) const {
    EpiDh e = *this;
    e.sc = sc + g * NSC;
    return e;
  }
  __device__ __forceinline__ EpiDh prepare() const {
    EpiDh e = *this;
    e.dq = sc[SC_DQ_DH2];
    e.sdp = sc[SC_S_DP];
    e.sh = sc[SC_S_H];
#ifndef TFB_DH_FASTCAST
#define TFB_DH_FASTCAST 1
#endif
    if (TFB_DH_FASTCAST) {
      e.fast_dp = pow2(e.sdp);
      e.inv_sdp = 1.0f / e.sdp;
      e.lim_dp = TFB_E5M2_MAX * e.inv_sdp;
      const float lim = fminf(hq_limit, TFB_E4M3_MAX);
      e.inv_sh = 1.0f / e.sh;
      e.lim_h = lim * e.inv_sh;
      e.fast_h = pow2(e.sh) && hq8 && !h && lim > 0.f && (__float_as_uint(e.lim_h) & 0xffffu) == 0;
    }
    return e;
  }
  typedef u32x4 pre_t;  // the 8 values of r this chunk needs, requested before the k-loop
  __device__ __forceinline__ pre_t prefetch(int p, int q) const {
    return __builtin_nontemporal_load((const u32x4*)(r + (long)q * F + p));   // read once
  }
  typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
  typedef short s2_t __attribute__((ext_vector_type(2)));
  template <int FMT>
  static __device__ __forceinline__ uint32_t cast4_scaled(uint32_t lo_pair, uint32_t hi_pair, float inv_scale) {
    s2_t o = {0, 0};
    if (FMT == TFB_FMT_E5M2) {
      o = __builtin_amdgcn_cvt_scalef32_pk_bf8_bf16(o, __builtin_bit_cast(bf2_t, lo_pair), inv_scale, false);
      o = __builtin_amdgcn_cvt_scalef32_pk_bf8_bf16(o, __builtin_bit_cast(bf2_t, hi_pair), inv_scale, true);
    } else {
      o = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(o, __builtin_bit_cast(bf2_t, lo_pair), inv_scale, false);
      o = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(o, __builtin_bit_cast(bf2_t, hi_pair), inv_scale, true);
    }
    return __builtin_bit_cast(uint32_t, o);
  }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], const pre_t& rv, int) const {
    const long off = (long)q * F + p;
    float rr[8], dp[8];
    unpack8bf(rv, rr);
    u32x4 dbits;
    if (fast_dp) {
#pragma unroll
      for (int i = 0; i < 8; ++i) dp[i] = (v[i] * dq) * rr[i];
      if (dpre) *(u32x4*)(dpre + off) = pack8bf(dp);                 // dpre = bf16((acc dq_dh2) r)
#pragma unroll
      for (int i = 0; i < 8; ++i) dp[i] = dp[i] != dp[i] ? dp[i] : fminf(fmaxf(dp[i], -lim_dp), lim_dp);
      dbits = pack8bf(dp);
      u32x2 o = {cast4_scaled<TFB_FMT_E5M2>(dbits[0], dbits[1], inv_sdp), cast4_scaled<TFB_FMT_E5M2>(dbits[2], dbits[3], inv_sdp)};
      *(u32x2*)(dp8 + off) = o;
    } else {
#pragma unroll
      for (int i = 0; i < 8; i += 2) {
        dp[i] = (v[i] * dq) * rr[i];
        dp[i + 1] = (v[i + 1] * dq) * rr[i + 1];
        dbits[i >> 1] = round2_bf(dp[i], dp[i + 1]);           // dpre = bf16((acc dq_dh2) r)
      }
      if (dpre) *(u32x4*)(dpre + off) = dbits;
      u32x2 o = {cvt4_fp8<TFB_FMT_E5M2>(dp[0] * sdp, dp[1] * sdp, dp[2] * sdp, dp[3] * sdp),
                 cvt4_fp8<TFB_FMT_E5M2>(dp[4] * sdp, dp[5] * sdp, dp[6] * sdp, dp[7] * sdp)};
      *(u32x2*)(dp8 + off) = o;
    }
    if (fast_h) {   // hq8 only: e4m3(min(bf16(r^2) s_h, limit)) = cast(bf16(min(r^2, limit / s_h)), 1 / s_h)
#pragma unroll
      for (int i = 0; i < 8; ++i) rr[i] = fminf(rr[i] * rr[i], lim_h);
      const u32x4 hb = pack8bf(rr);
      u32x2 q8 = {cast4_scaled<TFB_FMT_E4M3>(hb[0], hb[1], inv_sh), cast4_scaled<TFB_FMT_E4M3>(hb[2], hb[3], inv_sh)};
      *(u32x2*)(hq8 + off) = q8;
    } else if (h || hq8) {
      u32x4 hbits;
#pragma unroll
      for (int i = 0; i < 8; i += 2) {
        rr[i] = rr[i] * rr[i];
        rr[i + 1] = rr[i + 1] * rr[i + 1];
        hbits[i >> 1] = round2_bf(rr[i], rr[i + 1]);         // h = bf16(r^2)
      }
      if (h) *(u32x4*)(h + off) = hbits;
      if (hq8) {
        const float lim = fminf(hq_limit, TFB_E4M3_MAX);
#pragma unroll
        for (int i = 0; i < 8; ++i) rr[i] = fminf(rr[i] * sh, lim);   // 0 <= . <= lim: in range, no further clamp
        u32x2 q = {cvt4_fp8<TFB_FMT_E4M3, false>(rr[0], rr[1], rr[2], rr[3]),
                   cvt4_fp8<TFB_FMT_E4M3, false>(rr[4], rr[5], rr[6], rr[7])};
        *(u32x2*)(hq8 + off) = q;
      }
    }
  }
};

// h = bf16(r^2) applied to a fragment of 8 bf16 on its way into the MFMA (the dW_proj GEMM reads r, not h).
struct LoadSquare {
  __device__ __forceinline__ bf16x8 operator()(bf16x8 v) const {
    typedef float f32x8_t __attribute__((ext_vector_type(8)));
    f32x8_t f = __builtin_convertvector(v, f32x8_t);
    f = f * f;
    return __builtin_convertvector(f, bf16x8);
  }
};

inline bool shapes8(long M, int d, int F) { return M > 0 && M % 128 == 0 && d > 0 && d % 256 == 0 && F > 0 && F % 256 == 0; }

template <int FMT>
int launch_quant(const void* x, const float* sp, float si, void* out, long n, hipStream_t s) {
  if (n % 8) return TFB_ERR_SHAPE;
  long blocks = (n / 8 + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(quant_kernel<FMT>, dim3((unsigned)blocks), dim3(256), 0, s, (const bf16_t*)x, sp, si, (uint8_t*)out, n);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

constexpr int AMAX_BLOCKS = 1024;

}  // namespace

// Scratch the scale kernels need (fp32 elements): partial maxima and the per-row / per-column norms.
extern "C" long tfb_mlp8_scale_scratch_floats(int F) { return (2L + COL_SLICES) * F + 4L * AMAX_BLOCKS; }

// row_out: fp32 [16] device. e4m3_limit: 240 reproduces the reference's rows; 448 is the OCP maximum.
// The forward scale rows of `layers` MLPs whose weights sit `wz` elements apart (w_fc and w_proj alike): three launches
// whatever the layer count. scratch: layers x tfb_mlp8_scale_scratch_floats(F) floats; row_out: layers x 16 floats.
static int launch_forward_scales(const void* w_fc, const void* w_proj, void* row_out, void* scratch, int F, int d,
                                 float e4m3_limit, float x_scale, const void* x_scale_dev, int layers, long wz, hipStream_t s) {
  const long oz = tfb_mlp8_scale_scratch_floats(F);
  float* rowss = (float*)scratch;
  float* colss = rowss + F;
  float* colpart = colss + F;
  float* pa = colpart + (long)COL_SLICES * F;
  float* pb = pa + AMAX_BLOCKS;
  int nfc = (F + 3) / 4;
  if (nfc > AMAX_BLOCKS) nfc = AMAX_BLOCKS;
  int npj = (F + 511) / 512;
  int slices = AMAX_BLOCKS / npj < COL_SLICES ? AMAX_BLOCKS / npj : COL_SLICES;
  if (slices < 1) return TFB_ERR_SHAPE;
  hipLaunchKernelGGL(weight_stats_kernel, dim3(nfc + npj * slices, 1, layers), dim3(256), 0, s, (const bf16_t*)w_fc,
                     (const bf16_t*)w_proj, F, d, rowss, pa, colpart, pb, nfc, npj, slices, wz, oz);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(col_finish_kernel, dim3((F + 255) / 256, 1, layers), dim3(256), 0, s, colpart, F, slices, colss, oz);
  TFB_LAUNCH_CHECK();
  const float h_bound = (float)(1.3 * (double)d);
  hipLaunchKernelGGL(forward_scales_kernel, dim3(1, 1, layers), dim3(256), 0, s, rowss, F, pa, nfc, colss, pb, npj * slices,
                     e4m3_limit, h_bound, x_scale_dev ? 0.f : (float)(1.0 / (double)x_scale), (const float*)x_scale_dev,
                     (float*)row_out, oz);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

extern "C" int tfb_mlp8_forward_scales(const void* w_fc, const void* w_proj, void* row_out, void* scratch, int F, int d,
                                       float e4m3_limit, float x_scale, const void* x_scale_dev, void* stream) {
  if (!w_fc || !w_proj || !row_out || !scratch) return TFB_ERR_ARG;
  if (F <= 0 || d <= 0 || F % 8 || d % 8 || (!x_scale_dev && !(x_scale > 0.f))) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  return launch_forward_scales(w_fc, w_proj, row_out, scratch, F, d, e4m3_limit, x_scale, x_scale_dev, 1, 0, s);
}

extern "C" int tfb_mlp8_backward_scales(const void* dy, const void* row_in, void* row_out, void* scratch, long M, int d,
                                        void* stream) {
  if (!dy || !row_in || !row_out || !scratch) return TFB_ERR_ARG;
  long n = M * d;
  if (n <= 0 || n % 8) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  long blocks = (n / 8 + 255) / 256;
  if (blocks > AMAX_BLOCKS) blocks = AMAX_BLOCKS;
  hipLaunchKernelGGL(amax_partial_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (const bf16_t*)dy, n, (float*)scratch);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(backward_scales_kernel, dim3(1), dim3(256), 0, s, (const float*)scratch, (int)blocks,
                     (const float*)row_in, (float)(36.16 * (double)d), (float*)row_out);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// tfb_mlp8_backward_scales from amax partials that the producer of dy left (tfb_rmsnorm_bwd_amax: npart values whose
// maximum is amax(dy)): the same row, without the pass over dy. d = dy's row length.
extern "C" int tfb_mlp8_backward_scales_part(const void* amax_part, int npart, const void* row_in, void* row_out, int d,
                                             void* stream) {
  if (!amax_part || !row_in || !row_out) return TFB_ERR_ARG;
  if (npart <= 0 || d <= 0) return TFB_ERR_SHAPE;
  hipLaunchKernelGGL(backward_scales_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, (const float*)amax_part, npart,
                     (const float*)row_in, (float)(36.16 * (double)d), (float*)row_out);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// out: fp32 [3] device = {s, 1/s, amax}: per-tensor power-of-two scale from the exact amax.
extern "C" int tfb_amax_scale(const void* x, long n, float limit, int e_lo, int e_hi, void* out, void* scratch,
                              void* stream) {
  if (!x || !out || !scratch) return TFB_ERR_ARG;
  if (n <= 0 || n % 8) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  long blocks = (n / 8 + 255) / 256;
  if (blocks > AMAX_BLOCKS) blocks = AMAX_BLOCKS;
  hipLaunchKernelGGL(amax_partial_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (const bf16_t*)x, n, (float*)scratch);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(amax_scale_kernel, dim3(1), dim3(256), 0, s, (const float*)scratch, (int)blocks, limit, e_lo, e_hi,
                     (float*)out);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// out8 = fp8(x * scale): scale from device memory (scale_ptr) or immediate. fmt 0 = e4m3, 1 = e5m2.
extern "C" int tfb_quant_fp8(const void* x, const void* scale_ptr, float scale_imm, int fmt, void* out8, long n,
                             void* stream) {
  if (!x || !out8) return TFB_ERR_ARG;
  if (n <= 0) return TFB_ERR_SHAPE;
  if (fmt == TFB_FMT_E4M3) return launch_quant<TFB_FMT_E4M3>(x, (const float*)scale_ptr, scale_imm, out8, n, (hipStream_t)stream);
  if (fmt == TFB_FMT_E5M2) return launch_quant<TFB_FMT_E5M2>(x, (const float*)scale_ptr, scale_imm, out8, n, (hipStream_t)stream);
  return TFB_ERR_ARG;
}

// w8: uint8 [4][F*d] = wf8 [F][d], wf8T [d][F], wp8 [d][F], wp8T [F][d] (all e4m3, scaled by the row's s_w).
extern "C" int tfb_mlp8_precast(const void* w_fc, const void* w_proj, const void* row, void* w8, int F, int d, void* stream) {
  if (!w_fc || !w_proj || !row || !w8) return TFB_ERR_ARG;
  if (F <= 0 || d <= 0 || F % 64 || d % 64) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  uint8_t* b = (uint8_t*)w8;
  hipLaunchKernelGGL(precast_mlp_kernel, dim3(2 * (F / 64) * (d / 64), 1, 1), dim3(256), 0, s, (const bf16_t*)w_fc,
                     (const bf16_t*)w_proj, (const float*)row, b, F, d, 0L, 0L, 0L);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// The per-optimizer-step refresh of `layers` MLPs in four launches: scale rows [layers][16] and e4m3 packs [layers][4 F d]
// (layouts as tfb_mlp8_forward_scales / tfb_mlp8_precast) from weights laid out with one stride: layer i's w_fc at
// w_fc + i * layer_stride elements, its w_proj at w_proj + i * layer_stride. scratch: layers x
// tfb_mlp8_scale_scratch_floats(F) floats. The per-layer calls cost ~45 us of small launches each.
extern "C" int tfb_mlp8_refresh_layers(const void* w_fc, const void* w_proj, long layer_stride, int layers, void* rows, void* w8,
                                       void* scratch, int F, int d, float e4m3_limit, float x_scale, void* stream) {
  if (!w_fc || !w_proj || !rows || !w8 || !scratch) return TFB_ERR_ARG;
  if (F <= 0 || d <= 0 || F % 64 || d % 64 || layers <= 0 || layers > 65535 || layer_stride < 0 || layer_stride % 8 ||
      !(x_scale > 0.f))
    return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  int st = launch_forward_scales(w_fc, w_proj, rows, scratch, F, d, e4m3_limit, x_scale, nullptr, layers, layer_stride, s);
  if (st != TFB_OK) return st;
  uint8_t* b = (uint8_t*)w8;
  const long n = (long)F * d;
  hipLaunchKernelGGL(precast_mlp_kernel, dim3(2 * (F / 64) * (d / 64), 1, layers), dim3(256), 0, s, (const bf16_t*)w_fc,
                     (const bf16_t*)w_proj, (const float*)rows, b, F, d, layer_stride, (long)NSC, 4 * n);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// w [R][C] bf16 -> out8 [R][C] and outT8 [C][R], both e4m3(w * *scale_ptr): the two byte layouts a projection's forward
// (contraction over C) and input-gradient (contraction over R) GEMMs read k-contiguously.
extern "C" int tfb_precast8(const void* w, const void* scale_ptr, void* out8, void* outT8, int R, int C, void* stream) {
  if (!w || !scale_ptr || !out8 || !outT8) return TFB_ERR_ARG;
  if (R <= 0 || C <= 0 || R % 64 || C % 64) return TFB_ERR_SHAPE;
  hipLaunchKernelGGL(precast_kernel, dim3(C / 64, R / 64, 1), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)w,
                     (const float*)scale_ptr, (uint8_t*)out8, (uint8_t*)outT8, R, C, 0L, 0L, 0L);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

using Cfg8 = GemmCfg<128, 128, 2, 2, 1, TFB_K_CONTIG, TFB_K_CONTIG, TFB_FMT_E4M3, TFB_FMT_E4M3>;
using Cfg8g = GemmCfg<128, 128, 2, 2, 1, TFB_K_CONTIG, TFB_K_CONTIG, TFB_FMT_E4M3, TFB_FMT_E5M2>;

// A dense fp8 GEMM with both operands k-contiguous: the persistent 256 x 256 kernel where the shape allows it (the same
// sums in the same order, the epilogue's values bit for bit), else the 128 x 128 kernel.
template <class Cfg, class Epi>
static int launch8(GemmOperand P, GemmOperand Q, int np, int nq, long kbytes, Epi e, hipStream_t s) {
  // a contraction of 768 bytes (the fp8 attention projections of a 768-wide model): the weight-stationary kernel
  if (gemm_ws8_applies(np, nq, kbytes)) return gemm_ws8_launch<Cfg::FMTP, Cfg::FMTQ>(P, Q, np, nq, kbytes, e, s);
  if (gemm_pp_applies(np, nq, kbytes)) return gemm_pp_launch<1, Cfg::FMTP, Cfg::FMTQ>(P, Q, np, nq, kbytes, e, s);
  return gemm_launch<Cfg>(P, Q, np, nq, kbytes, 1, LoadIdentity{}, LoadIdentity{}, e, s);
}

// The MLP's two GEMMs that contract over d_model with a heavy epilogue (up-projection, dH): with d_model = 768 the
// weight-stationary kernel (the weights in registers, only the tokens stream), else the 128 x 128 kernel. The same sums in
// the same order, the same epilogue code.
template <class Cfg, class Epi>
static int launch_k768(GemmOperand P, GemmOperand Q, int np, int nq, long kbytes, Epi e, hipStream_t s) {
  if (gemm_ws8_applies(np, nq, kbytes)) return gemm_ws8_launch<Cfg::FMTP, Cfg::FMTQ>(P, Q, np, nq, kbytes, e, s);
  return gemm_launch<Cfg>(P, Q, np, nq, kbytes, 1, LoadIdentity{}, LoadIdentity{}, e, s);
}

// out [M][N] bf16 = bf16((a8 [M][K] @ b8 [N][K]^T) * dq): the fp8 projection GEMM. a8 is e4m3 (fmt_a 0: forward
// activations) or e5m2 (fmt_a 1: gradients); b8 is e4m3 (a pre-cast weight layout). dq = dq_imm * *dq_a * *dq_b, the
// pointers being device fp32 scalars (inverse power-of-two scales) or null.
extern "C" int tfb_gemm_fp8(const void* a8, int fmt_a, const void* b8, const void* dq_a, const void* dq_b, float dq_imm,
                            void* out, long M, int N, int K, void* stream) {
  if (!a8 || !b8 || !out) return TFB_ERR_ARG;
  if (fmt_a != TFB_FMT_E4M3 && fmt_a != TFB_FMT_E5M2) return TFB_ERR_ARG;
  if (M <= 0 || N <= 0 || K <= 0 || M % 128 || N % 128 || K % 128 || M > 0x7fffffffL) return TFB_ERR_SHAPE;
  GemmOperand P{(const uint8_t*)b8, (long)K}, Q{(const uint8_t*)a8, (long)K};
  EpiDescale e{(const float*)dq_a, (const float*)dq_b, dq_imm, (bf16_t*)out, (long)N};
  if (fmt_a == TFB_FMT_E4M3)
    return launch8<Cfg8>(P, Q, N, (int)M, (long)K, e, (hipStream_t)stream);
  return launch8<Cfg8g>(P, Q, N, (int)M, (long)K, e, (hipStream_t)stream);
}

// tfb_gemm_fp8 with the residual add in the store: out = bf16(res + bf16((a8 @ b8^T) * dq)), res [M][N] bf16; e4m3
// activations only (a forward projection). Equal to tfb_gemm_fp8 followed by a bf16 add, bit for bit.
// Replaces _proj8_fwd_ra_kernel (round2/source/kernels/nki_attn_nr8.py:1003).
extern "C" int tfb_gemm_fp8_res(const void* a8, const void* b8, const void* dq_a, const void* dq_b, float dq_imm, const void* res,
                                void* out, long M, int N, int K, void* stream) {
  if (!a8 || !b8 || !res || !out) return TFB_ERR_ARG;
  if (M <= 0 || N <= 0 || K <= 0 || M % 128 || N % 128 || K % 128 || M > 0x7fffffffL) return TFB_ERR_SHAPE;
  GemmOperand P{(const uint8_t*)b8, (long)K}, Q{(const uint8_t*)a8, (long)K};
  EpiDescaleRes e{nullptr, 0, (const float*)dq_a, (const float*)dq_b, dq_imm, (const bf16_t*)res, (bf16_t*)out, (long)N};
  return launch8<Cfg8>(P, Q, N, (int)M, (long)K, e, (hipStream_t)stream);
}

// out [O][D] (+)= ((g8 [M][O]^T @ a8 [M][D]) * imm / (*s_g * *s_a)): the fp8 weight gradient of a projection, contraction
// over the M tokens of two token-major byte tensors (fp32 accumulation over all tokens, one rounding; bf16 or fp32
// output, optionally accumulated into). (fmt_g, fmt_a) = (e5m2, e4m3): a gradient against the forward's activation
// bytes; (e4m3, e5m2): an activation on the g side (the MLP's h against dy). s_g, s_a: device fp32 scalars (the
// power-of-two scales the bytes were cast at) or null. Split-K through the workspace.
// Replaces dw8_grad (round2/source/train.py:8185) = K/nki_dw8.py:323 emulate_dw / _dw8_kernel.
extern "C" int tfb_gemm_fp8_tn(const void* g8, int fmt_g, const void* a8, int fmt_a, const void* s_g, const void* s_a, float imm,
                               void* out, long M, int O, int D, int out_f32, int accumulate, void* workspace,
                               long workspace_bytes, void* stream) {
  if (!g8 || !a8 || !out || !workspace) return TFB_ERR_ARG;
  const bool ga = fmt_g == TFB_FMT_E5M2 && fmt_a == TFB_FMT_E4M3, ag = fmt_g == TFB_FMT_E4M3 && fmt_a == TFB_FMT_E5M2;
  if (!ga && !ag) return TFB_ERR_ARG;
  if (M <= 0 || O <= 0 || D <= 0 || M % 128 || O % 128 || D % 128) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const long n = (long)O * D;
  // a long contraction over few 256 x 256 tiles (the MLP's weight gradients: 36 tiles of 256 k-tiles): the persistent kernel,
  // one k range per workgroup
#ifndef TFB_PP_DW8
#define TFB_PP_DW8 1
#endif
  if (TFB_PP && TFB_PP_DW8 && O % 256 == 0 && D % 256 == 0 && M / 128 >= 128) {
    const int sp = gemm_pp_fewtile_splits((long)(O / 256) * (D / 256), M / 128, n, workspace_bytes);
    if (sp > 1) {
      GemmOperand P{(const uint8_t*)a8, (long)D}, Q{(const uint8_t*)g8, (long)O};
      EpiSplit e{(float*)workspace, (long)D, n};
      int st = ga ? gemm_pp_launch_lay<1, TFB_FMT_E4M3, TFB_FMT_E5M2, TFB_K_STRIDED, TFB_K_STRIDED>(P, Q, D, O, M, sp, e, s)
                  : gemm_pp_launch_lay<1, TFB_FMT_E5M2, TFB_FMT_E4M3, TFB_K_STRIDED, TFB_K_STRIDED>(P, Q, D, O, M, sp, e, s);
      if (st != TFB_OK) return st;
      return splitk_reduce((const float*)workspace, out, n, sp, out_f32, accumulate, s, (const float*)s_g, (const float*)s_a, imm);
    }
  }
  const int splits = choose_splits(n / (128 * 128), (int)(M / 128), n, workspace_bytes);
  if ((long)splits * n * 4 > workspace_bytes) return TFB_ERR_SHAPE;
  float* ws = (float*)workspace;
  // D[p = dd][q = o] = sum_m a8[m][dd] g8[m][o] -> out[o][dd]
  GemmOperand P{(const uint8_t*)a8, (long)D}, Q{(const uint8_t*)g8, (long)O};
  EpiSplit e{ws, (long)D, n};
  int st = ga ? gemm_launch<GemmCfg<128, 128, 2, 2, 1, TFB_K_STRIDED, TFB_K_STRIDED, TFB_FMT_E4M3, TFB_FMT_E5M2>>(
                    P, Q, D, O, M, splits, LoadIdentity{}, LoadIdentity{}, e, s)
              : gemm_launch<GemmCfg<128, 128, 2, 2, 1, TFB_K_STRIDED, TFB_K_STRIDED, TFB_FMT_E5M2, TFB_FMT_E4M3>>(
                    P, Q, D, O, M, splits, LoadIdentity{}, LoadIdentity{}, e, s);
  if (st != TFB_OK) return st;
  return splitk_reduce(ws, out, n, splits, out_f32, accumulate, s, (const float*)s_g, (const float*)s_a, imm);
}

// Forward: x8 [M][d] e4m3 (already cast at s_x), w8 pack, row -> y [M][d] bf16, r [M][F] bf16, h8 [M][F] e4m3 scratch.
extern "C" int tfb_mlp8_fwd(const void* x8, const void* w8, const void* row, void* y, void* r, void* h8, long M, int d, int F,
                            void* stream) {
  if (!x8 || !w8 || !row || !y || !r || !h8) return TFB_ERR_ARG;
  if (!shapes8(M, d, F)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const uint8_t* b = (const uint8_t*)w8;
  const long n = (long)F * d;
  GemmOperand Pw{b, (long)d}, Qx{(const uint8_t*)x8, (long)d};
  EpiUp e1{(const float*)row, (bf16_t*)r, (uint8_t*)h8, (long)F};
  int st = launch_k768<Cfg8>(Pw, Qx, F, (int)M, (long)d, e1, s);
  if (st != TFB_OK) return st;
  GemmOperand Pp{b + 2 * n, (long)F}, Qh{(const uint8_t*)h8, (long)F};
  EpiScaleStore e2{(const float*)row, SC_DQ_PROJ, (bf16_t*)y, (long)d};
  return launch8<Cfg8>(Pp, Qh, d, (int)M, (long)F, e2, s);
}

// tfb_mlp8_fwd with the block's residual add in the second GEMM's store: y = bf16(res + bf16(MLP(x))), res [M][d] bf16 (the
// MLP's input before its norm). Equal to tfb_mlp8_fwd followed by a bf16 add, bit for bit.
// Replaces the residual half of _mlp8_fwd_nr_kernel (round2/source/kernels/nki_mlp_nr8.py:1032); its norm half is
// tfb_rmsnorm_fwd_q, which hands this call its x8.
extern "C" int tfb_mlp8_fwd_res(const void* x8, const void* w8, const void* row, const void* res, void* y, void* r, void* h8,
                                long M, int d, int F, void* stream) {
  if (!x8 || !w8 || !row || !res || !y || !r || !h8) return TFB_ERR_ARG;
  if (!shapes8(M, d, F)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const uint8_t* b = (const uint8_t*)w8;
  const long n = (long)F * d;
  GemmOperand Pw{b, (long)d}, Qx{(const uint8_t*)x8, (long)d};
  EpiUp e1{(const float*)row, (bf16_t*)r, (uint8_t*)h8, (long)F};
  int st = launch_k768<Cfg8>(Pw, Qx, F, (int)M, (long)d, e1, s);
  if (st != TFB_OK) return st;
  GemmOperand Pp{b + 2 * n, (long)F}, Qh{(const uint8_t*)h8, (long)F};
  EpiDescaleRes e2{(const float*)row, SC_DQ_PROJ, nullptr, nullptr, 1.0f, (const bf16_t*)res, (bf16_t*)y, (long)d};
  return launch8<Cfg8>(Pp, Qh, d, (int)M, (long)F, e2, s);
}

// Backward: dy8 [M][d] e5m2 (cast at the row's s_dy), r [M][F] -> dx [M][d], dpre [M][F] bf16, h [M][F] bf16 (optional,
// may be NULL), dp8 [M][F] e5m2 scratch.
// hq8 (optional, may be NULL) [M][F] = e4m3(min(bf16(r^2) * s_h, hq_limit)): the g-side operand of the fp8 weight
// gradient of w_proj (K/nki_dw8.py:323 with format E4M3C, round2/source/train.py:8226).
extern "C" int tfb_mlp8_bwd_q(const void* dy8, const void* r, const void* w8, const void* row, void* dx, void* h, void* dpre,
                              void* dp8, void* hq8, float hq_limit, long M, int d, int F, void* stream) {
  if (!dy8 || !r || !w8 || !row || !dx || !dp8) return TFB_ERR_ARG;  // dpre may be NULL: only dp8 is then written
  if (!shapes8(M, d, F)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const uint8_t* b = (const uint8_t*)w8;
  const long n = (long)F * d;
  GemmOperand Pw{b + 3 * n, (long)d}, Qg{(const uint8_t*)dy8, (long)d};  // wp8T [F][d]
  EpiDh e1{(const float*)row, (const bf16_t*)r, (bf16_t*)dpre, (uint8_t*)dp8, (bf16_t*)h, (uint8_t*)hq8, hq_limit, (long)F};
  int st = launch_k768<Cfg8g>(Pw, Qg, F, (int)M, (long)d, e1, s);
  if (st != TFB_OK) return st;
  GemmOperand Pf{b + n, (long)F}, Qd{(const uint8_t*)dp8, (long)F};  // wf8T [d][F]
  EpiScaleStore e2{(const float*)row, SC_DQ_DX, (bf16_t*)dx, (long)d};
  return launch8<Cfg8g>(Pf, Qd, d, (int)M, (long)F, e2, s);
}
extern "C" int tfb_mlp8_bwd(const void* dy8, const void* r, const void* w8, const void* row, void* dx, void* h, void* dpre,
                            void* dp8, long M, int d, int F, void* stream) {
  return tfb_mlp8_bwd_q(dy8, r, w8, row, dx, h, dpre, dp8, nullptr, 0.f, M, d, F, stream);
}

// The two weight gradients in fp8, from byte tensors the forward and backward already hold (token-major, contraction
// over the M tokens): dw_fc [F][d] = bf16((dp8^T @ x8) / (s_dp x_scale)) with dp8 = e5m2(dpre s_dp) and x8 = e4m3(x x_scale);
// dw_proj [d][F] = bf16((dy8^T @ hq8) / (s_dy s_h)) with dy8 = e5m2(dy s_dy) and hq8 from tfb_mlp8_bwd_q. row = the
// backward call's scale row. Outputs bf16 or fp32, optionally accumulated into; split-K through the workspace.
// Replaces mlp8_weight_grads under switch 9k (round2/source/train.py:8209-8229) = K/nki_dw8.py:323 emulate_dw.
extern "C" int tfb_mlp8_dw8(const void* x8, const void* dp8, const void* hq8, const void* dy8, const void* row, float x_scale,
                            void* dw_fc, void* dw_proj, long M, int d, int F, int out_f32, int accumulate, void* workspace,
                            long workspace_bytes, const void* x_scale_dev, void* stream) {
  if (!x8 || !dp8 || !hq8 || !dy8 || !row || !dw_fc || !dw_proj || !workspace) return TFB_ERR_ARG;
  if (!shapes8(M, d, F) || (!x_scale_dev && !(x_scale > 0.f))) return TFB_ERR_SHAPE;
  const float* sc = (const float*)row;
  // dw_fc[f][dd] = sum_m dp8[m][f] x8[m][dd]: g = dp8 (e5m2), a = x8 (e4m3); x8's scale from the device when it lives there
  int st = tfb_gemm_fp8_tn(dp8, TFB_FMT_E5M2, x8, TFB_FMT_E4M3, sc + SC_S_DP, x_scale_dev, x_scale_dev ? 1.0f : 1.0f / x_scale,
                           dw_fc, M, F, d, out_f32, accumulate, workspace, workspace_bytes, stream);
  if (st != TFB_OK) return st;
  // dw_proj[dd][f] = sum_m dy8[m][dd] hq8[m][f]: g = dy8 (e5m2), a = hq8 (e4m3)
  return tfb_gemm_fp8_tn(dy8, TFB_FMT_E5M2, hq8, TFB_FMT_E4M3, sc + SC_S_DY, sc + SC_S_H, 1.0f, dw_proj, M, d, F, out_f32,
                         accumulate, workspace, workspace_bytes, stream);
}

// dW_proj [d][F] (+)= dy^T @ bf16(r^2): the token-contraction GEMM with the square applied while r is staged, so h
// is never written. out bf16 or fp32; workspace fp32 for split-K (tokens are the long dimension).
extern "C" int tfb_mlp_dw_proj(const void* dy, const void* r, void* dw, long M, int d, int F, int out_f32, int accumulate,
                               void* workspace, long workspace_bytes, void* stream) {
  if (!dy || !r || !dw) return TFB_ERR_ARG;
  if (M <= 0 || M % 64 || d % 128 || F % 128) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  // 4 x 1 wavefronts: each wavefront squares one P fragment per k-step and every element of r is squared once
  using Cfg = GemmCfg<128, 128, 4, 1, 2, TFB_K_STRIDED, TFB_K_STRIDED>;
  GemmOperand P{(const uint8_t*)r, (long)F * 2}, Q{(const uint8_t*)dy, (long)d * 2};
  const long tiles = (long)(F / 128) * (d / 128);
  const int splits = workspace ? choose_splits(tiles, (int)(M / 64), (long)d * F, workspace_bytes) : 1;
  if (splits == 1) {
    EpiStore e{dw, (long)F, out_f32, accumulate};
    return gemm_launch<Cfg>(P, Q, F, d, M * 2, 1, LoadSquare{}, LoadIdentity{}, e, s);
  }
  EpiSplit e{(float*)workspace, (long)F, (long)d * F};
  int st = gemm_launch<Cfg>(P, Q, F, d, M * 2, splits, LoadSquare{}, LoadIdentity{}, e, s);
  if (st != TFB_OK) return st;
  return splitk_reduce((const float*)workspace, dw, (long)d * F, splits, out_f32, accumulate, s);
}

// ================================================================================================ grouped (MoE experts)
// The experts' rows live in one token-major buffer, expert e's rows contiguous and padded to a multiple of 128 (padding
// rows are zero), so every 128-row tile belongs to one expert: tile_expert[t] names it (-1 beyond the ragged extent).
// Each expert has its own weight pack (w8 + e * 4 F d bytes) and scale row (rows + e * 16).
// Replaces moe_experts8_local / moe_expert8_mlp (round2/source/train.py:10731-10776): one fp8 MLP call per expert there,
// one grouped launch per GEMM here, with no host-side knowledge of the experts' loads.
namespace {
template <class Cfg, class Epi>
int grouped_launch(const uint8_t* wbase, long wld, long wgroup_stride, const uint8_t* act, long ald, int np, long rmax, long kbytes,
                   const int* tile_expert, Epi e, hipStream_t s) {
  GemmArgs a;
  a.P = GemmOperand{wbase, wld};
  a.Q = GemmOperand{act, ald};
  a.np = np;
  a.nq = (int)rmax;
  a.nkt = (int)(kbytes / 128);
  a.ntp = np / Cfg::BP;
  a.q_group = tile_expert;
  a.p_group_stride = wgroup_stride;
  a.k_seg = nullptr;
  return gemm_launch_args<Cfg>(a, 1, 1, LoadIdentity{}, LoadIdentity{}, e, s);
}
}  // namespace

extern "C" int tfb_moe_mlp8_fwd(const void* x8, const void* w8, const void* rows, const void* tile_expert, void* y, void* r,
                                void* h8, long rmax, int d, int F, void* stream) {
  if (!x8 || !w8 || !rows || !tile_expert || !y || !r || !h8) return TFB_ERR_ARG;
  if (!shapes8(rmax, d, F)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const uint8_t* b = (const uint8_t*)w8;
  const long n = (long)F * d;
  EpiUp e1{(const float*)rows, (bf16_t*)r, (uint8_t*)h8, (long)F};
  int st = grouped_launch<Cfg8>(b, d, 4 * n, (const uint8_t*)x8, d, F, rmax, d, (const int*)tile_expert, e1, s);
  if (st != TFB_OK) return st;
  EpiScaleStore e2{(const float*)rows, SC_DQ_PROJ, (bf16_t*)y, (long)d};
  return grouped_launch<Cfg8>(b + 2 * n, F, 4 * n, (const uint8_t*)h8, F, d, rmax, F, (const int*)tile_expert, e2, s);
}

// dpre may be null (the fp8 weight gradients read dp8, not dpre); hq8 non-null: also hq8 [rmax][F] = e4m3(min(bf16(r^2) s_h,
// hq_limit)), the activation operand of the fp8 dW_proj (each expert at its own s_h).
extern "C" int tfb_moe_mlp8_bwd_q(const void* dy8, const void* r, const void* w8, const void* rows, const void* tile_expert,
                                  void* dx, void* dpre, void* dp8, void* hq8, float hq_limit, long rmax, int d, int F,
                                  void* stream) {
  if (!dy8 || !r || !w8 || !rows || !tile_expert || !dx || !dp8) return TFB_ERR_ARG;
  if (!shapes8(rmax, d, F) || (hq8 && !(hq_limit > 0.f))) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const uint8_t* b = (const uint8_t*)w8;
  const long n = (long)F * d;
  EpiDh e1{(const float*)rows, (const bf16_t*)r, (bf16_t*)dpre, (uint8_t*)dp8, nullptr, (uint8_t*)hq8, hq_limit, (long)F};
  int st = grouped_launch<Cfg8g>(b + 3 * n, d, 4 * n, (const uint8_t*)dy8, d, F, rmax, d, (const int*)tile_expert, e1, s);
  if (st != TFB_OK) return st;
  EpiScaleStore e2{(const float*)rows, SC_DQ_DX, (bf16_t*)dx, (long)d};
  return grouped_launch<Cfg8g>(b + n, F, 4 * n, (const uint8_t*)dp8, F, d, rmax, F, (const int*)tile_expert, e2, s);
}
extern "C" int tfb_moe_mlp8_bwd(const void* dy8, const void* r, const void* w8, const void* rows, const void* tile_expert,
                                void* dx, void* dpre, void* dp8, long rmax, int d, int F, void* stream) {
  if (!dpre) return TFB_ERR_ARG;
  return tfb_moe_mlp8_bwd_q(dy8, r, w8, rows, tile_expert, dx, dpre, dp8, nullptr, 0.f, rmax, d, F, stream);
}

namespace {
// out[g] (+)= acc imm / (rows[g][ca] rows[g][cb]): a grouped fp8 weight gradient leaves the accumulators at its expert's
// power-of-two scales (cb < 0: one scale)
struct EpiDescaleGrouped {
  EpiStore base;
  long slab;  // elements per group
  const float* rows;
  int ca, cb;
  float imm;
  float mul = 0.f;
  __device__ __forceinline__ EpiDescaleGrouped for_group(int g) const {
    EpiDescaleGrouped e = *this;
    e.base.out = base.f32 ? (void*)((float*)base.out + (long)g * slab) : (void*)((bf16_t*)base.out + (long)g * slab);
    e.rows = rows + (long)g * NSC;
    return e;
  }
  __device__ __forceinline__ EpiDescaleGrouped prepare() const {
    EpiDescaleGrouped e = *this;
    float dsc = rows[ca];
    if (cb >= 0) dsc *= rows[cb];
    e.mul = imm / dsc;
    return e;
  }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], int s) const {
    float w[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = v[i] * mul;
    base(p, q, w, s);
  }
};
}  // namespace

// The experts' two weight gradients in fp8 over each expert's row segment [seg[e], seg[e+1]) of the grouped byte buffers
// (every segment a multiple of 128 rows): dw_fc [E][F][d] (+)= bf16((dp8_e^T @ xs8_e) / (s_dp[e] x_scale)), dw_proj [E][d][F]
// (+)= bf16((dy8_e^T @ hq8_e) / (s_dy[e] s_h[e])), with the scales of rows fp32 [E][16] (the backward call's rows).
// xs8 e4m3 (the gather's), dp8 e5m2 and hq8 e4m3 (tfb_moe_mlp8_bwd_q's), dy8 e5m2 (the backward's input bytes).
// Replaces mlp8_weight_grads under its fp8 weight-gradient switch (round2/source/train.py:8209-8229) inside
// moe_expert8_mlp's backward, expert by expert.
extern "C" int tfb_moe_dw8(const void* xs8, const void* dp8, const void* hq8, const void* dy8, const void* rows, float x_scale,
                           const void* seg, void* dw_fc, void* dw_proj, int E, int d, int F, int out_f32, int accumulate,
                           void* stream) {
  if (!xs8 || !dp8 || !hq8 || !dy8 || !rows || !seg || !dw_fc || !dw_proj) return TFB_ERR_ARG;
  if (E <= 0 || d <= 0 || F <= 0 || d % 128 || F % 128 || !(x_scale > 0.f)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  using Cfg = GemmCfg<128, 128, 2, 2, 1, TFB_K_STRIDED, TFB_K_STRIDED, TFB_FMT_E4M3, TFB_FMT_E5M2>;
  GemmArgs a;
  a.q_group = nullptr;
  a.p_group_stride = 0;
  a.k_seg = (const int*)seg;
  a.nkt = 0;
  // dw_fc[e][f][j] = sum_m dp8[m][f] xs8[m][j]: output contiguous in j -> P = xs8 (e4m3), Q = dp8 (e5m2)
  a.P = GemmOperand{(const uint8_t*)xs8, (long)d};
  a.Q = GemmOperand{(const uint8_t*)dp8, (long)F};
  a.np = d;
  a.nq = F;
  a.ntp = d / 128;
  EpiDescaleGrouped e1{EpiStore{dw_fc, (long)d, out_f32, accumulate}, (long)F * d, (const float*)rows, SC_S_DP, -1, 1.0f / x_scale};
  int st = gemm_launch_args<Cfg>(a, E, 1, LoadIdentity{}, LoadIdentity{}, e1, s);
  if (st != TFB_OK) return st;
  // dw_proj[e][j][f] = sum_m dy8[m][j] hq8[m][f]: output contiguous in f -> P = hq8 (e4m3), Q = dy8 (e5m2)
  a.P = GemmOperand{(const uint8_t*)hq8, (long)F};
  a.Q = GemmOperand{(const uint8_t*)dy8, (long)d};
  a.np = F;
  a.nq = d;
  a.ntp = F / 128;
  EpiDescaleGrouped e2{EpiStore{dw_proj, (long)F, out_f32, accumulate}, (long)F * d, (const float*)rows, SC_S_DY, SC_S_H, 1.0f};
  return gemm_launch_args<Cfg>(a, E, 1, LoadIdentity{}, LoadIdentity{}, e2, s);
}

// Per-expert weight gradients over the expert's row segment [seg[e], seg[e+1]) of the grouped buffers:
// dw_fc [E][F][d] (+)= dpre_e^T @ xs_e; dw_proj [E][d][F] (+)= dys_e^T @ bf16(r_e^2). bf16 or fp32 outputs.
extern "C" int tfb_moe_dw(const void* dpre, const void* xs, const void* dys, const void* r, const void* seg, void* dw_fc,
                          void* dw_proj, int E, int d, int F, int out_f32, int accumulate, void* stream) {
  if (!dpre || !xs || !dys || !r || !seg || !dw_fc || !dw_proj) return TFB_ERR_ARG;
  if (E <= 0 || d % 128 || F % 128) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  using Cfg = GemmCfg<128, 128, 2, 2, 2, TFB_K_STRIDED, TFB_K_STRIDED>;
  GemmArgs a;
  a.q_group = nullptr;
  a.p_group_stride = 0;
  a.k_seg = (const int*)seg;
  a.nkt = 0;
  // dw_fc[e][f][j] = sum_m dpre[m][f] xs[m][j]: output contiguous in j (d) -> P = xs, Q = dpre
  a.P = GemmOperand{(const uint8_t*)xs, (long)d * 2};
  a.Q = GemmOperand{(const uint8_t*)dpre, (long)F * 2};
  a.np = d;
  a.nq = F;
  a.ntp = d / 128;
  EpiStoreGrouped e1{EpiStore{dw_fc, (long)d, out_f32, accumulate}, (long)F * d};
  int st = gemm_launch_args<Cfg>(a, E, 1, LoadIdentity{}, LoadIdentity{}, e1, s);
  if (st != TFB_OK) return st;
  // dw_proj[e][j][f] = sum_m dys[m][j] r[m][f]^2: output contiguous in f -> P = r (squared while staged), Q = dys
  a.P = GemmOperand{(const uint8_t*)r, (long)F * 2};
  a.Q = GemmOperand{(const uint8_t*)dys, (long)d * 2};
  a.np = F;
  a.nq = d;
  a.ntp = F / 128;
  EpiStoreGrouped e2{EpiStore{dw_proj, (long)F, out_f32, accumulate}, (long)F * d};
  using CfgSq = GemmCfg<128, 128, 4, 1, 2, TFB_K_STRIDED, TFB_K_STRIDED>;
  return gemm_launch_args<CfgSq>(a, E, 1, LoadSquare{}, LoadIdentity{}, e2, s);
}

// ---- bf16 experts ------------------------------------------------------------------------------------------------
// The routed experts in bf16, every expert on this GPU, on the grouped buffers of the slot tables: each expert e applies
// F.linear(relu(F.linear(x, w_fc[e])).square(), w_proj[e]) to its rows, with the bf16 roundings of those four operations
// (pre, r = relu(pre), h = r^2, y). Replaces moe_experts_local / the kit's expression of moe_expert_mlp
// (round2/source/train.py:10716-10727, 10711) and its autograd backward.
namespace {
struct EpiRelu2 {  // pre = bf16(acc); r = max(pre, 0); h = bf16(r r)
  bf16_t* r;
  bf16_t* h;
  long F;
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], int) const {
    u32x4 rb, hb;
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      float a = v[i], b = v[i + 1];
      round2_bf(a, b);
      a = fmaxf(a, 0.f);
      b = fmaxf(b, 0.f);
      rb[i >> 1] = pack2bf(a, b);  // exact: a and b are bf16 values
      a *= a;
      b *= b;
      hb[i >> 1] = round2_bf(a, b);
    }
    const long off = (long)q * F + p;
    __builtin_nontemporal_store(rb, (u32x4*)(r + off));   // (kept for the backward only, as the fp8 experts' r)
    *(u32x4*)(h + off) = hb;
  }
};
struct EpiDpre {  // dpre = bf16(bf16(acc) (2 r)): the gradient through h = r^2 and the ReLU (r = 0 where it was off)
  const bf16_t* r;
  bf16_t* dpre;
  long F;
  typedef u32x4 pre_t;
  __device__ __forceinline__ pre_t prefetch(int p, int q) const { return __builtin_nontemporal_load((const u32x4*)(r + (long)q * F + p)); }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], const pre_t& rv, int) const {
    float rr[8];
    unpack8bf(rv, rr);
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      float a = v[i], b = v[i + 1];
      round2_bf(a, b);
      a *= 2.f * rr[i];
      b *= 2.f * rr[i + 1];
      o[i >> 1] = round2_bf(a, b);
    }
    *(u32x4*)(dpre + (long)q * F + p) = o;
  }
};
inline bool shapes16(long rmax, int d, int F) { return rmax > 0 && rmax % 128 == 0 && d > 0 && d % 128 == 0 && F > 0 && F % 128 == 0; }
using CfgNT = GemmCfg<128, 128, 2, 2, 2, TFB_K_CONTIG, TFB_K_CONTIG>;
using CfgNN = GemmCfg<128, 128, 2, 2, 2, TFB_K_STRIDED, TFB_K_CONTIG>;
}  // namespace

// xs bf16 [rmax][d] (the gathered rows, padding rows zero), w_fc bf16 [E][F][d], w_proj bf16 [E][d][F], tile_expert int32
// [rmax / 128] -> ys bf16 [rmax][d], r bf16 [rmax][F] = relu(pre) and h bf16 [rmax][F] = r^2 (both kept for the backward).
extern "C" int tfb_moe_mlp_fwd(const void* xs, const void* w_fc, const void* w_proj, const void* tile_expert, void* ys, void* r,
                               void* h, long rmax, int d, int F, void* stream) {
  if (!xs || !w_fc || !w_proj || !tile_expert || !ys || !r || !h) return TFB_ERR_ARG;
  if (!shapes16(rmax, d, F)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const long n = (long)F * d;
  EpiRelu2 e1{(bf16_t*)r, (bf16_t*)h, (long)F};
  int st = grouped_launch<CfgNT>((const uint8_t*)w_fc, d * 2L, n * 2, (const uint8_t*)xs, d * 2L, F, rmax, d * 2L,
                                 (const int*)tile_expert, e1, s);
  if (st != TFB_OK) return st;
  EpiStore e2{ys, (long)d, 0, 0};
  return grouped_launch<CfgNT>((const uint8_t*)w_proj, F * 2L, n * 2, (const uint8_t*)h, F * 2L, d, rmax, F * 2L,
                               (const int*)tile_expert, e2, s);
}

// dys bf16 [rmax][d], r as the forward left it -> dpre bf16 [rmax][F] = bf16(bf16(dys w_proj[e]) 2 r), dxs bf16 [rmax][d] =
// dpre w_fc[e]. The weight gradients are tfb_moe_dw(dpre, xs, dys, r, ...): dw_proj contracts dys with bf16(r^2) = h.
extern "C" int tfb_moe_mlp_bwd(const void* dys, const void* r, const void* w_fc, const void* w_proj, const void* tile_expert,
                               void* dxs, void* dpre, long rmax, int d, int F, void* stream) {
  if (!dys || !r || !w_fc || !w_proj || !tile_expert || !dxs || !dpre) return TFB_ERR_ARG;
  if (!shapes16(rmax, d, F)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const long n = (long)F * d;
  // dh[row][f] = sum_j dys[row][j] w_proj[e][j][f]: the weight is the k-strided operand (k = j, contiguous in f)
  EpiDpre e1{(const bf16_t*)r, (bf16_t*)dpre, (long)F};
  int st = grouped_launch<CfgNN>((const uint8_t*)w_proj, F * 2L, n * 2, (const uint8_t*)dys, d * 2L, F, rmax, d * 2L,
                                 (const int*)tile_expert, e1, s);
  if (st != TFB_OK) return st;
  // dxs[row][j] = sum_f dpre[row][f] w_fc[e][f][j]
  EpiStore e2{dxs, (long)d, 0, 0};
  return grouped_launch<CfgNN>((const uint8_t*)w_fc, d * 2L, n * 2, (const uint8_t*)dpre, F * 2L, d, rmax, F * 2L,
                               (const int*)tile_expert, e2, s);
}

// ---- dense bf16 fused MLP ------------------------------------------------------------------------------------------
// y = bf16(h @ w_proj^T) with r = bf16(relu(x @ w_fc^T)), h = bf16(r r); backward dpre = bf16(((dy @ w_proj) 2) r) (ONE
// rounding: the fused kernel folds the factors into the product's evacuation), h = bf16(r r), dx = bf16(dpre @ w_fc).
// Replaces _mlp_fwd_kernel(x2, w_fc, w_proj, tb) -> (y, rT) and _mlp_bwd_kernel(dy2, rT, w_fc, w_proj, tb, dw_mode) ->
// (dx, h, dpre) (round2/source/kernels/nki_mlp_fused.py:242, 290; arithmetic emulate_forward / emulate_backward :372-392).
// The saved activation is token-major r [M][F] (the reference keeps its transpose for its SBUF layout).
namespace {
struct EpiDpre1 {  // dpre = bf16((acc 2) r); optionally h = bf16(r r)
  const bf16_t* r;
  bf16_t* dpre;
  bf16_t* h;  // or null
  long F;
  typedef u32x4 pre_t;
  __device__ __forceinline__ pre_t prefetch(int p, int q) const { return *(const u32x4*)(r + (long)q * F + p); }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], const pre_t& rv, int) const {
    float rr[8];
    unpack8bf(rv, rr);
    u32x4 o, hb;
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      o[i >> 1] = pack2bf((v[i] * 2.f) * rr[i], (v[i + 1] * 2.f) * rr[i + 1]);
      hb[i >> 1] = pack2bf(rr[i] * rr[i], rr[i + 1] * rr[i + 1]);
    }
    const long off = (long)q * F + p;
    *(u32x4*)(dpre + off) = o;
    if (h) *(u32x4*)(h + off) = hb;
  }
};
}  // namespace

// x bf16 [M][d], w_fc bf16 [F][d], w_proj bf16 [d][F] -> y bf16 [M][d], r bf16 [M][F] (saved for the backward), h bf16
// [M][F] (the second GEMM's operand; scratch for the caller). M, d, F multiples of 128.
extern "C" int tfb_mlp_fwd(const void* x, const void* w_fc, const void* w_proj, void* y, void* r, void* h, long M, int d, int F,
                           void* stream) {
  if (!x || !w_fc || !w_proj || !y || !r || !h) return TFB_ERR_ARG;
  if (!shapes16(M, d, F) || M > 0x7fffffffL) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  GemmOperand Pw{(const uint8_t*)w_fc, d * 2L}, Qx{(const uint8_t*)x, d * 2L};
  EpiRelu2 e1{(bf16_t*)r, (bf16_t*)h, (long)F};
  int st = gemm_launch<CfgNT>(Pw, Qx, F, (int)M, d * 2L, 1, LoadIdentity{}, LoadIdentity{}, e1, s);
  if (st != TFB_OK) return st;
  GemmOperand Pp{(const uint8_t*)w_proj, F * 2L}, Qh{(const uint8_t*)h, F * 2L};
  EpiStore e2{y, (long)d, 0, 0};
  return gemm_launch<CfgNT>(Pp, Qh, d, (int)M, F * 2L, 1, LoadIdentity{}, LoadIdentity{}, e2, s);
}

// dy bf16 [M][d], r as the forward left it -> dx bf16 [M][d], dpre bf16 [M][F], h bf16 [M][F] (optional, may be NULL):
// what the weight gradients dw_fc = dpre^T x and dw_proj = dy^T h contract (weight_grads, :394).
extern "C" int tfb_mlp_bwd(const void* dy, const void* r, const void* w_fc, const void* w_proj, void* dx, void* h, void* dpre,
                           long M, int d, int F, void* stream) {
  if (!dy || !r || !w_fc || !w_proj || !dx || !dpre) return TFB_ERR_ARG;
  if (!shapes16(M, d, F) || M > 0x7fffffffL) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  // dh[m][f] = sum_j dy[m][j] w_proj[j][f]: the weight is the k-strided operand (k = j, contiguous in f)
  GemmOperand Pp{(const uint8_t*)w_proj, F * 2L}, Qg{(const uint8_t*)dy, d * 2L};
  EpiDpre1 e1{(const bf16_t*)r, (bf16_t*)dpre, (bf16_t*)h, (long)F};
  int st = gemm_launch<CfgNN>(Pp, Qg, F, (int)M, d * 2L, 1, LoadIdentity{}, LoadIdentity{}, e1, s);
  if (st != TFB_OK) return st;
  // dx[m][j] = sum_f dpre[m][f] w_fc[f][j]
  GemmOperand Pf{(const uint8_t*)w_fc, d * 2L}, Qd{(const uint8_t*)dpre, F * 2L};
  EpiStore e2{dx, (long)d, 0, 0};
  return gemm_launch<CfgNN>(Pf, Qd, d, (int)M, F * 2L, 1, LoadIdentity{}, LoadIdentity{}, e2, s);
}

// RMSNorm family (bandwidth-bound): one wavefront per row, 128-bit coalesced loads, the row
// kept in registers, fp32 math, one rounding per output, wavefront shuffles for the row sums.
//
//   rmsnorm fwd / bwd, optionally with a fused residual add in front (s = x + res, y = norm(s))
//     and an optional per-channel weight                 round1/source/train.py:5594 (rmsnorm_fast),
//                                                        6117 (tail_norm2), 6826 (final_norm);
//                                                        round2/source/train.py:8805-8825 (nf_norm_rows / backward)
//   block head: x_new = l1*x + l2*x0 (+ l3*skip), x_norm = RMSNorm(x_new)
//                                                        round1/source/train.py:5578 (block_head), 6106 (head_skip)
//
// The value that is normalised is the bf16-rounded sum, as the eager chain normalises its bf16
// tensor. Gain / weight gradients are fp32 partial sums per workgroup finished by a column sum.
#include "common.hpp"

namespace {

constexpr int ROWS_PER_BLOCK = 4;  // one wavefront per row, 4 wavefronts per workgroup

// A row is held by G lanes (a whole wavefront, or half of one: two rows per wavefront when the row length is a multiple
// of 256 up to 1024, so that every lane has work in every chunk and a wavefront keeps two rows' loads in flight), each
// lane NCH chunks of 8 elements: chunk i of lane l covers columns 8 (l + G i) .. + 7. `lane` below is the lane's index
// inside its group.
template <int NCH, int G = 64>
struct Row {
  float v[NCH][8];
  __device__ __forceinline__ void load(const bf16_t* p, int C, int lane) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      int c = (lane + G * i) * 8;
      if (c < C) {
        u32x4 u = *(const u32x4*)(p + c);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          v[i][2 * k] = bflo(u[k]);
          v[i][2 * k + 1] = bfhi(u[k]);
        }
      } else {
#pragma unroll
        for (int k = 0; k < 8; ++k) v[i][k] = 0.f;
      }
    }
  }
  __device__ __forceinline__ void store(bf16_t* p, int C, int lane) const {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      int c = (lane + G * i) * 8;
      if (c < C) {
        u32x4 u;
#pragma unroll
        for (int k = 0; k < 4; ++k) u[k] = pack2bf(v[i][2 * k], v[i][2 * k + 1]);
        *(u32x4*)(p + c) = u;
      }
    }
  }
  __device__ __forceinline__ void round() {
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) v[i][k] = round_bf(v[i][k]);
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) v[i][k] = 0.f;
  }
};

// A row as loaded (bf16 pairs in 32-bit words), to be widened later: the kernels below request the NEXT row of a
// wavefront before they store the current one. A wait for loaded data also waits for every older memory operation, stores
// included (one counter orders both), so a loop that loads after its stores pays a full store round trip per row.
template <int NCH, int G = 64>
struct RawRow {
  u32x4 u[NCH];
  __device__ __forceinline__ void load(const bf16_t* p, int C, int lane) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = (lane + G * i) * 8;
      u[i] = c < C ? *(const u32x4*)(p + c) : u32x4{0u, 0u, 0u, 0u};
    }
  }
  __device__ __forceinline__ void widen(Row<NCH, G>& r) const {
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        r.v[i][2 * k] = bflo(u[i][k]);
        r.v[i][2 * k + 1] = bfhi(u[i][k]);
      }
  }
};

// sum / max over the G lanes that hold a row (the butterfly stays inside the group)
template <int G>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int o = G / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
template <int NCH, int G>
__device__ __forceinline__ float row_dot(const Row<NCH, G>& a, const Row<NCH, G>& b) {
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i)
#pragma unroll
    for (int k = 0; k < 8; ++k) s += a.v[i][k] * b.v[i][k];
  return group_sum<G>(s);
}

// ------------------------------------------------------------------------------------------
template <int NCH, int G>
__global__ __launch_bounds__(256) void rmsnorm_fwd_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ res,
                                                         const bf16_t* __restrict__ w, bf16_t* __restrict__ s_out,
                                                         bf16_t* __restrict__ y, float* __restrict__ inv, long nrows,
                                                         int C, float eps, uint8_t* __restrict__ y8, float y8_scale) {
  constexpr int RPW = 64 / G;  // rows per wavefront
  const int lane = threadIdx.x & (G - 1), sub = (threadIdx.x & 63) / G, wave = threadIdx.x >> 6;
  Row<NCH, G> wr;
  if (w) wr.load(w, C, lane);
  const long step = (long)gridDim.x * ROWS_PER_BLOCK * RPW;
  long row = ((long)blockIdx.x * ROWS_PER_BLOCK + wave) * RPW + sub;
  RawRow<NCH, G> xa, xr;
  if (row < nrows) {
    xa.load(x + row * C, C, lane);
    if (res) xr.load(res + row * C, C, lane);
  }
  for (; row < nrows; row += step) {
    Row<NCH, G> a;
    xa.widen(a);
    Row<NCH, G> r;
    if (res) xr.widen(r);
    if (row + step < nrows) {  // the next row's loads go out before this row's stores
      xa.load(x + (row + step) * C, C, lane);
      if (res) xr.load(res + (row + step) * C, C, lane);
    }
    if (res) {
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k) a.v[i][k] = round_bf(a.v[i][k] + r.v[i][k]);
      if (s_out) a.store(s_out + row * C, C, lane);
    }
    float ss = row_dot(a, a);
    float rs = 1.0f / sqrtf(ss * (1.0f / C) + eps);
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) a.v[i][k] = w ? a.v[i][k] * rs * wr.v[i][k] : a.v[i][k] * rs;
    if (y) a.store(y + row * C, C, lane);
    if (y8) {  // e4m3(bf16(y) * scale): the cast the fp8 GEMM that consumes y would otherwise make in a pass of its own
      a.round();
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int c = (lane + G * i) * 8;
        if (c < C) {
          u32x2 o;
          o.x = cvt4_fp8<TFB_FMT_E4M3>(a.v[i][0] * y8_scale, a.v[i][1] * y8_scale, a.v[i][2] * y8_scale, a.v[i][3] * y8_scale);
          o.y = cvt4_fp8<TFB_FMT_E4M3>(a.v[i][4] * y8_scale, a.v[i][5] * y8_scale, a.v[i][6] * y8_scale, a.v[i][7] * y8_scale);
          *(u32x2*)(y8 + row * C + c) = o;
        }
      }
    }
    if (inv && lane == 0) inv[row] = rs;
  }
}

// dx = gs + J^T(gy): J^T(gy) = inv * (gh - s * (gh . s) * inv^2 / C), gh = gy * w.
// dw partial [gridDim.x][C] = sum over the workgroup's rows of gy * s * inv.
template <int NCH, int G>
__global__ __launch_bounds__(256) void rmsnorm_bwd_kernel(const bf16_t* __restrict__ gy, const bf16_t* __restrict__ gs,
                                                         const bf16_t* __restrict__ s, const bf16_t* __restrict__ w,
                                                         const float* __restrict__ inv, bf16_t* __restrict__ dx,
                                                         float* __restrict__ dw_part, float* __restrict__ amax_part, long nrows,
                                                         int C) {
  constexpr int RPW = 64 / G, RPB = ROWS_PER_BLOCK * RPW;  // rows per wavefront, per workgroup
  __shared__ float red[RPB][NCH * G * 8];
  __shared__ float amred[ROWS_PER_BLOCK];
  const int lane = threadIdx.x & (G - 1), sub = (threadIdx.x & 63) / G, wave = threadIdx.x >> 6;
  float am = 0.f;   // amax of the rounded dx this wavefront wrote (amax_part: one value per workgroup)
  Row<NCH, G> wr, dwacc;
  if (w) wr.load(w, C, lane);
  dwacc.zero();
  const long step = (long)gridDim.x * RPB;
  long row = ((long)blockIdx.x * ROWS_PER_BLOCK + wave) * RPW + sub;
  RawRow<NCH, G> xg, xa, xr;
  float rs_next = 0.f;
  if (row < nrows) {
    xg.load(gy + row * C, C, lane);
    xa.load(s + row * C, C, lane);
    if (gs) xr.load(gs + row * C, C, lane);
    rs_next = inv[row];
  }
  for (; row < nrows; row += step) {
    Row<NCH, G> g, a, r;
    xg.widen(g);
    xa.widen(a);
    if (gs) xr.widen(r);
    const float rs = rs_next;
    if (row + step < nrows) {  // the next row's loads go out before this row's store
      xg.load(gy + (row + step) * C, C, lane);
      xa.load(s + (row + step) * C, C, lane);
      if (gs) xr.load(gs + (row + step) * C, C, lane);
      rs_next = inv[row + step];
    }
    if (w) {
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          dwacc.v[i][k] += g.v[i][k] * a.v[i][k] * rs;
          g.v[i][k] *= wr.v[i][k];
        }
    }
    float dot = row_dot(g, a);
    float coef = dot * rs * rs * (1.0f / C);
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) g.v[i][k] = rs * (g.v[i][k] - a.v[i][k] * coef);
    if (gs) {
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k) g.v[i][k] += r.v[i][k];
    }
    if (amax_part) {
      g.round();
#pragma unroll
      for (int i = 0; i < NCH; ++i)
        if ((lane + G * i) * 8 < C) {
#pragma unroll
          for (int k = 0; k < 8; ++k) am = fmaxf(am, fabsf(g.v[i][k]));
        }
    }
    g.store(dx + row * C, C, lane);
  }
  if (amax_part) {
    am = wave_max(am);
    if ((threadIdx.x & 63) == 0) amred[wave] = am;
    __syncthreads();
    if (threadIdx.x == 0) {
      float t = amred[0];
#pragma unroll
      for (int r = 1; r < ROWS_PER_BLOCK; ++r) t = fmaxf(t, amred[r]);
      amax_part[blockIdx.x] = t;
    }
  }
  if (w && dw_part) {
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) red[wave * RPW + sub][(lane + G * i) * 8 + k] = dwacc.v[i][k];
    __syncthreads();
    for (int c = threadIdx.x; c < C; c += 256) {
      float t = 0.f;
#pragma unroll
      for (int r = 0; r < RPB; ++r) t += red[r][c];
      dw_part[(long)blockIdx.x * C + c] = t;
    }
  }
}

// out[c] (+)= sum_r part[r][c]: 64 columns x 16 row lanes per workgroup, rows interleaved over the lanes.
// blockIdx.y selects one of several independent sums (part + y * part_stride -> out + y * out_stride).
__global__ __launch_bounds__(1024) void colsum_kernel(const float* __restrict__ part, float* __restrict__ out, int rows, int C,
                                                     int accumulate, long part_stride = 0, long out_stride = 0) {
  __shared__ float red[16][64];
  const int tx = threadIdx.x, ty = threadIdx.y;
  const int c = blockIdx.x * 64 + tx;
  part += (long)blockIdx.y * part_stride;
  out += (long)blockIdx.y * out_stride;
  float t = 0.f;
  if (c < C)
    for (int r = ty; r < rows; r += 16) t += part[(long)r * C + c];
  red[ty][tx] = t;
  __syncthreads();
  if (ty == 0 && c < C) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += red[i][tx];
    out[c] = accumulate ? out[c] + s : s;
  }
}

// ------------------------------------------------------------------------------------------ block head
template <int NCH>
__global__ __launch_bounds__(256) void block_head_fwd_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ x0,
                                                            const bf16_t* __restrict__ skip,
                                                            const float* __restrict__ gains, bf16_t* __restrict__ x_new,
                                                            bf16_t* __restrict__ x_norm, float* __restrict__ inv,
                                                            long nrows, int C, float eps) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float l1 = gains[0], l2 = gains[1], l3 = skip ? gains[2] : 0.f;
  for (long row = (long)blockIdx.x * ROWS_PER_BLOCK + wave; row < nrows; row += (long)gridDim.x * ROWS_PER_BLOCK) {
    Row<NCH> a, b;
    a.load(x + row * C, C, lane);
    b.load(x0 + row * C, C, lane);
    if (skip) {
      Row<NCH> c;
      c.load(skip + row * C, C, lane);
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k) a.v[i][k] = round_bf(l1 * (a.v[i][k] + l3 * c.v[i][k]) + l2 * b.v[i][k]);
    } else {
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k) a.v[i][k] = round_bf(l1 * a.v[i][k] + l2 * b.v[i][k]);
    }
    a.store(x_new + row * C, C, lane);
    float ss = row_dot(a, a);
    float rs = 1.0f / sqrtf(ss * (1.0f / C) + eps);
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) a.v[i][k] *= rs;
    a.store(x_norm + row * C, C, lane);
    if (lane == 0) inv[row] = rs;
  }
}

// x_new = l1 (x + l3 skip) + l2 x0. G = g_new + inv * (g_norm - x_new * (g_norm . x_new) * inv^2 / C);
// dx = l1 G, dx0 = l2 G, dskip = l1 l3 G; gain partials [gridDim.x][4] = sum G.(x + l3 skip), G.x0, l1 G.skip, 0
template <int NCH>
__global__ __launch_bounds__(256) void block_head_bwd_kernel(const bf16_t* __restrict__ g_new,
                                                            const bf16_t* __restrict__ g_norm,
                                                            const bf16_t* __restrict__ x, const bf16_t* __restrict__ x0,
                                                            const bf16_t* __restrict__ skip,
                                                            const bf16_t* __restrict__ x_new,
                                                            const float* __restrict__ inv, const float* __restrict__ gains,
                                                            bf16_t* __restrict__ dx, bf16_t* __restrict__ dx0,
                                                            bf16_t* __restrict__ dskip, float* __restrict__ gain_part,
                                                            long nrows, int C) {
  __shared__ float red[ROWS_PER_BLOCK][3];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float l1 = gains[0], l2 = gains[1], l3 = skip ? gains[2] : 0.f;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (long row = (long)blockIdx.x * ROWS_PER_BLOCK + wave; row < nrows; row += (long)gridDim.x * ROWS_PER_BLOCK) {
    Row<NCH> g, xn, t;
    g.load(g_norm + row * C, C, lane);
    xn.load(x_new + row * C, C, lane);
    const float rs = inv[row];
    float dot = row_dot(g, xn);
    float coef = dot * rs * rs * (1.0f / C);
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) g.v[i][k] = rs * (g.v[i][k] - xn.v[i][k] * coef);
    if (g_new) {
      t.load(g_new + row * C, C, lane);
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k) g.v[i][k] += t.v[i][k];
    }
    // g is G (fp32)
    t.load(x + row * C, C, lane);
    s1 += row_dot(g, t);
    if (skip) {
      Row<NCH> sk;
      sk.load(skip + row * C, C, lane);
      const float gs = row_dot(g, sk);
      s1 += l3 * gs;
      s3 += l1 * gs;
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) t.v[i][k] = l1 * g.v[i][k];
    t.store(dx + row * C, C, lane);
    t.load(x0 + row * C, C, lane);
    s2 += row_dot(g, t);
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) t.v[i][k] = l2 * g.v[i][k];
    t.store(dx0 + row * C, C, lane);
    if (skip) {
      const float l13 = l1 * l3;
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k) t.v[i][k] = l13 * g.v[i][k];
      t.store(dskip + row * C, C, lane);
    }
  }
  if (lane == 0) {
    red[wave][0] = s1;
    red[wave][1] = s2;
    red[wave][2] = s3;
  }
  __syncthreads();
  if (threadIdx.x < 3) {
    float t = 0.f;
    for (int r = 0; r < ROWS_PER_BLOCK; ++r) t += red[r][threadIdx.x];
    gain_part[(long)blockIdx.x * 4 + threadIdx.x] = t;
  }
  if (threadIdx.x == 3) gain_part[(long)blockIdx.x * 4 + 3] = 0.f;
}

// ------------------------------------------------------------------------------------------ mixer tail
// The attention-less block's causal one-token shift in front of the tail norm:
//   s1 = bf16(x + bf16(lam * shift1(x))), xn2 = RMSNorm(s1), inv saved; shift1 gives token t the row of token t - 1 of its
//   sequence (zeros at t = 0). One wavefront per row; the previous row is read again (it is the neighbour's row, from L2).
template <int NCH>
__global__ __launch_bounds__(256) void mix_tail_fwd_kernel(const bf16_t* __restrict__ x, const float* __restrict__ lam,
                                                          bf16_t* __restrict__ s1, bf16_t* __restrict__ xn2,
                                                          float* __restrict__ inv, long nrows, int C, int T, float eps) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float l = lam[0];
  for (long row = (long)blockIdx.x * ROWS_PER_BLOCK + wave; row < nrows; row += (long)gridDim.x * ROWS_PER_BLOCK) {
    Row<NCH> a, b;
    a.load(x + row * C, C, lane);
    if (row % T) b.load(x + (row - 1) * C, C, lane);
    else b.zero();
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) a.v[i][k] = round_bf(a.v[i][k] + round_bf(l * b.v[i][k]));
    a.store(s1 + row * C, C, lane);
    const float ss = row_dot(a, a);
    const float rs = 1.0f / sqrtf(ss * (1.0f / C) + eps);
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) a.v[i][k] *= rs;
    a.store(xn2 + row * C, C, lane);
    if (lane == 0) inv[row] = rs;
  }
}

// g = bf16(ge + inv (gy - s (gy . s) inv^2 / C)) (the tail norm's backward, one rounding; ge and/or gy may be absent);
// gx[t] = bf16(g[t] + bf16(lam g[t + 1])) (g[t + 1] = 0 at a sequence's last token: the shift's adjoint);
// dlam partial [gridDim.x] = sum over the workgroup's rows of the bf16 products bf16(g[t] x[t - 1]) in fp32.
// Row t + 1's g is recomputed by the wavefront that owns row t (the chain is per row: the same bits).
template <int NCH>
__global__ __launch_bounds__(256) void mix_tail_bwd_kernel(const bf16_t* __restrict__ s, const bf16_t* __restrict__ gy,
                                                          const bf16_t* __restrict__ ge, const float* __restrict__ inv,
                                                          const bf16_t* __restrict__ x, const float* __restrict__ lam,
                                                          bf16_t* __restrict__ gx, float* __restrict__ dlam_part, long nrows,
                                                          int C, int T) {
  __shared__ float red[ROWS_PER_BLOCK];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float l = lam[0];
  float dl = 0.f;
  auto g_row = [&](long row, Row<NCH>& g) {
    Row<NCH> a;
    a.load(s + row * C, C, lane);
    if (gy) {
      g.load(gy + row * C, C, lane);
      const float rs = inv[row];
      const float coef = row_dot(g, a) * rs * rs * (1.0f / C);
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k) g.v[i][k] = rs * (g.v[i][k] - a.v[i][k] * coef);
    } else {
      g.zero();
    }
    if (ge) {
      Row<NCH> e;
      e.load(ge + row * C, C, lane);
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k) g.v[i][k] += e.v[i][k];
    }
    g.round();
  };
  for (long row = (long)blockIdx.x * ROWS_PER_BLOCK + wave; row < nrows; row += (long)gridDim.x * ROWS_PER_BLOCK) {
    Row<NCH> g, gn, xp;
    g_row(row, g);
    if ((row + 1) % T) g_row(row + 1, gn);
    else gn.zero();
    if (row % T) xp.load(x + (row - 1) * C, C, lane);
    else xp.zero();
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        part += round_bf(g.v[i][k] * xp.v[i][k]);
        g.v[i][k] = g.v[i][k] + round_bf(l * gn.v[i][k]);
      }
    dl += wave_sum(part);
    g.store(gx + row * C, C, lane);
  }
  if (lane == 0) red[wave] = dl;
  __syncthreads();
  if (threadIdx.x == 0) dlam_part[blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
}

// out[0] = sum of part[0 .. n) in a fixed order (one workgroup)
__global__ __launch_bounds__(256) void sum_partials_kernel(const float* __restrict__ part, int n, float* __restrict__ out) {
  __shared__ float red[4];
  float t = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) t += part[i];
  t = wave_sum(t);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = t;
  __syncthreads();
  if (threadIdx.x == 0) out[0] = (red[0] + red[1]) + (red[2] + red[3]);
}

inline int grid_for(long nrows, int cap) {
  long b = (nrows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  return (int)(b < cap ? b : cap);
}

}  // namespace

#define DISPATCH_NCH(C, CALL)            \
  do {                                   \
    if ((C) <= 512) { CALL(1); }         \
    else if ((C) <= 1024) { CALL(2); }   \
    else if ((C) <= 2048) { CALL(4); }   \
    else { CALL(8); }                    \
  } while (0)
// the RMSNorm pair: rows of 256, 512, 768 or 1024 elements on half a wavefront each (two rows per wavefront), else a
// wavefront per row
#define DISPATCH_ROWS(C, CALL)                                   \
  do {                                                           \
    if ((C) % 256 == 0 && (C) <= 1024) {                         \
      if ((C) == 256) { CALL(1, 32); }                           \
      else if ((C) == 512) { CALL(2, 32); }                      \
      else if ((C) == 768) { CALL(3, 32); }                      \
      else { CALL(4, 32); }                                      \
    } else if ((C) <= 512) { CALL(1, 64); }                      \
    else if ((C) <= 1024) { CALL(2, 64); }                       \
    else if ((C) <= 2048) { CALL(4, 64); }                       \
    else { CALL(8, 64); }                                        \
  } while (0)
static inline int norm_rows_per_block(int C) { return (C % 256 == 0 && C <= 1024) ? 2 * ROWS_PER_BLOCK : ROWS_PER_BLOCK; }

static bool norm_shape_ok(long nrows, int C) { return nrows > 0 && C > 0 && C % 8 == 0 && C <= 4096; }

extern "C" int tfb_norm_bwd_blocks(long nrows) { return grid_for(nrows, 1024); }

// y8 (optional): e4m3(bf16(y) * y8_scale), [nrows][C] bytes - the operand cast of the fp8 GEMM that consumes y, made here
// instead of in a pass of its own.
static int rmsnorm_fwd_impl(const void* x, const void* res, const void* w, void* s_out, void* y, void* inv, void* y8,
                            float y8_scale, long nrows, int C, float eps, void* stream) {
  if (!x || (!y && !y8)) return TFB_ERR_ARG;   // y may be left out when only its fp8 cast is read (both MLP GEMM kinds in fp8)
  if (res && !s_out) return TFB_ERR_ARG;
  if (!norm_shape_ok(nrows, C)) return TFB_ERR_SHAPE;
  const long rpb = norm_rows_per_block(C), nb = (nrows + rpb - 1) / rpb;
  int grid = (int)(nb < 8192 ? nb : 8192);
#define CALL(N, G)                                                                                                    \
  hipLaunchKernelGGL((rmsnorm_fwd_kernel<N, G>), dim3(grid), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)x,     \
                     (const bf16_t*)res, (const bf16_t*)w, (bf16_t*)s_out, (bf16_t*)y, (float*)inv, nrows, C, eps,    \
                     (uint8_t*)y8, y8_scale)
  DISPATCH_ROWS(C, CALL);
#undef CALL
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}
extern "C" int tfb_rmsnorm_fwd(const void* x, const void* res, const void* w, void* s_out, void* y, void* inv, long nrows,
                               int C, float eps, void* stream) {
  return rmsnorm_fwd_impl(x, res, w, s_out, y, inv, nullptr, 0.f, nrows, C, eps, stream);
}
extern "C" int tfb_rmsnorm_fwd_q(const void* x, const void* res, const void* w, void* s_out, void* y, void* inv, void* y8,
                                 float y8_scale, long nrows, int C, float eps, void* stream) {
  if (!y8) return TFB_ERR_ARG;
  return rmsnorm_fwd_impl(x, res, w, s_out, y, inv, y8, y8_scale, nrows, C, eps, stream);
}

// dw_part: fp32 [tfb_norm_bwd_blocks(nrows)][C] scratch (only when w != NULL); dw: fp32 [C].
static int rmsnorm_bwd_impl(const void* gy, const void* gs, const void* s, const void* w, const void* inv, void* dx,
                            void* dw_part, void* dw, int dw_accumulate, void* amax_part, long nrows, int C, void* stream) {
  if (!gy || !s || !inv || !dx) return TFB_ERR_ARG;
  if (w && !dw_part) return TFB_ERR_ARG;
  if (!norm_shape_ok(nrows, C)) return TFB_ERR_SHAPE;
  // (the grid is tfb_norm_bwd_blocks(nrows) whatever the rows per workgroup: every partial row of dw_part / amax_part is
  // written, by a workgroup without rows as zeros)
  int grid = grid_for(nrows, 1024);
#define CALL(N, G)                                                                                                     \
  hipLaunchKernelGGL((rmsnorm_bwd_kernel<N, G>), dim3(grid), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)gy,     \
                     (const bf16_t*)gs, (const bf16_t*)s, (const bf16_t*)w, (const float*)inv, (bf16_t*)dx,            \
                     (float*)dw_part, (float*)amax_part, nrows, C)
  DISPATCH_ROWS(C, CALL);
#undef CALL
  TFB_LAUNCH_CHECK();
  if (w && dw) {
    hipLaunchKernelGGL(colsum_kernel, dim3((C + 63) / 64), dim3(64, 16), 0, (hipStream_t)stream, (const float*)dw_part,
                       (float*)dw, grid, C, dw_accumulate, 0L, 0L);
    TFB_LAUNCH_CHECK();
  }
  return TFB_OK;
}

extern "C" int tfb_rmsnorm_bwd(const void* gy, const void* gs, const void* s, const void* w, const void* inv, void* dx,
                               void* dw_part, void* dw, int dw_accumulate, long nrows, int C, void* stream) {
  return rmsnorm_bwd_impl(gy, gs, s, w, inv, dx, dw_part, dw, dw_accumulate, nullptr, nrows, C, stream);
}
// tfb_rmsnorm_bwd that also leaves amax_part fp32 [tfb_norm_bwd_blocks(nrows)]: per workgroup, the largest |dx| it wrote
// (of the rounded values). The fp8 MLP whose backward receives this dx as its dy takes its scales from these
// (tfb_mlp8_backward_scales_part) instead of reading dy once more for its amax.
extern "C" int tfb_rmsnorm_bwd_amax(const void* gy, const void* gs, const void* s, const void* w, const void* inv, void* dx,
                                    void* dw_part, void* dw, int dw_accumulate, void* amax_part, long nrows, int C,
                                    void* stream) {
  if (!amax_part) return TFB_ERR_ARG;
  return rmsnorm_bwd_impl(gy, gs, s, w, inv, dx, dw_part, dw, dw_accumulate, amax_part, nrows, C, stream);
}

// Finish `count` weight gradients at once: dw[i][c] (+)= sum_r part[i][r][c], part = count blocks of
// tfb_norm_bwd_blocks(nrows) x C floats as left by tfb_rmsnorm_bwd calls made with dw = NULL (part_stride, dw_stride in
// floats). One launch instead of one 12-workgroup launch per norm.
extern "C" int tfb_norm_dw_finish(const void* dw_part, void* dw, int count, long part_stride, long dw_stride, int dw_accumulate,
                                  long nrows, int C, void* stream) {
  if (!dw_part || !dw) return TFB_ERR_ARG;
  if (count <= 0 || count > 65535 || !norm_shape_ok(nrows, C) || part_stride < 0 || dw_stride < 0) return TFB_ERR_SHAPE;
  hipLaunchKernelGGL(colsum_kernel, dim3((C + 63) / 64, count), dim3(64, 16), 0, (hipStream_t)stream, (const float*)dw_part,
                     (float*)dw, grid_for(nrows, 1024), C, dw_accumulate, part_stride, dw_stride);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// gains: device fp32 [3] = l1, l2, l3 (l3 read only when skip != NULL)
extern "C" int tfb_block_head_fwd(const void* x, const void* x0, const void* skip, const void* gains, void* x_new,
                                  void* x_norm, void* inv, long nrows, int C, float eps, void* stream) {
  if (!x || !x0 || !gains || !x_new || !x_norm || !inv) return TFB_ERR_ARG;
  if (!norm_shape_ok(nrows, C)) return TFB_ERR_SHAPE;
  int grid = grid_for(nrows, 8192);
#define CALL(N)                                                                                                      \
  hipLaunchKernelGGL(block_head_fwd_kernel<N>, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)x,      \
                     (const bf16_t*)x0, (const bf16_t*)skip, (const float*)gains, (bf16_t*)x_new, (bf16_t*)x_norm,  \
                     (float*)inv, nrows, C, eps)
  DISPATCH_NCH(C, CALL);
#undef CALL
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// gain_part: fp32 [tfb_norm_bwd_blocks(nrows)][4] scratch; dgains: fp32 [4] (sum G.(x + l3 skip), G.x0, l1 G.skip, 0)
extern "C" int tfb_block_head_bwd(const void* g_new, const void* g_norm, const void* x, const void* x0, const void* skip,
                                  const void* x_new, const void* inv, const void* gains, void* dx, void* dx0,
                                  void* dskip, void* gain_part, void* dgains, long nrows, int C, void* stream) {
  if (!g_norm || !x || !x0 || !x_new || !inv || !gains || !dx || !dx0 || !gain_part || !dgains) return TFB_ERR_ARG;
  if (skip && !dskip) return TFB_ERR_ARG;
  if (!norm_shape_ok(nrows, C)) return TFB_ERR_SHAPE;
  int grid = grid_for(nrows, 1024);
#define CALL(N)                                                                                                        \
  hipLaunchKernelGGL(block_head_bwd_kernel<N>, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)g_new,    \
                     (const bf16_t*)g_norm, (const bf16_t*)x, (const bf16_t*)x0, (const bf16_t*)skip,                  \
                     (const bf16_t*)x_new, (const float*)inv, (const float*)gains, (bf16_t*)dx, (bf16_t*)dx0,          \
                     (bf16_t*)dskip, (float*)gain_part, nrows, C)
  DISPATCH_NCH(C, CALL);
#undef CALL
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(colsum_kernel, dim3(1), dim3(64, 16), 0, (hipStream_t)stream, (const float*)gain_part, (float*)dgains,
                     grid, 4, 0);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// ---- mixer tail (round1/source/train.py:7308 mix_tail; kernels _mix_fwd_kernel :7097, _mix_bwd_kernel :7145) -----------------
// x bf16 [nrows][C] (nrows = sequences x T tokens), lam: device fp32 scalar -> s1 = bf16(x + bf16(lam shift1(x))),
// xn2 = RMSNorm(s1) (no weight), inv fp32 [nrows].
extern "C" int tfb_mix_tail_fwd(const void* x, const void* lam, void* s1, void* xn2, void* inv, long nrows, int C, int T,
                                float eps, void* stream) {
  if (!x || !lam || !s1 || !xn2 || !inv) return TFB_ERR_ARG;
  if (!norm_shape_ok(nrows, C) || T <= 0 || nrows % T) return TFB_ERR_SHAPE;
  int grid = grid_for(nrows, 8192);
#define CALL(N)                                                                                                          \
  hipLaunchKernelGGL(mix_tail_fwd_kernel<N>, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)x,            \
                     (const float*)lam, (bf16_t*)s1, (bf16_t*)xn2, (float*)inv, nrows, C, T, eps)
  DISPATCH_NCH(C, CALL);
#undef CALL
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}
// s1, inv as the forward left them; gy (gradient of xn2) and ge (gradient of s1) bf16 [nrows][C], either may be NULL (not
// both); x the forward's input -> gx bf16 [nrows][C], dlam fp32 [1] = sum over all elements of bf16(g shift1(x)) (the
// caller rounds it to lam's dtype). part: fp32 [tfb_norm_bwd_blocks(nrows)] scratch.
extern "C" int tfb_mix_tail_bwd(const void* s1, const void* gy, const void* ge, const void* inv, const void* x, const void* lam,
                                void* gx, void* part, void* dlam, long nrows, int C, int T, void* stream) {
  if (!s1 || (!gy && !ge) || !inv || !x || !lam || !gx || !part || !dlam) return TFB_ERR_ARG;
  if (!norm_shape_ok(nrows, C) || T <= 0 || nrows % T) return TFB_ERR_SHAPE;
  int grid = grid_for(nrows, 1024);
#define CALL(N)                                                                                                          \
  hipLaunchKernelGGL(mix_tail_bwd_kernel<N>, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)s1,           \
                     (const bf16_t*)gy, (const bf16_t*)ge, (const float*)inv, (const bf16_t*)x, (const float*)lam,       \
                     (bf16_t*)gx, (float*)part, nrows, C, T)
  DISPATCH_NCH(C, CALL);
#undef CALL
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(sum_partials_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, (const float*)part, grid, (float*)dlam);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

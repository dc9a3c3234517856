// Bandwidth-bound elementwise kernels: ReLU^2 family, RoPE, residual-mix backward, embedding
// gather / scatter-add, fused AdamW. All use 128-bit coalesced accesses (8 bf16 or 4 fp32 per
// lane), fp32 math and one rounding per output.
//
//   relu2 fwd / bwd / bwd-from-output      round1/source/train.py:663, 597, 633 (625-631)
//   rope (half-split rotation)             round1/source/train.py:4188-4193
//   resmix backward                        round2/source/kernels/nki_resmix.py:148-162
//   embedding                              round1/source/train.py:8407 (embedding_fwd), 8303 (backward as dW = onehot^T dY)
//   adamw                                  round1/source/train.py:9670-9677, round2/source/train.py:13756-13766
#include "common.hpp"
// the optimizer's 3.8 GB of state stream past the caches once per step (AdamW -0.02 ms, the weight refresh after it -0.03)
#ifndef TFB_NT_D
#define TFB_NT_D 1
#endif

namespace {

inline int blocks_for(long nvec, int cap = 16384) {
  long b = (nvec + 255) / 256;
  return (int)(b < cap ? (b > 0 ? b : 1) : cap);
}

// mode 0: y = relu(x)^2 ; mode 1: dx = g * 2 relu(x) ; mode 2: dx = bf16(sqrt(4 h)) * g  (a = x or h, b = g)
template <int MODE>
__global__ __launch_bounds__(256) void relu2_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ b,
                                                   bf16_t* __restrict__ out, long n) {
  for (long i = ((long)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += (long)gridDim.x * 256 * 8) {
    u32x4 ua = *(const u32x4*)(a + i);
    u32x4 ub = {0, 0, 0, 0};
    if (MODE != 0) ub = *(const u32x4*)(b + i);
    u32x4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float x0 = bflo(ua[k]), x1 = bfhi(ua[k]);
      float r0, r1;
      if (MODE == 0) {
        x0 = fmaxf(x0, 0.f);
        x1 = fmaxf(x1, 0.f);
        r0 = x0 * x0;
        r1 = x1 * x1;
      } else if (MODE == 1) {
        r0 = bflo(ub[k]) * 2.0f * fmaxf(x0, 0.f);
        r1 = bfhi(ub[k]) * 2.0f * fmaxf(x1, 0.f);
      } else {
        r0 = round_bf(sqrtf(4.0f * x0)) * bflo(ub[k]);
        r1 = round_bf(sqrtf(4.0f * x1)) * bfhi(ub[k]);
      }
      o[k] = pack2bf(r0, r1);
    }
    *(u32x4*)(out + i) = o;
  }
}

// x [rows][row_stride] holds nheads heads of D contiguous elements starting at column 0; row r is token r % T.
// y1 = x1 c + x2 s, y2 = x2 c - x1 s  (inverse: y1 = x1 c - x2 s, y2 = x2 c + x1 s). In place when out == x.
__global__ __launch_bounds__(256) void rope_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ cs,
                                                  const bf16_t* __restrict__ sn, bf16_t* __restrict__ out, long rows, int T,
                                                  int nheads, int D, long row_stride, long out_stride, int inverse) {
  const int hc = D / 16;  // 8-element chunks per half head
  const long per_row = (long)nheads * hc;
  const long total = rows * per_row;
  for (long idx = (long)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (long)gridDim.x * 256) {
    long row = idx / per_row;
    int rem = (int)(idx % per_row);
    int head = rem / hc, c = rem % hc;
    int t = (int)(row % T);
    const bf16_t* p1 = x + row * row_stride + (long)head * D + c * 8;
    u32x4 a = *(const u32x4*)p1;
    u32x4 b = *(const u32x4*)(p1 + D / 2);
    u32x4 cc = *(const u32x4*)(cs + (long)t * (D / 2) + c * 8);
    u32x4 ss = *(const u32x4*)(sn + (long)t * (D / 2) + c * 8);
    u32x4 o1, o2;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float a0 = bflo(a[k]), a1 = bfhi(a[k]), b0 = bflo(b[k]), b1 = bfhi(b[k]);
      float c0 = bflo(cc[k]), c1 = bfhi(cc[k]);
      float s0 = bflo(ss[k]), s1 = bfhi(ss[k]);
      if (inverse) {
        s0 = -s0;
        s1 = -s1;
      }
      o1[k] = pack2bf(a0 * c0 + b0 * s0, a1 * c1 + b1 * s1);
      o2[k] = pack2bf(b0 * c0 - a0 * s0, b1 * c1 - a1 * s1);
    }
    bf16_t* q1 = out + row * out_stride + (long)head * D + c * 8;
    *(u32x4*)q1 = o1;
    *(u32x4*)(q1 + D / 2) = o2;
  }
}

// RoPE followed by the parameter-free RMSNorm of each head (the attention block's QK-norm): r = bf16(rope(x)),
// inv = rsqrt(mean(r^2) + eps) over the head's D elements, y = bf16(r inv). D / 16 lanes share a head (a lane holds 8
// elements of each half); heads laid out as in rope_kernel. r_out may be NULL.
__global__ __launch_bounds__(256) void rope_norm_fwd_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ cs,
                                                           const bf16_t* __restrict__ sn, bf16_t* __restrict__ r_out,
                                                           bf16_t* __restrict__ y_out, float* __restrict__ inv_out, long rows,
                                                           int T, int nheads, int D, long x_stride, long r_stride,
                                                           long y_stride, float eps) {
  const int hc = D / 16;  // lanes per head: 4 (D = 64) or 8 (D = 128), a power of two
  const long per_row = (long)nheads * hc;
  const long total = rows * per_row;
  const long span = ((total + 63) / 64) * 64;  // whole wavefronts stay in the loop for the shuffles
  for (long idx = (long)blockIdx.x * 256 + threadIdx.x; idx < span; idx += (long)gridDim.x * 256) {
    const bool live = idx < total;
    const long id = live ? idx : total - 1;
    const long row = id / per_row;
    const int rem = (int)(id % per_row);
    const int head = rem / hc, c = rem % hc;
    const int t = (int)(row % T);
    const bf16_t* p1 = x + row * x_stride + (long)head * D + c * 8;
    const u32x4 a = *(const u32x4*)p1, b = *(const u32x4*)(p1 + D / 2);
    const u32x4 cc = *(const u32x4*)(cs + (long)t * (D / 2) + c * 8), ss = *(const u32x4*)(sn + (long)t * (D / 2) + c * 8);
    float r1[8], r2[8], sq = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float a0 = bflo(a[k]), a1 = bfhi(a[k]), b0 = bflo(b[k]), b1 = bfhi(b[k]);
      const float c0 = bflo(cc[k]), c1 = bfhi(cc[k]), s0 = bflo(ss[k]), s1 = bfhi(ss[k]);
      r1[2 * k] = round_bf(a0 * c0 + b0 * s0);
      r1[2 * k + 1] = round_bf(a1 * c1 + b1 * s1);
      r2[2 * k] = round_bf(b0 * c0 - a0 * s0);
      r2[2 * k + 1] = round_bf(b1 * c1 - a1 * s1);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) sq += r1[k] * r1[k] + r2[k] * r2[k];
    for (int o = 1; o < hc; o <<= 1) sq += __shfl_xor(sq, o, 64);
    const float inv = rsqrtf(sq / (float)D + eps);
    if (!live) continue;
    if (r_out) {
      bf16_t* q = r_out + row * r_stride + (long)head * D + c * 8;
      *(u32x4*)q = pack8bf(r1);
      *(u32x4*)(q + D / 2) = pack8bf(r2);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      r1[k] *= inv;
      r2[k] *= inv;
    }
    bf16_t* q = y_out + row * y_stride + (long)head * D + c * 8;
    *(u32x4*)q = pack8bf(r1);
    *(u32x4*)(q + D / 2) = pack8bf(r2);
    if (c == 0) inv_out[row * nheads + head] = inv;
  }
}

// Gradient of rope_norm_fwd: rh = r inv, dr = bf16(inv (g - rh (g . rh) / D)), then the transposed rotation
// dx1 = dr1 c - dr2 s, dx2 = dr2 c + dr1 s, one rounding.
__global__ __launch_bounds__(256) void rope_norm_bwd_kernel(const bf16_t* __restrict__ g, const bf16_t* __restrict__ r,
                                                           const float* __restrict__ inv_in, const bf16_t* __restrict__ cs,
                                                           const bf16_t* __restrict__ sn, bf16_t* __restrict__ dx, long rows,
                                                           int T, int nheads, int D, long g_stride, long r_stride,
                                                           long dx_stride) {
  const int hc = D / 16;
  const long per_row = (long)nheads * hc;
  const long total = rows * per_row;
  const long span = ((total + 63) / 64) * 64;
  for (long idx = (long)blockIdx.x * 256 + threadIdx.x; idx < span; idx += (long)gridDim.x * 256) {
    const bool live = idx < total;
    const long id = live ? idx : total - 1;
    const long row = id / per_row;
    const int rem = (int)(id % per_row);
    const int head = rem / hc, c = rem % hc;
    const int t = (int)(row % T);
    const long off = (long)head * D + c * 8;
    const u32x4 ga = *(const u32x4*)(g + row * g_stride + off), gb = *(const u32x4*)(g + row * g_stride + off + D / 2);
    const u32x4 ra = *(const u32x4*)(r + row * r_stride + off), rb = *(const u32x4*)(r + row * r_stride + off + D / 2);
    const float inv = inv_in[row * nheads + head];
    float g1[8], g2[8], h1[8], h2[8], dot = 0.f;
    unpack8bf(ga, g1);
    unpack8bf(gb, g2);
    unpack8bf(ra, h1);
    unpack8bf(rb, h2);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      h1[k] *= inv;
      h2[k] *= inv;
      dot += g1[k] * h1[k] + g2[k] * h2[k];
    }
    for (int o = 1; o < hc; o <<= 1) dot += __shfl_xor(dot, o, 64);
    if (!live) continue;
    const float coef = dot / (float)D;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      g1[k] = round_bf(inv * (g1[k] - h1[k] * coef));
      g2[k] = round_bf(inv * (g2[k] - h2[k] * coef));
    }
    const u32x4 cc = *(const u32x4*)(cs + (long)t * (D / 2) + c * 8), ss = *(const u32x4*)(sn + (long)t * (D / 2) + c * 8);
    float cf[8], sf[8], o1[8], o2[8];
    unpack8bf(cc, cf);
    unpack8bf(ss, sf);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      o1[k] = g1[k] * cf[k] - g2[k] * sf[k];
      o2[k] = g2[k] * cf[k] + g1[k] * sf[k];
    }
    bf16_t* q = dx + row * dx_stride + off;
    *(u32x4*)q = pack8bf(o1);
    *(u32x4*)(q + D / 2) = pack8bf(o2);
  }
}

// dx = g * bf16(a), dx0 = g * bf16(b) (products rounded to bf16), partial sums of bf16(g x) and bf16(g x0) in fp32.
__global__ __launch_bounds__(256) void resmix_bwd_kernel(const bf16_t* __restrict__ g, const bf16_t* __restrict__ x,
                                                        const bf16_t* __restrict__ x0, const float* __restrict__ ab,
                                                        bf16_t* __restrict__ dx, bf16_t* __restrict__ dx0,
                                                        float* __restrict__ part, long n) {
  __shared__ float red[2][4];
  const float a = round_bf(ab[0]), b = round_bf(ab[1]);
  float sa = 0.f, sb = 0.f;
  for (long i = ((long)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += (long)gridDim.x * 256 * 8) {
    u32x4 ug = *(const u32x4*)(g + i), ux = *(const u32x4*)(x + i), u0 = *(const u32x4*)(x0 + i);
    u32x4 o1, o2;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float g0 = bflo(ug[k]), g1 = bfhi(ug[k]);
      o1[k] = pack2bf(g0 * a, g1 * a);
      o2[k] = pack2bf(g0 * b, g1 * b);
      sa += round_bf(g0 * bflo(ux[k])) + round_bf(g1 * bfhi(ux[k]));
      sb += round_bf(g0 * bflo(u0[k])) + round_bf(g1 * bfhi(u0[k]));
    }
    *(u32x4*)(dx + i) = o1;
    *(u32x4*)(dx0 + i) = o2;
  }
  sa = wave_sum(sa);
  sb = wave_sum(sb);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    red[0][wave] = sa;
    red[1][wave] = sb;
  }
  __syncthreads();
  if (threadIdx.x < 2) part[(long)blockIdx.x * 2 + threadIdx.x] = red[threadIdx.x][0] + red[threadIdx.x][1] + red[threadIdx.x][2] + red[threadIdx.x][3];
}

__global__ void sum_pairs_kernel(const float* __restrict__ part, int nblocks, float* __restrict__ out) {
  __shared__ float red[2][4];
  float s0 = 0.f, s1 = 0.f;
  for (int i = threadIdx.x; i < nblocks; i += 256) {
    s0 += part[2 * i];
    s1 += part[2 * i + 1];
  }
  s0 = wave_sum(s0);
  s1 = wave_sum(s1);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    red[0][wave] = s0;
    red[1][wave] = s1;
  }
  __syncthreads();
  if (threadIdx.x < 2) out[threadIdx.x] = red[threadIdx.x][0] + red[threadIdx.x][1] + red[threadIdx.x][2] + red[threadIdx.x][3];
}

template <typename IDX>
__global__ __launch_bounds__(256) void embedding_fwd_kernel(const IDX* __restrict__ idx, const bf16_t* __restrict__ w,
                                                           bf16_t* __restrict__ out, long n, int C, int V) {
  const int cpr = C / 8;
  const long total = n * cpr;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    long row = i / cpr;
    int c = (int)(i % cpr) * 8;
    long tok = (long)idx[row];
    // an id outside [0, V) never becomes an address: its row is zeros (and takes no gradient in the backward)
    u32x4 val = {0u, 0u, 0u, 0u};
    if ((unsigned long)tok < (unsigned long)V) val = *(const u32x4*)(w + tok * C + c);
    *(u32x4*)(out + row * C + c) = val;
  }
}

// dW[idx[row]] += dY[row] in fp32 with atomics (dW fp32, zeroed or accumulated into by the caller).
template <typename IDX>
__global__ __launch_bounds__(256) void embedding_bwd_kernel(const IDX* __restrict__ idx, const bf16_t* __restrict__ dy,
                                                           float* __restrict__ dw, long n, int C, int V) {
  const int cpr = C / 8;
  const long total = n * cpr;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    long row = i / cpr;
    int c = (int)(i % cpr) * 8;
    long tok = (long)idx[row];
    if ((unsigned long)tok >= (unsigned long)V) continue;  // out-of-range id: no gradient row
    u32x4 u = *(const u32x4*)(dy + row * C + c);
    float* d = dw + tok * C + c;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      atomicAdd(d + 2 * k, bflo(u[k]));
      atomicAdd(d + 2 * k + 1, bfhi(u[k]));
    }
  }
}

// ---- embedding backward without contended atomics: rows grouped by token (counting sort), then a segmented sum.
__global__ __launch_bounds__(256) void emb_zero_kernel(int* __restrict__ p, long n) {
  long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0;
}
template <typename IDX>
__device__ __forceinline__ int emb_bucket(IDX t, int V) {
  // ids outside [0, V) share the extra bucket V, which the sum skips
  return (unsigned long)(long)t < (unsigned long)V ? (int)t : V;
}
template <typename IDX>
__global__ __launch_bounds__(256) void emb_count_kernel(const IDX* __restrict__ idx, int* __restrict__ count, long n, int V) {
  long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) atomicAdd(count + emb_bucket(idx[i], V), 1);
}
// One workgroup: cursor[v] = exclusive prefix sum of count[v] (count is left untouched).
__global__ __launch_bounds__(1024) void emb_scan_kernel(const int* __restrict__ count, int* __restrict__ cursor, int V) {
  __shared__ int wsum[16];
  __shared__ int carry;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int base = 0; base < V; base += 1024) {
    const int v = base + tid;
    const int c = v < V ? count[v] : 0;
    int x = c;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      int y = __shfl_up(x, o, 64);
      if (lane >= o) x += y;
    }
    if (lane == 63) wsum[wave] = x;
    __syncthreads();
    int before = carry;
    for (int w = 0; w < wave; ++w) before += wsum[w];
    if (v < V) cursor[v] = before + x - c;
    __syncthreads();
    if (tid == 1023) carry = before + x;
    __syncthreads();
  }
}
template <typename IDX>
__global__ __launch_bounds__(256) void emb_place_kernel(const IDX* __restrict__ idx, int* __restrict__ cursor,
                                                       int* __restrict__ order, long n, int V) {
  long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) order[atomicAdd(cursor + emb_bucket(idx[i], V), 1)] = (int)i;
}
// The counting sort without contended global atomics, for a vocabulary whose counters fit a CU's LDS: a workgroup counts
// its EMB_TOK tokens in an LDS histogram (each token gets its rank among the workgroup's equal ones from the LDS atomic),
// then ONE thread per distinct token adds the workgroup's count to the global counter and the returned value places the
// workgroup's run inside the token's: rank[i] = position of row i among all rows of its token. A hot token of a Zipf batch
// then costs one global atomic per workgroup, not one per occurrence (the per-row atomics took 66 us each way at 32768 rows).
constexpr int EMB_TOK = 512;  // tokens per workgroup (two per thread)
template <typename IDX>
__global__ __launch_bounds__(256) void emb_rank_kernel(const IDX* __restrict__ idx, int* __restrict__ count,
                                                      int* __restrict__ rank, long n, int V) {
  extern __shared__ int hist[];  // V + 1 counters
  for (int i = threadIdx.x; i <= V; i += 256) hist[i] = 0;
  __syncthreads();
  const long base = (long)blockIdx.x * EMB_TOK;
  int tok[2], lr[2];
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const long i = base + k * 256 + threadIdx.x;
    tok[k] = -1;
    if (i < n) {
      tok[k] = emb_bucket(idx[i], V);
      lr[k] = atomicAdd(hist + tok[k], 1);
    }
  }
  __syncthreads();
  int mine[2];
#pragma unroll
  for (int k = 0; k < 2; ++k) mine[k] = tok[k] >= 0 && lr[k] == 0 ? hist[tok[k]] : 0;  // the first arrival speaks for its token
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 2; ++k)
    if (mine[k] > 0) hist[tok[k]] = atomicAdd(count + tok[k], mine[k]);
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const long i = base + k * 256 + threadIdx.x;
    if (i < n) rank[i] = hist[tok[k]] + lr[k];
  }
}
// Exclusive prefix sum of count[0 .. V) into cursor, one workgroup per tile of 1024 counters and no dependency between
// workgroups: each first adds up everything before its tile (at most 128 KB, loads eight tiles at a time), then scans its own.
__global__ __launch_bounds__(1024) void emb_scan_tiles_kernel(const int* __restrict__ count, int* __restrict__ cursor, int V) {
  __shared__ int wsum[16];
  __shared__ int wtot[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lo = blockIdx.x * 1024;
  int s = 0;
  for (int base = 0; base < lo; base += 8 * 1024) {
    int v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = base + j * 1024 + tid;
      v[j] = i < lo ? count[i] : 0;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) s += v[j];
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
  const int i = lo + tid;
  const int c = i < V ? count[i] : 0;
  int x = c;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    int y = __shfl_up(x, o, 64);
    if (lane >= o) x += y;
  }
  if (lane == 63) wsum[wave] = x;
  if (lane == 0) wtot[wave] = s;
  __syncthreads();
  int before = 0;
  for (int w = 0; w < 16; ++w) before += wtot[w];
  for (int w = 0; w < wave; ++w) before += wsum[w];
  if (i < V) cursor[i] = before + x - c;
}
template <typename IDX>
__global__ __launch_bounds__(256) void emb_scatter_kernel(const IDX* __restrict__ idx, const int* __restrict__ cursor,
                                                         const int* __restrict__ rank, int* __restrict__ order, long n, int V) {
  long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) order[cursor[emb_bucket(idx[i], V)] + rank[i]] = (int)i;
}

// A workgroup sums EMB_SEG consecutive rows of the token-grouped order, thread t owning columns 8t .. 8t+7. A run of
// equal tokens that lies inside the segment has a single owner and is added with plain loads/stores; the first and the
// last run may continue in the neighbouring segments and use atomics.
#ifndef TFB_EMB_SEG
#define TFB_EMB_SEG 32
#endif
constexpr int EMB_SEG = TFB_EMB_SEG;
template <typename IDX>
__global__ __launch_bounds__(128) void emb_reduce_kernel(const IDX* __restrict__ idx, const int* __restrict__ order,
                                                        const bf16_t* __restrict__ dy, float* __restrict__ dw, long n, int C,
                                                        int V) {
  __shared__ int rows[EMB_SEG];
  __shared__ int toks[EMB_SEG];
  __shared__ int edge[2];  // the tokens of the rows just before and just after this segment (-1: none)
  const long pos0 = (long)blockIdx.x * EMB_SEG;
  const int cnt = (int)min((long)EMB_SEG, n - pos0);
  if (threadIdx.x < cnt) {
    const int r = order[pos0 + threadIdx.x];
    rows[threadIdx.x] = r;
    toks[threadIdx.x] = emb_bucket(idx[r], V);
  } else if (threadIdx.x == EMB_SEG) {
    edge[0] = pos0 > 0 ? emb_bucket(idx[order[pos0 - 1]], V) : -1;
  } else if (threadIdx.x == EMB_SEG + 1) {
    edge[1] = pos0 + cnt < n ? emb_bucket(idx[order[pos0 + cnt]], V) : -1;
  }
  __syncthreads();
  const int c = (blockIdx.y * 128 + threadIdx.x) * 8;
  if (c >= C) return;
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  int run_start = 0;
  for (int i = 0; i < cnt; ++i) {
    u32x4 u = *(const u32x4*)(dy + (long)rows[i] * C + c);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      acc[2 * k] += bflo(u[k]);
      acc[2 * k + 1] += bfhi(u[k]);
    }
    if (i + 1 == cnt || toks[i + 1] != toks[i]) {
      float* d = dw + (long)toks[i] * C + c;
      if (toks[i] == V) {
        // the bucket of out-of-range ids: dropped
      } else if ((run_start == 0 && edge[0] == toks[i]) || (i + 1 == cnt && edge[1] == toks[i])) {
        // the token's run goes on in a neighbouring segment: another workgroup adds to the same row
#pragma unroll
        for (int k = 0; k < 8; ++k) atomicAdd(d + k, acc[k]);
      } else {
        f32x4 a0 = *(const f32x4*)d, a1 = *(const f32x4*)(d + 4);
        *(f32x4*)d = f32x4{a0[0] + acc[0], a0[1] + acc[1], a0[2] + acc[2], a0[3] + acc[3]};
        *(f32x4*)(d + 4) = f32x4{a1[0] + acc[4], a1[1] + acc[5], a1[2] + acc[6], a1[3] + acc[7]};
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) acc[k] = 0.f;
      run_start = i + 1;
    }
  }
}

struct AdamScalars {
  float lr, wd, omb1, omb2, eps, bias1, bias2;
};

__device__ __forceinline__ float lerp_torch(float a, float b, float w) {
  // torch.lerp: a + w (b - a) for w < 0.5, else b - (b - a)(1 - w)
  float d = b - a;
  return w < 0.5f ? fmaf(w, d, a) : fmaf(-d, 1.0f - w, b);  // torch's lerp contracts to one fma
}

__device__ __forceinline__ void adamw_one(float& pk, float& mk, float& vk, float gk, const AdamScalars& s) {
  if (s.wd > 0.f) pk = pk * (1.0f - s.lr * s.wd);
  mk = lerp_torch(mk, gk, s.omb1);
  vk = lerp_torch(vk, gk * gk, s.omb2);
  const float upd = mk / s.bias1 / (sqrtf(vk / s.bias2) + s.eps);
  pk = pk - upd * s.lr;
}

// p (fp32 master) updated in place; optional bf16 copy written; g is fp32 (GF32) or bf16. Groups of four elements
// take 128-bit accesses; the last n % 4 elements (one-element gains, odd-sized vectors) are finished one by one.
template <bool GF32>
__global__ __launch_bounds__(256) void adamw_kernel(float* __restrict__ p, const void* __restrict__ g, float* __restrict__ m,
                                                   float* __restrict__ v, bf16_t* __restrict__ p16, long n, AdamScalars s) {
  const long n4 = n & ~3L;
  const long step = (long)gridDim.x * 256 * 4;
  long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
  // the next group's four loads go out before this group's stores: a wait for loaded data also waits for every older
  // store (one counter orders both), so loading after the stores would cost a store round trip per group
  f32x4 pp, mm, vv, gg;
  u32x2 gb;
  auto fetch = [&](long j) {
    pp = tfb_load_nt((const f32x4*)(p + j), TFB_NT_D);
    mm = tfb_load_nt((const f32x4*)(m + j), TFB_NT_D);
    vv = tfb_load_nt((const f32x4*)(v + j), TFB_NT_D);
    if (GF32) gg = tfb_load_nt((const f32x4*)((const float*)g + j), TFB_NT_D);
    else gb = tfb_load_nt((const u32x2*)((const bf16_t*)g + j), TFB_NT_D);
  };
  if (i < n4) fetch(i);
  for (; i < n4; i += step) {
    f32x4 cp = pp, cm = mm, cv = vv, cg;
    if (GF32) cg = gg;
    else cg = f32x4{bflo(gb.x), bfhi(gb.x), bflo(gb.y), bfhi(gb.y)};
    if (i + step < n4) fetch(i + step);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float pk = cp[k], mk = cm[k], vk = cv[k];
      adamw_one(pk, mk, vk, cg[k], s);
      cp[k] = pk;
      cm[k] = mk;
      cv[k] = vk;
    }
    tfb_store_nt((f32x4*)(p + i), cp, TFB_NT_D);
    tfb_store_nt((f32x4*)(m + i), cm, TFB_NT_D);
    tfb_store_nt((f32x4*)(v + i), cv, TFB_NT_D);
    if (p16) {
      u32x2 o = {pack2bf(cp[0], cp[1]), pack2bf(cp[2], cp[3])};
      *(u32x2*)(p16 + i) = o;
    }
  }
  if (blockIdx.x == 0 && threadIdx.x < (int)(n - n4)) {
    const long i = n4 + threadIdx.x;
    float pk = p[i], mk = m[i], vk = v[i];
    const float gk = GF32 ? ((const float*)g)[i] : bf2f(((const bf16_t*)g)[i]);
    adamw_one(pk, mk, vk, gk, s);
    p[i] = pk;
    m[i] = mk;
    v[i] = vk;
    if (p16) p16[i] = f2bf(pk);
  }
}

__global__ __launch_bounds__(256) void fill_f32_kernel(float* __restrict__ p, float val, long n) {
  for (long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4; i < n; i += (long)gridDim.x * 256 * 4) {
    if (i + 3 < n) {
      *(f32x4*)(p + i) = f32x4{val, val, val, val};
    } else {
      for (long j = i; j < n; ++j) p[j] = val;
    }
  }
}

}  // namespace

extern "C" int tfb_relu2(const void* a, const void* b, void* out, long n, int mode, void* stream) {
  if (!a || !out || (mode != 0 && !b)) return TFB_ERR_ARG;
  if (n <= 0 || n % 8) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  int nb = blocks_for(n / 8);
  if (mode == 0) hipLaunchKernelGGL(relu2_kernel<0>, dim3(nb), dim3(256), 0, s, (const bf16_t*)a, (const bf16_t*)b, (bf16_t*)out, n);
  else if (mode == 1) hipLaunchKernelGGL(relu2_kernel<1>, dim3(nb), dim3(256), 0, s, (const bf16_t*)a, (const bf16_t*)b, (bf16_t*)out, n);
  else if (mode == 2) hipLaunchKernelGGL(relu2_kernel<2>, dim3(nb), dim3(256), 0, s, (const bf16_t*)a, (const bf16_t*)b, (bf16_t*)out, n);
  else return TFB_ERR_ARG;
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

extern "C" int tfb_rope(const void* x, const void* cos_t, const void* sin_t, void* out, long rows, int T, int nheads, int D,
                        long row_stride, long out_stride, int inverse, void* stream) {
  if (!x || !cos_t || !sin_t || !out) return TFB_ERR_ARG;
  if (rows <= 0 || T <= 0 || nheads <= 0 || D <= 0 || D % 16 || row_stride % 8 || out_stride % 8) return TFB_ERR_SHAPE;
  long total = rows * nheads * (D / 16);
  hipLaunchKernelGGL(rope_kernel, dim3(blocks_for(total)), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)x,
                     (const bf16_t*)cos_t, (const bf16_t*)sin_t, (bf16_t*)out, rows, T, nheads, D, row_stride, out_stride, inverse);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// x [rows][x_stride] holds nheads heads of D elements from column 0 (row = token, row % T its position): y = the
// RMS-normalised rotation, r (NULL to skip) the rotation before the norm, inv fp32 [rows][nheads]. D = 64 or 128.
extern "C" int tfb_rope_norm_fwd(const void* x, const void* cos_t, const void* sin_t, void* r, void* y, void* inv, long rows, int T,
                                 int nheads, int D, long x_stride, long r_stride, long y_stride, float eps, void* stream) {
  if (!x || !cos_t || !sin_t || !y || !inv) return TFB_ERR_ARG;
  if (rows <= 0 || T <= 0 || nheads <= 0 || (D != 64 && D != 128) || x_stride % 8 || r_stride % 8 || y_stride % 8)
    return TFB_ERR_SHAPE;
  const long total = rows * nheads * (D / 16);
  hipLaunchKernelGGL(rope_norm_fwd_kernel, dim3(blocks_for(total)), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)x,
                     (const bf16_t*)cos_t, (const bf16_t*)sin_t, (bf16_t*)r, (bf16_t*)y, (float*)inv, rows, T, nheads, D,
                     x_stride, r_stride, y_stride, eps);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// dx = gradient of tfb_rope_norm_fwd's input from g = gradient of y, the saved r and inv. dx may alias g.
extern "C" int tfb_rope_norm_bwd(const void* g, const void* r, const void* inv, const void* cos_t, const void* sin_t, void* dx,
                                 long rows, int T, int nheads, int D, long g_stride, long r_stride, long dx_stride,
                                 void* stream) {
  if (!g || !r || !inv || !cos_t || !sin_t || !dx) return TFB_ERR_ARG;
  if (rows <= 0 || T <= 0 || nheads <= 0 || (D != 64 && D != 128) || g_stride % 8 || r_stride % 8 || dx_stride % 8)
    return TFB_ERR_SHAPE;
  const long total = rows * nheads * (D / 16);
  hipLaunchKernelGGL(rope_norm_bwd_kernel, dim3(blocks_for(total)), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)g,
                     (const bf16_t*)r, (const float*)inv, (const bf16_t*)cos_t, (const bf16_t*)sin_t, (bf16_t*)dx, rows, T,
                     nheads, D, g_stride, r_stride, dx_stride);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

extern "C" int tfb_resmix_bwd_blocks(long n) { return blocks_for(n / 8, 1024); }

// ab: device fp32 [2] gains; part: fp32 [2 * tfb_resmix_bwd_blocks(n)] scratch; dab: fp32 [2] = (sum g x, sum g x0)
extern "C" int tfb_resmix_bwd(const void* g, const void* x, const void* x0, const void* ab, void* dx, void* dx0, void* part,
                              void* dab, long n, void* stream) {
  if (!g || !x || !x0 || !ab || !dx || !dx0 || !part || !dab) return TFB_ERR_ARG;
  if (n <= 0 || n % 8) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  int nb = blocks_for(n / 8, 1024);
  hipLaunchKernelGGL(resmix_bwd_kernel, dim3(nb), dim3(256), 0, s, (const bf16_t*)g, (const bf16_t*)x, (const bf16_t*)x0,
                     (const float*)ab, (bf16_t*)dx, (bf16_t*)dx0, (float*)part, n);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(sum_pairs_kernel, dim3(1), dim3(256), 0, s, (const float*)part, nb, (float*)dab);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

extern "C" int tfb_embedding_fwd(const void* idx, int idx64, const void* w, void* out, long n, int C, int V, void* stream) {
  if (!idx || !w || !out) return TFB_ERR_ARG;
  if (n <= 0 || C <= 0 || C % 8 || V <= 0) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  int nb = blocks_for(n * (C / 8));
  if (idx64) hipLaunchKernelGGL(embedding_fwd_kernel<long>, dim3(nb), dim3(256), 0, s, (const long*)idx, (const bf16_t*)w, (bf16_t*)out, n, C, V);
  else hipLaunchKernelGGL(embedding_fwd_kernel<int>, dim3(nb), dim3(256), 0, s, (const int*)idx, (const bf16_t*)w, (bf16_t*)out, n, C, V);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

extern "C" int tfb_embedding_bwd(const void* idx, int idx64, const void* dy, void* dw_f32, long n, int C, int V, void* stream) {
  if (!idx || !dy || !dw_f32) return TFB_ERR_ARG;
  if (n <= 0 || C <= 0 || C % 8 || V <= 0) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  int nb = blocks_for(n * (C / 8));
  if (idx64) hipLaunchKernelGGL(embedding_bwd_kernel<long>, dim3(nb), dim3(256), 0, s, (const long*)idx, (const bf16_t*)dy, (float*)dw_f32, n, C, V);
  else hipLaunchKernelGGL(embedding_bwd_kernel<int>, dim3(nb), dim3(256), 0, s, (const int*)idx, (const bf16_t*)dy, (float*)dw_f32, n, C, V);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// Scratch (int32 elements) of tfb_embedding_bwd_grouped.
extern "C" long tfb_embedding_bwd_scratch_ints(long n, int V) { return 2L * (V + 1) + 2 * n; }

// The same sum as tfb_embedding_bwd, rows grouped by token first: hot tokens (a Zipf batch) no longer serialize on atomics.
extern "C" int tfb_embedding_bwd_grouped(const void* idx, int idx64, const void* dy, void* dw_f32, long n, int C, int V,
                                         void* scratch, void* stream) {
  if (!idx || !dy || !dw_f32 || !scratch) return TFB_ERR_ARG;
  if (n <= 0 || n > 0x7fffffffL || C <= 0 || C % 8 || V <= 0) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  int* count = (int*)scratch;
  int* cursor = count + (V + 1);  // bucket V collects the ids outside [0, V)
  int* order = cursor + (V + 1);
  int* rank = order + n;
  const unsigned nb = (unsigned)((n + 255) / 256);
  hipLaunchKernelGGL(emb_zero_kernel, dim3((unsigned)((V + 256) / 256)), dim3(256), 0, s, count, (long)V + 1);
  const size_t hist_bytes = ((size_t)V + 1) * 4;
  if (hist_bytes <= 144 * 1024) {
    // the counters of the whole vocabulary fit a CU's LDS: workgroup-level counting, no atomics in the placement
    const unsigned nw = (unsigned)((n + EMB_TOK - 1) / EMB_TOK);
    const void* fn = idx64 ? (const void*)emb_rank_kernel<long> : (const void*)emb_rank_kernel<int>;
    if (hist_bytes > 48 * 1024 &&
        hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)hist_bytes) != hipSuccess)
      return TFB_ERR_LAUNCH;
    if (idx64) hipLaunchKernelGGL(emb_rank_kernel<long>, dim3(nw), dim3(256), hist_bytes, s, (const long*)idx, count, rank, n, V);
    else hipLaunchKernelGGL(emb_rank_kernel<int>, dim3(nw), dim3(256), hist_bytes, s, (const int*)idx, count, rank, n, V);
    hipLaunchKernelGGL(emb_scan_tiles_kernel, dim3((unsigned)((V + 1 + 1023) / 1024)), dim3(1024), 0, s, count, cursor, V + 1);
    if (idx64) hipLaunchKernelGGL(emb_scatter_kernel<long>, dim3(nb), dim3(256), 0, s, (const long*)idx, cursor, rank, order, n, V);
    else hipLaunchKernelGGL(emb_scatter_kernel<int>, dim3(nb), dim3(256), 0, s, (const int*)idx, cursor, rank, order, n, V);
  } else {
    if (idx64) hipLaunchKernelGGL(emb_count_kernel<long>, dim3(nb), dim3(256), 0, s, (const long*)idx, count, n, V);
    else hipLaunchKernelGGL(emb_count_kernel<int>, dim3(nb), dim3(256), 0, s, (const int*)idx, count, n, V);
    hipLaunchKernelGGL(emb_scan_kernel, dim3(1), dim3(1024), 0, s, count, cursor, V + 1);
    if (idx64) hipLaunchKernelGGL(emb_place_kernel<long>, dim3(nb), dim3(256), 0, s, (const long*)idx, cursor, order, n, V);
    else hipLaunchKernelGGL(emb_place_kernel<int>, dim3(nb), dim3(256), 0, s, (const int*)idx, cursor, order, n, V);
  }
  dim3 grid((unsigned)((n + EMB_SEG - 1) / EMB_SEG), (unsigned)((C / 8 + 127) / 128));
  if (idx64) hipLaunchKernelGGL(emb_reduce_kernel<long>, grid, dim3(128), 0, s, (const long*)idx, order, (const bf16_t*)dy, (float*)dw_f32, n, C, V);
  else hipLaunchKernelGGL(emb_reduce_kernel<int>, grid, dim3(128), 0, s, (const int*)idx, order, (const bf16_t*)dy, (float*)dw_f32, n, C, V);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// One AdamW update over n elements: p fp32 master in place, m / v fp32 in place, optional bf16 copy of p.
extern "C" int tfb_adamw(void* p, const void* g, int g_f32, void* m, void* v, void* p_bf16, long n, float lr, float wd,
                         float one_minus_beta1, float one_minus_beta2, float eps, float bias1, float bias2, void* stream) {
  if (!p || !g || !m || !v) return TFB_ERR_ARG;
  if (n <= 0) return TFB_ERR_SHAPE;
  // the groups of four are 128-bit accesses (64-bit for bf16 tensors)
  if ((((uintptr_t)p | (uintptr_t)m | (uintptr_t)v) & 15) || ((uintptr_t)g & (g_f32 ? 15 : 7)) || ((uintptr_t)p_bf16 & 7))
    return TFB_ERR_ARG;
  AdamScalars sc{lr, wd, one_minus_beta1, one_minus_beta2, eps, bias1, bias2};
  hipStream_t s = (hipStream_t)stream;
  int nb = blocks_for((n + 3) / 4);
  if (g_f32) hipLaunchKernelGGL(adamw_kernel<true>, dim3(nb), dim3(256), 0, s, (float*)p, g, (float*)m, (float*)v, (bf16_t*)p_bf16, n, sc);
  else hipLaunchKernelGGL(adamw_kernel<false>, dim3(nb), dim3(256), 0, s, (float*)p, g, (float*)m, (float*)v, (bf16_t*)p_bf16, n, sc);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// A fill kernel in place of hipMemsetAsync (safe to record into a HIP graph).
extern "C" int tfb_fill_f32(void* p, float val, long n, void* stream) {
  if (!p) return TFB_ERR_ARG;
  if (n <= 0) return TFB_ERR_SHAPE;
  hipLaunchKernelGGL(fill_f32_kernel, dim3(blocks_for((n + 3) / 4)), dim3(256), 0, (hipStream_t)stream, (float*)p, val, n);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// ---- gradient norm -------------------------------------------------------------------------------------------------
// The sums of squares of the step's gradient buffers (a bf16 one: the matrices' flat gradient; an fp32 one: embedding and
// norm weights) in one pass, and from them the global norm and the clipping factor, all left on the device.
// Replaces _gradnorm_kernel (round1/source/train.py:1480) and the norm / gate arithmetic of reduce_fused (:1634-1720):
// gnorm = sqrt(sum of squares), scale = min(clip / (gnorm + 1e-6), 1) for clip > 0, else 1.
namespace {
constexpr int GN_BLOCKS = 1024;
__global__ __launch_bounds__(256) void gradnorm_partial_kernel(const bf16_t* __restrict__ gb, long nb, const float* __restrict__ gf,
                                                              long nf, float* __restrict__ part) {
  __shared__ float red[2][4];
  float sb = 0.f, sf = 0.f;
  const long t = (long)blockIdx.x * 256 + threadIdx.x, stride = (long)gridDim.x * 256;
  const long nb8 = nb / 8, nf4 = nf / 4;
  for (long i = t; i < nb8; i += stride) {
    const u32x4 u = __builtin_nontemporal_load((const u32x4*)gb + i);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float a = bflo(u[k]), b = bfhi(u[k]);
      sb += a * a;
      sb += b * b;
    }
  }
  for (long i = nb8 * 8 + t; i < nb; i += stride) sb += bf2f(gb[i]) * bf2f(gb[i]);
  for (long i = t; i < nf4; i += stride) {
    const f32x4 v = __builtin_nontemporal_load((const f32x4*)gf + i);
    sf += v[0] * v[0];
    sf += v[1] * v[1];
    sf += v[2] * v[2];
    sf += v[3] * v[3];
  }
  for (long i = nf4 * 4 + t; i < nf; i += stride) sf += gf[i] * gf[i];
  sb = wave_sum(sb);
  sf = wave_sum(sf);
  if ((threadIdx.x & 63) == 0) {
    red[0][threadIdx.x >> 6] = sb;
    red[1][threadIdx.x >> 6] = sf;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    part[2 * blockIdx.x] = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
    part[2 * blockIdx.x + 1] = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
  }
}
// out[0], out[1] = the two sums (partials added in a fixed order), out[2] = gnorm, out[3] = the clipping factor
__global__ __launch_bounds__(256) void gradnorm_finish_kernel(const float* __restrict__ part, int blocks, float clip,
                                                             float* __restrict__ out) {
  __shared__ float red[2][4];
  float sb = 0.f, sf = 0.f;
  for (int i = threadIdx.x; i < blocks; i += 256) {
    sb += part[2 * i];
    sf += part[2 * i + 1];
  }
  sb = wave_sum(sb);
  sf = wave_sum(sf);
  if ((threadIdx.x & 63) == 0) {
    red[0][threadIdx.x >> 6] = sb;
    red[1][threadIdx.x >> 6] = sf;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    const float a = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
    const float b = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
    const float gn = sqrtf(a + b);
    out[0] = a;
    out[1] = b;
    out[2] = gn;
    out[3] = clip > 0.f ? fminf(clip / (gn + 1e-6f), 1.0f) : 1.0f;
  }
}
}  // namespace

extern "C" long tfb_gradnorm_scratch_floats(void) { return 2L * GN_BLOCKS; }

// g_bf16 [n_bf16] (may be NULL with n 0), g_f32 [n_f32] (likewise), both 16-byte aligned; scratch fp32
// [tfb_gradnorm_scratch_floats()]; out fp32 [4] = (sum of squares of g_bf16, of g_f32, the norm of both together,
// min(clip / (norm + 1e-6), 1) or 1 when clip <= 0). Two launches, deterministic.
extern "C" int tfb_gradnorm(const void* g_bf16, long n_bf16, const void* g_f32, long n_f32, float clip, void* scratch, void* out,
                            void* stream) {
  if (!scratch || !out || (n_bf16 > 0 && !g_bf16) || (n_f32 > 0 && !g_f32)) return TFB_ERR_ARG;
  if (n_bf16 < 0 || n_f32 < 0 || n_bf16 + n_f32 <= 0) return TFB_ERR_SHAPE;
  if (((uintptr_t)g_bf16 | (uintptr_t)g_f32) & 15) return TFB_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const long work = n_bf16 / 8 + n_f32 / 4;
  int blocks = (int)((work + 255) / 256);
  blocks = blocks < 1 ? 1 : (blocks > GN_BLOCKS ? GN_BLOCKS : blocks);
  hipLaunchKernelGGL(gradnorm_partial_kernel, dim3(blocks), dim3(256), 0, s, (const bf16_t*)g_bf16, n_bf16, (const float*)g_f32,
                     n_f32, (float*)scratch);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(gradnorm_finish_kernel, dim3(1), dim3(256), 0, s, (const float*)scratch, blocks, clip, (float*)out);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// Loss head: softcap + log-softmax + cross-entropy on bf16 logits, and the LM-head GEMM with the
// log-sum-exp fused into its epilogue.
//
// Replaces _loss_fwd_kernel / _loss_bwd_kernel behind fused_loss(logits, targets, reduction, softcap)
// (round1/source/train.py:4543, 4584, 4691; eager form 4481-4495), the row-weighted form of
// round2/source/train.py:6364-6391 (ignore_index -1 = weight 0), and the lm_head matmul in front of
// them (round1/source/train.py:8668, 9191-9212).
//
// Math per row, fp32 from the bf16-rounded logits x: s_v = c tanh(x_v / c) (or s_v = x_v without a
// softcap), lse = log sum_v exp(s_v), loss = lse - s_target; d x_v = g (softmax_v - [v = target])
// (1 - tanh^2). Only lse is saved; the backward recomputes tanh / exp.
//
// lmhead_fwd is the GEMM logits = x @ W^T (W [V, d]) whose epilogue rounds each accumulator to bf16,
// stores it, and reduces exp(s - shift) over the 64 vocabulary columns a wavefront holds for each row
// (in registers: a lane owns 32 of them, its partner lane the rest) into a [rows][V/64] table of
// (max, sum) pairs; a finishing kernel merges a row's pairs, reads the target logit and writes lse and
// the row loss. The logits make one trip to HBM (written once, read once by the backward).
#include "gemm_core.hpp"

namespace {

__device__ __forceinline__ float fexp(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }

// c * tanh(x / c) and tanh(x / c)
__device__ __forceinline__ float tanh_fast(float y) {
  // tanh(y) = 1 - 2 / (exp(2y) + 1); exp overflow gives 1, underflow gives -1
  float e = __builtin_amdgcn_exp2f(y * 2.8853900817779268f);
  return 1.0f - 2.0f / (e + 1.0f);
}

struct MS {
  float m, s;
};
__device__ __forceinline__ MS ms_merge(MS a, MS b) {
  float m = fmaxf(a.m, b.m);
  MS r;
  r.m = m;
  r.s = a.s * fexp(a.m - m) + b.s * fexp(b.m - m);
  return r;
}

// ------------------------------------------------------------------------------------ row weights
// One workgroup: w[i] = valid_i / max(1, #valid) for the mean over the rows that count (mean != 0), else valid_i; a row
// counts when 0 <= t_i < V (V <= 0: when 0 <= t_i): the rows the loss kernels give a loss to.
template <typename IDX>
__global__ __launch_bounds__(1024) void loss_row_weights_kernel(const IDX* __restrict__ tg, float* __restrict__ w, long rows,
                                                               int mean, long V) {
  auto valid = [&](IDX t) { return t >= 0 && (long)t < V; };
  __shared__ int cnt[16];
  float each = 1.0f;
  if (mean) {
    int c = 0;
    for (long i = threadIdx.x; i < rows; i += 4096) {
      IDX t[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) t[k] = i + 1024 * k < rows ? tg[i + 1024 * k] : (IDX)-1;
#pragma unroll
      for (int k = 0; k < 4; ++k) c += valid(t[k]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o);
    if ((threadIdx.x & 63) == 0) cnt[threadIdx.x >> 6] = c;
    __syncthreads();
    int n = 0;
#pragma unroll
    for (int k = 0; k < 16; ++k) n += cnt[k];
    each = 1.0f / (float)(n > 1 ? n : 1);
  }
  for (long i = threadIdx.x; i < rows; i += 1024) w[i] = valid(tg[i]) ? each : 0.f;
}

// ------------------------------------------------------------------------------------ loss on logits
// One workgroup per row. loss_row = w * (lse - s_t) with w = row_w[row] (or 1), 0 for target < 0.
template <typename IDX>
__global__ __launch_bounds__(256) void loss_fwd_kernel(const bf16_t* __restrict__ x, const IDX* __restrict__ tg,
                                                      const float* __restrict__ row_w, float* __restrict__ loss,
                                                      float* __restrict__ lse, int V, float cap) {
  __shared__ float rm[4], rs[4];
  const long row = blockIdx.x;
  const bf16_t* xr = x + row * V;
  const float icap = cap > 0.f ? 1.0f / cap : 0.f;
  MS a{-1e30f, 0.f};
  for (int i = threadIdx.x * 8; i < V; i += 256 * 8) {
    u32x4 u = *(const u32x4*)(xr + i);
    float v[8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[2 * k] = bflo(u[k]);
      v[2 * k + 1] = bfhi(u[k]);
    }
    if (cap > 0.f) {
      // fixed shift: every s is in [-cap, cap]
#pragma unroll
      for (int k = 0; k < 8; ++k) a.s += fexp(cap * tanh_fast(v[k] * icap) - cap);
      a.m = cap;
    } else {
      float mx = a.m;
#pragma unroll
      for (int k = 0; k < 8; ++k) mx = fmaxf(mx, v[k]);
      float sc = fexp(a.m - mx), t = 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k) t += fexp(v[k] - mx);
      a.s = a.s * sc + t;
      a.m = mx;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    MS b{__shfl_xor(a.m, o, 64), __shfl_xor(a.s, o, 64)};
    a = ms_merge(a, b);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    rm[wave] = a.m;
    rs[wave] = a.s;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    MS t{rm[0], rs[0]};
    for (int i = 1; i < 4; ++i) t = ms_merge(t, MS{rm[i], rs[i]});
    float l = t.m + logf(t.s);
    lse[row] = l;
    long tt = (long)tg[row];
    float out = 0.f;
    if ((unsigned long)tt < (unsigned long)V) {  // a target outside [0, V) is an ignored row, never an address
      float xt = bf2f(xr[tt]);
      float st = cap > 0.f ? cap * tanh_fast(xt * icap) : xt;
      out = (l - st) * (row_w ? row_w[row] : 1.0f);
    }
    loss[row] = out;
  }
}

// d x_v = g_row (softmax_v - [v == t]) (1 - tanh^2); g_row = grow[row] (upstream grad x row weight); target < 0 -> 0.
template <typename IDX>
__global__ __launch_bounds__(256) void loss_bwd_kernel(const bf16_t* __restrict__ x, const IDX* __restrict__ tg,
                                                      const float* __restrict__ lse, const float* __restrict__ grow,
                                                      bf16_t* __restrict__ dx, int V, float cap) {
  const long row = blockIdx.x;
  const bf16_t* xr = x + row * V;
  bf16_t* dr = dx + row * V;
  const long tt = (long)tg[row];
  const float g = (unsigned long)tt < (unsigned long)V ? grow[row] : 0.f;  // out of range = ignored
  const float l = lse[row];
  const float icap = cap > 0.f ? 1.0f / cap : 0.f;
  // (the next chunk is requested before this chunk's store: a wait for loaded data also waits for every older store)
  u32x4 unext = {0u, 0u, 0u, 0u};
  if ((int)threadIdx.x * 8 < V) unext = *(const u32x4*)(xr + threadIdx.x * 8);
  for (int i = threadIdx.x * 8; i < V; i += 256 * 8) {
    const u32x4 u = unext;
    if (i + 256 * 8 < V) unext = *(const u32x4*)(xr + i + 256 * 8);
    float v[8], d[8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[2 * k] = bflo(u[k]);
      v[2 * k + 1] = bfhi(u[k]);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      float hot = (i + k == tt) ? 1.0f : 0.0f;
      if (cap > 0.f) {
        float t = tanh_fast(v[k] * icap);
        float p = fexp(cap * t - l);
        d[k] = g * (p - hot) * (1.0f - t * t);
      } else {
        d[k] = g * (fexp(v[k] - l) - hot);
      }
    }
    u32x4 o = {pack2bf(d[0], d[1]), pack2bf(d[2], d[3]), pack2bf(d[4], d[5]), pack2bf(d[6], d[7])};
    *(u32x4*)(dr + i) = o;
  }
}

// loss_fwd_kernel and loss_bwd_kernel for grow = row_w in ONE pass over the logits: a workgroup keeps its row in registers
// (NCH chunks of eight values per thread, V <= 2048 NCH), reduces it to lse in the order of loss_fwd_kernel, writes lse and
// the weighted row loss, and overwrites the row with d x_v = w (softmax_v - [v = t]) (1 - tanh^2): the gradient for an
// upstream gradient of one, which the caller's two gradient GEMMs scale by the real one. The logits are read once and
// written once where the two kernels read them twice; values equal theirs bit for bit.
template <typename IDX, int NCH>
__global__ __launch_bounds__(256) void loss_fwd_bwd_kernel(bf16_t* x, const IDX* __restrict__ tg, const float* __restrict__ row_w,
                                                          float* __restrict__ loss, float* __restrict__ lse, int V, float cap) {
  __shared__ float rm[4], rs[4], lsh;
  const long row = blockIdx.x;
  bf16_t* xr = x + row * V;
  const float icap = cap > 0.f ? 1.0f / cap : 0.f;
  u32x4 u[NCH];
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const int i = threadIdx.x * 8 + j * 2048;
    u[j] = i < V ? *(const u32x4*)(xr + i) : u32x4{0u, 0u, 0u, 0u};
  }
  MS a{-1e30f, 0.f};
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    if (threadIdx.x * 8 + j * 2048 < V) {
      float v[8];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        v[2 * k] = bflo(u[j][k]);
        v[2 * k + 1] = bfhi(u[j][k]);
      }
      if (cap > 0.f) {
#pragma unroll
        for (int k = 0; k < 8; ++k) a.s += fexp(cap * tanh_fast(v[k] * icap) - cap);
        a.m = cap;
      } else {
        float mx = a.m;
#pragma unroll
        for (int k = 0; k < 8; ++k) mx = fmaxf(mx, v[k]);
        float sc = fexp(a.m - mx), t = 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) t += fexp(v[k] - mx);
        a.s = a.s * sc + t;
        a.m = mx;
      }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    MS b{__shfl_xor(a.m, o, 64), __shfl_xor(a.s, o, 64)};
    a = ms_merge(a, b);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    rm[wave] = a.m;
    rs[wave] = a.s;
  }
  __syncthreads();
  const long tt = (long)tg[row];
  const bool valid = (unsigned long)tt < (unsigned long)V;  // a target outside [0, V) is an ignored row, never an address
  const float w = valid ? (row_w ? row_w[row] : 1.0f) : 0.f;
  if (threadIdx.x == 0) {
    MS t{rm[0], rs[0]};
    for (int i = 1; i < 4; ++i) t = ms_merge(t, MS{rm[i], rs[i]});
    const float l = t.m + logf(t.s);
    lse[row] = l;
    float out = 0.f;
    if (valid) {
      const float xt = bf2f(xr[tt]);   // (read before any thread overwrites the row: the barrier below)
      const float st = cap > 0.f ? cap * tanh_fast(xt * icap) : xt;
      out = (l - st) * w;
    }
    loss[row] = out;
    lsh = l;
  }
  __syncthreads();
  const float l = lsh;
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const int i = threadIdx.x * 8 + j * 2048;
    if (i < V) {
      float v[8], d[8];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        v[2 * k] = bflo(u[j][k]);
        v[2 * k + 1] = bfhi(u[j][k]);
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const float hot = (i + k == tt) ? 1.0f : 0.0f;
        if (cap > 0.f) {
          const float t = tanh_fast(v[k] * icap);
          const float p = fexp(cap * t - l);
          d[k] = w * (p - hot) * (1.0f - t * t);
        } else {
          d[k] = w * (fexp(v[k] - l) - hot);
        }
      }
      u32x4 o = {pack2bf(d[0], d[1]), pack2bf(d[2], d[3]), pack2bf(d[4], d[5]), pack2bf(d[6], d[7])};
      *(u32x4*)(xr + i) = o;
    }
  }
}

// ------------------------------------------------------------------------------------ several targets / label smoothing
// loss_row = sum_k rw_k (lse - (1 - eps) s_{t_k} - (eps / V) sum_v s_v), targets tg [K][rows] and weights rw [K][rows]
// (a target < 0 counts with weight 0). K > 1 is the multi-token-prediction loss (round1/source/train.py:4725), eps > 0
// the label-smoothed loss (round2/source/train.py:5697); K = 1, eps = 0 is loss_fwd_kernel with row weights.
// d x_v = g (1 - tanh^2) (W softmax_v - (1 - eps) sum_k rw_k [v = t_k] - W eps / V), W = sum_k rw_k.
constexpr int LOSS_KMAX = 8;

template <typename IDX>
__global__ __launch_bounds__(256) void loss_multi_fwd_kernel(const bf16_t* __restrict__ x, const IDX* __restrict__ tg,
                                                            const float* __restrict__ rw, int K, long rows,
                                                            float* __restrict__ loss, float* __restrict__ lse, int V, float cap,
                                                            float eps) {
  __shared__ float rm[4], rs[4], rt[4];
  const long row = blockIdx.x;
  const bf16_t* xr = x + row * V;
  const float icap = cap > 0.f ? 1.0f / cap : 0.f;
  MS a{-1e30f, 0.f};
  float ssum = 0.f;  // sum_v s_v (label smoothing)
  for (int i = threadIdx.x * 8; i < V; i += 256 * 8) {
    u32x4 u = *(const u32x4*)(xr + i);
    float v[8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[2 * k] = bflo(u[k]);
      v[2 * k + 1] = bfhi(u[k]);
    }
    if (cap > 0.f) {
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const float sv = cap * tanh_fast(v[k] * icap);
        ssum += sv;
        a.s += fexp(sv - cap);
      }
      a.m = cap;
    } else {
      float mx = a.m;
#pragma unroll
      for (int k = 0; k < 8; ++k) mx = fmaxf(mx, v[k]);
      float sc = fexp(a.m - mx), t = 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        t += fexp(v[k] - mx);
        ssum += v[k];
      }
      a.s = a.s * sc + t;
      a.m = mx;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    MS b{__shfl_xor(a.m, o, 64), __shfl_xor(a.s, o, 64)};
    a = ms_merge(a, b);
    ssum += __shfl_xor(ssum, o, 64);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    rm[wave] = a.m;
    rs[wave] = a.s;
    rt[wave] = ssum;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    MS t{rm[0], rs[0]};
    for (int i = 1; i < 4; ++i) t = ms_merge(t, MS{rm[i], rs[i]});
    const float l = t.m + logf(t.s);
    const float mean_s = (rt[0] + rt[1] + rt[2] + rt[3]) / (float)V;
    lse[row] = l;
    float out = 0.f;
    for (int k = 0; k < K; ++k) {
      const long tt = (long)tg[(long)k * rows + row];
      if ((unsigned long)tt >= (unsigned long)V) continue;  // negative or beyond the vocabulary: weight 0
      const float xt = bf2f(xr[tt]);
      const float st = cap > 0.f ? cap * tanh_fast(xt * icap) : xt;
      out += rw[(long)k * rows + row] * (l - (1.0f - eps) * st - eps * mean_s);
    }
    loss[row] = out;
  }
}

template <typename IDX>
__global__ __launch_bounds__(256) void loss_multi_bwd_kernel(const bf16_t* __restrict__ x, const IDX* __restrict__ tg,
                                                            const float* __restrict__ rw, int K, long rows,
                                                            const float* __restrict__ lse, const float* __restrict__ g,
                                                            bf16_t* __restrict__ dx, int V, float cap, float eps) {
  const long row = blockIdx.x;
  const bf16_t* xr = x + row * V;
  bf16_t* dr = dx + row * V;
  long tk[LOSS_KMAX];
  float wk[LOSS_KMAX];
  float W = 0.f;
#pragma unroll
  for (int k = 0; k < LOSS_KMAX; ++k) {
    tk[k] = -1;
    wk[k] = 0.f;
    if (k < K) {
      tk[k] = (long)tg[(long)k * rows + row];
      if ((unsigned long)tk[k] < (unsigned long)V) {
        wk[k] = rw[(long)k * rows + row];
        W += wk[k];
      }
    }
  }
  const float gr = g[row];
  const float l = lse[row];
  const float icap = cap > 0.f ? 1.0f / cap : 0.f;
  const float flat = W * eps / (float)V, keep = 1.0f - eps;
  for (int i = threadIdx.x * 8; i < V; i += 256 * 8) {
    u32x4 u = *(const u32x4*)(xr + i);
    float v[8], d[8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      v[2 * k] = bflo(u[k]);
      v[2 * k + 1] = bfhi(u[k]);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float hot = 0.f;
#pragma unroll
      for (int k = 0; k < LOSS_KMAX; ++k) hot += (i + e == tk[k]) ? wk[k] : 0.f;
      if (cap > 0.f) {
        const float t = tanh_fast(v[e] * icap);
        d[e] = gr * (W * fexp(cap * t - l) - keep * hot - flat) * (1.0f - t * t);
      } else {
        d[e] = gr * (W * fexp(v[e] - l) - keep * hot - flat);
      }
    }
    u32x4 o = {pack2bf(d[0], d[1]), pack2bf(d[2], d[3]), pack2bf(d[4], d[5]), pack2bf(d[6], d[7])};
    *(u32x4*)(dr + i) = o;
  }
}

// ------------------------------------------------------------------------------------ LM head GEMM + lse partials
struct EpiLmHead {
  static constexpr bool kTileEpilogue = true;
  bf16_t* logits;  // [rows][V]
  float* part;     // [V/64][rows][2] (max, sum): slab-major, so that a wavefront's 32 rows of one slab are one 256-byte store
  long V, rows;
  int nchunk;      // V / 64
  float cap;
  template <int TP, int TQ>
  __device__ __forceinline__ void tile(const f32x16 (&acc)[TP][TQ], int pw, int qw, int lr, int lh, int, int) const {
    static_assert(TP == 2, "a wavefront spans 64 vocabulary columns");
    const float icap = cap > 0.f ? 1.0f / cap : 0.f;
#pragma unroll
    for (int j = 0; j < TQ; ++j) {
      const long row = qw + j * 32 + lr;
      float v[TP * 16];
#pragma unroll
      for (int i = 0; i < TP; ++i)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int p = pw + i * 32 + jj * 8 + lh * 4;
          uint32_t w0 = pack2bf(acc[i][j][4 * jj], acc[i][j][4 * jj + 1]);
          uint32_t w1 = pack2bf(acc[i][j][4 * jj + 2], acc[i][j][4 * jj + 3]);
          u32x2 o = {w0, w1};
          *(u32x2*)(logits + row * V + p) = o;
          v[i * 16 + 4 * jj] = bflo(w0);
          v[i * 16 + 4 * jj + 1] = bfhi(w0);
          v[i * 16 + 4 * jj + 2] = bflo(w1);
          v[i * 16 + 4 * jj + 3] = bfhi(w1);
        }
      MS a;
      if (cap > 0.f) {
        a.m = cap;
        a.s = 0.f;
#pragma unroll
        for (int k = 0; k < TP * 16; ++k) a.s += fexp(cap * tanh_fast(v[k] * icap) - cap);
        a.s += __shfl_xor(a.s, 32, 64);
      } else {
        float mx = v[0];
#pragma unroll
        for (int k = 1; k < TP * 16; ++k) mx = fmaxf(mx, v[k]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < TP * 16; ++k) t += fexp(v[k] - mx);
        t += __shfl_xor(t, 32, 64);
        a.m = mx;
        a.s = t;
      }
      if (lh == 0) *(f32x2_t*)(part + ((long)(pw >> 6) * rows + row) * 2) = f32x2_t{a.m, a.s};
    }
  }
};

// A workgroup per 64 rows, a lane per row: each wavefront merges a quarter of the row's slab pairs (eight coalesced 512-byte
// loads in flight), the four quarters meet in LDS, then the target logit is read and lse and the row loss are written.
template <typename IDX>
__global__ __launch_bounds__(256) void lmhead_finish_kernel(const float* __restrict__ part, const bf16_t* __restrict__ logits,
                                                           const IDX* __restrict__ tg, const float* __restrict__ row_w,
                                                           float* __restrict__ loss, float* __restrict__ lse, long rows, long V,
                                                           int nchunk, float cap) {
  __shared__ float rm[4][64], rs[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long row = (long)blockIdx.x * 64 + lane;
  const long rr = row < rows ? row : rows - 1;
  const int q = (nchunk + 3) / 4, c0 = wave * q, c1 = c0 + q < nchunk ? c0 + q : nchunk;
  MS a{-1e30f, 0.f};
  for (int c = c0; c < c1; c += 8) {
    f32x2_t v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      v[j] = c + j < c1 ? *(const f32x2_t*)(part + ((long)(c + j) * rows + rr) * 2) : f32x2_t{-1e30f, 0.f};
#pragma unroll
    for (int j = 0; j < 8; ++j) a = ms_merge(a, MS{v[j][0], v[j][1]});
  }
  rm[wave][lane] = a.m;
  rs[wave][lane] = a.s;
  __syncthreads();
  if (wave == 0 && row < rows) {
#pragma unroll
    for (int w = 1; w < 4; ++w) a = ms_merge(a, MS{rm[w][lane], rs[w][lane]});
    float l = a.m + logf(a.s);
    lse[row] = l;
    long tt = (long)tg[row];
    float out = 0.f;
    if ((unsigned long)tt < (unsigned long)V) {  // a target outside [0, V) is an ignored row, never an address
      float xt = bf2f(logits[row * V + tt]);
      float st = cap > 0.f ? cap * tanh_fast(xt / cap) : xt;
      out = (l - st) * (row_w ? row_w[row] : 1.0f);
    }
    loss[row] = out;
  }
}

}  // namespace

// logits bf16 [rows][V]; targets int64 (idx64) or int32, negative = ignored; row_w fp32 [rows] or NULL;
// loss fp32 [rows] (already weighted); lse fp32 [rows]. softcap <= 0 means no softcap.
extern "C" int tfb_loss_fwd(const void* logits, const void* targets, int idx64, const void* row_w, void* loss, void* lse,
                            long rows, int V, float softcap, void* stream) {
  if (!logits || !targets || !loss || !lse) return TFB_ERR_ARG;
  if (rows <= 0 || V <= 0 || V % 8) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (idx64)
    hipLaunchKernelGGL(loss_fwd_kernel<long>, dim3((unsigned)rows), dim3(256), 0, s, (const bf16_t*)logits, (const long*)targets,
                       (const float*)row_w, (float*)loss, (float*)lse, V, softcap);
  else
    hipLaunchKernelGGL(loss_fwd_kernel<int>, dim3((unsigned)rows), dim3(256), 0, s, (const bf16_t*)logits, (const int*)targets,
                       (const float*)row_w, (float*)loss, (float*)lse, V, softcap);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// w fp32 [rows]: the weight of each row's loss in the reduction, valid / max(1, number of valid rows) for the mean over the
// rows that count (mean != 0: F.cross_entropy(ignore_index < 0) semantics), valid for the sum; valid = 0 <= t < V, the rows
// the loss kernels give a loss to (V <= 0: no upper bound). One small launch in place of a compare, a cast, a sum, a clamp
// and a division.
extern "C" int tfb_loss_row_weights(const void* targets, int idx64, void* w, long rows, int mean, int V, void* stream) {
  if (!targets || !w) return TFB_ERR_ARG;
  if (rows <= 0) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const long vmax = V > 0 ? (long)V : (1L << 62);
  if (idx64)
    hipLaunchKernelGGL(loss_row_weights_kernel<long>, dim3(1), dim3(1024), 0, s, (const long*)targets, (float*)w, rows, mean, vmax);
  else
    hipLaunchKernelGGL(loss_row_weights_kernel<int>, dim3(1), dim3(1024), 0, s, (const int*)targets, (float*)w, rows, mean, vmax);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// tfb_loss_fwd followed by tfb_loss_bwd with grow = row_w (an upstream gradient of one), in place and in one pass over the
// logits: loss and lse as tfb_loss_fwd writes them, and logits overwritten by that gradient, bit for bit what the two calls
// give. V <= 65536 (a row is held in one workgroup's registers); status TFB_ERR_SHAPE beyond, for the caller to take the two calls.
extern "C" int tfb_loss_fwd_bwd(void* logits, const void* targets, int idx64, const void* row_w, void* loss, void* lse, long rows,
                                int V, float softcap, void* stream) {
  if (!logits || !targets || !loss || !lse) return TFB_ERR_ARG;
  if (rows <= 0 || V <= 0 || V % 8 || V > 65536) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
#define TFB_LFB(IDX, NCH)                                                                                                  \
  hipLaunchKernelGGL((loss_fwd_bwd_kernel<IDX, NCH>), dim3((unsigned)rows), dim3(256), 0, s, (bf16_t*)logits,             \
                     (const IDX*)targets, (const float*)row_w, (float*)loss, (float*)lse, V, softcap)
  if (V <= 16384) {
    if (idx64) TFB_LFB(long, 8); else TFB_LFB(int, 8);
  } else if (V <= 32768) {
    if (idx64) TFB_LFB(long, 16); else TFB_LFB(int, 16);
  } else {
    if (idx64) TFB_LFB(long, 32); else TFB_LFB(int, 32);
  }
#undef TFB_LFB
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// dlogits may alias logits (in place). grow fp32 [rows] = upstream gradient of each row's loss times its weight.
extern "C" int tfb_loss_bwd(const void* logits, const void* targets, int idx64, const void* lse, const void* grow, void* dlogits,
                            long rows, int V, float softcap, void* stream) {
  if (!logits || !targets || !lse || !grow || !dlogits) return TFB_ERR_ARG;
  if (rows <= 0 || V <= 0 || V % 8) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (idx64)
    hipLaunchKernelGGL(loss_bwd_kernel<long>, dim3((unsigned)rows), dim3(256), 0, s, (const bf16_t*)logits, (const long*)targets,
                       (const float*)lse, (const float*)grow, (bf16_t*)dlogits, V, softcap);
  else
    hipLaunchKernelGGL(loss_bwd_kernel<int>, dim3((unsigned)rows), dim3(256), 0, s, (const bf16_t*)logits, (const int*)targets,
                       (const float*)lse, (const float*)grow, (bf16_t*)dlogits, V, softcap);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// Several targets per row and / or label smoothing: targets [K][rows], row_w fp32 [K][rows], 1 <= K <= 8, 0 <= eps < 1.
extern "C" int tfb_loss_multi_fwd(const void* logits, const void* targets, int idx64, const void* row_w, int K, float eps,
                                  void* loss, void* lse, long rows, int V, float softcap, void* stream) {
  if (!logits || !targets || !row_w || !loss || !lse) return TFB_ERR_ARG;
  if (rows <= 0 || V <= 0 || V % 8 || K < 1 || K > LOSS_KMAX || !(eps >= 0.f && eps < 1.f)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (idx64)
    hipLaunchKernelGGL(loss_multi_fwd_kernel<long>, dim3((unsigned)rows), dim3(256), 0, s, (const bf16_t*)logits,
                       (const long*)targets, (const float*)row_w, K, rows, (float*)loss, (float*)lse, V, softcap, eps);
  else
    hipLaunchKernelGGL(loss_multi_fwd_kernel<int>, dim3((unsigned)rows), dim3(256), 0, s, (const bf16_t*)logits,
                       (const int*)targets, (const float*)row_w, K, rows, (float*)loss, (float*)lse, V, softcap, eps);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// g fp32 [rows] = upstream gradient of each row's loss (the weights are applied here). dlogits may alias logits.
extern "C" int tfb_loss_multi_bwd(const void* logits, const void* targets, int idx64, const void* row_w, int K, float eps,
                                  const void* lse, const void* g, void* dlogits, long rows, int V, float softcap, void* stream) {
  if (!logits || !targets || !row_w || !lse || !g || !dlogits) return TFB_ERR_ARG;
  if (rows <= 0 || V <= 0 || V % 8 || K < 1 || K > LOSS_KMAX || !(eps >= 0.f && eps < 1.f)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (idx64)
    hipLaunchKernelGGL(loss_multi_bwd_kernel<long>, dim3((unsigned)rows), dim3(256), 0, s, (const bf16_t*)logits,
                       (const long*)targets, (const float*)row_w, K, rows, (const float*)lse, (const float*)g,
                       (bf16_t*)dlogits, V, softcap, eps);
  else
    hipLaunchKernelGGL(loss_multi_bwd_kernel<int>, dim3((unsigned)rows), dim3(256), 0, s, (const bf16_t*)logits,
                       (const int*)targets, (const float*)row_w, K, rows, (const float*)lse, (const float*)g,
                       (bf16_t*)dlogits, V, softcap, eps);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// Fused LM head forward: x bf16 [rows][d], W bf16 [V][d] -> logits bf16 [rows][V], loss fp32 [rows], lse fp32 [rows].
// part: fp32 scratch [rows][V/64][2].
extern "C" int tfb_lmhead_fwd(const void* x, const void* W, const void* targets, int idx64, const void* row_w, void* logits,
                              void* part, void* loss, void* lse, long rows, int d, int V, float softcap, void* stream) {
  if (!x || !W || !targets || !logits || !part || !loss || !lse) return TFB_ERR_ARG;
  if (rows <= 0 || rows % 128 || V <= 0 || V % 128 || d <= 0 || d % 64) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  // 128 x 128 tiles, two workgroups per CU started half a tile apart (gemm_core.hpp): the epilogue of one (2.1 GB of
  // logits written, exp / max / sum per element) runs under the other's MFMAs. Measured at V = 32768, 32768 rows:
  // 2.08 ms, against 2.26 ms for 256 x 256 tiles on 8 wavefronts (half the operand bytes per flop, but one resident
  // workgroup and nothing to hide its epilogue behind); a wavefront spans 64 vocabulary columns.
  using Cfg = GemmCfg<128, 128, 2, 2, 2, TFB_K_CONTIG, TFB_K_CONTIG>;
  GemmOperand P{(const uint8_t*)W, (long)d * 2}, Q{(const uint8_t*)x, (long)d * 2};
  EpiLmHead e{(bf16_t*)logits, (float*)part, (long)V, rows, V / 64, softcap};
  int st = gemm_launch<Cfg>(P, Q, V, (int)rows, (long)d * 2, 1, LoadIdentity{}, LoadIdentity{}, e, s);
  if (st != TFB_OK) return st;
  unsigned nb = (unsigned)((rows + 63) / 64);
  if (idx64)
    hipLaunchKernelGGL(lmhead_finish_kernel<long>, dim3(nb), dim3(256), 0, s, (const float*)part, (const bf16_t*)logits,
                       (const long*)targets, (const float*)row_w, (float*)loss, (float*)lse, rows, (long)V, V / 64, softcap);
  else
    hipLaunchKernelGGL(lmhead_finish_kernel<int>, dim3(nb), dim3(256), 0, s, (const float*)part, (const bf16_t*)logits,
                       (const int*)targets, (const float*)row_w, (float*)loss, (float*)lse, rows, (long)V, V / 64, softcap);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

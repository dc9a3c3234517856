// Mixture-of-experts routing, dispatch and combine for gfx950 (top-1 / top-2, experts local to the GPU).
//
// Replaces the host-side torch graph of MoeMLP.forward (round2/source/train.py:10941-11001): moe_route / moe_tournament
// (10505-10553: softmax of fp32 router logits, the k best experts by first-maximum, gates renormalised over the two),
// moe_positions / moe_gather_tables (10555-10634: each assignment's slot), MoeDispatch2 / MoeCombine2 (10652-10688) and
// the gated combine (10990-10992). The reference counts a fixed capacity per sequence and drops the overflow because
// its compiler needs static shapes; here the slot buffer is ragged and dropless: expert e's assignments are contiguous,
// in token order, padded to a multiple of 128 rows, and a device-side table names the expert of every 128-row tile, so
// the grouped fp8 GEMMs need no host knowledge of the loads (no sync, no recompilation when routing is skewed).
// With a capacity that drops nothing the reference computes the same function.
//
// Tables (int32, device): cnt[E]; seg[E+1] padded segment offsets; tile_expert[rmax/128]; slot[N][k]; tok[rmax] (token
// of each row or -1); ksel[rmax] (which choice a row holds).
#include "common.hpp"

namespace {

constexpr int MAXE = 16;
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
#ifndef TFB_ROUTE_EIGHT
#define TFB_ROUTE_EIGHT 1  // E <= 8: the eight-tokens-per-wavefront router (0: one token per wavefront)
#endif

__device__ __forceinline__ void load8(const bf16_t* p, float (&v)[8]) {
  u32x4 u = *(const u32x4*)p;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    v[2 * k] = bflo(u[k]);
    v[2 * k + 1] = bfhi(u[k]);
  }
}
__device__ __forceinline__ void store8(bf16_t* p, const float (&v)[8]) {
  u32x4 u = {pack2bf(v[0], v[1]), pack2bf(v[2], v[3]), pack2bf(v[4], v[5]), pack2bf(v[6], v[7])};
  *(u32x4*)p = u;
}

// ------------------------------------------------------------------------------------------------ router
// One wavefront per token: logits = h . Wr[e] (+ bias) in fp32, softmax, first-maximum top-k, gates.
// The EP (8 or 16) per-lane partial sums are reduced over the wavefront together: at each of the first log2(EP) butterfly
// steps a lane keeps half of its values and hands the other half to its partner, so the whole reduction is EP - 1 + 6 -
// log2(EP) shuffles instead of 6 EP, with the same additions in the same order as a butterfly sum of every value
// (a + b is b + a bit for bit), so two experts with equal weights still get equal logits.
template <int EP>
__device__ __forceinline__ float route_reduce(const float (&acc)[EP], int lane) {
  float v[EP];
#pragma unroll
  for (int e = 0; e < EP; ++e) v[e] = acc[e];
  int n = EP, off = 32;
#pragma unroll
  for (int lvl = 0; lvl < (EP == 16 ? 4 : 3); ++lvl) {
    const bool hi = (lane & off) != 0;
    n >>= 1;
#pragma unroll
    for (int j = 0; j < EP / 2; ++j) {
      if (j < n) {
        const float keep = hi ? v[n + j] : v[j], send = hi ? v[j] : v[n + j];
        v[j] = keep + __shfl_xor(send, off, 64);
      }
    }
    off >>= 1;
  }
  float r = v[0];
#pragma unroll
  for (int o = (EP == 16 ? 2 : 4); o > 0; o >>= 1) r += __shfl_xor(r, o, 64);
  return r;  // the total of expert (lane >> (EP == 16 ? 2 : 3)) with its index bits in the order the steps split them
}
// the lane whose route_reduce result is expert e's total: step k (offset 32 >> k) split on bit (log2(EP) - 1 - k) of e
template <int EP>
__device__ __forceinline__ int route_lane_of(int e) {
  return EP == 16 ? (e << 2) : (e << 3);
}

// One token's logits from the lanes' partial sums, then softmax, the first-maximum top-k and the gates; lane 0 stores.
template <int EP>
__device__ __forceinline__ void route_finish(const float (&acc)[EP], int lane, long n, long N, int E, int topk,
                                             const float* __restrict__ bias, float* __restrict__ logits_out,
                                             float* __restrict__ p_out, int* __restrict__ idx_out,
                                             float* __restrict__ gate_out) {
  float lg[EP];
  float mx = -INFINITY;
  if constexpr (EP <= 8) {
    const float mine = route_reduce<EP>(acc, lane);
#pragma unroll
    for (int e = 0; e < EP; ++e) lg[e] = e < E ? __shfl(mine, route_lane_of<EP>(e), 64) + (bias ? bias[e] : 0.f) : 0.f;
  } else {  // (the joint reduction of sixteen values measured slower than sixteen butterflies: 114 against 102 us)
#pragma unroll
    for (int e = 0; e < EP; ++e) lg[e] = e < E ? wave_sum(acc[e]) + (bias ? bias[e] : 0.f) : 0.f;
  }
#pragma unroll
  for (int e = 0; e < EP; ++e)
    if (e < E) mx = fmaxf(mx, lg[e]);
  float p[EP], den = 0.f;
#pragma unroll
  for (int e = 0; e < EP; ++e) {
    p[e] = e < E ? expf(lg[e] - mx) : 0.f;
    den += p[e];
  }
  int i1 = 0, i2 = 0;
  float v1 = -1.f, v2 = -1.f;
#pragma unroll
  for (int e = 0; e < EP; ++e) {
    if (e < E) {
      p[e] = p[e] / den;
      if (p[e] > v1) {
        v1 = p[e];
        i1 = e;
      }
    }
  }
#pragma unroll
  for (int e = 0; e < EP; ++e) {
    if (e < E && e != i1 && p[e] > v2) {
      v2 = p[e];
      i2 = e;
    }
  }
  if (n >= N) return;
  if (lane < E) {   // lane e stores expert e's probability and logit: one store instruction each instead of E
    float pe = p[0], le = lg[0];
#pragma unroll
    for (int e = 1; e < EP; ++e) {
      pe = lane == e ? p[e] : pe;
      le = lane == e ? lg[e] : le;
    }
    p_out[n * E + lane] = pe;
    if (logits_out) logits_out[n * E + lane] = le;
  }
  if (lane == 0) {
    if (topk == 2) {
      const float s = v1 + v2;
      *(i32x2*)(idx_out + n * 2) = i32x2{i1, i2};
      *(f32x2*)(gate_out + n * 2) = f32x2{v1 / s, v2 / s};
    } else {
      idx_out[n] = i1;
      gate_out[n] = v1;
    }
  }
}

// TPW tokens per wavefront at a time (sharing one fetch of the router's weights) was measured at 2 and 4: slower than 1
// (41 and 49 us against 36 for 16384 tokens of d = 1024), as was staging the weights in LDS under one round of workgroups.
template <int EP, int TPW>
__global__ __launch_bounds__(256) void moe_route_kernel(const bf16_t* __restrict__ h, const float* __restrict__ wr,
                                                       const float* __restrict__ bias, float* __restrict__ logits_out,
                                                       float* __restrict__ p_out, int* __restrict__ idx_out,
                                                       float* __restrict__ gate_out, long N, int d, int E, int topk) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (long n0 = ((long)blockIdx.x * 4 + wave) * TPW; n0 < N; n0 += (long)gridDim.x * 4 * TPW) {
    float acc[TPW][EP];
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
      for (int e = 0; e < EP; ++e) acc[t][e] = 0.f;
    for (int c = lane * 8; c < d; c += 512) {
      float x[TPW][8];
#pragma unroll
      for (int t = 0; t < TPW; ++t) load8(h + (n0 + t < N ? n0 + t : N - 1) * d + c, x[t]);  // (a group's tail re-reads the last token)
      if constexpr (EP <= 8) {
        // no branch on e < E here: behind one, each expert's two loads wait for the previous expert's (2 E dependent round
        // trips to the L2 per chunk: 42 -> 36 us); an expert beyond E re-reads the last one's weights, its sum is never used
        f32x4 w0[EP], w1[EP];
#pragma unroll
        for (int e = 0; e < EP; ++e) {
          const float* w = wr + (long)(e < E ? e : E - 1) * d + c;
          w0[e] = *(const f32x4*)w;
          w1[e] = *(const f32x4*)(w + 4);
        }
#pragma unroll
        for (int t = 0; t < TPW; ++t)
#pragma unroll
          for (int e = 0; e < EP; ++e)
            acc[t][e] += x[t][0] * w0[e][0] + x[t][1] * w0[e][1] + x[t][2] * w0[e][2] + x[t][3] * w0[e][3] + x[t][4] * w1[e][0] +
                         x[t][5] * w1[e][1] + x[t][6] * w1[e][2] + x[t][7] * w1[e][3];
      } else {
        // sixteen experts' weights of a chunk would be 128 registers: one expert at a time (102 us against 135 at d = 2048)
#pragma unroll
        for (int e = 0; e < EP; ++e) {
          if (e < E) {
            const float* w = wr + (long)e * d + c;
            const f32x4 w0 = *(const f32x4*)w, w1 = *(const f32x4*)(w + 4);
#pragma unroll
            for (int t = 0; t < TPW; ++t)
              acc[t][e] += x[t][0] * w0[0] + x[t][1] * w0[1] + x[t][2] * w0[2] + x[t][3] * w0[3] + x[t][4] * w1[0] +
                           x[t][5] * w1[1] + x[t][6] * w1[2] + x[t][7] * w1[3];
          }
        }
      }
    }
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
      const long n = n0 + t;
      route_finish<EP>(acc[t], lane, n, N, E, topk, bias, logits_out, p_out, idx_out, gate_out);
    }
  }
}

// Eight tokens per wavefront, finished one (token, expert) pair per lane. The 64 per-lane partial sums (8 tokens x 8
// experts) go through ONE joint butterfly (63 shuffles for eight tokens; value t * 8 + e ends up complete in lane t * 8 + e,
// added in the order of a butterfly sum, so a token's logits are the bits the one-token kernel above gives), and the
// softmax, the first-maximum top-k and the gates then run once over the wavefront with a token's eight experts in eight
// neighbouring lanes, instead of once per token with every lane repeating the same arithmetic. A chunk of the router's
// weights is fetched once per eight tokens. 16384 tokens of d = 1024: 36 -> 15 us. E <= 8.
template <int HALF>
__device__ __forceinline__ void route_fold(float (&v)[64], int lane) {   // a lane keeps HALF of its 2 HALF values, its partner (lane ^ HALF) the others
  const bool hi = (lane & HALF) != 0;
#pragma unroll
  for (int j = 0; j < HALF; ++j) {
    const float keep = hi ? v[HALF + j] : v[j], send = hi ? v[j] : v[HALF + j];
    v[j] = keep + __shfl_xor(send, HALF, 64);
  }
}
__device__ __forceinline__ float route_reduce64(float (&v)[64], int lane) {
  route_fold<32>(v, lane);
  route_fold<16>(v, lane);
  route_fold<8>(v, lane);
  route_fold<4>(v, lane);
  route_fold<2>(v, lane);
  route_fold<1>(v, lane);
  return v[0];
}

__global__ __launch_bounds__(256) void moe_route8_kernel(const bf16_t* __restrict__ h, const float* __restrict__ wr,
                                                        const float* __restrict__ bias, float* __restrict__ logits_out,
                                                        float* __restrict__ p_out, int* __restrict__ idx_out,
                                                        float* __restrict__ gate_out, long N, int d, int E, int topk) {
  const int lane = threadIdx.x & 63;
  const long n0 = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * 8;
  if (n0 >= N) return;
  float acc[64];
#pragma unroll
  for (int i = 0; i < 64; ++i) acc[i] = 0.f;
  for (int c = lane * 8; c < d; c += 512) {
    u32x4 raw[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) raw[t] = *(const u32x4*)(h + (n0 + t < N ? n0 + t : N - 1) * d + c);  // (a tail re-reads the last token)
    f32x4 w0[8], w1[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {   // an expert beyond E re-reads the last one's weights; its sums are never used
      const float* w = wr + (long)(e < E ? e : E - 1) * d + c;
      w0[e] = *(const f32x4*)w;
      w1[e] = *(const f32x4*)(w + 4);
    }
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      float x[8];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        x[2 * k] = bflo(raw[t][k]);
        x[2 * k + 1] = bfhi(raw[t][k]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e)
        acc[t * 8 + e] += x[0] * w0[e][0] + x[1] * w0[e][1] + x[2] * w0[e][2] + x[3] * w0[e][3] + x[4] * w1[e][0] +
                          x[5] * w1[e][1] + x[6] * w1[e][2] + x[7] * w1[e][3];
    }
  }
  const int e = lane & 7;
  const long n = n0 + (lane >> 3);
  const bool live = e < E;
  const float lg = route_reduce64(acc, lane) + (bias && live ? bias[e] : 0.f);
  float mx = live ? lg : -INFINITY;
#pragma unroll
  for (int o = 1; o < 8; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  float p = live ? expf(lg - mx) : 0.f;
  float den = p;
#pragma unroll
  for (int o = 1; o < 8; o <<= 1) den += __shfl_xor(den, o, 64);
  p = p / den;
  // first maximum over the token's eight lanes: the larger value wins, equal values go to the lower expert
  auto best_of = [&](float v, int i, float& bv, int& bi) {
    bv = v;
    bi = i;
#pragma unroll
    for (int o = 1; o < 8; o <<= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
  };
  float v1, v2;
  int i1, i2;
  best_of(live ? p : -1.f, e, v1, i1);
  best_of(live && e != i1 ? p : -1.f, e, v2, i2);
  if (n >= N) return;
  if (live) {
    p_out[n * E + e] = p;
    if (logits_out) logits_out[n * E + e] = lg;
  }
  if (e == 0) {
    if (topk == 2) {
      const float s = v1 + v2;
      *(i32x2*)(idx_out + n * 2) = i32x2{i1, i2};
      *(f32x2*)(gate_out + n * 2) = f32x2{v1 / s, v2 / s};
    } else {
      idx_out[n] = i1;
      gate_out[n] = v1;
    }
  }
}

// ------------------------------------------------------------------------------------------------ slot tables
// Per wavefront of 64 tokens: how many assignments each expert receives.
__global__ __launch_bounds__(256) void moe_count_kernel(const int* __restrict__ idx, int* __restrict__ wave_cnt, long N, int E,
                                                       int topk) {
  const int lane = threadIdx.x & 63;
  const long w = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const long n = w * 64 + lane;
  if (w * 64 >= N) return;
  int a0 = -1, a1 = -1;
  if (n < N) {
    a0 = idx[n * topk];
    if (topk == 2) a1 = idx[n * 2 + 1];
  }
  for (int e = 0; e < E; ++e) {
    int c = __popcll(__ballot(a0 == e)) + __popcll(__ballot(a1 == e));
    if (lane == 0) wave_cnt[w * E + e] = c;
  }
}

// One workgroup: exclusive scan of the per-wavefront counts per expert (a wavefront per expert, each lane a run of
// consecutive entries), padded segment offsets, tile -> expert table.
__global__ __launch_bounds__(256) void moe_scan_kernel(int* __restrict__ wave_cnt, int nwaves, int E, int* __restrict__ cnt,
                                                      int* __restrict__ seg, int* __restrict__ tile_expert, int ntiles) {
  __shared__ int s_seg[MAXE + 1];
  __shared__ int s_cnt[MAXE];
  const int lane = threadIdx.x & 63;
  const int run_len = (nwaves + 63) / 64;
  const int w0 = lane * run_len < nwaves ? lane * run_len : nwaves;
  const int w1 = w0 + run_len < nwaves ? w0 + run_len : nwaves;
  for (int e = threadIdx.x >> 6; e < E; e += 4) {
    int tot = 0;
    for (int w = w0; w < w1; ++w) tot += wave_cnt[(long)w * E + e];
    int inc = tot;
    for (int o = 1; o < 64; o <<= 1) {
      const int t = __shfl_up(inc, o);
      if (lane >= o) inc += t;
    }
    int run = inc - tot;
    for (int w = w0; w < w1; ++w) {
      const int c = wave_cnt[(long)w * E + e];
      wave_cnt[(long)w * E + e] = run;  // becomes the wavefront's offset inside the expert's segment
      run += c;
    }
    if (lane == 63) {
      cnt[e] = inc;
      s_cnt[e] = inc;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int off = 0;
    for (int e = 0; e < E; ++e) {
      s_seg[e] = off;
      off += (s_cnt[e] + 127) / 128 * 128;
    }
    s_seg[E] = off;
    for (int e = 0; e <= E; ++e) seg[e] = s_seg[e];
  }
  __syncthreads();
  for (int t = threadIdx.x; t < ntiles; t += 256) {
    int row = t * 128, ex = -1;
    for (int e = 0; e < E; ++e)
      if (row >= s_seg[e] && row < s_seg[e + 1]) ex = e;
    tile_expert[t] = ex;
  }
}

// The reference's per-sequence capacity (round2/source/train.py:10555 moe_positions, :10600 keep = pos < cap): an assignment's
// position is the number of assignments to its expert at EARLIER tokens of the same sequence (both choices count); the
// first `cap` of a sequence are kept, the rest are skipped. One thread per (sequence, expert) walks the sequence's
// wavefronts (a sequence is a whole number of 64-token wavefronts): pre[w][e] = assignments before wavefront w inside its
// sequence, wave_cnt[w][e] becomes the number KEPT in the wavefront (the earliest lanes), cnt_all[e] every assignment.
__global__ __launch_bounds__(256) void moe_cap_kernel(int* __restrict__ wave_cnt, int* __restrict__ pre, int* __restrict__ cnt_all,
                                                     int nseq, int wps, int E, int cap) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= nseq * E) return;
  const int b = i / E, e = i % E;
  int prefix = 0;
  for (int w = b * wps; w < (b + 1) * wps; ++w) {
    const int raw = wave_cnt[(long)w * E + e];
    pre[(long)w * E + e] = prefix;
    const int room = cap - prefix;
    wave_cnt[(long)w * E + e] = room <= 0 ? 0 : (raw < room ? raw : room);
    prefix += raw;
  }
  atomicAdd(cnt_all + e, prefix);
}

// Every assignment's row: seg[e] + (assignments to e from earlier wavefronts) + (from earlier lanes of this one). With a
// capacity (pre != NULL) wave_off counts kept assignments only, and an assignment whose position inside its sequence
// (pre + earlier lanes) reaches cap gets slot -1 and no row.
__global__ __launch_bounds__(256) void moe_place_kernel(const int* __restrict__ idx, const int* __restrict__ wave_off,
                                                       const int* __restrict__ seg, int* __restrict__ slot,
                                                       int* __restrict__ tok, int* __restrict__ ksel, long N, int E, int topk,
                                                       const int* __restrict__ pre, int cap) {
  const int lane = threadIdx.x & 63;
  const long w = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const long n = w * 64 + lane;
  if (w * 64 >= N) return;
  int a0 = -1, a1 = -1;
  if (n < N) {
    a0 = idx[n * topk];
    if (topk == 2) a1 = idx[n * 2 + 1];
  }
  const unsigned long long lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  int r0 = 0, r1 = 0;
  for (int e = 0; e < E; ++e) {
    unsigned long long b0 = __ballot(a0 == e), b1 = __ballot(a1 == e);
    int before = __popcll(b0 & lt) + __popcll(b1 & lt);
    if (a0 == e) r0 = before;
    if (a1 == e) r1 = before;
  }
  if (n < N) {
    const bool keep0 = !pre || pre[w * E + a0] + r0 < cap;
    int s0 = keep0 ? seg[a0] + wave_off[w * E + a0] + r0 : -1;
    slot[n * topk] = s0;
    if (keep0) {
      tok[s0] = (int)n;
      ksel[s0] = 0;
    }
    if (topk == 2) {
      const bool keep1 = !pre || pre[w * E + a1] + r1 < cap;
      int s1 = keep1 ? seg[a1] + wave_off[w * E + a1] + r1 : -1;
      slot[n * 2 + 1] = s1;
      if (keep1) {
        tok[s1] = (int)n;
        ksel[s1] = 1;
      }
    }
  }
}

__global__ void fill_i32_kernel(int* __restrict__ p, int val, long n) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) p[i] = val;
}

// ------------------------------------------------------------------------------------------------ dispatch / combine
// xs[row] = h[tok[row]] (zero rows for padding), and / or its e4m3 cast at `scale`.
__global__ __launch_bounds__(256) void moe_gather_kernel(const bf16_t* __restrict__ h, const int* __restrict__ tok,
                                                        const float* __restrict__ scale_ptr, float scale_imm,
                                                        bf16_t* __restrict__ xs, uint8_t* __restrict__ xs8, long rmax, int d) {
  const float sc = scale_ptr ? *scale_ptr : scale_imm;
  const int cpr = d / 8;
  const long total = rmax * cpr;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    long row = i / cpr;
    int c = (int)(i % cpr) * 8;
    int t = tok[row];
    float v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (t >= 0) load8(h + (long)t * d + c, v);
    if (xs) store8(xs + row * d + c, v);
    if (xs8) {
      u32x2 o = {cvt4_fp8<TFB_FMT_E4M3>(v[0] * sc, v[1] * sc, v[2] * sc, v[3] * sc),
                 cvt4_fp8<TFB_FMT_E4M3>(v[4] * sc, v[5] * sc, v[6] * sc, v[7] * sc)};
      *(u32x2*)(xs8 + row * d + c) = o;
    }
  }
}

// out[n] = bf16(bf16(g1) y[slot1]) + bf16(bf16(g2) y[slot2]), rounded again (the eager bf16 expression).
__global__ __launch_bounds__(256) void moe_combine_kernel(const bf16_t* __restrict__ ys, const int* __restrict__ slot,
                                                         const float* __restrict__ gate, bf16_t* __restrict__ out, long N,
                                                         int d, int topk) {
  const int cpr = d / 8;
  const long total = N * cpr;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    long n = i / cpr;
    int c = (int)(i % cpr) * 8;
    // a skipped assignment (slot -1: over the sequence's capacity) reads the reference's zero row
    float a[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, r[8];
    const int s1 = slot[n * topk];
    if (s1 >= 0) load8(ys + (long)s1 * d + c, a);
    const float g1 = round_bf(gate[n * topk]);
#pragma unroll
    for (int k = 0; k < 8; ++k) r[k] = round_bf(g1 * a[k]);
    if (topk == 2) {
      float b[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      const int s2 = slot[n * 2 + 1];
      if (s2 >= 0) load8(ys + (long)s2 * d + c, b);
      const float g2 = round_bf(gate[n * 2 + 1]);
#pragma unroll
      for (int k = 0; k < 8; ++k) r[k] += round_bf(g2 * b[k]);
    }
    store8(out + n * d + c, r);
  }
}

// One wavefront per slot row: dys[row] = bf16(bf16(g_k) dout[tok]); dgate[tok][k] = bf16(sum_d dout[tok] ys[row]).
// ROWMAX: rowmax[row] = max |dys[row]| of the rounded values (0 for a padding row), from which the experts' backward scales
// are taken without another pass over dys.
template <bool ROWMAX>
__global__ __launch_bounds__(256) void moe_combine_bwd_kernel(const bf16_t* __restrict__ dout, const bf16_t* __restrict__ ys,
                                                             const int* __restrict__ tok, const int* __restrict__ ksel,
                                                             const float* __restrict__ gate, bf16_t* __restrict__ dys,
                                                             float* __restrict__ dgate, float* __restrict__ rowmax, long rmax,
                                                             int d, int topk) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (long row = (long)blockIdx.x * 4 + wave; row < rmax; row += (long)gridDim.x * 4) {
    const int t = tok[row];
    if (t < 0) {
      for (int c = lane * 8; c < d; c += 512) *(u32x4*)(dys + row * d + c) = u32x4{0, 0, 0, 0};
      if (ROWMAX && lane == 0) rowmax[row] = 0.f;
      continue;
    }
    const int k = ksel[row];
    const float g = round_bf(gate[(long)t * topk + k]);
    float dot = 0.f, m = 0.f;
    for (int c = lane * 8; c < d; c += 512) {
      float go[8], y[8];
      load8(dout + (long)t * d + c, go);
      load8(ys + row * d + c, y);
#pragma unroll
      for (int j = 0; j < 8; ++j) dot += go[j] * y[j];
      const u32x4 u = {pack2bf(g * go[0], g * go[1]), pack2bf(g * go[2], g * go[3]), pack2bf(g * go[4], g * go[5]),
                       pack2bf(g * go[6], g * go[7])};
      *(u32x4*)(dys + row * d + c) = u;
      if (ROWMAX) {
#pragma unroll
        for (int j = 0; j < 4; ++j) m = fmaxf(m, fmaxf(fabsf(bflo(u[j])), fabsf(bfhi(u[j]))));
      }
    }
    dot = wave_sum(dot);
    if (ROWMAX) m = wave_max(m);
    if (lane == 0) {
      dgate[(long)t * topk + k] = round_bf(dot);
      if (ROWMAX) rowmax[row] = m;
    }
  }
}

// dlogits[n][e] = p_e (dp_e - sum_j p_j dp_j), dp from the gate gradients through the renormalisation.
// With the auxiliary router terms (terms != NULL: [0] lb, [1] z, [2..] f_e as left by moe_aux_finish_kernel; lse[n]; g =
// *gaux, the gradient arriving at the weighted sum alpha lb + beta z): dp_e += g alpha (E / N) f_e (f carries no
// gradient) and, after the softmax Jacobian, dlogits_e += g beta (2 / N) lse_n p_e. With the per-sequence balance term
// (fs != NULL: fs[b][e] the load shares of sequence b = n / T as left by moe_aux_seq_kernel, weight gamma):
// dp_e += g gamma (E / N) fs[b][e] (the term is a mean over the N / T sequences of E sum_e fs ps, ps a mean over T tokens).
__global__ __launch_bounds__(256) void moe_dlogits_kernel(const float* __restrict__ dgate, const float* __restrict__ p,
                                                         const int* __restrict__ idx, float* __restrict__ dlogits, long N,
                                                         int E, int topk, const float* __restrict__ terms,
                                                         const float* __restrict__ lse, const float* __restrict__ gaux,
                                                         float alpha, float beta, const float* __restrict__ fs, float gamma,
                                                         long T) {
  long n = (long)blockIdx.x * 256 + threadIdx.x;
  if (n >= N) return;
  float dp[MAXE];
  for (int e = 0; e < E; ++e) dp[e] = 0.f;
  if (topk == 2) {
    const int i1 = idx[n * 2], i2 = idx[n * 2 + 1];
    const float v1 = p[n * E + i1], v2 = p[n * E + i2], den = v1 + v2;
    const float dg1 = dgate[n * 2], dg2 = dgate[n * 2 + 1];
    // g1 = v1 / den, g2 = v2 / den
    const float inv2 = 1.0f / (den * den);
    const float dv1 = (dg1 - dg2) * v2 * inv2, dv2 = (dg2 - dg1) * v1 * inv2;
    for (int e = 0; e < E; ++e) dp[e] = e == i1 ? dv1 : (e == i2 ? dv2 : 0.f);
  } else {
    const int i1 = idx[n];
    for (int e = 0; e < E; ++e) dp[e] = e == i1 ? dgate[n] : 0.f;
  }
  float zc = 0.f;
  if (terms) {
    const float g = *gaux;
    const float ca = g * alpha * (float)E / (float)N;
    for (int e = 0; e < E; ++e) dp[e] += ca * terms[2 + e];
    zc = g * beta * 2.0f / (float)N * lse[n];
    if (fs) {
      const float cs = g * gamma * (float)E / (float)N;
      const float* fb = fs + (n / T) * E;
      for (int e = 0; e < E; ++e) dp[e] += cs * fb[e];
    }
  }
  float dot = 0.f;
  for (int e = 0; e < E; ++e) dot += p[n * E + e] * dp[e];
  for (int e = 0; e < E; ++e) dlogits[n * E + e] = p[n * E + e] * (dp[e] - dot + zc);
}

// Auxiliary router terms (round2/source/train.py:10779 moe_aux_terms): partial column sums of p and of lse^2, lse[n] =
// logsumexp(logits[n]); part [gridDim.x][MAXE + 1].
__global__ __launch_bounds__(256) void moe_aux_partial_kernel(const float* __restrict__ p, const float* __restrict__ logits,
                                                             float* __restrict__ lse_out, float* __restrict__ part, long N,
                                                             int E) {
  __shared__ float red[4][MAXE + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float acc[MAXE + 1];
#pragma unroll
  for (int e = 0; e <= MAXE; ++e) acc[e] = 0.f;
  for (long n = (long)blockIdx.x * 256 + threadIdx.x; n < N; n += (long)gridDim.x * 256) {
    float mx = -INFINITY;
    for (int e = 0; e < E; ++e) mx = fmaxf(mx, logits[n * E + e]);
    float den = 0.f;
    for (int e = 0; e < E; ++e) den += expf(logits[n * E + e] - mx);
    const float l = mx + logf(den);
    lse_out[n] = l;
    acc[MAXE] += l * l;
#pragma unroll
    for (int e = 0; e < MAXE; ++e)
      if (e < E) acc[e] += p[n * E + e];
  }
#pragma unroll
  for (int e = 0; e <= MAXE; ++e) {
    const float v = wave_sum(acc[e]);
    if (lane == 0) red[wave][e] = v;
  }
  __syncthreads();
  if (threadIdx.x <= MAXE)
    part[(long)blockIdx.x * (MAXE + 1) + threadIdx.x] = red[0][threadIdx.x] + red[1][threadIdx.x] + red[2][threadIdx.x] + red[3][threadIdx.x];
}
// terms[0] = lb = E sum_e f_e P_e, terms[1] = z = mean lse^2, terms[2 + e] = f_e = cnt_e / (N topk), P_e = mean_n p[n][e]
__global__ void moe_aux_finish_kernel(const float* __restrict__ part, int nparts, const int* __restrict__ cnt,
                                      float* __restrict__ terms, long N, int E, int topk) {
  __shared__ float tot[MAXE + 1];
  if (threadIdx.x <= MAXE) {
    float s = 0.f;
    for (int b = 0; b < nparts; ++b) s += part[(long)b * (MAXE + 1) + threadIdx.x];
    tot[threadIdx.x] = s;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float lb = 0.f;
    for (int e = 0; e < E; ++e) {
      const float f = (float)cnt[e] / ((float)N * (float)topk);
      terms[2 + e] = f;
      lb += f * (tot[e] / (float)N);
    }
    terms[0] = (float)E * lb;
    terms[1] = tot[MAXE] / (float)N;
  }
}

// The per-sequence form of the balance term (round2/source/train.py:10789-10792): one workgroup per sequence b of T tokens.
// fs[b][e] = (assignments of the sequence's tokens to e) / (T topk), from ALL selections (idx), dropped or not;
// part[b] = E sum_e fs[b][e] ps[b][e] with ps[b][e] the mean of p over the sequence's tokens.
__global__ __launch_bounds__(256) void moe_aux_seq_kernel(const float* __restrict__ p, const int* __restrict__ idx,
                                                         float* __restrict__ fs, float* __restrict__ part, long T, int E,
                                                         int topk) {
  __shared__ float red[4][2 * MAXE];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long n0 = (long)blockIdx.x * T;
  float ps[MAXE], cn[MAXE];
#pragma unroll
  for (int e = 0; e < MAXE; ++e) ps[e] = cn[e] = 0.f;
  for (long i = threadIdx.x; i < T; i += 256) {
    const long n = n0 + i;
    const int i1 = idx[n * topk], i2 = topk == 2 ? idx[n * 2 + 1] : -1;
#pragma unroll
    for (int e = 0; e < MAXE; ++e)
      if (e < E) {
        ps[e] += p[n * E + e];
        cn[e] += (float)((e == i1) + (e == i2));   // whole numbers below 2^24: exact whatever the order
      }
  }
#pragma unroll
  for (int e = 0; e < MAXE; ++e) {
    const float a = wave_sum(ps[e]), c = wave_sum(cn[e]);
    if (lane == 0) {
      red[wave][e] = a;
      red[wave][MAXE + e] = c;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float acc = 0.f;
    for (int e = 0; e < E; ++e) {
      const float psum = (red[0][e] + red[1][e]) + (red[2][e] + red[3][e]);
      const float cnt = (red[0][MAXE + e] + red[1][MAXE + e]) + (red[2][MAXE + e] + red[3][MAXE + e]);
      const float f = cnt / ((float)T * (float)topk);
      fs[(long)blockIdx.x * E + e] = f;
      acc += f * (psum / (float)T);
    }
    part[blockIdx.x] = (float)E * acc;
  }
}
// term = the mean of part over the nseq sequences, summed in sequence order
__global__ void moe_aux_seq_finish_kernel(const float* __restrict__ part, long nseq, float* __restrict__ term) {
  if (threadIdx.x == 0) {
    float s = 0.f;
    for (long b = 0; b < nseq; ++b) s += part[b];
    *term = s / (float)nseq;
  }
}

// dh[n] = dxs[slot1] + dxs[slot2] + sum_e dlogits[n][e] Wr[e] (fp32 sum, one rounding).
// A thread keeps ONE 8-column chunk for all the tokens it visits (the launch makes the thread count a multiple of the chunks
// per row), so its slice of every expert's router weights stays in registers: fetched per token from the L2 they were 16
// times the bytes of the output (537 MB for 16384 tokens of d = 1024) and what the kernel waited for.
template <int EP>
__global__ __launch_bounds__(256) void moe_dispatch_bwd_kernel(const bf16_t* __restrict__ dxs, const int* __restrict__ slot,
                                                              const float* __restrict__ dlogits, const float* __restrict__ wr,
                                                              bf16_t* __restrict__ dh, long N, int d, int E, int topk) {
  const int cpr = d / 8;
  const long tid = (long)blockIdx.x * 256 + threadIdx.x, nthreads = (long)gridDim.x * 256;
  const int c = (int)(tid % cpr) * 8;
  const long nstep = nthreads / cpr;
  f32x4 w0[EP], w1[EP];
  if (dlogits) {
#pragma unroll
    for (int e = 0; e < EP; ++e) {
      const float* w = wr + (long)(e < E ? e : E - 1) * d + c;   // (an expert beyond E: the last one's, with a zero gradient)
      w0[e] = *(const f32x4*)w;
      w1[e] = *(const f32x4*)(w + 4);
    }
  }
  // Software-pipelined over the thread's tokens: a token's slots and router gradients are requested one token ahead, and
  // its two rows of dxs are loaded without a branch between them (a skipped assignment reads row 0 and is zeroed by a
  // select), so a token costs one round trip to memory instead of three dependent ones (36 -> 28 us for 16384 x 1024).
  auto fetch_meta = [&](long n, int& s1, int& s2, float (&g)[EP]) {
    if (topk == 2) {
      const i32x2 sv = *(const i32x2*)(slot + n * 2);
      s1 = sv.x;
      s2 = sv.y;
    } else {
      s1 = slot[n];
      s2 = -1;
    }
    if (dlogits) {
#pragma unroll
      for (int e = 0; e < EP; ++e) g[e] = dlogits[n * E + (e < E ? e : E - 1)];
    }
  };
  long n = tid / cpr;
  int s1 = -1, s2 = -1, t1 = -1, t2 = -1;
  float g[EP], gn[EP];
#pragma unroll
  for (int e = 0; e < EP; ++e) g[e] = gn[e] = 0.f;
  if (n < N) fetch_meta(n, s1, s2, g);
  for (; n < N; n += nstep) {
    const u32x4 ra = *(const u32x4*)(dxs + (long)(s1 >= 0 ? s1 : 0) * d + c);
    const u32x4 rb = *(const u32x4*)(dxs + (long)(s2 >= 0 ? s2 : 0) * d + c);
    if (n + nstep < N) fetch_meta(n + nstep, t1, t2, gn);
    float r[8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float a0 = s1 >= 0 ? bflo(ra[k]) : 0.f, a1 = s1 >= 0 ? bfhi(ra[k]) : 0.f;
      const float b0 = s2 >= 0 ? bflo(rb[k]) : 0.f, b1 = s2 >= 0 ? bfhi(rb[k]) : 0.f;
      r[2 * k] = a0 + b0;
      r[2 * k + 1] = a1 + b1;
    }
    if (dlogits) {
#pragma unroll
      for (int e = 0; e < EP; ++e) {
        const float ge = e < E ? g[e] : 0.f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          r[k] += ge * w0[e][k];
          r[4 + k] += ge * w1[e][k];
        }
      }
    }
    store8(dh + n * d + c, r);
    s1 = t1;
    s2 = t2;
#pragma unroll
    for (int e = 0; e < EP; ++e) g[e] = gn[e];
  }
}

// dWr[e][c] (+)= sum_n dlogits[n][e] h[n][c] in two launches with a fixed summation order: workgroup (x, y) owns 64 columns
// and the y-th chunk of the tokens (32 row lanes stride over it) and leaves its sums in part[y][e][c]; the finish adds the
// chunks in order. DWR_CHUNKS chunks at most: part is fp32 [DWR_CHUNKS][E][d].
constexpr int DWR_CHUNKS = 64;
#ifndef DWR_WANT
#define DWR_WANT 0
#endif
__global__ __launch_bounds__(256) void moe_dwr_partial_kernel(const float* __restrict__ dlogits, const bf16_t* __restrict__ h,
                                                             float* __restrict__ part, long N, long chunk, int d, int E) {
  __shared__ __align__(16) float red[4][8][64];
  __shared__ __align__(16) float gs[256][8];
  const int cl = threadIdx.x & 7, rl = threadIdx.x >> 3;
  const int c = blockIdx.x * 64 + cl * 8;
  const long n0 = blockIdx.y * chunk, n1 = n0 + chunk < N ? n0 + chunk : N;
  for (int e0 = 0; e0 < E; e0 += 8) {
    float acc[8][8];
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
      for (int k = 0; k < 8; ++k) acc[e][k] = 0.f;
    // 256 tokens at a time: their dlogits go to LDS (so no registers wait for them) while all eight of a row lane's rows of
    // h are in flight together; 16384 tokens are one such round per workgroup (one row at a time it was eight dependent
    // round trips to memory, 28 us for 16384 x 1024)
    for (long nb = n0; nb < n1; nb += 256) {
      __syncthreads();   // (the previous round's dlogits have been read)
      {
        const long n = nb + threadIdx.x;
#pragma unroll
        for (int e = 0; e < 8; ++e) gs[threadIdx.x][e] = n < n1 && e0 + e < E ? dlogits[n * E + e0 + e] : 0.f;
      }
      u32x4 raw[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const long nj = nb + rl + 32 * j;
        raw[j] = *(const u32x4*)(h + (nj < n1 ? nj : n1 - 1) * d + c);
      }
      __syncthreads();
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (nb + rl + 32 * j < n1) {
          const f32x4 g0 = *(const f32x4*)&gs[rl + 32 * j][0], g1 = *(const f32x4*)&gs[rl + 32 * j][4];
          const float g[8] = {g0[0], g0[1], g0[2], g0[3], g1[0], g1[1], g1[2], g1[3]};
          float x[8];
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            x[2 * k] = bflo(raw[j][k]);
            x[2 * k + 1] = bfhi(raw[j][k]);
          }
#pragma unroll
          for (int e = 0; e < 8; ++e)
#pragma unroll
            for (int k = 0; k < 8; ++k) acc[e][k] += g[e] * x[k];
        }
      }
    }
    // the wavefront's eight row lanes first, by the joint butterfly over lane bits 3..5 (56 shuffles; the lane of row-lane
    // index e is left with expert e's eight columns), then the four wavefronts through LDS: one barrier instead of sixteen
    float v[64];
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
      for (int k = 0; k < 8; ++k) v[e * 8 + k] = acc[e][k];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    route_fold<32>(v, lane);
    route_fold<16>(v, lane);
    route_fold<8>(v, lane);
    __syncthreads();   // (the previous group of experts has been read)
    {
      const int e = (lane >> 3) & 7;
      *(f32x4*)&red[wave][e][cl * 8] = f32x4{v[0], v[1], v[2], v[3]};
      *(f32x4*)&red[wave][e][cl * 8 + 4] = f32x4{v[4], v[5], v[6], v[7]};
    }
    __syncthreads();
    {
      const int e = threadIdx.x >> 5, col = (threadIdx.x & 31) * 2;
      if (e0 + e < E) {
        f32x2 s2 = *(const f32x2*)&red[0][e][col];
#pragma unroll
        for (int w = 1; w < 4; ++w) s2 += *(const f32x2*)&red[w][e][col];
        *(f32x2*)(part + ((long)blockIdx.y * E + e0 + e) * d + blockIdx.x * 64 + col) = s2;
      }
    }
  }
}

__global__ __launch_bounds__(256) void moe_dwr_finish_kernel(const float* __restrict__ part, float* __restrict__ dwr, int chunks,
                                                            long ED, int accumulate) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= ED) return;
  float s = accumulate ? dwr[i] : 0.f;
  int y = 0;
  for (; y + 8 <= chunks; y += 8) {   // eight loads in flight, added in order
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = part[(y + j) * ED + i];
#pragma unroll
    for (int j = 0; j < 8; ++j) s += v[j];
  }
  for (; y < chunks; ++y) s += part[y * ED + i];
  dwr[i] = s;
}

// ------------------------------------------------------------------------------------------------ per-expert scales
// amax of each 128-row tile of g (four workgroups of 32 rows each), merged into its expert's slot (non-negative floats order
// like their bit patterns).
__global__ __launch_bounds__(256) void moe_amax_kernel(const bf16_t* __restrict__ g, const int* __restrict__ tile_expert,
                                                      unsigned* __restrict__ amax_bits, int d) {
  __shared__ float red[4];
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const bf16_t* base = g + ((long)blockIdx.x * 128 + blockIdx.y * 32) * d;
  float m = 0.f;
  for (long i = (long)threadIdx.x * 8; i < 32L * d; i += 256 * 8) {
    u32x4 u = *(const u32x4*)(base + i);
#pragma unroll
    for (int k = 0; k < 4; ++k) m = fmaxf(m, fmaxf(fabsf(bflo(u[k])), fabsf(bfhi(u[k]))));
  }
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    atomicMax(amax_bits + e, __float_as_uint(m));
  }
}

__device__ void pow2_le_moe(float v, float limit, int e_lo, int e_hi, float* s_out, float* inv_out) {
  float s = ldexpf(1.0f, e_lo), inv = ldexpf(1.0f, -e_lo);
  const float top = ldexpf(1.0f, e_hi);
  const int span = e_hi - e_lo;
  for (int b = 64; b >= 1; b >>= 1) {
    if (b > span) continue;
    float cand = s * ldexpf(1.0f, b);
    if ((v * cand <= limit) && (cand <= top)) {
      s = cand;
      inv = inv * ldexpf(1.0f, -b);
    }
  }
  *s_out = s;
  *inv_out = inv;
}

// rows_out[e] = rows_in[e] with the four backward columns filled from the expert's amax(dy)
// (round2/source/kernels/nki_mlp_fused8.py:803-813, once per expert).
__device__ void moe_backward_scale_row(const float* in, float* out, float amax_dy, float dp_factor) {
  for (int i = 0; i < 16; ++i) out[i] = in[i];
  float s_dy, i_dy, s_dp, i_dp;
  pow2_le_moe(amax_dy, TFB_E5M2_MAX / 2.0f, -40, 60, &s_dy, &i_dy);
  float bound = sqrtf(in[9] * in[10]) * amax_dy * dp_factor;
  pow2_le_moe(bound, TFB_E5M2_MAX, -40, 60, &s_dp, &i_dp);
  out[5] = s_dy;
  out[6] = i_dy * in[12] * 2.0f;
  out[7] = s_dp;
  out[8] = i_dp * in[11];
}
__global__ void moe_backward_scales_kernel(const unsigned* __restrict__ amax_bits, const float* __restrict__ rows_in,
                                           float* __restrict__ rows_out, int E, float dp_factor) {
  int e = threadIdx.x;
  if (e >= E) return;
  moe_backward_scale_row(rows_in + e * 16, rows_out + e * 16, __uint_as_float(amax_bits[e]), dp_factor);
}
// The same from the row maxima the combine backward left: workgroup e takes the maximum over expert e's rows
// seg[e] .. seg[e + 1] (a maximum does not depend on the order, so the scales are those of the kernel above bit for bit).
__global__ __launch_bounds__(256) void moe_backward_scales_rowmax_kernel(const float* __restrict__ rowmax, const int* __restrict__ seg,
                                                                        const float* __restrict__ rows_in,
                                                                        float* __restrict__ rows_out, float dp_factor) {
  __shared__ float red[4];
  const int e = blockIdx.x;
  float m = 0.f;
  const int end = seg[e + 1];
  for (int r = seg[e] + threadIdx.x; r < end; r += 256 * 8) {   // eight loads in flight per thread
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = r + 256 * j < end ? rowmax[r + 256 * j] : 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) m = fmaxf(m, v[j]);
  }
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0)
    moe_backward_scale_row(rows_in + e * 16, rows_out + e * 16, fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])), dp_factor);
}

// out8[row] = fp8(x[row] * rows[expert of row][col]) for the rows of live tiles; padding tiles are zero-filled.
template <int FMT>
__global__ __launch_bounds__(256) void moe_quant_kernel(const bf16_t* __restrict__ x, const int* __restrict__ tile_expert,
                                                       const float* __restrict__ rows, int col, uint8_t* __restrict__ out,
                                                       long rmax, int d) {
  const int cpr = d / 8;
  const long total = rmax * cpr;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    long row = i / cpr;
    int c = (int)(i % cpr) * 8;
    int e = tile_expert[row >> 7];
    u32x2 o = {0, 0};
    if (e >= 0) {
      const float s = rows[e * 16 + col];
      float v[8];
      load8(x + row * d + c, v);
      o.x = cvt4_fp8<FMT>(v[0] * s, v[1] * s, v[2] * s, v[3] * s);
      o.y = cvt4_fp8<FMT>(v[4] * s, v[5] * s, v[6] * s, v[7] * s);
    }
    *(u32x2*)(out + row * d + c) = o;
  }
}

inline int nblocks(long n, int cap = 8192) {
  long b = (n + 255) / 256;
  return (int)(b < 1 ? 1 : (b < cap ? b : cap));
}

}  // namespace

// Upper bound of the padded slot rows for N tokens: every expert's segment rounds up to 128 (host helper).
extern "C" long tfb_moe_max_rows(long N, int E, int topk) { return (N * topk + (long)E * 127) / 128 * 128; }

// h bf16 [N][d], wr fp32 [E][d], bias fp32 [E] or NULL -> logits (optional) / p fp32 [N][E], idx int32 [N][topk],
// gate fp32 [N][topk]. E <= 16, topk 1 or 2, d % 8 == 0.
// Replaces F.linear(h.float(), router.float()) + moe_route (round2/source/train.py:10525-10553, 10961).
extern "C" int tfb_moe_route(const void* h, const void* wr, const void* bias, void* logits, void* p, void* idx, void* gate, long N,
                             int d, int E, int topk, void* stream) {
  if (!h || !wr || !p || !idx || !gate) return TFB_ERR_ARG;
  if (N <= 0 || d <= 0 || d % 8 || E < 2 || E > MAXE || (topk != 1 && topk != 2)) return TFB_ERR_SHAPE;
  if (E <= 8 && TFB_ROUTE_EIGHT)
    hipLaunchKernelGGL(moe_route8_kernel, dim3((unsigned)((N + 31) / 32)), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)h,
                       (const float*)wr, (const float*)bias, (float*)logits, (float*)p, (int*)idx, (float*)gate, N, d, E, topk);
  else if (E <= 8)
    hipLaunchKernelGGL((moe_route_kernel<8, 1>), dim3(nblocks(N * 64)), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)h,
                       (const float*)wr, (const float*)bias, (float*)logits, (float*)p, (int*)idx, (float*)gate, N, d, E, topk);
  else
    hipLaunchKernelGGL((moe_route_kernel<16, 1>), dim3(nblocks(N * 64)), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)h,
                       (const float*)wr, (const float*)bias, (float*)logits, (float*)p, (int*)idx, (float*)gate, N, d, E, topk);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// idx int32 [N][topk] -> cnt [E], seg [E+1], tile_expert [rmax/128], slot [N][topk], tok [rmax], ksel [rmax];
// scratch: int32 [ceil(N/64) * E]. rmax = tfb_moe_max_rows(N, E, topk).
// Replaces moe_positions + moe_gather_tables (round2/source/train.py:10555-10634), dropless.
extern "C" int tfb_moe_tables(const void* idx, void* cnt, void* seg, void* tile_expert, void* slot, void* tok, void* ksel,
                              void* scratch, long N, int E, int topk, long rmax, void* stream) {
  if (!idx || !cnt || !seg || !tile_expert || !slot || !tok || !ksel || !scratch) return TFB_ERR_ARG;
  if (N <= 0 || E < 2 || E > MAXE || (topk != 1 && topk != 2) || rmax % 128 || rmax < tfb_moe_max_rows(N, E, topk))
    return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const int nwaves = (int)((N + 63) / 64);
  const int nb = (nwaves + 3) / 4;
  hipLaunchKernelGGL(fill_i32_kernel, dim3(nblocks(rmax)), dim3(256), 0, s, (int*)tok, -1, rmax);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_count_kernel, dim3(nb), dim3(256), 0, s, (const int*)idx, (int*)scratch, N, E, topk);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_scan_kernel, dim3(1), dim3(256), 0, s, (int*)scratch, nwaves, E, (int*)cnt, (int*)seg,
                     (int*)tile_expert, (int)(rmax / 128));
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_place_kernel, dim3(nb), dim3(256), 0, s, (const int*)idx, (const int*)scratch, (const int*)seg,
                     (int*)slot, (int*)tok, (int*)ksel, N, E, topk, (const int*)nullptr, 0);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// tfb_moe_tables with the reference's per-sequence capacity (round2/source/train.py:10555-10600): the tokens are N / T
// sequences of T; of a sequence's assignments to one expert (both choices, in token order) the first `cap` keep a row, the
// rest get slot -1 (the reference's zero row: they add nothing to the output and receive no gradient). cnt [E] counts the
// kept assignments (the segments' extents), cnt_all [E] every assignment (what the load-balance term's f_e is made of).
// scratch: int32 [2 * ceil(N/64) * E]. T % 64 == 0 (a sequence is a whole number of wavefronts), N % T == 0, cap >= 1.
extern "C" int tfb_moe_tables_cap(const void* idx, void* cnt, void* cnt_all, void* seg, void* tile_expert, void* slot, void* tok,
                                  void* ksel, void* scratch, long N, long T, int cap, int E, int topk, long rmax, void* stream) {
  if (!idx || !cnt || !cnt_all || !seg || !tile_expert || !slot || !tok || !ksel || !scratch) return TFB_ERR_ARG;
  if (N <= 0 || E < 2 || E > MAXE || (topk != 1 && topk != 2) || rmax % 128 || rmax < tfb_moe_max_rows(N, E, topk))
    return TFB_ERR_SHAPE;
  if (T <= 0 || T % 64 || N % T || cap < 1) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const int nwaves = (int)(N / 64);
  const int nb = (nwaves + 3) / 4;
  const int nseq = (int)(N / T), wps = (int)(T / 64);
  int* wave_cnt = (int*)scratch;
  int* pre = wave_cnt + (long)nwaves * E;
  hipLaunchKernelGGL(fill_i32_kernel, dim3(nblocks(rmax)), dim3(256), 0, s, (int*)tok, -1, rmax);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(fill_i32_kernel, dim3(1), dim3(256), 0, s, (int*)cnt_all, 0, (long)E);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_count_kernel, dim3(nb), dim3(256), 0, s, (const int*)idx, wave_cnt, N, E, topk);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_cap_kernel, dim3((nseq * E + 255) / 256), dim3(256), 0, s, wave_cnt, pre, (int*)cnt_all, nseq, wps, E, cap);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_scan_kernel, dim3(1), dim3(256), 0, s, wave_cnt, nwaves, E, (int*)cnt, (int*)seg, (int*)tile_expert,
                     (int)(rmax / 128));
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_place_kernel, dim3(nb), dim3(256), 0, s, (const int*)idx, (const int*)wave_cnt, (const int*)seg,
                     (int*)slot, (int*)tok, (int*)ksel, N, E, topk, (const int*)pre, cap);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// xs bf16 [rmax][d] = h[tok] (zero padding rows), xs8 = e4m3(xs * scale). Replaces MoeDispatch2.forward (10652-10660).
extern "C" int tfb_moe_gather(const void* h, const void* tok, const void* scale_ptr, float scale_imm, void* xs, void* xs8,
                              long rmax, int d, void* stream) {
  if (!h || !tok || (!xs && !xs8)) return TFB_ERR_ARG;   // either copy may be left out (bf16 experts take no fp8 rows; fp8 experts
                                                        // with fp8 weight gradients no bf16 ones)
  if (rmax <= 0 || d <= 0 || d % 8) return TFB_ERR_SHAPE;
  hipLaunchKernelGGL(moe_gather_kernel, dim3(nblocks(rmax * (d / 8))), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)h,
                     (const int*)tok, (const float*)scale_ptr, scale_imm, (bf16_t*)xs, (uint8_t*)xs8, rmax, d);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// out bf16 [N][d] = sum_k bf16(gate_k) ys[slot_k]. Replaces MoeCombine2.forward + the gated sum (10672-10676, 10990-10992).
extern "C" int tfb_moe_combine(const void* ys, const void* slot, const void* gate, void* out, long N, int d, int topk,
                               void* stream) {
  if (!ys || !slot || !gate || !out) return TFB_ERR_ARG;
  if (N <= 0 || d <= 0 || d % 8 || (topk != 1 && topk != 2)) return TFB_ERR_SHAPE;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(nblocks(N * (d / 8))), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)ys,
                     (const int*)slot, (const float*)gate, (bf16_t*)out, N, d, topk);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// dys bf16 [rmax][d], dgate fp32 [N][topk] from dout bf16 [N][d]. Replaces MoeCombine2.backward (10678-10688).
// Only the assignments that hold a row are written: with a capacity in use the caller zero-fills dgate first.
extern "C" int tfb_moe_combine_bwd(const void* dout, const void* ys, const void* tok, const void* ksel, const void* gate,
                                   void* dys, void* dgate, long rmax, int d, int topk, void* stream) {
  if (!dout || !ys || !tok || !ksel || !gate || !dys || !dgate) return TFB_ERR_ARG;
  if (rmax <= 0 || d <= 0 || d % 8 || (topk != 1 && topk != 2)) return TFB_ERR_SHAPE;
  hipLaunchKernelGGL(moe_combine_bwd_kernel<false>, dim3(nblocks(rmax * 64)), dim3(256), 0, (hipStream_t)stream,
                     (const bf16_t*)dout, (const bf16_t*)ys, (const int*)tok, (const int*)ksel, (const float*)gate, (bf16_t*)dys,
                     (float*)dgate, (float*)nullptr, rmax, d, topk);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}
// tfb_moe_combine_bwd that also leaves rowmax fp32 [rmax] = max |dys[row]| (0 for a padding row) for
// tfb_moe_backward_scales_rowmax: the experts' backward scales then cost no pass of their own over dys.
extern "C" int tfb_moe_combine_bwd_rowmax(const void* dout, const void* ys, const void* tok, const void* ksel, const void* gate,
                                          void* dys, void* dgate, void* rowmax, long rmax, int d, int topk, void* stream) {
  if (!dout || !ys || !tok || !ksel || !gate || !dys || !dgate || !rowmax) return TFB_ERR_ARG;
  if (rmax <= 0 || d <= 0 || d % 8 || (topk != 1 && topk != 2)) return TFB_ERR_SHAPE;
  hipLaunchKernelGGL(moe_combine_bwd_kernel<true>, dim3(nblocks(rmax * 64)), dim3(256), 0, (hipStream_t)stream,
                     (const bf16_t*)dout, (const bf16_t*)ys, (const int*)tok, (const int*)ksel, (const float*)gate, (bf16_t*)dys,
                     (float*)dgate, (float*)rowmax, rmax, d, topk);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// Router backward + dispatch backward: dlogits fp32 [N][E] (scratch/output), dh bf16 [N][d] = dxs[slots] + dlogits Wr,
// dwr fp32 [E][d] (+)= dlogits^T h. Replaces MoeDispatch2.backward (10662-10666) and autograd through moe_route.
static int moe_route_bwd_impl(const void* dgate, const void* p, const void* idx, const void* dxs, const void* slot,
                              const void* h, const void* wr, void* dlogits, void* dh, void* dwr, int dwr_accumulate,
                              void* scratch, long N, int d, int E, int topk, const void* terms, const void* lse,
                              const void* gaux, float alpha, float beta, const void* fs, float gamma, long T, void* stream) {
  if (!dgate || !p || !idx || !dxs || !slot || !h || !wr || !dlogits || !dh || !dwr || !scratch) return TFB_ERR_ARG;
  if (N <= 0 || d <= 0 || d % 64 || E < 2 || E > MAXE || (topk != 1 && topk != 2)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(moe_dlogits_kernel, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, s, (const float*)dgate,
                     (const float*)p, (const int*)idx, (float*)dlogits, N, E, topk, (const float*)terms, (const float*)lse,
                     (const float*)gaux, alpha, beta, (const float*)fs, gamma, T > 0 ? T : N);
  TFB_LAUNCH_CHECK();
  {
    // a thread count that is a multiple of the 8-column chunks per row: every thread then stays on one chunk
    const int cpr = d / 8;
    int g = cpr, b = 256;
    while (b) {
      const int t = g % b;
      g = b;
      b = t;
    }
    const int m = cpr / g;   // blocks per whole number of rows
    int blocks = nblocks(N * cpr, 2048);
    blocks = blocks < m ? m : blocks / m * m;
    if (E <= 8)
      hipLaunchKernelGGL(moe_dispatch_bwd_kernel<8>, dim3(blocks), dim3(256), 0, s, (const bf16_t*)dxs, (const int*)slot,
                         (const float*)dlogits, (const float*)wr, (bf16_t*)dh, N, d, E, topk);
    else
      hipLaunchKernelGGL(moe_dispatch_bwd_kernel<16>, dim3(blocks), dim3(256), 0, s, (const bf16_t*)dxs, (const int*)slot,
                         (const float*)dlogits, (const float*)wr, (bf16_t*)dh, N, d, E, topk);
  }
  TFB_LAUNCH_CHECK();
  // as many token chunks as give one round of resident workgroups (three per CU at this kernel's registers), DWR_CHUNKS at most
  const int resident = tfb_resident_slots(3) / (d / 64);
  const int want = DWR_WANT ? DWR_WANT : (resident < 1 ? 1 : (resident < DWR_CHUNKS ? resident : DWR_CHUNKS));
  const long chunk = ((N + want - 1) / want + 31) / 32 * 32;
  const int chunks = (int)((N + chunk - 1) / chunk);
  hipLaunchKernelGGL(moe_dwr_partial_kernel, dim3(d / 64, chunks), dim3(256), 0, s, (const float*)dlogits, (const bf16_t*)h,
                     (float*)scratch, N, chunk, d, E);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_dwr_finish_kernel, dim3(nblocks((long)E * d)), dim3(256), 0, s, (const float*)scratch, (float*)dwr,
                     chunks, (long)E * d, dwr_accumulate);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

extern "C" int tfb_moe_route_bwd(const void* dgate, const void* p, const void* idx, const void* dxs, const void* slot,
                                 const void* h, const void* wr, void* dlogits, void* dh, void* dwr, int dwr_accumulate,
                                 void* scratch, long N, int d, int E, int topk, void* stream) {
  return moe_route_bwd_impl(dgate, p, idx, dxs, slot, h, wr, dlogits, dh, dwr, dwr_accumulate, scratch, N, d, E, topk, nullptr,
                            nullptr, nullptr, 0.f, 0.f, nullptr, 0.f, 0, stream);
}
// tfb_moe_route_bwd with the gradient of the auxiliary router terms folded into dlogits: the weighted sum
// alpha lb + beta z of tfb_moe_aux_fwd received the gradient *gaux (device fp32 scalar); terms and lse as that call left them.
extern "C" int tfb_moe_route_bwd_aux(const void* dgate, const void* p, const void* idx, const void* dxs, const void* slot,
                                     const void* h, const void* wr, void* dlogits, void* dh, void* dwr, int dwr_accumulate,
                                     void* scratch, const void* terms, const void* lse, const void* gaux, float alpha,
                                     float beta, long N, int d, int E, int topk, void* stream) {
  if (!terms || !lse || !gaux) return TFB_ERR_ARG;
  return moe_route_bwd_impl(dgate, p, idx, dxs, slot, h, wr, dlogits, dh, dwr, dwr_accumulate, scratch, N, d, E, topk, terms,
                            lse, gaux, alpha, beta, nullptr, 0.f, 0, stream);
}
// tfb_moe_route_bwd_aux with the per-sequence balance term as well: the weighted sum alpha lb + beta z + gamma seq received
// the gradient *gaux; fs fp32 [N / T][E] as tfb_moe_aux_seq_fwd left it, T the sequence length (N % T == 0).
extern "C" int tfb_moe_route_bwd_aux_seq(const void* dgate, const void* p, const void* idx, const void* dxs, const void* slot,
                                         const void* h, const void* wr, void* dlogits, void* dh, void* dwr, int dwr_accumulate,
                                         void* scratch, const void* terms, const void* lse, const void* gaux, float alpha,
                                         float beta, const void* fs, float gamma, long T, long N, int d, int E, int topk,
                                         void* stream) {
  if (!terms || !lse || !gaux || !fs) return TFB_ERR_ARG;
  if (T <= 0 || N % T) return TFB_ERR_SHAPE;
  return moe_route_bwd_impl(dgate, p, idx, dxs, slot, h, wr, dlogits, dh, dwr, dwr_accumulate, scratch, N, d, E, topk, terms,
                            lse, gaux, alpha, beta, fs, gamma, T, stream);
}

// The router's auxiliary terms: terms fp32 [2 + E] = (lb = E sum_e f_e P_e, z = mean_n logsumexp(logits_n)^2, f_e) with
// f_e = cnt_e / (N topk) the share of the assignments that chose e (from the slot tables' counts) and P_e the mean
// router probability; lse fp32 [N] (kept for the backward); scratch: fp32 [64][17].
// Replaces moe_aux_terms (round2/source/train.py:10779-10788; its per-sequence term is tfb_moe_aux_seq_fwd).
extern "C" int tfb_moe_aux_fwd(const void* p, const void* logits, const void* cnt, void* terms, void* lse, void* scratch, long N,
                               int E, int topk, void* stream) {
  if (!p || !logits || !cnt || !terms || !lse || !scratch) return TFB_ERR_ARG;
  if (N <= 0 || E < 2 || E > MAXE || (topk != 1 && topk != 2)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const int nb = (int)((N + 255) / 256 < 64 ? (N + 255) / 256 : 64);
  hipLaunchKernelGGL(moe_aux_partial_kernel, dim3(nb), dim3(256), 0, s, (const float*)p, (const float*)logits, (float*)lse,
                     (float*)scratch, N, E);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_aux_finish_kernel, dim3(1), dim3(64), 0, s, (const float*)scratch, nb, (const int*)cnt, (float*)terms, N,
                     E, topk);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// The per-sequence balance term of moe_aux_terms (round2/source/train.py:10789-10792, the reference's R2_MOE_AUX_SEQ):
// term fp32 [1] = mean over the N / T sequences of E sum_e fs[b][e] ps[b][e], fs fp32 [N / T][E] the sequences' load shares
// (kept for the backward; no gradient), ps the sequences' mean router probabilities. idx int32 [N][topk] the selections
// (all of them: a capacity drops rows, not assignments, from this count); scratch fp32 [N / T].
extern "C" int tfb_moe_aux_seq_fwd(const void* p, const void* idx, void* fs, void* term, void* scratch, long N, long T, int E,
                                   int topk, void* stream) {
  if (!p || !idx || !fs || !term || !scratch) return TFB_ERR_ARG;
  if (N <= 0 || T <= 0 || N % T || T >= (1L << 23) || E < 2 || E > MAXE || (topk != 1 && topk != 2)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const long nseq = N / T;
  if (nseq > (1L << 30)) return TFB_ERR_SHAPE;
  hipLaunchKernelGGL(moe_aux_seq_kernel, dim3((unsigned)nseq), dim3(256), 0, s, (const float*)p, (const int*)idx, (float*)fs,
                     (float*)scratch, T, E, topk);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_aux_seq_finish_kernel, dim3(1), dim3(64), 0, s, (const float*)scratch, nseq, (float*)term);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// rows_out fp32 [E][16]: each expert's backward scale row from the amax of its rows of dys; amax_scratch: uint32 [E].
extern "C" int tfb_moe_backward_scales(const void* dys, const void* tile_expert, const void* rows_in, void* rows_out,
                                       void* amax_scratch, long rmax, int d, int E, void* stream) {
  if (!dys || !tile_expert || !rows_in || !rows_out || !amax_scratch) return TFB_ERR_ARG;
  if (rmax <= 0 || rmax % 128 || d % 8 || E < 1 || E > MAXE) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(fill_i32_kernel, dim3(1), dim3(256), 0, s, (int*)amax_scratch, 0, (long)E);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_amax_kernel, dim3((unsigned)(rmax / 128), 4), dim3(256), 0, s, (const bf16_t*)dys, (const int*)tile_expert,
                     (unsigned*)amax_scratch, d);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_backward_scales_kernel, dim3(1), dim3(64), 0, s, (const unsigned*)amax_scratch, (const float*)rows_in,
                     (float*)rows_out, E, (float)(36.16 * (double)d));
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// tfb_moe_backward_scales from rowmax fp32 [rmax] (tfb_moe_combine_bwd_rowmax) and the segment offsets seg int32 [E + 1]
// (tfb_moe_tables): the same rows, one small launch. d is the experts' model width (it sets the bound of dpre).
extern "C" int tfb_moe_backward_scales_rowmax(const void* rowmax, const void* seg, const void* rows_in, void* rows_out, int d, int E,
                                              void* stream) {
  if (!rowmax || !seg || !rows_in || !rows_out) return TFB_ERR_ARG;
  if (d <= 0 || d % 8 || E < 1 || E > MAXE) return TFB_ERR_SHAPE;
  hipLaunchKernelGGL(moe_backward_scales_rowmax_kernel, dim3(E), dim3(256), 0, (hipStream_t)stream, (const float*)rowmax,
                     (const int*)seg, (const float*)rows_in, (float*)rows_out, (float)(36.16 * (double)d));
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// out8 = fp8(x * rows[expert][col]) row-wise by the tile's expert (fmt 0 e4m3, 1 e5m2).
extern "C" int tfb_moe_quant(const void* x, const void* tile_expert, const void* rows, int col, int fmt, void* out8, long rmax,
                             int d, void* stream) {
  if (!x || !tile_expert || !rows || !out8) return TFB_ERR_ARG;
  if (rmax <= 0 || rmax % 128 || d % 8 || col < 0 || col >= 16) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  int nb = nblocks(rmax * (d / 8));
  if (fmt == TFB_FMT_E4M3)
    hipLaunchKernelGGL(moe_quant_kernel<TFB_FMT_E4M3>, dim3(nb), dim3(256), 0, s, (const bf16_t*)x, (const int*)tile_expert,
                       (const float*)rows, col, (uint8_t*)out8, rmax, d);
  else if (fmt == TFB_FMT_E5M2)
    hipLaunchKernelGGL(moe_quant_kernel<TFB_FMT_E5M2>, dim3(nb), dim3(256), 0, s, (const bf16_t*)x, (const int*)tile_expert,
                       (const float*)rows, col, (uint8_t*)out8, rmax, d);
  else
    return TFB_ERR_ARG;
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

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
// Layout of the work on the MFMA (32x32x16 bf16, 64-lane wavefronts): a wavefront owns 32
// queries (forward, dQ) or 32 keys (dK/dV) as the MFMA *column* index, so every row statistic
// (max, sum, lse, D) is one scalar per lane, and the score tile's accumulator registers, packed
// to bf16, are directly the B operand of the next product (P never touches LDS). The operand
// that must be contracted along its token dimension (V, K in dQ; Q, dO in dK/dV) is written
// into LDS transposed through 4 x 8 register micro-blocks while it is staged.
//
// Tensors are addressed by (batch, head, token) element strides with the head dimension
// contiguous, so q/k/v may be thirds of a fused qkv [B,T,3C] buffer and o / dO are [B,T,H,D].
#include "common.hpp"

#ifndef TFB_ATTN128_XCD
#define TFB_ATTN128_XCD 1  // re-deal workgroups so that a (batch, head) pair's blocks share an XCD's L2
#endif
#ifndef TFB_FWD128_WPE
#define TFB_FWD128_WPE 2  // D = 128 forward: 262 registers at one wavefront per SIMD, 70 KB of LDS: two workgroups fit a CU at 256
#endif
#ifndef TFB_FWD_WPE
#define TFB_FWD_WPE 3  // wavefronts per SIMD the forward kernel is compiled for (register budget 512 / WPE)
#endif
#ifndef TFB_DKDV128_WPE
#define TFB_DKDV128_WPE 1  // D = 128 dK/dV: 326 registers; at two wavefronts per SIMD it spills 36 and runs 0.90 vs 0.80 ms
#endif
#ifndef TFB_DKDV_WPE
#define TFB_DKDV_WPE 2
#endif
#ifndef TFB_BWD_NBUF
#define TFB_BWD_NBUF 1  // LDS buffers of the backward kernels' staged tiles
#endif
#ifndef TFB_DQ_WPE
#define TFB_DQ_WPE 2
#endif
#ifndef TFB_FWD_QG2
#define TFB_FWD_QG2 0  // two query groups per wavefront: measured slower (373 VGPRs, one wavefront per SIMD)
#endif

namespace {

struct AttnT {
  bf16_t* p;
  long sb, sh, st;
};

__device__ __forceinline__ bf16x8 lds16(const uint8_t* base, int off) { return *(const bf16x8*)(base + off); }
__device__ __forceinline__ bf16x8 lds8x2(const uint8_t* base, int off) {
  u32x2 a = *(const u32x2*)(base + off);
  u32x2 b = *(const u32x2*)(base + off + 16);
  u32x4 v = {a.x, a.y, b.x, b.y};
  return __builtin_bit_cast(bf16x8, v);
}
__device__ __forceinline__ bf16x8 frag_from(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  u32x4 v = {a, b, c, d};
  return __builtin_bit_cast(bf16x8, v);
}
__device__ __forceinline__ f32x16 mfma_bf16(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// 4 rows x 8 columns of bf16 held as four 128-bit rows.
struct MicroBlock {
  u32x4 g[4];
  __device__ __forceinline__ void load(const bf16_t* base, long stride, int row0, int col0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) g[j] = *(const u32x4*)(base + (long)(row0 + j) * stride + col0);
  }
  __device__ __forceinline__ void store_normal(uint8_t* lds, int rowbytes, int row0, int col0) const {
#pragma unroll
    for (int j = 0; j < 4; ++j) *(u32x4*)(lds + (row0 + j) * rowbytes + col0 * 2) = g[j];
  }
  // lds[col][row]: 8 rows of the transposed tile get 4 consecutive elements each
  __device__ __forceinline__ void store_transposed(uint8_t* lds, int rowbytes, int row0, int col0) const {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      u32x2 lo, hi;
      lo.x = (g[0][w] & 0xffffu) | (g[1][w] << 16);
      lo.y = (g[2][w] & 0xffffu) | (g[3][w] << 16);
      hi.x = (g[0][w] >> 16) | (g[1][w] & 0xffff0000u);
      hi.y = (g[2][w] >> 16) | (g[3][w] & 0xffff0000u);
      *(u32x2*)(lds + (col0 + 2 * w) * rowbytes + row0 * 2) = lo;
      *(u32x2*)(lds + (col0 + 2 * w + 1) * rowbytes + row0 * 2) = hi;
    }
  }
};

// s_waitcnt vmcnt(0) before a main loop: the register fragments loaded from global memory ahead of the loop are then
// known to have arrived, and the compiler does not repeat (in every iteration, against the tile loads in flight) the
// waits it would otherwise keep for them.
__device__ __forceinline__ void wait_all_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
// Workgroup -> (block along the sequence, batch*head): consecutive workgroup ids go round-robin to the 8 XCDs, each with
// its own L2, so the ids are re-dealt to keep all sequence blocks of one (batch, head) - which stream the same K / V (or
// Q / dO) tiles - on one XCD (the D = 64 kernels do the same). nx = blocks per (batch, head), nbh = batch*head count.
__device__ __forceinline__ void xcd_block128(int nx, int nbh, int& bx, int& bh) {
  const int lin = blockIdx.y * nx + blockIdx.x;
  if (TFB_ATTN128_XCD && nbh % 8 == 0) {
    const int xcd = lin & 7, idx = lin >> 3;
    bh = xcd + 8 * (idx / nx);
    bx = idx % nx;
  } else {
    bh = blockIdx.y;
    bx = blockIdx.x;
  }
}

// LDS row of a transposed tile: 64 tokens + 8 bytes of pad. With 32 banks and 64-bit accesses resolved per 16 lanes,
// a 136-byte stride puts the 16 rows a half-wavefront's fragment read touches on 16 different bank pairs, and the
// transposing writes (16 consecutive lanes along the tokens of one row) are conflict-free as well.
constexpr int TROW = 64 * 2 + 8;

// =========================================================================================== forward
// QG = query groups of 32 per wavefront. With QG = 2 every K / V^T fragment read from LDS feeds two MFMAs (half the LDS
// traffic per flop) and the two groups' softmax arithmetic and MFMAs are independent instruction streams that co-execute.
template <int D, int QG>
__global__ __launch_bounds__(256, (D == 64 && QG == 1) ? TFB_FWD_WPE : (QG == 1 ? TFB_FWD128_WPE : 1)) void attn_fwd_kernel(AttnT q, AttnT k, AttnT v, AttnT o, float* __restrict__ lse, int T,
                                                      int H, float sl2, int nw) {
  constexpr int DS = D / 16, DT = D / 32, NV = D / 64;
  constexpr int KROW = D * 2 + 16;
  constexpr int KBYTES = 64 * KROW, VBYTES = D * TROW, BUF = KBYTES + VBYTES;
  constexpr int QB = 128 * QG, QW = 32 * QG;  // queries per workgroup / per wavefront
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  int bx, bh;
  xcd_block128(gridDim.x, gridDim.y, bx, bh);
  const int qb = gridDim.x - 1 - bx;  // longest rows first
  const int b = bh / H, h = bh % H;
  const bf16_t* qp = q.p + b * q.sb + h * q.sh;
  const bf16_t* kp = k.p + b * k.sb + h * k.sh;
  const bf16_t* vp = v.p + b * v.sb + h * v.sh;
  bf16_t* op = o.p + b * o.sb + h * o.sh;
  const int q0 = qb * QB, qw0 = q0 + wave * QW;

  bf16x8 qf[QG][DS];
#pragma unroll
  for (int g = 0; g < QG; ++g)
#pragma unroll
    for (int s = 0; s < DS; ++s) qf[g][s] = *(const bf16x8*)(qp + (long)(qw0 + 32 * g + lr) * q.st + 16 * s + 8 * lh);

  const int ntiles = (q0 + QB) / 64;
  const bool vrole = wave < 2;
  const int t2 = tid & 127;
  MicroBlock mb[NV];  // V micro-blocks (waves 0,1) or DS K chunks (waves 2,3) share these registers

  auto gload = [&](int tile) {
    const int k0 = tile * 64;
    if (vrole) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        int m = t2 + i * 128;
        mb[i].load(vp, v.st, k0 + 4 * (m & 15), 8 * (m >> 4));
      }
    } else {
#pragma unroll
      for (int i = 0; i < DS; ++i) {
        int c = t2 + i * 128;
        int row = c / (D / 8), cc = c % (D / 8);
        mb[i / 4].g[i % 4] = *(const u32x4*)(kp + (long)(k0 + row) * k.st + cc * 8);
      }
    }
  };
  auto sstore = [&](uint8_t* buf) {
    if (vrole) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        int m = t2 + i * 128;
        mb[i].store_transposed(buf + KBYTES, TROW, 4 * (m & 15), 8 * (m >> 4));
      }
    } else {
#pragma unroll
      for (int i = 0; i < DS; ++i) {
        int c = t2 + i * 128;
        int row = c / (D / 8), cc = c % (D / 8);
        *(u32x4*)(buf + row * KROW + cc * 16) = mb[i / 4].g[i % 4];
      }
    }
  };

  f32x16 oacc[QG][DT];
  float m[QG], l[QG];
#pragma unroll
  for (int g = 0; g < QG; ++g) {
    m[g] = -1e30f;  // running maximum of the raw scores
    l[g] = 0.f;
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) oacc[g][i][e] = 0.f;
  }

  // band (nw > 0, QG = 1): the queries of 128-token tile qb see key tiles qb - nw + 1 .. qb only
  const int t0 = nw > 0 ? 2 * (qb - nw + 1 > 0 ? qb - nw + 1 : 0) : 0;
  gload(t0);
  sstore(smem);
  wait_all_loads();
  __syncthreads();

  for (int t = t0; t < ntiles; ++t) {
    const uint8_t* cur = smem + (t & 1) * BUF;
    const bool more = t + 1 < ntiles;
    if (more) gload(t + 1);
    const int k0 = t * 64;
    if (k0 <= qw0 + QW - 1) {
      f32x16 st[QG][2];
#pragma unroll
      for (int g = 0; g < QG; ++g)
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int e = 0; e < 16; ++e) st[g][kt][e] = 0.f;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int s = 0; s < DS; ++s) {
          bf16x8 a = lds16(cur, (kt * 32 + lr) * KROW + s * 32 + lh * 16);
#pragma unroll
          for (int g = 0; g < QG; ++g) st[g][kt] = mfma_bf16(a, qf[g][s], st[g][kt]);
        }
      const uint8_t* vt = cur + KBYTES;
#pragma unroll
      for (int g = 0; g < QG; ++g) {
        const int qg0 = qw0 + 32 * g;
        const bool diag = k0 + 63 > qg0;
        const int kbase = k0 + lh * 4 - (qg0 + lr);  // key - q for element (kt, e) is kbase + kt*32 + (e>>2)*8 + (e&3)
        float mx = m[g];
        if (diag) {  // wavefront-uniform; the per-element masking below is branch-free selects
#pragma unroll
          for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
              const bool future = kbase + kt * 32 + (e >> 2) * 8 + (e & 3) > 0;
              st[g][kt][e] = future ? -INFINITY : st[g][kt][e];
            }
        }
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int e = 0; e < 16; e += 2) mx = fmaxf(fmaxf(mx, st[g][kt][e]), st[g][kt][e + 1]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float alpha = fast_exp2((m[g] - mx) * sl2);
        m[g] = mx;
        l[g] *= alpha;
#pragma unroll
        for (int i = 0; i < DT; ++i)
#pragma unroll
          for (int e = 0; e < 16; ++e) oacc[g][i][e] *= alpha;
        const float negm = -mx * sl2;
        // 16 keys at a time: exponentials and packing (VALU) of one chunk run beside the PV MFMAs of the previous one
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int hf = 0; hf < 2; ++hf) {
            uint32_t w[4];
#pragma unroll
            for (int x = 0; x < 4; ++x) {
              const int e = 8 * hf + 2 * x;
              float p0 = fast_exp2(fmaf(st[g][kt][e], sl2, negm)), p1 = fast_exp2(fmaf(st[g][kt][e + 1], sl2, negm));
              w[x] = pack2bf(p0, p1);
              l[g] = sum2bf(w[x], l[g]);  // the row sum runs over the rounded values
            }
            const bf16x8 bb = frag_from(w[0], w[1], w[2], w[3]);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
              bf16x8 a = lds8x2(vt, (dt * 32 + lr) * TROW + (kt * 32 + 16 * hf + 4 * lh) * 2);
              oacc[g][dt] = mfma_bf16(a, bb, oacc[g][dt]);
            }
          }
      }
    }
    if (more) sstore(smem + ((t + 1) & 1) * BUF);
    __syncthreads();
  }

#pragma unroll
  for (int g = 0; g < QG; ++g) {
    const int myq = qw0 + 32 * g + lr;
    float lt = l[g] + __shfl_xor(l[g], 32, 64);
    const float inv = 1.0f / lt;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int d = dt * 32 + 8 * j + 4 * lh;
        u32x2 w = {pack2bf(oacc[g][dt][4 * j] * inv, oacc[g][dt][4 * j + 1] * inv),
                   pack2bf(oacc[g][dt][4 * j + 2] * inv, oacc[g][dt][4 * j + 3] * inv)};
        *(u32x2*)(op + (long)myq * o.st + d) = w;
      }
    if (lh == 0) lse[(long)bh * T + myq] = (m[g] * sl2 + log2f(lt)) * LN2;  // m is the raw-score maximum
  }
}

// =========================================================================================== delta
// delta[bh][t] = sum_d dO[b,t,h,d] * O[b,t,h,d] (fp32 of the bf16 values); 4 lanes per row.
template <int D>
__global__ __launch_bounds__(256) void attn_delta_kernel(AttnT o, AttnT go, float* __restrict__ delta, int T, int H, long rows) {
  long idx = (long)blockIdx.x * 256 + threadIdx.x;
  long row = idx >> 2;
  int part = (int)(idx & 3);
  if (row >= rows) return;
  int t = (int)(row % T);
  long bh = row / T;
  int b = (int)(bh / H), h = (int)(bh % H);
  const bf16_t* op = o.p + b * o.sb + h * o.sh + (long)t * o.st + part * (D / 4);
  const bf16_t* gp = go.p + b * go.sb + h * go.sh + (long)t * go.st + part * (D / 4);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < D / 32; ++i) {
    u32x4 a = *(const u32x4*)(op + 8 * i);
    u32x4 g = *(const u32x4*)(gp + 8 * i);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      s += bflo(a[w]) * bflo(g[w]);
      s += bfhi(a[w]) * bfhi(g[w]);
    }
  }
  s += __shfl_xor(s, 1, 64);
  s += __shfl_xor(s, 2, 64);
  if (part == 0) delta[row] = s;
}

// =========================================================================================== dK / dV
template <int D>
__global__ __launch_bounds__(256, D == 64 ? TFB_DKDV_WPE : TFB_DKDV128_WPE) void attn_bwd_dkdv_kernel(AttnT q, AttnT k, AttnT v, AttnT go, AttnT dk, AttnT dv,
                                                           const float* __restrict__ lse, const float* __restrict__ delta,
                                                           int T, int H, float scale, float sl2, int nw) {
  constexpr int DS = D / 16, DT = D / 32, NV = D / 64;
  constexpr int KROW = D * 2 + 16;
  constexpr int NBYTES = 64 * KROW, TBYTES = D * TROW;
  constexpr int OFF_QN = 0, OFF_GN = NBYTES, OFF_QT = 2 * NBYTES, OFF_GT = 2 * NBYTES + TBYTES;
  constexpr int OFF_L = 2 * NBYTES + 2 * TBYTES, BUF = OFF_L + 512;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  int kb, bh;  // low key blocks see the most query tiles: already longest first
  xcd_block128(gridDim.x, gridDim.y, kb, bh);
  const int b = bh / H, h = bh % H;
  const bf16_t* qp = q.p + b * q.sb + h * q.sh;
  const bf16_t* kp = k.p + b * k.sb + h * k.sh;
  const bf16_t* vp = v.p + b * v.sb + h * v.sh;
  const bf16_t* gp = go.p + b * go.sb + h * go.sh;
  const float* lsep = lse + (long)bh * T;
  const float* delp = delta + (long)bh * T;
  const int kw0 = kb * 128 + wave * 32, mykey = kw0 + lr;

  bf16x8 kf[DS], vf[DS];
#pragma unroll
  for (int s = 0; s < DS; ++s) {
    kf[s] = *(const bf16x8*)(kp + (long)mykey * k.st + 16 * s + 8 * lh);
    vf[s] = *(const bf16x8*)(vp + (long)mykey * v.st + 16 * s + 8 * lh);
  }

  // band (nw > 0): key tile kb is seen by the queries of tiles kb .. kb + nw - 1 only
  const int qt0 = kb * 2, nqt = nw > 0 && (kb + nw) * 2 < T / 64 ? (kb + nw) * 2 : T / 64;
  const bool qrole = wave < 2;
  const int t2 = tid & 127;
  MicroBlock mb[NV];
  float stat = 0.f;
  const float* statp = tid < 64 ? lsep : delp;  // wavefront 0 stages lse, the others delta (wavefront 1's copy is stored)

  auto gload = [&](int qt) {
    const int r0 = qt * 64;
    const bf16_t* src = qrole ? qp : gp;
    const long st_ = qrole ? q.st : go.st;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      int m = t2 + i * 128;
      mb[i].load(src, st_, r0 + 4 * (m & 15), 8 * (m >> 4));
    }
    // raw value only: any arithmetic here would make the wavefront wait for the loads it has just issued
    stat = statp[r0 + (tid & 63)];
  };
  auto sstore = [&](uint8_t* buf) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      int m = t2 + i * 128;
      mb[i].store_normal(buf + (qrole ? OFF_QN : OFF_GN), KROW, 4 * (m & 15), 8 * (m >> 4));
      mb[i].store_transposed(buf + (qrole ? OFF_QT : OFF_GT), TROW, 4 * (m & 15), 8 * (m >> 4));
    }
    if (tid < 128) ((float*)(buf + OFF_L))[tid] = tid < 64 ? -stat * LOG2E : stat;  // negated lse: the exponent is one fma
  };

  f32x16 dka[DT], dva[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      dka[i][e] = 0.f;
      dva[i][e] = 0.f;
    }

  gload(qt0);
  sstore(smem);
  wait_all_loads();
  __syncthreads();

  for (int qt = qt0; qt < nqt; ++qt) {
    const uint8_t* cur = smem + (TFB_BWD_NBUF == 2 ? ((qt - qt0) & 1) * BUF : 0);
    const bool more = qt + 1 < nqt;
    if (more) gload(qt + 1);
    const float* ls = (const float*)(cur + OFF_L);
#pragma unroll
    for (int qs = 0; qs < 2; ++qs) {
      const int qlo = qt * 64 + qs * 32;
      if (qlo + 31 < kw0) continue;  // every key of this wavefront is in the future of these queries
      f32x16 S, dP;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        S[e] = 0.f;
        dP[e] = 0.f;
      }
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        S = mfma_bf16(lds16(cur + OFF_QN, (qs * 32 + lr) * KROW + s * 32 + lh * 16), kf[s], S);
        dP = mfma_bf16(lds16(cur + OFF_GN, (qs * 32 + lr) * KROW + s * 32 + lh * 16), vf[s], dP);
      }
      const bool diag = kw0 + 31 > qlo;
      const int kq = mykey - (qlo + 4 * lh);  // key - q for element e is kq - (e>>2)*8 - (e&3)
      if (diag) {  // wavefront-uniform; masked scores become -inf (P = 0) through branch-free selects
#pragma unroll
        for (int e = 0; e < 16; ++e) S[e] = (kq - 8 * (e >> 2) - (e & 3) > 0) ? -INFINITY : S[e];
      }
      uint32_t pw[8], dsw[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        f32x4 L = *(const f32x4*)(ls + qs * 32 + 8 * j + 4 * lh);
        f32x4 Dl = *(const f32x4*)(ls + 64 + qs * 32 + 8 * j + 4 * lh);
        float p[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          p[i] = fast_exp2(fmaf(S[4 * j + i], sl2, L[i]));
        }
        uint32_t w0 = pack2bf(p[0], p[1]), w1 = pack2bf(p[2], p[3]);
        pw[2 * j] = w0;
        pw[2 * j + 1] = w1;
        float d0 = bflo(w0) * (dP[4 * j] - Dl[0]), d1 = bfhi(w0) * (dP[4 * j + 1] - Dl[1]);
        float d2 = bflo(w1) * (dP[4 * j + 2] - Dl[2]), d3 = bfhi(w1) * (dP[4 * j + 3] - Dl[3]);
        dsw[2 * j] = pack2bf(d0, d1);
        dsw[2 * j + 1] = pack2bf(d2, d3);
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          const int off = (dt * 32 + lr) * TROW + (qs * 32 + 16 * ks + 4 * lh) * 2;
          bf16x8 pb = frag_from(pw[4 * ks], pw[4 * ks + 1], pw[4 * ks + 2], pw[4 * ks + 3]);
          bf16x8 db = frag_from(dsw[4 * ks], dsw[4 * ks + 1], dsw[4 * ks + 2], dsw[4 * ks + 3]);
          dva[dt] = mfma_bf16(lds8x2(cur + OFF_GT, off), pb, dva[dt]);
          dka[dt] = mfma_bf16(lds8x2(cur + OFF_QT, off), db, dka[dt]);
        }
    }
    if (TFB_BWD_NBUF == 1) __syncthreads();
    if (more) sstore(smem + (TFB_BWD_NBUF == 2 ? ((qt + 1 - qt0) & 1) * BUF : 0));
    __syncthreads();
  }

  bf16_t* dkp = dk.p + b * dk.sb + h * dk.sh + (long)mykey * dk.st;
  bf16_t* dvp = dv.p + b * dv.sb + h * dv.sh + (long)mykey * dv.st;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int d = dt * 32 + 8 * j + 4 * lh;
      u32x2 wk = {pack2bf(dka[dt][4 * j] * scale, dka[dt][4 * j + 1] * scale),
                  pack2bf(dka[dt][4 * j + 2] * scale, dka[dt][4 * j + 3] * scale)};
      u32x2 wv = {pack2bf(dva[dt][4 * j], dva[dt][4 * j + 1]), pack2bf(dva[dt][4 * j + 2], dva[dt][4 * j + 3])};
      *(u32x2*)(dkp + d) = wk;
      *(u32x2*)(dvp + d) = wv;
    }
}

// =========================================================================================== dQ
template <int D>
__global__ __launch_bounds__(256, D == 64 ? TFB_DQ_WPE : 1) void attn_bwd_dq_kernel(AttnT q, AttnT k, AttnT v, AttnT go, AttnT dq,
                                                         const float* __restrict__ lse, const float* __restrict__ delta,
                                                         int T, int H, float scale, float sl2, int nw) {
  constexpr int DS = D / 16, DT = D / 32, NV = D / 64;
  constexpr int KROW = D * 2 + 16;
  constexpr int NBYTES = 64 * KROW, TBYTES = D * TROW;
  constexpr int OFF_KN = 0, OFF_VN = NBYTES, OFF_KT = 2 * NBYTES, BUF = 2 * NBYTES + TBYTES;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  int bx, bh;
  xcd_block128(gridDim.x, gridDim.y, bx, bh);
  const int qb = gridDim.x - 1 - bx;
  const int b = bh / H, h = bh % H;
  const bf16_t* qp = q.p + b * q.sb + h * q.sh;
  const bf16_t* kp = k.p + b * k.sb + h * k.sh;
  const bf16_t* vp = v.p + b * v.sb + h * v.sh;
  const bf16_t* gp = go.p + b * go.sb + h * go.sh;
  const int q0 = qb * 128, qw0 = q0 + wave * 32, myq = qw0 + lr;

  bf16x8 qf[DS], gf[DS];
#pragma unroll
  for (int s = 0; s < DS; ++s) {
    qf[s] = *(const bf16x8*)(qp + (long)myq * q.st + 16 * s + 8 * lh);
    gf[s] = *(const bf16x8*)(gp + (long)myq * go.st + 16 * s + 8 * lh);
  }
  const float myL = -lse[(long)bh * T + myq] * LOG2E;
  const float myD = delta[(long)bh * T + myq];

  const int ntiles = (q0 + 128) / 64;
  const bool krole = wave < 2;
  const int t2 = tid & 127;
  MicroBlock mb[NV];

  auto gload = [&](int tile) {
    const int k0 = tile * 64;
    if (krole) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        int m = t2 + i * 128;
        mb[i].load(kp, k.st, k0 + 4 * (m & 15), 8 * (m >> 4));
      }
    } else {
#pragma unroll
      for (int i = 0; i < DS; ++i) {
        int c = t2 + i * 128;
        int row = c / (D / 8), cc = c % (D / 8);
        mb[i / 4].g[i % 4] = *(const u32x4*)(vp + (long)(k0 + row) * v.st + cc * 8);
      }
    }
  };
  auto sstore = [&](uint8_t* buf) {
    if (krole) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        int m = t2 + i * 128;
        mb[i].store_normal(buf + OFF_KN, KROW, 4 * (m & 15), 8 * (m >> 4));
        mb[i].store_transposed(buf + OFF_KT, TROW, 4 * (m & 15), 8 * (m >> 4));
      }
    } else {
#pragma unroll
      for (int i = 0; i < DS; ++i) {
        int c = t2 + i * 128;
        int row = c / (D / 8), cc = c % (D / 8);
        *(u32x4*)(buf + OFF_VN + row * KROW + cc * 16) = mb[i / 4].g[i % 4];
      }
    }
  };

  f32x16 dqa[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) dqa[i][e] = 0.f;

  const int t0 = nw > 0 ? 2 * (qb - nw + 1 > 0 ? qb - nw + 1 : 0) : 0;  // band: key tiles qb - nw + 1 .. qb
  gload(t0);
  sstore(smem);
  wait_all_loads();
  __syncthreads();

  for (int t = t0; t < ntiles; ++t) {
    const uint8_t* cur = smem + (TFB_BWD_NBUF == 2 ? (t & 1) * BUF : 0);
    const bool more = t + 1 < ntiles;
    if (more) gload(t + 1);
    const int k0 = t * 64;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      const int klo = k0 + kt * 32;
      if (klo > qw0 + 31) continue;
      f32x16 S, dP;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        S[e] = 0.f;
        dP[e] = 0.f;
      }
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        S = mfma_bf16(lds16(cur + OFF_KN, (kt * 32 + lr) * KROW + s * 32 + lh * 16), qf[s], S);
        dP = mfma_bf16(lds16(cur + OFF_VN, (kt * 32 + lr) * KROW + s * 32 + lh * 16), gf[s], dP);
      }
      const bool diag = klo + 31 > qw0;
      const int kbase = klo + lh * 4 - myq;
      if (diag) {
#pragma unroll
        for (int e = 0; e < 16; ++e) S[e] = (kbase + (e >> 2) * 8 + (e & 3) > 0) ? -INFINITY : S[e];
      }
      uint32_t dsw[8];
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        float p0 = fast_exp2(fmaf(S[e], sl2, myL)), p1 = fast_exp2(fmaf(S[e + 1], sl2, myL));
        uint32_t w = pack2bf(p0, p1);
        dsw[e >> 1] = pack2bf(bflo(w) * (dP[e] - myD), bfhi(w) * (dP[e + 1] - myD));
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          bf16x8 a = lds8x2(cur + OFF_KT, (dt * 32 + lr) * TROW + (kt * 32 + 16 * ks + 4 * lh) * 2);
          bf16x8 bb = frag_from(dsw[4 * ks], dsw[4 * ks + 1], dsw[4 * ks + 2], dsw[4 * ks + 3]);
          dqa[dt] = mfma_bf16(a, bb, dqa[dt]);
        }
    }
    if (TFB_BWD_NBUF == 1) __syncthreads();
    if (more) sstore(smem + (TFB_BWD_NBUF == 2 ? ((t + 1) & 1) * BUF : 0));
    __syncthreads();
  }

  bf16_t* dqp = dq.p + b * dq.sb + h * dq.sh + (long)myq * dq.st;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int d = dt * 32 + 8 * j + 4 * lh;
      u32x2 w = {pack2bf(dqa[dt][4 * j] * scale, dqa[dt][4 * j + 1] * scale),
                 pack2bf(dqa[dt][4 * j + 2] * scale, dqa[dt][4 * j + 3] * scale)};
      *(u32x2*)(dqp + d) = w;
    }
}

template <class K>
int set_lds(K kern, int bytes) {
  return hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess ? TFB_OK
                                                                                                                 : TFB_ERR_LAUNCH;
}

AttnT mk(const void* p, const long* s) { return AttnT{(bf16_t*)p, s[0], s[1], s[2]}; }

bool strides_ok(const long* s) { return s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0; }

template <int D, int QG>
int fwd_launch(AttnT q, AttnT k, AttnT v, AttnT o, float* lse, int B, int H, int T, float scale, int nw, hipStream_t s) {
  constexpr int BUF = 64 * (D * 2 + 16) + D * TROW;
  static bool once = false;
  if (!once) {
    if (set_lds(attn_fwd_kernel<D, QG>, 2 * BUF) != TFB_OK) return TFB_ERR_LAUNCH;
    once = true;
  }
  hipLaunchKernelGGL((attn_fwd_kernel<D, QG>), dim3(T / (128 * QG), B * H), dim3(256), 2 * BUF, s, q, k, v, o, lse, T, H,
                     scale * LOG2E, nw);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

template <int D>
int fwd_impl(AttnT q, AttnT k, AttnT v, AttnT o, float* lse, int B, int H, int T, float scale, int nw, hipStream_t s) {
  // two query groups per wavefront when the sequence splits into 256-query blocks and the registers allow (D = 64);
  // a band needs one 128-token tile per workgroup
  if (TFB_FWD_QG2 && D == 64 && T % 256 == 0 && nw <= 0)
    return fwd_launch<D, (D == 64 ? 2 : 1)>(q, k, v, o, lse, B, H, T, scale, 0, s);
  return fwd_launch<D, 1>(q, k, v, o, lse, B, H, T, scale, nw, s);
}

template <int D>
int bwd_impl(AttnT q, AttnT k, AttnT v, AttnT o, AttnT go, AttnT dq, AttnT dk, AttnT dv, const float* lse, float* delta, int B,
             int H, int T, float scale, int nw, hipStream_t s) {
  constexpr int NB = 64 * (D * 2 + 16), TB = D * TROW;
  constexpr int BUF1 = 2 * NB + 2 * TB + 512, BUF2 = 2 * NB + TB;
  static bool once = false;
  if (!once) {
    if (set_lds(attn_bwd_dkdv_kernel<D>, TFB_BWD_NBUF * BUF1) != TFB_OK) return TFB_ERR_LAUNCH;
    if (set_lds(attn_bwd_dq_kernel<D>, TFB_BWD_NBUF * BUF2) != TFB_OK) return TFB_ERR_LAUNCH;
    once = true;
  }
  const long rows = (long)B * H * T;
  hipLaunchKernelGGL(attn_delta_kernel<D>, dim3((unsigned)((rows * 4 + 255) / 256)), dim3(256), 0, s, o, go, delta, T, H, rows);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(attn_bwd_dkdv_kernel<D>, dim3(T / 128, B * H), dim3(256), TFB_BWD_NBUF * BUF1, s, q, k, v, go, dk, dv, lse, delta, T, H,
                     scale, scale * LOG2E, nw);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(attn_bwd_dq_kernel<D>, dim3(T / 128, B * H), dim3(256), TFB_BWD_NBUF * BUF2, s, q, k, v, go, dq, lse, delta, T, H, scale,
                     scale * LOG2E, nw);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

}  // namespace

// D = 64 runs the kernels of attention64.hip (direct-to-LDS tile loads, transposed LDS fragment reads).
int tfb_attn64_fwd_impl(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs, void* o,
                        const long* os, float* lse, int B, int H, int T, float scale, int nw, hipStream_t s);
int tfb_attn64_bwd_impl(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs,
                        const void* o, const long* os, const void* go, const long* gos, void* dq, const long* dqs, void* dk,
                        const long* dks, void* dv, const long* dvs, const float* lse, float* stats, int B, int H, int T,
                        float scale, const void* cos_t, const void* sin_t, int nw, hipStream_t s);

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
  return fwd_impl<128>(mk(q, qs), mk(k, ks), mk(v, vs), mk(o, os), (float*)lse, B, H, T, scale, nw, s);
}
extern "C" int tfb_attn_fwd(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs, void* o,
                            const long* os, void* lse, int B, int H, int T, int D, float scale, void* stream) {
  return tfb_attn_fwd_band(q, qs, k, ks, v, vs, o, os, lse, B, H, T, D, scale, 0, stream);
}

// delta: fp32 [2][B*H][T] scratch (row dot products, then -lse log2 e). dq, dk, dv may alias thirds of one dqkv buffer.
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
  return bwd_impl<128>(mk(q, qs), mk(k, ks), mk(v, vs), mk(o, os), mk(go, gos), mk(dq, dqs), mk(dk, dks), mk(dv, dvs),
                       (const float*)lse, (float*)delta, B, H, T, scale, nw, s);
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
// tfb_attn_bwd needs fp32 [2][B*H][T] of device scratch (the row statistics its first kernel leaves for the second:
// a pre-pass's for D = 128, the dQ kernel's for D = 64) and takes it from the caller. Code under HIP graph capture, tight serving loops and harnesses that forbid
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

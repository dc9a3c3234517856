// Causal flash attention for head dimension 64 on gfx950: the kernels the C-ABI entry points in attention.hip run for
// D = 64 (their arithmetic contract and the reference citations are stated there).
//
// Data movement: a 64-token x 64-element bf16 tile is 64 rows of 128 bytes. Tiles go from global memory straight
// into LDS with global_load_lds_dwordx4 (8 tokens per instruction, no staging registers); 16-byte chunk c of token t
// sits at slot c ^ swz(t), swz(t) = 4 ((t >> 1) & 1) | ((t >> 2) & 3). One copy of a tile then serves both MFMA
// operand forms without bank conflicts (LDS: 64 banks of 4 bytes):
//   * token-major fragments (token = MFMA row, contraction over d): one ds_read_b128 per lane; 16 consecutive tokens
//     of one chunk fall on 16 different 16-byte bank groups;
//   * transposed fragments (d = MFMA row, contraction over tokens): two ds_read_b64_tr_b16 per lane, whose 16-lane
//     transpose hands lane i four consecutive tokens of element i when lane j points at (token0 + j / 4, d0 + 4 (j % 4));
//     the four tokens of a 32-lane access fall on four different 64-byte bank quarters.
// Two LDS stages (separate __shared__ objects: the compiler can tell reads of one stage from the loads in flight into
// the other), one barrier per tile.
//
// Work layout: a wavefront owns 32 queries (forward, dQ) or 32 keys (dK/dV) as the MFMA column index, so every row
// statistic is one scalar per lane and the packed score registers are directly the B operand of the next product.
//
// What bounds these kernels is the SIMD's vector issue port, not the matrix pipe: measured on gfx950 with one
// wavefront issuing MFMAs and another VALU instructions on the same SIMD, a 32x32x16 MFMA costs the port about 18
// cycles, a v_exp_f32 8 and any other VALU instruction 4, and the main loops below run at 80-93 % of the time that sum
// predicts (dQ: 12 MFMA + 16 exp + 66 other per 32x32 block = 608 cycles against 384 cycles of matrix pipe). The
// forward and dQ main loops are therefore software-pipelined: the scores of the next block are issued while the vector
// ALU turns the current block's into P (dS), dealt out 1 MFMA : ~10 VALU by scheduling-group barriers, so the matrix
// pipe's work hides under the vector work inside one wavefront instead of depending on the other resident wavefront
// being in the opposite phase. dK/dV has no registers left for a second set of scores at two wavefronts per SIMD and
// keeps the plain loop.
#include <type_traits>
#include "common.hpp"

// wavefronts per SIMD the kernels are compiled for (register budget 512 / n)
#ifndef TFB_DKDV64_QT
#define TFB_DKDV64_QT 2
#endif
#ifndef TFB_DKDV64_PIPE
#define TFB_DKDV64_PIPE 1  // dK/dV: the stages after the diagonal one as a software pipeline over 32-query blocks
#endif
#ifndef TFB_DKDV64_VALU_PER_MFMA
#define TFB_DKDV64_VALU_PER_MFMA 10
#endif
#ifndef TFB_DQ64_WPE
#define TFB_DQ64_WPE 2
#endif
#ifndef TFB_DQ64_VALU_PER_MFMA
#define TFB_DQ64_VALU_PER_MFMA 10
#endif
#ifndef TFB_FWD64_VALU_PER_MFMA
#define TFB_FWD64_VALU_PER_MFMA 12
#endif
#ifndef TFB_FWD64_WPE
#define TFB_FWD64_WPE 2
#endif
#ifndef TFB_ATTN_DELTA_IN_DQ
#define TFB_ATTN_DELTA_IN_DQ 1  // the dQ kernel makes the rows' -delta and -lse / scale itself (0: the separate pre-pass)
#endif

namespace {

struct AttnT {
  bf16_t* p;
  long sb, sh, st;
};

typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void glb_void_t;
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4_t;

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
constexpr int TILE = 64 * 128;  // bytes of one staged tile

__device__ __forceinline__ f32x16 mfma_bf16(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ bf16x8 frag_from(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  u32x4 v = {a, b, c, d};
  return __builtin_bit_cast(bf16x8, v);
}
__device__ __forceinline__ void wait_all_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }  // s_waitcnt vmcnt(0)

// Workgroup -> (block along the sequence, batch*head): consecutive workgroup ids are dealt round-robin to the 8 XCDs,
// each with its own L2, so the ids are re-dealt to keep all sequence blocks of one (batch, head) - which stream the same
// K/V (or Q/dO) tiles - on one XCD. nx = blocks per (batch, head), nbh = batch*head count.
__device__ __forceinline__ void xcd_block(int nx, int nbh, int& bx, int& bh) {
  const int lin = blockIdx.y * nx + blockIdx.x;
  if (nbh % 8 == 0) {
    const int xcd = lin & 7, idx = lin >> 3;
    bh = xcd + 8 * (idx / nx);
    bx = idx % nx;
  } else {
    bh = blockIdx.y;
    bx = blockIdx.x;
  }
}

// Causal work per 128-token block grows linearly along the sequence, and workgroups are dispatched in id order: with one
// block per workgroup the heaviest blocks of the last (batch, head) pairs start when most of the grid has drained and
// run on alone (for 16 blocks x 192 pairs on 512 slots: 17 % of the kernel's time). When the block count nx is even a
// workgroup therefore does block i and then block nx - 1 - i (gridDim.x = nx / 2): every workgroup carries the same
// work. `heavy_last` = the work grows with the block index (query blocks) rather than falls (key blocks); the heavier
// block of the pair runs first either way.
__device__ __forceinline__ int paired_passes(int nx) { return (int)gridDim.x * 2 == nx ? 2 : 1; }
__device__ __forceinline__ int paired_block(int nx, int bx, int pass, bool heavy_last) {
  const int first = heavy_last ? nx - 1 - bx : bx;
  return pass == 0 ? first : nx - 1 - first;
}
// First 64-key tile a 128-token query tile qb sees under a band of nw key tiles (a query of tile i sees the keys k <= q
// of tiles i - nw + 1 .. i: band_mask, round2/source/kernels/nki_attn_bandpro.py:1654); 0 without a band (nw <= 0).
__device__ __forceinline__ int band_first_tile(int qb, int nw) { return nw > 0 && qb - nw + 1 > 0 ? 2 * (qb - nw + 1) : 0; }
__host__ inline unsigned paired_grid(int nx) { return (unsigned)(nx % 2 == 0 ? nx / 2 : nx); }

__device__ __forceinline__ int swz(int t) { return (((t >> 1) & 1) << 2) | ((t >> 2) & 3); }

// Of the two workgroups that start together on a CU, the one in an odd wavefront slot (HW_ID.wave_id bit 0) begins
// ~3.6 us late, once, in the first round: the pair then alternates between its memory-bound and MFMA-bound phases
// instead of running them in lockstep (measured -0.17 ms per training step over the three kernels).
#ifndef TFB_ATTN_STAGGER
#define TFB_ATTN_STAGGER 1
#endif
__device__ __forceinline__ void stagger_start(int slots) {  // slots: workgroups resident at once (the first round)
  if (TFB_ATTN_STAGGER > 0 && (int)(blockIdx.x + gridDim.x * blockIdx.y) < slots) {
    if (__builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 4) & 1)  // getreg(size 4, offset 0, HW_REG_HW_ID)
      for (int i = 0; i < TFB_ATTN_STAGGER; ++i) __builtin_amdgcn_s_sleep(127);
  }
}

// This wavefront's share (NI of the 4 NI instructions) of a (32 NI)-token tile load. `rows` points at token 0 of the
// tile, `stride` = bytes between tokens.
template <int NI>
struct TileLoad {
  uint32_t voff;
  int wave;
  __device__ __forceinline__ void init(long stride, int wave_, int lane) {
    wave = wave_;
    const int lrow = lane >> 3;
    // token = 8 g + lrow with g = wave + 4 i: swz depends on g only through g & 1 = wave & 1
    const int chunk = (lane & 7) ^ swz(8 * wave + lrow);
    voff = (uint32_t)(lrow * stride + chunk * 16);
  }
  __device__ __forceinline__ void issue(const uint8_t* rows, long stride, uint8_t* lds) const {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int g = wave + 4 * i;
      __builtin_amdgcn_global_load_lds((glb_void_t*)(rows + 8L * g * stride + (size_t)voff), (lds_void_t*)(lds + g * 1024), 16,
                                       0, 0);
    }
  }
};

// token-major fragment: token = 32 * half + (lane & 31), elements 16 s + 8 (lane >> 5) .. + 7
__device__ __forceinline__ bf16x8 frag_rows(const uint8_t* tile, int half, int s, int lr, int lh) {
  const int t = 32 * half + lr;
  return *(const bf16x8*)(tile + t * 128 + (((2 * s + lh) ^ swz(t)) << 4));
}
// transposed fragment: element (MFMA row) 32 dt + (lane & 31); tokens tok0 + 4 lh + {0..3} and tok0 + 8 + 4 lh + {0..3}
// (the order in which a lane's packed score registers hold a 16-token block)
__device__ __forceinline__ bf16x8 frag_cols(const uint8_t* tile, int dt, int tok0, int lane) {
  const int g4 = lane >> 4, j = lane & 15;
  const int d = 32 * dt + 16 * (g4 & 1) + 4 * (j & 3);
  const int t = tok0 + 4 * (g4 >> 1) + (j >> 2);
  const int off0 = t * 128 + ((((d >> 3) ^ swz(t))) << 4) + ((d & 4) << 1);
  const int off1 = (t + 8) * 128 + ((((d >> 3) ^ swz(t + 8))) << 4) + ((d & 4) << 1);
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)(tile + off0));
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)(tile + off1));
  const s16x8 v = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  return __builtin_bit_cast(bf16x8, v);
}

// Store one token's gradient row from the two 32-element halves a lane's accumulators hold (elements 8 j + 4 lh + i of
// each half), scaled and rounded once to bf16; with cos / sin tables ([T][32] bf16) the inverse RoPE rotation
// (y1 = x1 c - x2 s, y2 = x2 c + x1 s on the rounded values, rounded again: what a separate pass over the bf16
// gradient computes) is applied on the way out.
__device__ __forceinline__ void store_grad_row(const f32x16 (&acc)[2], float scale, bf16_t* row, const bf16_t* cs,
                                               const bf16_t* sn, int tok, int lh) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int d = 8 * j + 4 * lh;
    u32x2 w1 = {pack2bf(acc[0][4 * j] * scale, acc[0][4 * j + 1] * scale),
                pack2bf(acc[0][4 * j + 2] * scale, acc[0][4 * j + 3] * scale)};
    u32x2 w2 = {pack2bf(acc[1][4 * j] * scale, acc[1][4 * j + 1] * scale),
                pack2bf(acc[1][4 * j + 2] * scale, acc[1][4 * j + 3] * scale)};
    if (cs) {
      const u32x2 c = *(const u32x2*)(cs + (long)tok * 32 + d), s = *(const u32x2*)(sn + (long)tok * 32 + d);
      u32x2 o1, o2;
#pragma unroll
      for (int x = 0; x < 2; ++x) {
        const float a0 = bflo(w1[x]), a1 = bfhi(w1[x]), b0 = bflo(w2[x]), b1 = bfhi(w2[x]);
        const float c0 = bflo(c[x]), c1 = bfhi(c[x]), s0 = -bflo(s[x]), s1 = -bfhi(s[x]);
        o1[x] = pack2bf(a0 * c0 + b0 * s0, a1 * c1 + b1 * s1);
        o2[x] = pack2bf(b0 * c0 - a0 * s0, b1 * c1 - a1 * s1);
      }
      w1 = o1;
      w2 = o2;
    }
    *(u32x2*)(row + d) = w1;
    *(u32x2*)(row + 32 + d) = w2;
  }
}

// =========================================================================================== forward
__global__ __launch_bounds__(256, TFB_FWD64_WPE) void attn64_fwd_kernel(AttnT q, AttnT k, AttnT v, AttnT o, float* __restrict__ lse,
                                                            int T, int H, float sl2, int nw, int slots) {
  __shared__ __attribute__((aligned(1024))) uint8_t st0[2 * TILE];
  __shared__ __attribute__((aligned(1024))) uint8_t st1[2 * TILE];
  const int tid = threadIdx.x, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  stagger_start(slots);
  int bx, bh;
  xcd_block(gridDim.x, gridDim.y, bx, bh);
  const int b = bh / H, h = bh % H;
  const bf16_t* qp = q.p + b * q.sb + h * q.sh;
  const uint8_t* kp = (const uint8_t*)(k.p + b * k.sb + h * k.sh);
  const uint8_t* vp = (const uint8_t*)(v.p + b * v.sb + h * v.sh);
  bf16_t* op = o.p + b * o.sb + h * o.sh;
  const int nx = T / 128, npass = paired_passes(nx);
  for (int pass = 0; pass < npass; ++pass) {
  const int qb = paired_block(nx, bx, pass, true);
  const int q0 = qb * 128, qw0 = q0 + wave * 32;
  const long kst = k.st * 2, vst = v.st * 2;

  bf16x8 qf[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) qf[s] = *(const bf16x8*)(qp + (long)(qw0 + lr) * q.st + 16 * s + 8 * lh);

  TileLoad<2> lk, lv;
  lk.init(kst, wave, lane);
  lv.init(vst, wave, lane);
  auto issue = [&](uint8_t* st, int tile) {
    lk.issue(kp + (long)tile * 64 * kst, kst, st);
    lv.issue(vp + (long)tile * 64 * vst, vst, st + TILE);
  };

  f32x16 oacc[2];
  float m = -1e30f, l = 0.f;  // running maximum of the raw scores, running sum
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[i][e] = 0.f;

  // One 64-key tile against the wavefront's 32 queries, in steps that the main loop overlaps across tiles.
  // (1) raw scores S = K Q^T (key = MFMA row: a lane holds 32 keys of one query)
  auto scores = [&](const uint8_t* st, f32x16 (&sc)[2]) {
    bf16x8 ka[2][4];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int s = 0; s < 4; ++s) ka[kt][s] = frag_rows(st, kt, s, lr, lh);
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) sc[kt][e] = 0.f;
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) sc[kt] = mfma_bf16(ka[kt][s], qf[s], sc[kt]);
  };
  // (2) the V^T fragments of the second product
  auto load_vT = [&](const uint8_t* st, bf16x8 (&va)[2][2][2]) {
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) va[kt][hf][dt] = frag_cols(st + TILE, dt, kt * 32 + 16 * hf, lane);
  };
  // (3) the row maximum including this tile
  auto row_max = [&](const f32x16 (&sc)[2]) {
    float mx = m;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 16; e += 2) mx = fmaxf(fmaxf(mx, sc[kt][e]), sc[kt][e + 1]);
    return fmaxf(mx, __shfl_xor(mx, 32, 64));
  };
  // (4) The reference point m of the exponentials only has to keep them in range: it follows the running maximum when
  // some row's maximum has grown by more than 2^8 (always on a row's first tile, m = -1e30), which after the first few
  // tiles is rare, and the 33 multiplications that rescale l and the output accumulators are skipped otherwise.
  // O = sum p v / sum p and lse = m + log(sum p) do not depend on the reference point.
  auto follow_max = [&](float mx) {
    if (__builtin_amdgcn_ballot_w64((mx - m) * sl2 > 8.0f)) {
      const float alpha = fast_exp2((m - mx) * sl2);
      m = mx;
      l *= alpha;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[i][e] *= alpha;
    }
  };
  // (5) P = exp2(sl2 (S - m)) rounded to bf16 and packed as B operands; the row sum runs over the rounded values
  auto softmax = [&](const f32x16 (&sc)[2], uint32_t (&pw)[2][2][4]) {
    const float negm = -m * sl2;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          const int e = 8 * hf + 2 * x;
          const float p0 = fast_exp2(fmaf(sc[kt][e], sl2, negm)), p1 = fast_exp2(fmaf(sc[kt][e + 1], sl2, negm));
          pw[kt][hf][x] = pack2bf(p0, p1);
          l = sum2bf(pw[kt][hf][x], l);
        }
  };
  // (6) O += P V
  auto accumulate = [&](const bf16x8 (&va)[2][2][2], const uint32_t (&pw)[2][2][4]) {
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const bf16x8 bb = frag_from(pw[kt][hf][0], pw[kt][hf][1], pw[kt][hf][2], pw[kt][hf][3]);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) oacc[dt] = mfma_bf16(va[kt][hf][dt], bb, oacc[dt]);
      }
  };
  // MFMA and VALU instructions of one scheduling region dealt out alternately (8 MFMAs, `per` VALU instructions each)
  auto interleave = [&](auto per) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x402, decltype(per)::value, 0);
    }
  };

  // State carried between tiles: the scores of the tile about to be normalised (computed one step ahead, while the
  // previous tile's exponentials ran) and the P / V^T operands of the previous tile, whose product into O runs under
  // this tile's row maximum.
  f32x16 scA[2], scB[2];
  bf16x8 pva[2][2][2];
  uint32_t ppw[2][2][4];
#pragma unroll
  for (int kt = 0; kt < 2; ++kt)
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
      for (int x = 0; x < 4; ++x) ppw[kt][hf][x] = 0u;
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) pva[kt][hf][dt] = bf16x8{};
    }
  // a tile with all keys before the workgroup's queries: `cur` holds tile t (scores in scC), `nxt` tile t + 1 (scores
  // left in scN); tile t + 2 replaces t
  auto full_tile = [&](uint8_t* cur, const uint8_t* nxt, int t, f32x16 (&scC)[2], f32x16 (&scN)[2]) {
    const float mx = row_max(scC);
    accumulate(pva, ppw);
    interleave(std::integral_constant<int, 3>{});
    follow_max(mx);
    load_vT(cur, pva);
    __syncthreads();  // tile t + 1 has landed; every wavefront has its fragments of tile t
    issue(cur, t + 2);
    scores(nxt, scN);
    softmax(scC, ppw);
    interleave(std::integral_constant<int, TFB_FWD64_VALU_PER_MFMA>{});
  };
  // one of the two tiles over the workgroup's own tokens: skipped when in the wavefront's future, masked on its diagonal
  auto diagonal_tile = [&](const uint8_t* st, int tile, f32x16 (&sc)[2]) {
    const int k0 = tile * 64;
    if (k0 > qw0 + 31) return;
    bf16x8 va[2][2][2];
    uint32_t pw[2][2][4];
    load_vT(st, va);
    if (k0 + 63 > qw0) {  // wavefront-uniform; the per-element masking is branch-free selects
      const int kbase = k0 + lh * 4 - (qw0 + lr);  // key - q for element (kt, e) is kbase + kt*32 + (e>>2)*8 + (e&3)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const bool future = kbase + kt * 32 + (e >> 2) * 8 + (e & 3) > 0;
          sc[kt][e] = future ? -INFINITY : sc[kt][e];
        }
    }
    follow_max(row_max(sc));
    softmax(sc, pw);
    accumulate(va, pw);
  };

  const int n = (q0 + 128) / 64;  // even; tiles n - 2 and n - 1 cover the workgroup's own 128 tokens
  const int t0 = band_first_tile(qb, nw);  // even; 0 without a band
  issue(st0, t0);
  wait_all_loads();
  __syncthreads();
  issue(st1, t0 + 1);
  scores(st0, scA);
  for (int t = t0; t + 2 < n; t += 2) {
    full_tile(st0, st1, t, scA, scB);
    full_tile(st1, st0, t + 1, scB, scA);
  }
  accumulate(pva, ppw);  // the last full tile's product (zeros when there was none)
  diagonal_tile(st0, n - 2, scA);
  __syncthreads();
  scores(st1, scB);
  diagonal_tile(st1, n - 1, scB);

  const int myq = qw0 + lr;
  const float lt = l + __shfl_xor(l, 32, 64);
  const float inv = 1.0f / lt;
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int d = dt * 32 + 8 * j + 4 * lh;
      u32x2 w = {pack2bf(oacc[dt][4 * j] * inv, oacc[dt][4 * j + 1] * inv),
                 pack2bf(oacc[dt][4 * j + 2] * inv, oacc[dt][4 * j + 3] * inv)};
      *(u32x2*)(op + (long)myq * o.st + d) = w;
    }
  if (lh == 0) lse[(long)bh * T + myq] = (m * sl2 + log2f(lt)) * LN2;  // m is the raw-score maximum
  __syncthreads();  // the stages are free for the partner block
  }
}

// =========================================================================================== delta
// stats[0][bh][t] = -sum_d dO * O (fp32 of the bf16 values); stats[1][bh][t] = -lse / scale; 4 lanes per row. Both are
// the values the backward kernels start their dP and S accumulators from: the MFMAs then deliver dP - delta and
// S - lse / scale, and P = exp2(scale log2(e) (S - lse / scale)) needs no further row term.
__global__ __launch_bounds__(256) void attn64_delta_kernel(AttnT o, AttnT go, const float* __restrict__ lse,
                                                           float* __restrict__ stats, int T, int H, long rows, float inv_scale) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long row = idx >> 2;
  const int part = (int)(idx & 3);
  if (row >= rows) return;
  const int t = (int)(row % T);
  const long bh = row / T;
  const int b = (int)(bh / H), h = (int)(bh % H);
  const bf16_t* op = o.p + b * o.sb + h * o.sh + (long)t * o.st + part * 16;
  const bf16_t* gp = go.p + b * go.sb + h * go.sh + (long)t * go.st + part * 16;
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
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
  if (part == 0) {
    stats[row] = -s;
    stats[rows + row] = -lse[row] * inv_scale;
  }
}

// =========================================================================================== dK / dV
__global__ __launch_bounds__(256, 2) void attn64_dkdv_kernel(AttnT q, AttnT k, AttnT v, AttnT go, AttnT dk, AttnT dv,
                                                             const float* __restrict__ stats, long rows, int T, int H,
                                                             float scale, float sl2, const bf16_t* __restrict__ cs,
                                                             const bf16_t* __restrict__ sn, int nw, int slots) {
  constexpr int QT = TFB_DKDV64_QT;       // 64-query tiles per LDS stage (one barrier per stage)
  constexpr int R = 64 * QT, RT = R * 128;  // rows and bytes of a staged Q (dO) tile
  constexpr int STAGE = 2 * RT + 8 * R;    // Q tile, dO tile, R x (-lse / scale), R x (-delta)
  __shared__ __attribute__((aligned(1024))) uint8_t st0[STAGE];
  __shared__ __attribute__((aligned(1024))) uint8_t st1[STAGE];
  const int tid = threadIdx.x, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  stagger_start(slots);
  int bx, bh;
  xcd_block(gridDim.x, gridDim.y, bx, bh);
  const int b = bh / H, h = bh % H;
  const uint8_t* qp = (const uint8_t*)(q.p + b * q.sb + h * q.sh);
  const uint8_t* gp = (const uint8_t*)(go.p + b * go.sb + h * go.sh);
  const bf16_t* kp = k.p + b * k.sb + h * k.sh;
  const bf16_t* vp = v.p + b * v.sb + h * v.sh;
  const float* delp = stats + (long)bh * T;
  const float* nlp = stats + rows + (long)bh * T;
  const int nx = T / 128, npass = paired_passes(nx);
  for (int pass = 0; pass < npass; ++pass) {
  const int kb = paired_block(nx, bx, pass, false);  // low key blocks see the most query tiles
  const int kw0 = kb * 128 + wave * 32, mykey = kw0 + lr;
  const long qst = q.st * 2, gst = go.st * 2;

  bf16x8 kf[4], vf[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    kf[s] = *(const bf16x8*)(kp + (long)mykey * k.st + 16 * s + 8 * lh);
    vf[s] = *(const bf16x8*)(vp + (long)mykey * v.st + 16 * s + 8 * lh);
  }

  TileLoad<2 * QT> lq, lg;
  lq.init(qst, wave, lane);
  lg.init(gst, wave, lane);
  // T / 64 - 2 kb is even; with a band the keys of tile kb are seen by the queries of tiles kb .. kb + nw - 1 only
  const int qt0 = kb * 2, nall = (T / 64 - qt0) / QT, n = nw > 0 && nw < nall ? nw : nall;
  static_assert(QT == 2, "a stage is one 128-token tile of queries");
  auto issue = [&](uint8_t* st, int i) {
    const long r0 = (long)qt0 * 64 + (long)i * R;
    lq.issue(qp + r0 * qst, qst, st);
    lg.issue(gp + r0 * gst, gst, st + RT);
    // the row statistics: R floats each, 4-byte loads (wavefront 0: -lse / scale, wavefront 1: -delta)
    if (wave < 2) {
      const float* src = (wave == 0 ? nlp : delp) + r0;
#pragma unroll
      for (int x = 0; x < QT; ++x)
        __builtin_amdgcn_global_load_lds((glb_void_t*)(src + 64 * x + lane), (lds_void_t*)(st + 2 * RT + wave * 4 * R + 256 * x),
                                         4, 0, 0);
    }
  };

  f32x16 dka[2], dva[2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      dka[i][e] = 0.f;
      dva[i][e] = 0.f;
    }

  auto compute = [&](const uint8_t* st, int i) __attribute__((always_inline)) {
    const uint8_t* qt_ = st;
    const uint8_t* gt_ = st + RT;
    const float* ls = (const float*)(st + 2 * RT);
    const int qbase = qt0 * 64 + i * R;
#pragma unroll
    for (int qs = 0; qs < 2 * QT; ++qs) {
      const int qlo = qbase + qs * 32;
      if (qlo + 31 < kw0) continue;  // every key of this wavefront is in the future of these queries
      bf16x8 qa[4], ga[4];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        qa[s] = frag_rows(qt_, qs, s, lr, lh);
        ga[s] = frag_rows(gt_, qs, s, lr, lh);
      }
      // the accumulators start from the rows' -lse / scale and -delta
      f32x16 S, dP;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x4 L = *(const f32x4*)(ls + qs * 32 + 8 * j + 4 * lh);
        const f32x4 Dl = *(const f32x4*)(ls + R + qs * 32 + 8 * j + 4 * lh);
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          S[4 * j + x] = L[x];
          dP[4 * j + x] = Dl[x];
        }
      }
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        S = mfma_bf16(qa[s], kf[s], S);
        dP = mfma_bf16(ga[s], vf[s], dP);
      }
      // transposed fragments for the second pair of products: independent of the arithmetic below, so they are
      // requested first and arrive while the exponentials run
      bf16x8 gT[2][2], qT[2][2];
#pragma unroll
      for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          gT[dt][ks] = frag_cols(gt_, dt, qs * 32 + 16 * ks, lane);
          qT[dt][ks] = frag_cols(qt_, dt, qs * 32 + 16 * ks, lane);
        }
      const int kq = mykey - (qlo + 4 * lh);  // key - q for element e is kq - (e>>2)*8 - (e&3)
      if (kw0 + 31 > qlo) {  // wavefront-uniform; masked scores become -inf (P = 0) through branch-free selects
#pragma unroll
        for (int e = 0; e < 16; ++e) S[e] = (kq - 8 * (e >> 2) - (e & 3) > 0) ? -INFINITY : S[e];
      }
      uint32_t pw[8], dsw[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float p[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) p[x] = fast_exp2(S[4 * j + x] * sl2);
        const uint32_t w0 = pack2bf(p[0], p[1]), w1 = pack2bf(p[2], p[3]);
        pw[2 * j] = w0;
        pw[2 * j + 1] = w1;
        const float d0 = bflo(w0) * dP[4 * j], d1 = bfhi(w0) * dP[4 * j + 1];
        const float d2 = bflo(w1) * dP[4 * j + 2], d3 = bfhi(w1) * dP[4 * j + 3];
        dsw[2 * j] = pack2bf(d0, d1);
        dsw[2 * j + 1] = pack2bf(d2, d3);
      }
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const bf16x8 pb = frag_from(pw[4 * ks], pw[4 * ks + 1], pw[4 * ks + 2], pw[4 * ks + 3]);
        const bf16x8 db = frag_from(dsw[4 * ks], dsw[4 * ks + 1], dsw[4 * ks + 2], dsw[4 * ks + 3]);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
          dva[dt] = mfma_bf16(gT[dt][ks], pb, dva[dt]);
          dka[dt] = mfma_bf16(qT[dt][ks], db, dka[dt]);
        }
      }
    }
  };

  // A stage whose queries all come after the workgroup's keys (every stage but the first), as a software pipeline over its
  // four 32-query blocks: the dV / dK products of block j are issued between the vector instructions that turn block
  // j + 1's scores into P and dS, so half of the wavefront's MFMAs run under its own vector work.
  // The stages whose queries all come after the workgroup's keys (every stage but the first) run as a software pipeline
  // over their four 32-query blocks: the dV / dK products of block j are issued between the vector instructions that turn
  // block j + 1's scores into P and dS, so half of the wavefront's MFMAs run under its own vector work (294 -> 282 us at
  // B16 H12 T2048). Carrying the pipeline across stages (the barrier in the middle of a stage's last block) was slower
  // (299 us).
  auto scores = [&](const uint8_t* st, int qs, f32x16& S, f32x16& dP) __attribute__((always_inline)) {
    const float* ls = (const float*)(st + 2 * RT);
    bf16x8 qa[4], ga[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      qa[s] = frag_rows(st, qs, s, lr, lh);
      ga[s] = frag_rows(st + RT, qs, s, lr, lh);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const f32x4 L = *(const f32x4*)(ls + qs * 32 + 8 * j + 4 * lh);
      const f32x4 Dl = *(const f32x4*)(ls + R + qs * 32 + 8 * j + 4 * lh);
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        S[4 * j + x] = L[x];
        dP[4 * j + x] = Dl[x];
      }
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      S = mfma_bf16(qa[s], kf[s], S);
      dP = mfma_bf16(ga[s], vf[s], dP);
    }
  };
  auto softmax_ds = [&](const f32x16& S, const f32x16& dP, uint32_t (&pw)[8], uint32_t (&dsw)[8]) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float p[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) p[x] = fast_exp2(S[4 * j + x] * sl2);
      const uint32_t w0 = pack2bf(p[0], p[1]), w1 = pack2bf(p[2], p[3]);
      pw[2 * j] = w0;
      pw[2 * j + 1] = w1;
      dsw[2 * j] = pack2bf(bflo(w0) * dP[4 * j], bfhi(w0) * dP[4 * j + 1]);
      dsw[2 * j + 1] = pack2bf(bflo(w1) * dP[4 * j + 2], bfhi(w1) * dP[4 * j + 3]);
    }
  };
  auto full_stage = [&](const uint8_t* st) __attribute__((always_inline)) {
    f32x16 S, dP;
    uint32_t pws[2][8], dsws[2][8];  // P and dS of block j in [j & 1]
    scores(st, 0, S, dP);
    softmax_ds(S, dP, pws[0], dsws[0]);
#pragma unroll
    for (int qs = 0; qs < 4; ++qs) {
      uint32_t(&pw)[8] = pws[qs & 1];
      uint32_t(&dsw)[8] = dsws[qs & 1];
      if (qs < 3) scores(st, qs + 1, S, dP);
      __builtin_amdgcn_sched_barrier(0);
      bf16x8 gT[2][2], qT[2][2];
#pragma unroll
      for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          gT[dt][ks] = frag_cols(st + RT, dt, qs * 32 + 16 * ks, lane);
          qT[dt][ks] = frag_cols(st, dt, qs * 32 + 16 * ks, lane);
        }
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const bf16x8 pb = frag_from(pw[4 * ks], pw[4 * ks + 1], pw[4 * ks + 2], pw[4 * ks + 3]);
        const bf16x8 db = frag_from(dsw[4 * ks], dsw[4 * ks + 1], dsw[4 * ks + 2], dsw[4 * ks + 3]);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
          dva[dt] = mfma_bf16(gT[dt][ks], pb, dva[dt]);
          dka[dt] = mfma_bf16(qT[dt][ks], db, dka[dt]);
        }
      }
      if (qs < 3) {
        softmax_ds(S, dP, pws[(qs & 1) ^ 1], dsws[(qs & 1) ^ 1]);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x402, TFB_DKDV64_VALU_PER_MFMA, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  issue(st0, 0);
  wait_all_loads();
  __syncthreads();
  if (!TFB_DKDV64_PIPE) {
    for (int t = 0; t + 2 <= n; t += 2) {
      issue(st1, t + 1);
      compute(st0, t);
      __syncthreads();
      issue(st0, t + 2 < n ? t + 2 : n - 1);
      compute(st1, t + 1);
      __syncthreads();
    }
    if (n & 1) compute(st0, n - 1);
  } else {
    if (n > 1) issue(st1, 1);
    compute(st0, 0);  // the diagonal stage: blocks in a wavefront's past skipped, its own block masked
    if (n > 1) {
      __syncthreads();
      issue(st0, 2 < n ? 2 : n - 1);
      full_stage(st1);
      __syncthreads();
      for (int t = 2; t + 2 <= n; t += 2) {
        issue(st1, t + 1);
        full_stage(st0);
        __syncthreads();
        issue(st0, t + 2 < n ? t + 2 : n - 1);
        full_stage(st1);
        __syncthreads();
      }
      if (n & 1) full_stage(st0);
    }
  }

  bf16_t* dkp = dk.p + b * dk.sb + h * dk.sh + (long)mykey * dk.st;
  bf16_t* dvp = dv.p + b * dv.sb + h * dv.sh + (long)mykey * dv.st;
  store_grad_row(dka, scale, dkp, cs, sn, mykey, lh);
  store_grad_row(dva, 1.0f, dvp, nullptr, nullptr, mykey, lh);
  __syncthreads();  // the stages are free for the partner block
  }
}

// =========================================================================================== dQ
__global__ __launch_bounds__(256, TFB_DQ64_WPE) void attn64_dq_kernel(AttnT q, AttnT k, AttnT v, AttnT go, AttnT dq,
                                                           float* __restrict__ stats, long rows, int T, int H,
                                                           float scale, float sl2, const bf16_t* __restrict__ cs,
                                                           const bf16_t* __restrict__ sn, int nw, int slots, AttnT o,
                                                           const float* __restrict__ lse) {
  __shared__ __attribute__((aligned(1024))) uint8_t st0[2 * TILE];
  __shared__ __attribute__((aligned(1024))) uint8_t st1[2 * TILE];
  const int tid = threadIdx.x, lane = tid & 63, lr = lane & 31, lh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  stagger_start(slots);
  int bx, bh;
  xcd_block(gridDim.x, gridDim.y, bx, bh);
  const int b = bh / H, h = bh % H;
  const bf16_t* qp = q.p + b * q.sb + h * q.sh;
  const bf16_t* gp = go.p + b * go.sb + h * go.sh;
  const uint8_t* kp = (const uint8_t*)(k.p + b * k.sb + h * k.sh);
  const uint8_t* vp = (const uint8_t*)(v.p + b * v.sb + h * v.sh);
  const int nx = T / 128, npass = paired_passes(nx);
  for (int pass = 0; pass < npass; ++pass) {
  const int qb = paired_block(nx, bx, pass, true);
  const int q0 = qb * 128, qw0 = q0 + wave * 32, myq = qw0 + lr;
  const long kst = k.st * 2, vst = v.st * 2;

  bf16x8 qf[4], gf[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    qf[s] = *(const bf16x8*)(qp + (long)myq * q.st + 16 * s + 8 * lh);
    gf[s] = *(const bf16x8*)(gp + (long)myq * go.st + 16 * s + 8 * lh);
  }
  float myD, myL;
  if (TFB_ATTN_DELTA_IN_DQ) {
    // the row statistics of this wavefront's queries, made here (this kernel runs first) from the dO fragments it holds
    // anyway and the same elements of O, and left in `stats` for the dK/dV kernel: -sum_d dO O and -lse / scale
    const bf16_t* orow = o.p + b * o.sb + h * o.sh + (long)myq * o.st;
    float dot = 0.f;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const u32x4 ov = *(const u32x4*)(orow + 16 * s + 8 * lh);
      const u32x4 gv = __builtin_bit_cast(u32x4, gf[s]);
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        dot += bflo(ov[w]) * bflo(gv[w]);
        dot += bfhi(ov[w]) * bfhi(gv[w]);
      }
    }
    dot += __shfl_xor(dot, 32, 64);
    myD = -dot;
    myL = -lse[(long)bh * T + myq] * (1.0f / scale);   // (stored with the block's dQ at the end: a store here would sit in
                                                       // front of the first tile's wait for its loads)
  } else {
    myD = stats[(long)bh * T + myq];
    myL = stats[rows + (long)bh * T + myq];
  }

  TileLoad<2> lk, lv;
  lk.init(kst, wave, lane);
  lv.init(vst, wave, lane);
  auto issue = [&](uint8_t* st, int tile) {
    lk.issue(kp + (long)tile * 64 * kst, kst, st);
    lv.issue(vp + (long)tile * 64 * vst, vst, st + TILE);
  };

  f32x16 dqa[2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) dqa[i][e] = 0.f;

  // One 32-key block of the tile at `st`, in four steps that the main loop overlaps across blocks.
  // (1) S and dP, started from the query's -lse / scale and -delta
  auto scores = [&](const uint8_t* st, int kt, f32x16& S, f32x16& dP) {
    bf16x8 ka[4], va[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      ka[s] = frag_rows(st, kt, s, lr, lh);
      va[s] = frag_rows(st + TILE, kt, s, lr, lh);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      S[e] = myL;
      dP[e] = myD;
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      S = mfma_bf16(ka[s], qf[s], S);
      dP = mfma_bf16(va[s], gf[s], dP);
    }
  };
  // (2) the K^T fragments of the last product
  auto load_kT = [&](const uint8_t* st, int kt, bf16x8 (&kT)[2][2]) {
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) kT[dt][ks] = frag_cols(st, dt, kt * 32 + 16 * ks, lane);
  };
  // (3) dS = bf16(P) (dP - delta), packed as the B operand; `klo` = first key of the block when it can reach past the
  // wavefront's queries (masked scores become -inf, P = 0, through branch-free selects), -1 when it cannot
  auto softmax_ds = [&](f32x16& S, const f32x16& dP, uint32_t (&dsw)[8], int klo) {
    if (klo >= 0) {
      const int kbase = klo + lh * 4 - myq;
#pragma unroll
      for (int e = 0; e < 16; ++e) S[e] = (kbase + (e >> 2) * 8 + (e & 3) > 0) ? -INFINITY : S[e];
    }
#pragma unroll
    for (int e = 0; e < 16; e += 2) {
      const float p0 = fast_exp2(S[e] * sl2), p1 = fast_exp2(S[e + 1] * sl2);
      const uint32_t w = pack2bf(p0, p1);  // the reference multiplies dP - delta by the rounded P
      dsw[e >> 1] = pack2bf(bflo(w) * dP[e], bfhi(w) * dP[e + 1]);
    }
  };
  // (4) dQ += dS K
  auto accumulate = [&](const bf16x8 (&kT)[2][2], const uint32_t (&dsw)[8]) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const bf16x8 db = frag_from(dsw[4 * ks], dsw[4 * ks + 1], dsw[4 * ks + 2], dsw[4 * ks + 3]);
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) dqa[dt] = mfma_bf16(kT[dt][ks], db, dqa[dt]);
    }
  };
  // MFMA and VALU instructions of one scheduling region dealt out alternately: the matrix pipe works on the next block's
  // scores while the vector ALU turns the current block's into dS
  auto interleave = [&]() {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x402, TFB_DQ64_VALU_PER_MFMA, 0);
    }
  };

  f32x16 Sa, dPa;  // the scores of the next tile's first block, computed one step ahead
  // a tile with all keys before the workgroup's queries: `cur` holds tile t, `nxt` tile t + 1; tile t + 2 replaces t
  auto full_tile = [&](uint8_t* cur, const uint8_t* nxt, int t) {
    bf16x8 kTa[2][2], kTb[2][2];
    uint32_t dsa[8], dsb[8];
    f32x16 Sb, dPb;
    load_kT(cur, 0, kTa);
    scores(cur, 1, Sb, dPb);
    softmax_ds(Sa, dPa, dsa, -1);
    interleave();
    accumulate(kTa, dsa);
    __builtin_amdgcn_sched_barrier(0);  // the second block's fragments are not requested while the first's are live
    load_kT(cur, 1, kTb);
    __syncthreads();  // tile t + 1 has landed; every wavefront has its fragments of tile t
    issue(cur, t + 2);
    scores(nxt, 0, Sa, dPa);
    softmax_ds(Sb, dPb, dsb, -1);
    interleave();
    accumulate(kTb, dsb);
  };
  // one of the two tiles over the workgroup's own tokens: blocks in the wavefront's future are skipped, its diagonal
  // block masked; `first_ready`: block 0's scores are already in Sa / dPa
  auto diagonal_tile = [&](const uint8_t* st, int tile, bool first_ready) {
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      const int klo = tile * 64 + kt * 32;
      if (klo > qw0 + 31) continue;
      if (!(first_ready && kt == 0)) scores(st, kt, Sa, dPa);
      bf16x8 kT[2][2];
      uint32_t dsw[8];
      load_kT(st, kt, kT);
      softmax_ds(Sa, dPa, dsw, klo + 31 > qw0 ? klo : -1);
      accumulate(kT, dsw);
    }
  };

  const int n = (q0 + 128) / 64;  // even; tiles n - 2 and n - 1 cover the workgroup's own 128 tokens
  const int t0 = band_first_tile(qb, nw);  // even; 0 without a band
  issue(st0, t0);
  wait_all_loads();
  __syncthreads();
  issue(st1, t0 + 1);
  scores(st0, 0, Sa, dPa);
  for (int t = t0; t + 2 < n; t += 2) {
    full_tile(st0, st1, t);
    full_tile(st1, st0, t + 1);
  }
  diagonal_tile(st0, n - 2, true);
  __syncthreads();
  diagonal_tile(st1, n - 1, false);

  bf16_t* dqp = dq.p + b * dq.sb + h * dq.sh + (long)myq * dq.st;
  store_grad_row(dqa, scale, dqp, cs, sn, myq, lh);
  if (TFB_ATTN_DELTA_IN_DQ && lh == 0) {
    stats[(long)bh * T + myq] = myD;
    stats[rows + (long)bh * T + myq] = myL;
  }
  __syncthreads();  // the stages are free for the partner block
  }
}

AttnT mk(const void* p, const long* s) { return AttnT{(bf16_t*)p, s[0], s[1], s[2]}; }

}  // namespace

// Called by tfb_attn_fwd / tfb_attn_bwd for D = 64 (arguments already validated there: T % 128 == 0, strides % 8 == 0).
int tfb_attn64_fwd_impl(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs, void* o,
                        const long* os, float* lse, int B, int H, int T, float scale, int nw, hipStream_t s) {
  hipLaunchKernelGGL(attn64_fwd_kernel, dim3(paired_grid(T / 128), B * H), dim3(256), 0, s, mk(q, qs), mk(k, ks), mk(v, vs), mk(o, os), lse,
                     T, H, scale * LOG2E, nw, tfb_resident_slots(2));
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// stats: fp32 [2][B*H][T] scratch (-delta, then -lse / scale). cos_t / sin_t: bf16 [T][32] or null; when given, dq and dk
// leave the kernels with the inverse RoPE rotation applied (the gradient w.r.t. the un-rotated projections).
int tfb_attn64_bwd_impl(const void* q, const long* qs, const void* k, const long* ks, const void* v, const long* vs,
                        const void* o, const long* os, const void* go, const long* gos, void* dq, const long* dqs, void* dk,
                        const long* dks, void* dv, const long* dvs, const float* lse, float* stats, int B, int H, int T,
                        float scale, const void* cos_t, const void* sin_t, int nw, hipStream_t s) {
  const long rows = (long)B * H * T;
  // dQ first: it makes the row statistics of its own queries on the way (from fragments it loads anyway) and leaves them
  // for dK/dV, so no pass of its own reads O and dO for them (the separate pre-pass took 16.6 us at B16 H12 T2048)
  if (!TFB_ATTN_DELTA_IN_DQ) {
    hipLaunchKernelGGL(attn64_delta_kernel, dim3((unsigned)((rows * 4 + 255) / 256)), dim3(256), 0, s, mk(o, os), mk(go, gos), lse,
                       stats, T, H, rows, 1.0f / scale);
    TFB_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(attn64_dq_kernel, dim3(paired_grid(T / 128), B * H), dim3(256), 0, s, mk(q, qs), mk(k, ks), mk(v, vs), mk(go, gos),
                     mk(dq, dqs), stats, rows, T, H, scale, scale * LOG2E, (const bf16_t*)cos_t, (const bf16_t*)sin_t, nw,
                     tfb_resident_slots(2), mk(o, os), lse);
  TFB_LAUNCH_CHECK();
  hipLaunchKernelGGL(attn64_dkdv_kernel, dim3(paired_grid(T / 128), B * H), dim3(256), 0, s, mk(q, qs), mk(k, ks), mk(v, vs), mk(go, gos),
                     mk(dk, dks), mk(dv, dvs), stats, rows, T, H, scale, scale * LOG2E, (const bf16_t*)cos_t, (const bf16_t*)sin_t, nw, tfb_resident_slots(2));
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

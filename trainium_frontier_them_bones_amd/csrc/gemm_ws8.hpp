// Weight-stationary fp8 GEMM for a contraction of 768 bytes: D[q][p] = sum_k Q[q][k] P[p][k], P = a weight layout [np][768]
// (rows = the output's contiguous dimension), Q = token-major fp8 activations [nq][768]. For the MLP's up-projection and
// its dH GEMM (32768 x 3072 outputs from K = d_model = 768), whose cost on the tiled kernels is not the matrix pipe but
// the CU's vector-memory path: a 128 x 128 tile fetches 196 KB of operands for 48 KB of output, and ~24 bytes per clock
// and CU is what that path sustains.
//
// Here a workgroup (8 wavefronts, one per CU) keeps a PANEL of 256 weight rows in registers for its whole life - a
// wavefront holds 32 rows x 768 bytes as the twelve A fragments of v_mfma_scale_f32_32x32x64_f8f6f4 (96 registers) - and
// only the tokens stream: 64-token tiles (48 KB) through a two-stage LDS ring by global_load_lds_dwordx4, every
// wavefront reading all of a tile as B fragments. Operand traffic per output falls by four.
//
// The wavefronts form two groups (0-3, 4-7: one of each on every SIMD) that alternate roles in phases separated by one
// s_barrier: while one group multiplies tile t (24 MFMAs per wavefront) and leaves its fp32 accumulators in LDS, the
// other turns its previous tile's accumulators into outputs (the epilogue's vector work, loads and stores). The
// accumulators pass through LDS so that a wavefront pair (64 consecutive p) can finish whole 128-byte rows: after the
// phase's barrier wavefront 2m takes the first 32 tokens of the pair's 64 x 64 block, wavefront 2m + 1 the other 32, a lane
// 8 consecutive p of one token - the operator()(p, q, v[8] [, prefetched], split) protocol of the 128 x 128 kernel's
// epilogues, which run here unchanged and see the same sums in the same order (k ascending in steps of 64).
//
// Work: XCD x (= workgroup & 7) owns a slice of the token tiles and walks all panels over it in panel-major order, cut into
// equal runs for its workgroups (C4: 64 tiles x 12 panels = 768 steps = 24 per workgroup), so the slice (3 MB of fp8)
// stays in that XCD's L2 while the panels pass over it. A run that crosses a panel border reloads its registers once.
#pragma once
#include "gemm_pp.hpp"

struct Ws8Args {
  GemmOperand P, Q;
  int tq_x;     // token tiles (64 tokens) per XCD
  int steps_x;  // panels * tq_x: the steps of one XCD, panel-major
  int per_wg;   // steps per workgroup
  FastDiv d_tq;
};

#ifndef TFB_WS8
#define TFB_WS8 1  // 0: these GEMMs stay on the tiled kernels
#endif
#ifndef TFB_WS8_DEPTH
#define TFB_WS8_DEPTH 1  // k-steps the B fragment reads run ahead of the MFMAs (1 or 2)
#endif

template <int FMTP, int FMTQ, class Epi>
__global__ __launch_bounds__(512, 2) void gemm_ws8_kernel(Ws8Args a, Epi epi_in) {
  constexpr int STAGE = 6 * 8192;  // 64 tokens x 768 bytes, as six k-tiles of [64 rows][128 bytes]
  __shared__ __attribute__((aligned(1024))) uint8_t ring[2 * STAGE];
  __shared__ __attribute__((aligned(1024))) uint8_t stg_all[4 * 16384];  // per wavefront pair: 64 tokens x 64 p fp32
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int grp = wave >> 2;  // wavefronts w and w + 4 share a SIMD
  const int lr = lane & 31, lh = lane >> 5;

  const int x = blockIdx.x & 7, wi = blockIdx.x >> 3;
  const int s0 = wi * a.per_wg;
  int T = a.steps_x - s0;
  if (T > a.per_wg) T = a.per_wg;
  if (T <= 0) return;  // (whole workgroup, before any barrier)
  const Epi epi = epi_prepare(epi_in);

  // step -> panel, first token
  auto where = [&](int t, int& panel, long& q0) {
    const int s = s0 + t;
    panel = fastdiv(s, a.d_tq);
    q0 = 64L * (x * a.tq_x + (s - panel * a.tq_x));
  };

  // ---- token tile -> LDS stage: instruction (kt, wave) = rows 8 wave .. + 7 of k-tile kt, chunk c of row r at slot
  // c ^ tfb_kc_swz(r) (the k-contiguous layout of the tiled kernels: conflict-free 128-bit fragment reads)
  const uint32_t qv = (uint32_t)((lane >> 3) * a.Q.ld + (((lane & 7) ^ tfb_kc_swz((lane >> 3) + 8 * wave)) << 4));
  auto dma = [&](int t) {
    int panel;
    long q0;
    where(t, panel, q0);
    const uint8_t* g = a.Q.base + (q0 + 8 * wave) * a.Q.ld;
    uint8_t* d = ring + (t & 1) * STAGE + wave * 1024;
#pragma unroll
    for (int kt = 0; kt < 6; ++kt)
      __builtin_amdgcn_global_load_lds((tfb_glb_void_t*)(g + kt * 128 + (size_t)qv), (tfb_lds_void_t*)(d + kt * 8192), 16, 0, 0);
  };

  // ---- the panel's rows in registers: lane (lr, lh) holds bytes 64 ks + 32 lh .. + 31 of row 32 wave + lr per k-step
  // (loaded and waited for in inline assembly: behind compiler-visible loads the first MFMA of EVERY tile would wait for
  // all vector-memory operations in flight, the next tile's among them, because a run may have crossed a panel border)
  i32x4 Alo[12], Ahi[12];
  int cur_panel = -1;
  auto load_panel = [&](int panel) __attribute__((always_inline)) {
    const uint8_t* g = a.P.base + ((long)panel * 256 + 32 * wave + lr) * a.P.ld + 32 * lh;
#pragma unroll
    for (int ks = 0; ks < 12; ++ks) {
      asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(Alo[ks]) : "v"(g + 64 * ks));
      asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(Ahi[ks]) : "v"(g + 64 * ks));
    }
#pragma unroll
    for (int ks = 0; ks < 12; ks += 4)
      asm volatile("s_waitcnt vmcnt(0)"
                   : "+v"(Alo[ks]), "+v"(Ahi[ks]), "+v"(Alo[ks + 1]), "+v"(Ahi[ks + 1]), "+v"(Alo[ks + 2]), "+v"(Ahi[ks + 2]),
                     "+v"(Alo[ks + 3]), "+v"(Ahi[ks + 3]));
    cur_panel = panel;
  };

  // ---- B fragment addresses in stage 0: token row lr (+ 32 j as an immediate), k-step 2 kt + u: chunks 4 u + 2 lh + e
  uint32_t ab[4];
  {
    const uint32_t lbase = (uint32_t)(size_t)(tfb_lds_u8*)ring;
    const int f = tfb_kc_swz(lr);
#pragma unroll
    for (int ue = 0; ue < 4; ++ue) {
      const int c = 4 * (ue >> 1) + 2 * lh + (ue & 1);
      ab[ue] = lbase + lr * 128 + (((c ^ f) & 7) << 4);
    }
  }

  uint8_t* stg = stg_all + (wave >> 1) * 16384;

  // An epilogue's own operand (the saved activation of the dH GEMM) is requested when the wavefront starts to multiply the
  // tile and used one phase later: asked for in the epilogue itself, its round trip to HBM was that phase's length.
  constexpr bool kPrefetch = has_prefetch<Epi>::value;
  typedef typename prefetch_type<Epi>::type pre_t;
  [[maybe_unused]] pre_t pre[4];

  // ---- one tile: 24 MFMAs, the accumulators to the pair's staging block (row q = 256 bytes of fp32, 16-byte chunk c at
  // slot c ^ (q & 15))
  auto multiply = [&](int t) __attribute__((always_inline)) {
    int panel;
    long q0;
    where(t, panel, q0);
    if constexpr (kPrefetch) {
      const int p = panel * 256 + 64 * (wave >> 1) + 8 * (lane & 7), ql = 32 * (wave & 1) + (lane >> 3);
#pragma unroll
      for (int k = 0; k < 4; ++k) pre[k] = epi.prefetch(p, (int)q0 + ql + 8 * k);
    }
    if (panel != cur_panel) load_panel(panel);
    const uint32_t so = (t & 1) * STAGE;
    f32x16 acc0, acc1;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc0[e] = acc1[e] = 0.f;
    i32x4 b0[4], b1[4];
    auto rd = [&](auto KS, i32x4(&b)[4]) __attribute__((always_inline)) {
      constexpr int ks = decltype(KS)::value, off = (ks >> 1) * 8192, u = ks & 1;
      b[0] = tfb_lds_read128<off, i32x4>(ab[2 * u] + so);
      b[1] = tfb_lds_read128<off, i32x4>(ab[2 * u + 1] + so);
      b[2] = tfb_lds_read128<off + 4096, i32x4>(ab[2 * u] + so);
      b[3] = tfb_lds_read128<off + 4096, i32x4>(ab[2 * u + 1] + so);
    };
    auto mm = [&](auto KS, i32x4(&b)[4], auto NEWER) __attribute__((always_inline)) {
      constexpr int ks = decltype(KS)::value, newer = decltype(NEWER)::value;
      // `newer` reads were issued behind this k-step's four: all but those have to be there
      if (newer == 8) asm volatile("s_waitcnt lgkmcnt(8)" : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));
      else if (newer == 4) asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));
      else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));
      const i32x8 bv0 = {b[0].x, b[0].y, b[0].z, b[0].w, b[1].x, b[1].y, b[1].z, b[1].w};
      const i32x8 bv1 = {b[2].x, b[2].y, b[2].z, b[2].w, b[3].x, b[3].y, b[3].z, b[3].w};
      const i32x4 al = Alo[ks], ah = Ahi[ks];
      const i32x8 av = {al.x, al.y, al.z, al.w, ah.x, ah.y, ah.z, ah.w};
      acc0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv0, acc0, FMTP, FMTQ, 0, 127, 0, 127);
      acc1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv1, acc1, FMTP, FMTQ, 0, 127, 0, 127);
    };
#define TFB_WS_KS(n) std::integral_constant<int, n> {}
    __builtin_amdgcn_s_setprio(1);
#if TFB_WS8_DEPTH == 2
    // fragments two k-steps ahead of the MFMAs (three register sets)
    i32x4 b2[4];
    rd(TFB_WS_KS(0), b0);
    rd(TFB_WS_KS(1), b1);
    rd(TFB_WS_KS(2), b2);  mm(TFB_WS_KS(0), b0, TFB_WS_KS(8));
    rd(TFB_WS_KS(3), b0);  mm(TFB_WS_KS(1), b1, TFB_WS_KS(8));
    rd(TFB_WS_KS(4), b1);  mm(TFB_WS_KS(2), b2, TFB_WS_KS(8));
    rd(TFB_WS_KS(5), b2);  mm(TFB_WS_KS(3), b0, TFB_WS_KS(8));
    rd(TFB_WS_KS(6), b0);  mm(TFB_WS_KS(4), b1, TFB_WS_KS(8));
    rd(TFB_WS_KS(7), b1);  mm(TFB_WS_KS(5), b2, TFB_WS_KS(8));
    rd(TFB_WS_KS(8), b2);  mm(TFB_WS_KS(6), b0, TFB_WS_KS(8));
    rd(TFB_WS_KS(9), b0);  mm(TFB_WS_KS(7), b1, TFB_WS_KS(8));
    rd(TFB_WS_KS(10), b1); mm(TFB_WS_KS(8), b2, TFB_WS_KS(8));
    rd(TFB_WS_KS(11), b2); mm(TFB_WS_KS(9), b0, TFB_WS_KS(8));
    mm(TFB_WS_KS(10), b1, TFB_WS_KS(4));
    mm(TFB_WS_KS(11), b2, TFB_WS_KS(0));
#else
    rd(TFB_WS_KS(0), b0);
    rd(TFB_WS_KS(1), b1);  mm(TFB_WS_KS(0), b0, TFB_WS_KS(4));
    rd(TFB_WS_KS(2), b0);  mm(TFB_WS_KS(1), b1, TFB_WS_KS(4));
    rd(TFB_WS_KS(3), b1);  mm(TFB_WS_KS(2), b0, TFB_WS_KS(4));
    rd(TFB_WS_KS(4), b0);  mm(TFB_WS_KS(3), b1, TFB_WS_KS(4));
    rd(TFB_WS_KS(5), b1);  mm(TFB_WS_KS(4), b0, TFB_WS_KS(4));
    rd(TFB_WS_KS(6), b0);  mm(TFB_WS_KS(5), b1, TFB_WS_KS(4));
    rd(TFB_WS_KS(7), b1);  mm(TFB_WS_KS(6), b0, TFB_WS_KS(4));
    rd(TFB_WS_KS(8), b0);  mm(TFB_WS_KS(7), b1, TFB_WS_KS(4));
    rd(TFB_WS_KS(9), b1);  mm(TFB_WS_KS(8), b0, TFB_WS_KS(4));
    rd(TFB_WS_KS(10), b0); mm(TFB_WS_KS(9), b1, TFB_WS_KS(4));
    rd(TFB_WS_KS(11), b1); mm(TFB_WS_KS(10), b0, TFB_WS_KS(4));
    mm(TFB_WS_KS(11), b1, TFB_WS_KS(0));
#endif
    __builtin_amdgcn_s_setprio(0);
#undef TFB_WS_KS
    // acc_j[4 jj + e] = D[p = 8 jj + 4 lh + e][q = 32 j + lr]
    const int cw = 8 * (wave & 1) + lh;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const f32x4 v0 = {acc0[4 * jj], acc0[4 * jj + 1], acc0[4 * jj + 2], acc0[4 * jj + 3]};
      const f32x4 v1 = {acc1[4 * jj], acc1[4 * jj + 1], acc1[4 * jj + 2], acc1[4 * jj + 3]};
      *(f32x4*)(stg + lr * 256 + (((cw + 2 * jj) ^ (lr & 15)) << 4)) = v0;
      *(f32x4*)(stg + (32 + lr) * 256 + (((cw + 2 * jj) ^ (lr & 15)) << 4)) = v1;
    }
  };

  // ---- the epilogue of a tile: this wavefront's 32 tokens of the pair's block, four passes of 8 tokens x 64 p
  auto finish = [&](int t) __attribute__((always_inline)) {
    int panel;
    long q0;
    where(t, panel, q0);
    const int p = panel * 256 + 64 * (wave >> 1) + 8 * (lane & 7);
    const int ql = 32 * (wave & 1) + (lane >> 3);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int row = ql + 8 * k, c = 2 * (lane & 7);
      const f32x4 lo = *(const f32x4*)(stg + row * 256 + ((c ^ (row & 15)) << 4));
      const f32x4 hi = *(const f32x4*)(stg + row * 256 + (((c + 1) ^ (row & 15)) << 4));
      const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      if constexpr (kPrefetch) epi(p, (int)q0 + row, v, pre[k], 0);
      else epi(p, (int)q0 + row, v, 0);
    }
  };

  // ---- prologue: tile 0 on its way, the first panel into registers
  dma(0);
  {
    int panel;
    long q0;
    where(0, panel, q0);
    load_panel(panel);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  TFB_SBAR();

  // Phase ph: group 0 multiplies tile ph / 2 (ph even) or finishes it (ph odd); group 1 one phase later. Tile t + 1 is
  // requested in phase 2 t - by group 0 in front of its MFMAs, by group 1 behind its epilogue - into the stage whose tile
  // (t - 1) group 1 stopped reading in phase 2 t - 1, and waited for in phase 2 t + 1, a phase after the request: by group 1
  // behind its MFMAs with nothing younger outstanding, by group 0 in front of its epilogue, where only the epilogue's own
  // four operand loads (if it has any) are younger - behind the epilogue the wait would be for its stores' round trips
  // (completion is reported in issue order, stores included).
  for (int ph = 0; ph <= 2 * T; ++ph) {
    if ((ph & 1) == grp) {
      const int t = (ph - grp) >> 1;
      if (t < T) {
        if (grp == 0 && t + 1 < T) dma(t + 1);
        multiply(t);
        if (grp == 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
    } else {
      const int t = (ph - 1 - grp) >> 1;  // group 0: (ph - 1) / 2; group 1: (ph - 2) / 2
      if (grp == 0) {
        if (kPrefetch) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      if (ph - 1 - grp >= 0 && t < T) finish(t);
      if (grp == 1) {
        const int tn = (ph >> 1) + 1;
        if (tn < T) dma(tn);
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the staging block is complete (or read) before the roles swap
    TFB_SBAR();
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// np % 256 == 0, nq % 512 == 0 (64-token tiles dealt to the 8 XCDs), kbytes == 768, rows 16-byte aligned; at least one
// step for every CU
static inline bool gemm_ws8_applies(long np, long nq, long kbytes) {
  return TFB_WS8 && kbytes == 768 && np > 0 && nq > 0 && np % 256 == 0 && nq % 512 == 0 &&
         (np / 256) * (nq / 64) >= tfb_resident_slots(1);
}

template <int FMTP, int FMTQ, class Epi>
static int gemm_ws8_launch(GemmOperand P, GemmOperand Q, int np, int nq, long kbytes, Epi epi, hipStream_t stream) {
  if (kbytes != 768 || np <= 0 || nq <= 0 || np % 256 || nq % 512) return TFB_ERR_SHAPE;
  if (P.ld <= 0 || Q.ld <= 0 || P.ld > (1L << 24) || Q.ld > (1L << 24)) return TFB_ERR_SHAPE;
  if (((uintptr_t)P.base | (uintptr_t)Q.base | (uintptr_t)P.ld | (uintptr_t)Q.ld) & 15) return TFB_ERR_ARG;
  Ws8Args a = {};
  a.P = P;
  a.Q = Q;
  a.tq_x = nq / 512;
  a.steps_x = (np / 256) * a.tq_x;
  int per_x = tfb_resident_slots(1) / 8;  // workgroups per XCD: one per CU
  if (per_x < 1) per_x = 1;
  a.per_wg = (a.steps_x + per_x - 1) / per_x;
  const int wgs_x = (a.steps_x + a.per_wg - 1) / a.per_wg;
  a.d_tq = fastdiv_make(a.tq_x);
  hipLaunchKernelGGL((gemm_ws8_kernel<FMTP, FMTQ, Epi>), dim3(8 * wgs_x), dim3(512), 0, stream, a, epi);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

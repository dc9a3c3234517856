// Persistent 256 x 256 MFMA GEMM for gfx950: D[p][q] = sum_k P[p][k] * Q[q][k], fp32 accumulation, k-contiguous operands.
//
// One workgroup of eight wavefronts per CU (two per SIMD) walks output tiles. The wavefronts form two groups of four (one
// wavefront of each group on every SIMD) that alternate between a MEMORY cluster (fragment reads from LDS, operand loads
// global -> LDS) and an MFMA cluster (8 MFMAs of 32 x 32), one barrier per cluster, group 1 running one cluster behind
// group 0: each SIMD's matrix pipe is fed by one wavefront while the other one waits on the memory path, and a vector
// memory instruction (which holds the wavefront that issues it for 70-110 cycles) never delays an MFMA.
//
// A wavefront owns 2 x 64 rows of P (64 in each 128-row half of the tile) and 2 x 32 rows of Q: four accumulator blocks of
// 64 x 32. A k-tile (128 bytes of k per row) is consumed as: block (P half 0, Q half 0), (0, 1), (1, 0), (1, 1); an operand
// quarter (128 rows x 128 bytes = 16 KB, one of P half 0/1, Q half 0/1) is refilled with the k-tile two ahead as soon as
// both groups have it in registers, so two 64 KB stages keep the loads ~1.5 k-tiles ahead of the MFMAs. The load stream
// does not stop at an output tile's end: the last two k-tiles of a tile already fetch the first two of the workgroup's next
// tile, and the epilogue (accumulators -> bf16 -> global, straight from registers: a lane pair exchange with
// v_permlane32_swap gives every lane 8 consecutive outputs of a row) runs while those loads are in flight.
//
// Fragment reads are inline assembly (ds_read_b128 with immediate offsets) with explicit s_waitcnt: left to the compiler,
// every LDS read beside global -> LDS loads in flight would wait for vmcnt(0).
//
// LDS map (bytes): stage S at S * 65536: P half 0, P half 1, Q half 0, Q half 1 (16 KB each); row r of a half at r * 128,
// 16-byte chunk c at slot c ^ tfb_kc_swz(r) (no bank conflicts for the 128-bit fragment reads).
#pragma once
#include "gemm_core.hpp"

typedef __attribute__((address_space(3))) uint8_t tfb_lds_u8;
typedef unsigned tfb_u32x2 __attribute__((ext_vector_type(2)));

template <int OFF, class T>
__device__ __forceinline__ T tfb_lds_read128(uint32_t addr) {
  static_assert(sizeof(T) == 16, "128-bit fragment");
  T v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
#define TFB_SBAR()                          \
  do {                                      \
    __builtin_amdgcn_sched_barrier(0);      \
    asm volatile("s_barrier" ::: "memory"); \
    __builtin_amdgcn_sched_barrier(0);      \
  } while (0)

struct PpArgs {
  GemmOperand P, Q;
  int nkt;      // k-tiles per output tile (>= 2)
  int ntiles;   // output tiles
  int nwg;      // workgroups launched (a multiple of 8 when rect)
  int p_fast;   // the fast-walking operand is P
  int nfast;    // tiles of that operand
  // rect: XCD x (= work item & 7) owns R consecutive tile rows of the slow operand and walks them in panels of GW
  // columns (GW * R ~ the XCD's 32 CUs), so the tiles that run together on an XCD form a compact block and share their
  // operand rows in that XCD's L2
  int rect, R, GW, panel;  // panel = GW * R
  int gw_last;             // width of the last panel (nfast % GW, or GW)
  FastDiv d_nfast, d_panel, d_gw, d_gw_last;
};

// Epilogue protocol of this kernel (every epilogue of the library rounds f(accumulator) to bf16 first):
//   float pre(float acc)                      applied to every accumulator before its rounding to bf16;
//   void chunk(p, q, v [, vp] [, pre_t])      8 consecutive rounded outputs D[p .. p + 7][q] as four packed bf16 pairs
//                                             (p % 8 == 0); with kPartner32 also the 8 values 32 outputs away (p ^ 32); with a
//                                             pre_t / prefetch(p, q) the operand requested before the block was staged.
// Plain bf16 store: out [q][ld] = bf16(D)
struct EpiStoreBf16 {
  bf16_t* out;
  long ld;
  __device__ __forceinline__ float pre(float x) const { return x; }
  __device__ __forceinline__ void chunk(int p, int q, const u32x4& v) const { *(u32x4*)(out + (long)q * ld + p) = v; }
};

#ifdef PP_DBG
__device__ unsigned long long pp_dbg[256 * 4];
#endif
// ES: element size (2: bf16, 1: OCP fp8 with FMTP / FMTQ = 0 e4m3, 1 e5m2 per side)
template <int ES, int FMTP, int FMTQ, class Epi>
__global__ __launch_bounds__(512, 2) void gemm_pp_kernel(PpArgs a, Epi epi_in) {
#ifdef PP_DBG
  const unsigned long long c_start = __builtin_readcyclecounter();
  unsigned long long c_epi = 0, c_loop = 0;
  int n_tiles = 0;
#endif
  __shared__ __attribute__((aligned(1024))) uint8_t lds[2 * 65536];
  __shared__ __attribute__((aligned(1024))) uint8_t stg_all[8 * 4096];  // epilogue staging, 4 KB per wavefront
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int wr = wave >> 2, wc = wave & 3;  // wr: the group (wavefronts 0-3 / 4-7 sit on SIMDs 0-3 each)
  const int lr = lane & 31, lh = lane >> 5;
  const int nkt = a.nkt;
  uint8_t* stg = stg_all + wave * 4096;

  // work item -> output tile origin (rows of P, rows of Q)
  auto tile_of = [&](int w, long& p0, long& q0) {
    int fast, slow;
    if (a.rect) {
      const int x = w & 7, j = w >> 3;
      const int pn = fastdiv(j, a.d_panel), rem = j - pn * a.panel;
      const int first = pn * a.GW;
      const bool last = first + a.GW > a.nfast;
      const int row = last ? fastdiv(rem, a.d_gw_last) : fastdiv(rem, a.d_gw);
      const int gw = last ? a.gw_last : a.GW;
      fast = first + rem - row * gw;
      slow = x * a.R + row;
    } else {
      slow = fastdiv(w, a.d_nfast);
      fast = w - slow * a.nfast;
    }
    p0 = (long)(a.p_fast ? fast : slow) * 256;
    q0 = (long)(a.p_fast ? slow : fast) * 256;
  };

  // ---- operand loads: a quarter = 16 instructions of 8 rows x 128 B; this wavefront issues rows 8 wave + {0, 64} + lane / 8
  const int lrow = lane >> 3;
  const int dch = (lane & 7) ^ tfb_kc_swz(lrow + 8 * wave);
  const uint32_t vp = (uint32_t)(lrow * a.P.ld + dch * 16), vq = (uint32_t)(lrow * a.Q.ld + dch * 16);
  const long p64 = 64 * a.P.ld, q64 = 64 * a.Q.ld;
  const uint8_t* bp = a.P.base + 8L * wave * a.P.ld;
  const uint8_t* bq = a.Q.base + 8L * wave * a.Q.ld;
  // quarter (X: 0 P, 1 Q; half h) of stage S <- 128 bytes of k at g (the operand's row-0 address of the tile + k offset)
  auto dma = [&](int S, int X, int h, const uint8_t* g) {
    const long r64 = X ? q64 : p64;
    const uint32_t v = X ? vq : vp;
    uint8_t* d = lds + S * 65536 + X * 32768 + h * 16384 + wave * 1024;
#pragma unroll
    for (int i = 0; i < 2; ++i)
      __builtin_amdgcn_global_load_lds((tfb_glb_void_t*)(g + (2 * h + i) * r64 + (size_t)v), (tfb_lds_void_t*)(d + i * 8192),
                                       16, 0, 0);
  };

  // ---- fragment addresses (stage 0; the stage bit is toggled after every k-tile)
  uint32_t ap[4], aq[4];
  {
    const uint32_t lbase = (uint32_t)(size_t)(tfb_lds_u8*)lds;
    const int rp = wr * 64 + lr, rq = wc * 32 + lr;
    // bf16: k-step s (16 k) of a row is chunk 2 s + lh; fp8: k-step s (64 k) is chunks 4 s + 2 lh, + 1: entry 2 s + u
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int c = ES == 2 ? 2 * s + lh : 4 * (s >> 1) + 2 * lh + (s & 1);
      ap[s] = lbase + rp * 128 + (((c ^ tfb_kc_swz(rp)) & 7) << 4);
      aq[s] = lbase + 32768 + rq * 128 + (((c ^ tfb_kc_swz(rq)) & 7) << 4);
    }
  }

  f32x16 acc[2][2][2];  // [P half][i][Q half]
  // fragments: bf16 four k-steps of 16 (one 128-bit read each), fp8 two k-steps of 64 (two 128-bit reads each)
  typedef std::conditional_t<ES == 2, bf16x8, i32x4> r128_t;
  r128_t fa[2][4], fb0[4], fb1[4];
  auto readA = [&](auto H) {
    constexpr int h = decltype(H)::value;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      fa[0][s] = tfb_lds_read128<h * 16384, r128_t>(ap[s]);
      fa[1][s] = tfb_lds_read128<h * 16384 + 4096, r128_t>(ap[s]);
    }
  };
  auto readB = [&](auto H, r128_t(&fb)[4]) {
    constexpr int h = decltype(H)::value;
#pragma unroll
    for (int s = 0; s < 4; ++s) fb[s] = tfb_lds_read128<h * 16384, r128_t>(aq[s]);
  };
  // the fragments pass through the wait as in/out operands, so that no MFMA that reads them is scheduled ahead of it
  auto waitA = [&]() {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(fa[0][0]), "+v"(fa[0][1]), "+v"(fa[0][2]), "+v"(fa[0][3]), "+v"(fa[1][0]), "+v"(fa[1][1]),
                   "+v"(fa[1][2]), "+v"(fa[1][3]));
  };
  auto waitB = [&](r128_t(&fb)[4]) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]));
  };
  auto mma = [&](auto FIRST, auto HP, auto HQ, const r128_t(&fb)[4]) __attribute__((always_inline)) {
    constexpr bool first = decltype(FIRST)::value;
    constexpr int hp = decltype(HP)::value, hq = decltype(HQ)::value;
    __builtin_amdgcn_s_setprio(1);
    if constexpr (ES == 2) {
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          f32x16 c = acc[hp][i][hq];
          if (first && s == 0) {
#pragma unroll
            for (int e = 0; e < 16; ++e) c[e] = 0.f;
          }
          acc[hp][i][hq] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i][s], fb[s], c, 0, 0, 0);
        }
    } else {
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          f32x16 c = acc[hp][i][hq];
          if (first && s == 0) {
#pragma unroll
            for (int e = 0; e < 16; ++e) c[e] = 0.f;
          }
          const i32x4 al = fa[i][2 * s], ah = fa[i][2 * s + 1], bl = fb[2 * s], bh = fb[2 * s + 1];
          const i32x8 av = {al.x, al.y, al.z, al.w, ah.x, ah.y, ah.z, ah.w};
          const i32x8 bv = {bl.x, bl.y, bl.z, bl.w, bh.x, bh.y, bh.z, bh.w};
          // formats: 0 = e4m3, 1 = e5m2; E8M0 scale byte 127 = 2^0
          acc[hp][i][hq] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, c, FMTP, FMTQ, 0, 127, 0, 127);
        }
    }
    __builtin_amdgcn_s_setprio(0);
    // the MFMAs have no side effects: without a use here they may sink below the barriers that follow
    asm volatile("" : "+v"(acc[hp][0][hq]), "+v"(acc[hp][1][hq]));
  };
  typedef std::integral_constant<int, 0> H0;
  typedef std::integral_constant<int, 1> H1;

  const Epi epi = epi_prepare(epi_in);
  int w = blockIdx.x;
  if (w >= a.ntiles) return;  // (whole workgroup)
#ifdef PP_STAG
  for (int i = 0; i < (int)((blockIdx.x >> 3) & 3) * PP_STAG; ++i) __builtin_amdgcn_s_sleep(32);
#endif
  long p0, q0;
  tile_of(w, p0, q0);
  const uint8_t* gp = bp + p0 * a.P.ld;  // current tile
  const uint8_t* gq = bq + q0 * a.Q.ld;

  // ---- prologue: all of k-tile 0 into stage 0, three quarters of k-tile 1 into stage 1
  dma(0, 1, 0, gq);
  dma(0, 0, 0, gp);
  dma(0, 1, 1, gq);
  dma(0, 0, 1, gp);
  dma(1, 0, 0, gp + 128);
  dma(1, 1, 0, gq + 128);
  dma(1, 1, 1, gq + 128);
  asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
  TFB_SBAR();               // k-tile 0 is there for everybody
  if (wr == 1) TFB_SBAR();  // group 1 runs one cluster behind from here on

  // ---- epilogue of one 64 (p) x 32 (q) accumulator block, acc[hp][i][hq][4 jj + e] = D[pb + 32 i + 8 jj + 4 lh + e][qb + lr]:
  // every accumulator goes through epi.pre() and is rounded to bf16, the block passes through the wavefront's own 4 KB of
  // LDS (row q = 128 bytes, 16-byte chunk c at slot c ^ ((q >> 1) & 7): the 8-byte writes and the 16-byte reads then use
  // the banks evenly), and every lane finishes 8 consecutive outputs of a row, a row's 64 outputs (128 bytes) on 8
  // consecutive lanes: epi.chunk(p, q, v [, partner] [, prefetched]).
  constexpr bool kPrefetch = has_prefetch<Epi>::value;
  auto store_block = [&](auto HP, auto HQ, long tp0, long tq0) __attribute__((always_inline)) {
    constexpr int hp = decltype(HP)::value, hq = decltype(HQ)::value;
    const int pb = (int)tp0 + hp * 128 + wr * 64, qb = (int)tq0 + hq * 128 + wc * 32;
    const int ch = lane & 7, r8 = lane >> 3;
    // the epilogue's own operand: all four chunks requested up front when that is 16 registers, else one ahead
    typedef typename prefetch_type<Epi>::type pre_t;
    constexpr int kAhead = sizeof(pre_t) <= 16 ? 4 : 1;
    [[maybe_unused]] pre_t pre[4];
    if constexpr (kPrefetch) {
#pragma unroll
      for (int k = 0; k < kAhead; ++k) pre[k] = epi.prefetch(pb + 8 * ch, qb + r8 + 8 * k);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const f32x16& c = acc[hp][i][hq];
        u32x2 v = {pack2bf(epi.pre(c[4 * jj + 0]), epi.pre(c[4 * jj + 1])),
                   pack2bf(epi.pre(c[4 * jj + 2]), epi.pre(c[4 * jj + 3]))};
        *(u32x2*)(stg + lr * 128 + (((4 * i + jj) ^ ((lr >> 1) & 7)) << 4) + 8 * lh) = v;
      }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int row = r8 + 8 * k;
      const u32x4 v = *(const u32x4*)(stg + row * 128 + ((ch ^ ((row >> 1) & 7)) << 4));
      const int p = pb + 8 * ch, q = qb + row;
      if constexpr (kPrefetch && kAhead < 4) {
        if (k + kAhead < 4) pre[k + kAhead] = epi.prefetch(pb + 8 * ch, qb + r8 + 8 * (k + kAhead));
      }
      if constexpr (has_partner32<Epi>::value) {
        const u32x4 vp = *(const u32x4*)(stg + row * 128 + (((ch ^ 4) ^ ((row >> 1) & 7)) << 4));  // 32 outputs away
        if constexpr (kPrefetch) epi.chunk(p, q, v, vp, pre[k]);
        else epi.chunk(p, q, v, vp);
      } else if constexpr (kPrefetch) {
        epi.chunk(p, q, v, pre[k]);
      } else {
        epi.chunk(p, q, v);
      }
    }
    __builtin_amdgcn_wave_barrier();
  };

  int S = 0;
  bool have_prev = false;  // the previous tile's accumulators are still to be stored
  long pp0 = 0, pq0 = 0;   // its origin
  for (;;) {
    // the workgroup's next tile (its first k-tiles are requested by this tile's last iterations); past the end: this tile
    // again (loads nobody reads, from valid memory)
    const int wn = w + a.nwg;
    long pn = p0, qn = q0;
    if (wn < a.ntiles) tile_of(wn, pn, qn);
    const uint8_t* gpn = bp + pn * a.P.ld;
    const uint8_t* gqn = bq + qn * a.Q.ld;

    // One k-tile. In a tile's first iteration the MFMAs start from zero, and each accumulator block of the PREVIOUS tile is
    // stored in the memory cluster in front of the MFMA cluster that overwrites it: the stores of one group (4 KB per
    // wavefront and cluster) run under the other group's MFMAs.
    auto iter = [&](auto FIRST, int kt) __attribute__((always_inline)) {
      constexpr bool first = decltype(FIRST)::value;
      // k positions one and two ahead in the workgroup's stream of k-tiles
      const bool in1 = kt + 1 < nkt, in2 = kt + 2 < nkt;
      const long k1 = (long)(in1 ? kt + 1 : 0) * 128, k2 = (long)(in2 ? kt + 2 : kt + 2 - nkt) * 128;
      const uint8_t* gp1 = (in1 ? gp : gpn) + k1;
      const uint8_t* gp2 = (in2 ? gp : gpn) + k2;
      const uint8_t* gq2 = (in2 ? gq : gqn) + k2;
      // c0
      readB(H0{}, fb0);
      readA(H0{});
      dma(S ^ 1, 0, 1, gp1);
      if (first && have_prev) store_block(H0{}, H0{}, pp0, pq0);
      TFB_SBAR();
      // c1
      waitB(fb0);
      waitA();
      mma(FIRST, H0{}, H0{}, fb0);
      TFB_SBAR();
      // c2
      readB(H1{}, fb1);
      dma(S, 0, 0, gp2);
      if (first && have_prev) store_block(H0{}, H1{}, pp0, pq0);
      TFB_SBAR();
      // c3
      waitB(fb1);
      mma(FIRST, H0{}, H1{}, fb1);
      TFB_SBAR();
      // c4
      readA(H1{});
      dma(S, 1, 0, gq2);
      if (first && have_prev) store_block(H1{}, H0{}, pp0, pq0);
      TFB_SBAR();
      // c5
      waitA();
      mma(FIRST, H1{}, H0{}, fb0);
      TFB_SBAR();
      // c6
      dma(S, 1, 1, gq2);
      // Completion is reported in issue order, stores included. Everything up to the quarter requested in c0 has to be
      // there: all but the three quarters requested since (6 instructions), and in a first iteration with stores all but
      // those and the 16 stores (c0's four were issued behind its loads).
      if (first && have_prev) {
        store_block(H1{}, H1{}, pp0, pq0);
        asm volatile("s_waitcnt vmcnt(22)" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
      }
      TFB_SBAR();
      // c7
      mma(FIRST, H1{}, H1{}, fb1);
      TFB_SBAR();
      S ^= 1;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        ap[s] ^= 0x10000u;
        aq[s] ^= 0x10000u;
      }
    };
#ifdef PP_DBG
    const unsigned long long c_l0 = __builtin_readcyclecounter();
#endif
    iter(std::true_type{}, 0);
#ifdef PP_DBG
    const unsigned long long c_e0 = __builtin_readcyclecounter();
    c_epi += c_e0 - c_l0;
#endif
    for (int kt = 1; kt < nkt; ++kt) iter(std::false_type{}, kt);
#ifdef PP_DBG
    c_loop += __builtin_readcyclecounter() - c_e0;
    ++n_tiles;
#endif
    have_prev = true;
    pp0 = p0;
    pq0 = q0;
    w = wn;
    if (w >= a.ntiles) break;
    p0 = pn;
    q0 = qn;
    gp = gpn;
    gq = gqn;
  }
  // the last tile's accumulators
  store_block(H0{}, H0{}, pp0, pq0);
  store_block(H0{}, H1{}, pp0, pq0);
  store_block(H1{}, H0{}, pp0, pq0);
  store_block(H1{}, H1{}, pp0, pq0);
#ifdef PP_DBG
  if (tid == 0 && blockIdx.x < 256) {
    pp_dbg[blockIdx.x * 4 + 0] = __builtin_readcyclecounter() - c_start;
    pp_dbg[blockIdx.x * 4 + 1] = c_loop;
    pp_dbg[blockIdx.x * 4 + 2] = c_epi;
    pp_dbg[blockIdx.x * 4 + 3] = n_tiles;
  }
#endif
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stream's last (unused) loads must have landed before LDS is released
}

// Shapes this kernel takes (both operands k-contiguous): np, nq multiples of 256, at least two k-tiles of 128 bytes.
// Shapes it is USED for: contractions of at least 16 k-tiles, or outputs of at least 4096 tiles. Measured inside the training
// step against the 128 x 128 kernel (two workgroups per CU, one's epilogue under the other's k-loop): the 32768 x 32768 x 768
// LM-head product 1728 -> 1532 us, the fp8 GEMMs with 24 k-tiles 82.5 -> 74.7 and 84.8 -> 83.2 us; but with 6 to 12 k-tiles and
// a heavy epilogue per tile (rotary embedding, residual add, the MLP's activation) 141 -> 148, 55 -> 60, 112 -> 111 us: those stay.
#ifndef TFB_PP
#define TFB_PP 1  // 0: every GEMM on the 128 x 128 kernel; 2: every shape the kernel takes (for comparisons)
#endif
static inline bool gemm_pp_applies(long np, long nq, long kbytes) {
  if (!TFB_PP || np <= 0 || nq <= 0 || np % 256 || nq % 256 || kbytes < 256 || kbytes % 128) return false;
  const long tiles = (np / 256) * (nq / 256);
  if (tiles < 8) return false;
  return TFB_PP == 2 || kbytes / 128 >= 16 || tiles >= 4096;
}

template <int ES, int FMTP, int FMTQ, class Epi>
static int gemm_pp_launch(GemmOperand P, GemmOperand Q, int np, int nq, long kbytes, Epi epi, hipStream_t stream) {
  if (np <= 0 || nq <= 0 || kbytes < 256 || np % 256 || nq % 256 || kbytes % 128) return TFB_ERR_SHAPE;
  if (P.ld <= 0 || Q.ld <= 0 || P.ld > (1L << 28) || Q.ld > (1L << 28)) return TFB_ERR_SHAPE;
  if (((uintptr_t)P.base | (uintptr_t)Q.base | (uintptr_t)P.ld | (uintptr_t)Q.ld) & 15) return TFB_ERR_ARG;
  PpArgs a = {};
  a.P = P;
  a.Q = Q;
  a.nkt = (int)(kbytes / 128);
  const int ntp = np / 256, ntq = nq / 256;
  if ((long)ntp * ntq >= (1L << 30)) return TFB_ERR_SHAPE;
  a.ntiles = ntp * ntq;
  const int cus = tfb_resident_slots(1);
  a.p_fast = np <= nq;
  a.nfast = a.p_fast ? ntp : ntq;
  const int nslow = a.p_fast ? ntq : ntp;
  a.rect = (nslow % 8 == 0) && a.ntiles >= 8;
  a.nwg = a.ntiles < cus ? a.ntiles : cus;
  if (a.rect) a.nwg &= ~7;
  a.R = a.rect ? nslow / 8 : 1;
  // panel width: GW * R ~ the 32 workgroups an XCD runs together, at least 1 and at most all columns
  int gw = a.R >= 32 ? 1 : (32 + a.R - 1) / a.R;
  if (a.R > 8 && a.R < 32) gw = 32 / a.R > 0 ? 32 / a.R : 1;
  if (gw > a.nfast) gw = a.nfast;
  a.GW = gw;
  a.panel = a.GW * a.R;
  a.gw_last = a.nfast % a.GW ? a.nfast % a.GW : a.GW;
  a.d_nfast = fastdiv_make(a.nfast);
  a.d_panel = fastdiv_make(a.panel);
  a.d_gw = fastdiv_make(a.GW);
  a.d_gw_last = fastdiv_make(a.gw_last);
  hipLaunchKernelGGL((gemm_pp_kernel<ES, FMTP, FMTQ, Epi>), dim3(a.nwg), dim3(512), 0, stream, a, epi);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

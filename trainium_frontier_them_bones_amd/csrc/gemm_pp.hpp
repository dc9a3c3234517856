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
// LDS map (bytes): stage S at S * 65536: P half 0, P half 1, Q half 0, Q half 1 (16 KB each). A k-contiguous operand
// ([rows][K]) keeps row r of a half at r * 128, 16-byte chunk c at slot c ^ tfb_kc_swz(r) (no bank conflicts for the 128-bit
// fragment reads). A k-strided bf16 operand ([K][rows], the token-contraction GEMMs) keeps one k per 256-byte LDS row,
// chunk c of k-row k at slot c ^ (4 (k & 3)), and its fragments come through ds_read_b64_tr_b16 (two per fragment), the
// layout and lane map of the 128 x 128 kernel's K_STRIDED reader. A k-strided fp8 operand keeps one k per 128-byte LDS row
// (128 k-rows per quarter), chunk c of k-row k at slot c ^ (2 ((k >> 1) & 3)), fragments through ds_read_b64_tr_b8 (four
// per 64-k fragment).
//
// Long contractions with few output tiles (the LM head's gradients: 384 tiles of 512 k-tiles) are split along k into
// work items of equal length; each leaves its fp32 partial tile in a workspace (epilogues with kSplitF32, staged as
// fp32) and splitk_reduce_kernel finishes them.
#pragma once
#include "gemm_core.hpp"

#ifndef TFB_PP_EARLYB
#define TFB_PP_EARLYB 1  // a k-tile's first Q fragments requested in the previous k-tile's last MFMA cluster
#endif

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
  int nk_total; // k-tiles of the contraction; split s of `splits` takes [s nk / splits, (s + 1) nk / splits), >= 2 each
  int ntiles;   // work items = output tiles * splits (item w: split w / nout, output tile w % nout)
  int nout;     // output tiles
  int splits;
  int ipx;      // > 0 (few output tiles, one work item per workgroup): XCD x (= workgroup & 7) takes the ipx consecutive
                // work items from x * ipx, so that an XCD's workgroups share one or two k ranges of the operands in its L2
  FastDiv d_nout;
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
typedef short tfb_s16x8 __attribute__((ext_vector_type(8)));
template <int OFF>
__device__ __forceinline__ tfb_s16x4 tfb_lds_read_tr64(uint32_t addr) {
  tfb_s16x4 v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
typedef int tfb_pp_i32x2 __attribute__((ext_vector_type(2)));
template <int OFF>
__device__ __forceinline__ tfb_pp_i32x2 tfb_lds_read_tr64_b8(uint32_t addr) {
  tfb_pp_i32x2 v;
  asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}

// An epilogue with the static member kSplitF32 receives the raw fp32 accumulators, operator()(p, q, v[8], split): the
// partial tile of a k-split.
template <class T, class = void>
struct has_split_f32 : std::false_type {};
template <class T>
struct has_split_f32<T, std::void_t<decltype(T::kSplitF32)>> : std::true_type {};

// ES: element size (2: bf16, 1: OCP fp8 with FMTP / FMTQ = 0 e4m3, 1 e5m2 per side); LAYP / LAYQ: TFB_K_CONTIG or
// TFB_K_STRIDED
template <int ES, int FMTP, int FMTQ, int LAYP, int LAYQ, class Epi>
__global__ __launch_bounds__(512, 2) void gemm_pp_kernel(PpArgs a, Epi epi_in) {
  constexpr bool kF32 = has_split_f32<Epi>::value;
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
  int nkt;  // k-tiles of the current work item
  uint8_t* stg = stg_all + wave * 4096;

  // ---- operand loads. A quarter is 16 instructions of 1 KB, two per wavefront (g = wave and wave + 8):
  //   k-contiguous: instruction g = rows 8 g .. 8 g + 7 x 128 bytes of k, lane l -> row l / 8, chunk (l % 8) ^ swizzle;
  //   k-strided:    instruction g = k-rows 4 g .. 4 g + 3 x 128 rows (256 bytes), lane l -> k-row l / 16, chunk (l % 16) ^ 4 (k & 3);
  //                 fp8: k-rows 8 g .. 8 g + 7 x 128 rows (128 bytes), lane l -> k-row l / 8, chunk (l % 8) ^ 2 ((k >> 1) & 3).
  // Per operand: v = the lane's byte offset, istep = from instruction g to g + 8, hstep = from half 0 to half 1,
  // kstep = from one k-tile to the next, and the byte origin of output tile row-block r0.
  struct Side {
    const uint8_t* base;  // operand base + this wavefront's first instruction
    uint32_t v;
    long istep, hstep, kstep, tstep;  // tstep: bytes per row of the output tile origin
  };
  auto make_side = [&](const GemmOperand& o, int lay) {
    Side sd;
    if (lay == TFB_K_CONTIG) {
      const int lrow = lane >> 3;
      const int dch = (lane & 7) ^ tfb_kc_swz(lrow + 8 * wave);
      sd.base = o.base + 8L * wave * o.ld;
      sd.v = (uint32_t)(lrow * o.ld + dch * 16);
      sd.istep = 64 * o.ld;
      sd.hstep = 128 * o.ld;
      sd.kstep = 128;
      sd.tstep = o.ld;
    } else if (ES == 2) {
      const int kl = lane >> 4, slot = lane & 15;
      sd.base = o.base + 4L * wave * o.ld;
      sd.v = (uint32_t)(kl * o.ld + ((slot ^ (4 * kl)) << 4));
      sd.istep = 32 * o.ld;
      sd.hstep = 256;
      sd.kstep = 64 * o.ld;
      sd.tstep = 2;
    } else {
      const int kl = lane >> 3, slot = lane & 7;
      sd.base = o.base + 8L * wave * o.ld;
      sd.v = (uint32_t)(kl * o.ld + ((slot ^ (2 * ((kl >> 1) & 3))) << 4));
      sd.istep = 64 * o.ld;
      sd.hstep = 128;
      sd.kstep = 128 * o.ld;
      sd.tstep = 1;
    }
    return sd;
  };
  const Side sp = make_side(a.P, LAYP), sq = make_side(a.Q, LAYQ);

  // work item -> operand addresses of its first k-tile (P side, Q side), output tile origin and split
  auto tile_of = [&](int w, long& p0, long& q0, int& split) {
    split = 0;
    if (a.splits > 1) {
      split = fastdiv(w, a.d_nout);
      w -= split * a.nout;
    }
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
  auto krange = [&](int split, int& k0, int& n) {
    k0 = 0;
    n = a.nk_total;
    if (a.splits > 1) {
      k0 = (int)((long)split * a.nk_total / a.splits);
      n = (int)((long)(split + 1) * a.nk_total / a.splits) - k0;
    }
  };
  auto origin = [&](const Side& sd, long r0, int k0) { return sd.base + r0 * sd.tstep + (long)k0 * sd.kstep; };

  // quarter (X: 0 P, 1 Q; half h) of stage S <- the k-tile at g (the side's address of that k-tile of the output tile)
  auto dma = [&](int S, int X, int h, const uint8_t* g) {
    const Side& sd = X ? sq : sp;
    uint8_t* d = lds + S * 65536 + X * 32768 + h * 16384 + wave * 1024;
#pragma unroll
    for (int i = 0; i < 2; ++i)
      __builtin_amdgcn_global_load_lds((tfb_glb_void_t*)(g + h * sd.hstep + i * sd.istep + (size_t)sd.v),
                                       (tfb_lds_void_t*)(d + i * 8192), 16, 0, 0);
  };

  // ---- fragment addresses (stage 0; the stage bit is toggled after every k-tile)
  uint32_t ap[4], aq[4];
  {
    const uint32_t lbase = (uint32_t)(size_t)(tfb_lds_u8*)lds;
    const int rp = wr * 64 + lr, rq = wc * 32 + lr;
    // k-contiguous, one address per k-step. bf16: k-step s (16 k) of a row is chunk 2 s + lh; fp8: k-step s (64 k) is
    // chunks 4 s + 2 lh, + 1: entry 2 s + u
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int c = ES == 2 ? 2 * s + lh : 4 * (s >> 1) + 2 * lh + (s & 1);
      ap[s] = lbase + rp * 128 + (((c ^ tfb_kc_swz(rp)) & 7) << 4);
      aq[s] = lbase + 32768 + rq * 128 + (((c ^ tfb_kc_swz(rq)) & 7) << 4);
    }
    // k-strided: 16-lane group g4 reads rows 16 (g4 & 1) .. + 15 of an MFMA tile, k-group g4 >> 1; lane j of the group
    // points at k-row j / 4 (of four consecutive k), rows 4 (j % 4) .. + 3. One address per 32-row tile (ap[0], ap[1]:
    // the second tile's chunk index differs in bit 2, which the swizzle also touches, so it is not an immediate offset);
    // k-step s is 16 k-rows further (an immediate), the fragment's upper four k another 4 k-rows.
    const int g4 = lane >> 4, j = lane & 15, kq = j >> 2;
    // fp8: lane j of the group points at k-row j / 2 (of eight consecutive k), rows 8 (j % 2) .. + 7; the group's k-half
    // is 32 k-rows further, a k-step 64, the fragment's next eight k 8 (immediates).
    auto tr_addr = [&](int row0) {
      if (ES == 2) {
        const int p = row0 + 16 * (g4 & 1) + 4 * (j & 3);
        return (uint32_t)((8 * (g4 >> 1) + kq) * 256 + ((((p >> 3) ^ (4 * kq)) << 4) | ((p & 4) << 1)));
      }
      const int p = row0 + 16 * (g4 & 1) + 8 * (j & 1), k8 = j >> 1;
      return (uint32_t)((32 * (g4 >> 1) + k8) * 128 + ((((p >> 4) ^ (2 * ((k8 >> 1) & 3))) << 4) | (p & 8)));
    };
    if (LAYP == TFB_K_STRIDED) {
      ap[0] = lbase + tr_addr(wr * 64);
      ap[1] = lbase + tr_addr(wr * 64 + 32);
    }
    if (LAYQ == TFB_K_STRIDED) aq[0] = lbase + 32768 + tr_addr(wc * 32);
  }
  constexpr int NAP = LAYP == TFB_K_STRIDED ? 2 : 4, NAQ = LAYQ == TFB_K_STRIDED ? 1 : 4;  // addresses in use

  f32x16 acc[2][2][2];  // [P half][i][Q half]
  // fragments: bf16 four k-steps of 16 (one 128-bit read each), fp8 two k-steps of 64 (two 128-bit reads each)
  typedef std::conditional_t<ES == 2, bf16x8, i32x4> r128_t;
  r128_t fa[2][4], fb0[4], fb1[4];
  auto tr_frag = [&](auto OFF, uint32_t addr) {
    constexpr int off = decltype(OFF)::value;
    if constexpr (ES == 2) {  // k-step off / 4096: 16 k-rows of 256 bytes; the upper four k 4 rows further
      const tfb_s16x4 lo = tfb_lds_read_tr64<off>(addr), hi = tfb_lds_read_tr64<off + 1024>(addr);
      const tfb_s16x8 v = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      return __builtin_bit_cast(r128_t, v);
    } else {  // half a 64-k fragment: 16 k of a row, two reads 8 k-rows (1 KB) apart
      const tfb_pp_i32x2 lo = tfb_lds_read_tr64_b8<off>(addr), hi = tfb_lds_read_tr64_b8<off + 1024>(addr);
      return r128_t{lo.x, lo.y, hi.x, hi.y};
    }
  };
  // fragment entry e (bf16: k-step e of 16 k; fp8: half e & 1 of k-step e >> 1 of 64 k) -> byte offset in a quarter
  constexpr int TR1 = ES == 2 ? 4096 : 2048, TR2 = 8192, TR3 = ES == 2 ? 12288 : 8192 + 2048;
  auto readA = [&](auto H) __attribute__((always_inline)) {
    constexpr int h = decltype(H)::value;
    if constexpr (LAYP == TFB_K_CONTIG) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        fa[0][s] = tfb_lds_read128<h * 16384, r128_t>(ap[s]);
        fa[1][s] = tfb_lds_read128<h * 16384 + 4096, r128_t>(ap[s]);
      }
    } else {
      fa[0][0] = tr_frag(std::integral_constant<int, h * 16384>{}, ap[0]);
      fa[1][0] = tr_frag(std::integral_constant<int, h * 16384>{}, ap[1]);
      fa[0][1] = tr_frag(std::integral_constant<int, h * 16384 + TR1>{}, ap[0]);
      fa[1][1] = tr_frag(std::integral_constant<int, h * 16384 + TR1>{}, ap[1]);
      fa[0][2] = tr_frag(std::integral_constant<int, h * 16384 + TR2>{}, ap[0]);
      fa[1][2] = tr_frag(std::integral_constant<int, h * 16384 + TR2>{}, ap[1]);
      fa[0][3] = tr_frag(std::integral_constant<int, h * 16384 + TR3>{}, ap[0]);
      fa[1][3] = tr_frag(std::integral_constant<int, h * 16384 + TR3>{}, ap[1]);
    }
  };
  // flip = 0x10000: the fragments of the OTHER stage (the next k-tile)
  auto readB = [&](auto H, r128_t(&fb)[4], uint32_t flip = 0) __attribute__((always_inline)) {
    constexpr int h = decltype(H)::value;
    if constexpr (LAYQ == TFB_K_CONTIG) {
#pragma unroll
      for (int s = 0; s < 4; ++s) fb[s] = tfb_lds_read128<h * 16384, r128_t>(aq[s] ^ flip);
    } else {
      fb[0] = tr_frag(std::integral_constant<int, h * 16384>{}, aq[0] ^ flip);
      fb[1] = tr_frag(std::integral_constant<int, h * 16384 + TR1>{}, aq[0] ^ flip);
      fb[2] = tr_frag(std::integral_constant<int, h * 16384 + TR2>{}, aq[0] ^ flip);
      fb[3] = tr_frag(std::integral_constant<int, h * 16384 + TR3>{}, aq[0] ^ flip);
    }
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
  if (a.ipx > 0) {
    if ((w >> 3) >= a.ipx) return;
    w = (w & 7) * a.ipx + (w >> 3);
  }
  if (w >= a.ntiles) return;  // (whole workgroup)
  long p0, q0;
  int split, k0;
  tile_of(w, p0, q0, split);
  krange(split, k0, nkt);
  const uint8_t* gp = origin(sp, p0, k0);  // current work item: the sides' addresses of its first k-tile
  const uint8_t* gq = origin(sq, q0, k0);

  // ---- prologue: all of k-tile 0 into stage 0, three quarters of k-tile 1 into stage 1
  dma(0, 1, 0, gq);
  dma(0, 0, 0, gp);
  dma(0, 1, 1, gq);
  dma(0, 0, 1, gp);
  dma(1, 0, 0, gp + sp.kstep);
  dma(1, 1, 0, gq + sq.kstep);
  dma(1, 1, 1, gq + sq.kstep);
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
        if constexpr (!kF32) {
          u32x2 v = {pack2bf(epi.pre(c[4 * jj + 0]), epi.pre(c[4 * jj + 1])),
                     pack2bf(epi.pre(c[4 * jj + 2]), epi.pre(c[4 * jj + 3]))};
          *(u32x2*)(stg + lr * 128 + (((4 * i + jj) ^ ((lr >> 1) & 7)) << 4) + 8 * lh) = v;
        }
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
      } else if constexpr (!kF32) {
        epi.chunk(p, q, v);
      }
    }
    __builtin_amdgcn_wave_barrier();
  };

  // The same for the partial tile of a k-split (epilogues with kSplitF32): sixteen output rows at a time pass through the
  // 4 KB as fp32 (row = 256 bytes, 16-byte chunk c at slot c ^ row), and a lane finishes 8 consecutive fp32 outputs.
  auto store_block_f32 = [&](auto HP, auto HQ, long tp0, long tq0, int sp_) __attribute__((always_inline)) {
    constexpr int hp = decltype(HP)::value, hq = decltype(HQ)::value;
    const int pb = (int)tp0 + hp * 128 + wr * 64, qb = (int)tq0 + hq * 128 + wc * 32;
    const int ch = lane & 7, r8 = lane >> 3;
#pragma unroll
    for (int qh = 0; qh < 2; ++qh) {
      if ((lr >> 4) == qh) {
        const int row = lr & 15;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
            const f32x16& c = acc[hp][i][hq];
            const f32x4 v = {c[4 * jj + 0], c[4 * jj + 1], c[4 * jj + 2], c[4 * jj + 3]};
            *(f32x4*)(stg + row * 256 + (((8 * i + 2 * jj + lh) ^ row) << 4)) = v;
          }
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int row = r8 + 8 * k;
        const f32x4 lo = *(const f32x4*)(stg + row * 256 + (((2 * ch) ^ row) << 4));
        const f32x4 hi = *(const f32x4*)(stg + row * 256 + (((2 * ch + 1) ^ row) << 4));
        const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        if constexpr (kF32) epi(pb + 8 * ch, qb + 16 * qh + row, v, sp_);
      }
      __builtin_amdgcn_wave_barrier();
    }
  };

  int S = 0;
  if (TFB_PP_EARLYB) readB(H0{}, fb0);
  bool have_prev = false;  // the previous tile's accumulators are still to be stored
  long pp0 = 0, pq0 = 0;   // its origin
  for (;;) {
    // the workgroup's next work item (its first k-tiles are requested by this one's last iterations); past the end: this
    // one again (loads nobody reads, from valid memory)
    const int wn = a.ipx > 0 ? a.ntiles : w + a.nwg;
    long pn = p0, qn = q0;
    int splitn = split, k0n = k0, nktn = nkt;
    if (wn < a.ntiles) {
      tile_of(wn, pn, qn, splitn);
      krange(splitn, k0n, nktn);
    }
    const uint8_t* gpn = origin(sp, pn, k0n);
    const uint8_t* gqn = origin(sq, qn, k0n);

    // One k-tile. In a tile's first iteration the MFMAs start from zero, and each accumulator block of the PREVIOUS tile is
    // stored in the memory cluster in front of the MFMA cluster that overwrites it: the stores of one group (4 KB per
    // wavefront and cluster) run under the other group's MFMAs.
    auto iter = [&](auto FIRST, int kt) __attribute__((always_inline)) {
      constexpr bool first = decltype(FIRST)::value;
      // k positions one and two ahead in the workgroup's stream of k-tiles
      const bool in1 = kt + 1 < nkt, in2 = kt + 2 < nkt;
      const long k1 = in1 ? kt + 1 : 0, k2 = in2 ? kt + 2 : kt + 2 - nkt;
      const uint8_t* gp1 = (in1 ? gp : gpn) + k1 * sp.kstep;
      const uint8_t* gp2 = (in2 ? gp : gpn) + k2 * sp.kstep;
      const uint8_t* gq2 = (in2 ? gq : gqn) + k2 * sq.kstep;
      // c0 (the Q fragments of half 0 were requested in the previous k-tile's c7)
      if (!TFB_PP_EARLYB) readB(H0{}, fb0);
      readA(H0{});
      dma(S ^ 1, 0, 1, gp1);
      if constexpr (!kF32) {
        if (first && have_prev) store_block(H0{}, H0{}, pp0, pq0);
      }
      TFB_SBAR();
      // c1
      waitB(fb0);
      waitA();
      mma(FIRST, H0{}, H0{}, fb0);
      TFB_SBAR();
      // c2
      readB(H1{}, fb1);
      dma(S, 0, 0, gp2);
      if constexpr (!kF32) {
        if (first && have_prev) store_block(H0{}, H1{}, pp0, pq0);
      }
      TFB_SBAR();
      // c3
      waitB(fb1);
      mma(FIRST, H0{}, H1{}, fb1);
      TFB_SBAR();
      // c4
      readA(H1{});
      dma(S, 1, 0, gq2);
      if constexpr (!kF32) {
        if (first && have_prev) store_block(H1{}, H0{}, pp0, pq0);
      }
      TFB_SBAR();
      // c5
      waitA();
      mma(FIRST, H1{}, H0{}, fb0);
      if (TFB_PP_EARLYB) {
        // Completion is reported in issue order, stores included. Everything up to the quarter requested in c0 has to be
        // there one cluster before the other group's matching wait: all but the two quarters requested since (4
        // instructions), and in a first iteration with stores all but those and the 12 stores (c0's four were issued
        // behind its loads). After the barrier that ends c6 both groups have waited, so the next k-tile is complete.
        if (!kF32 && first && have_prev) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      }
      TFB_SBAR();
      // c6
      dma(S, 1, 1, gq2);
      if (!kF32 && first && have_prev) {
        if constexpr (!kF32) store_block(H1{}, H1{}, pp0, pq0);
        if (!TFB_PP_EARLYB) asm volatile("s_waitcnt vmcnt(22)" ::: "memory");
      } else {
        if (!TFB_PP_EARLYB) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
      }
      TFB_SBAR();
      // c7: the next k-tile's first Q fragments are requested under this cluster's MFMAs (fb0 was last read in c5)
      if (TFB_PP_EARLYB) readB(H0{}, fb0, 0x10000u);
      mma(FIRST, H1{}, H1{}, fb1);
      TFB_SBAR();
      S ^= 1;
#pragma unroll
      for (int s = 0; s < NAP; ++s) ap[s] ^= 0x10000u;
#pragma unroll
      for (int s = 0; s < NAQ; ++s) aq[s] ^= 0x10000u;
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
    if constexpr (kF32) {
      // a k-split's partial tile: stored here, both groups together (a work item is hundreds of k-tiles long)
      if (wr == 0) TFB_SBAR();  // group 0 waits for group 1's last cluster
      store_block_f32(H0{}, H0{}, p0, q0, split);
      store_block_f32(H0{}, H1{}, p0, q0, split);
      store_block_f32(H1{}, H0{}, p0, q0, split);
      store_block_f32(H1{}, H1{}, p0, q0, split);
    } else {
      have_prev = true;
      pp0 = p0;
      pq0 = q0;
    }
    w = wn;
    if (w >= a.ntiles) break;
    p0 = pn;
    q0 = qn;
    split = splitn;
    k0 = k0n;
    nkt = nktn;
    gp = gpn;
    gq = gqn;
    if constexpr (kF32) {
      if (wr == 1) TFB_SBAR();  // group 1 falls one cluster behind again
    }
  }
  if constexpr (!kF32) {
    // the last tile's accumulators
    store_block(H0{}, H0{}, pp0, pq0);
    store_block(H0{}, H1{}, pp0, pq0);
    store_block(H1{}, H0{}, pp0, pq0);
    store_block(H1{}, H1{}, pp0, pq0);
  }
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

// np, nq multiples of 256; kbytes = the contraction in bytes of a k-contiguous row (elements * ES), a multiple of 128
// with at least two k-tiles per split. With splits > 1 the epilogue is one with kSplitF32 (EpiSplit); when all work items
// fit one round of the CUs they are dealt to the XCDs in consecutive runs (PpArgs::ipx).
template <int ES, int FMTP, int FMTQ, int LAYP, int LAYQ, class Epi>
static int gemm_pp_launch_lay(GemmOperand P, GemmOperand Q, int np, int nq, long kbytes, int splits, Epi epi, hipStream_t stream) {
  if (np <= 0 || nq <= 0 || splits <= 0 || np % 256 || nq % 256 || kbytes % 128 || kbytes / 128 / splits < 2)
    return TFB_ERR_SHAPE;
  if (P.ld <= 0 || Q.ld <= 0 || P.ld > (1L << 28) || Q.ld > (1L << 28)) return TFB_ERR_SHAPE;
  if (((uintptr_t)P.base | (uintptr_t)Q.base | (uintptr_t)P.ld | (uintptr_t)Q.ld) & 15) return TFB_ERR_ARG;
  if ((splits > 1) != has_split_f32<Epi>::value) return TFB_ERR_ARG;
  PpArgs a = {};
  a.P = P;
  a.Q = Q;
  a.splits = splits;
  a.nk_total = (int)(kbytes / 128);
  const int ntp = np / 256, ntq = nq / 256;
  if ((long)ntp * ntq * splits >= (1L << 30)) return TFB_ERR_SHAPE;
  a.nout = ntp * ntq;
  a.ntiles = a.nout * splits;
  const int cus = tfb_resident_slots(1);
  a.p_fast = np <= nq;
  a.nfast = a.p_fast ? ntp : ntq;
  const int nslow = a.p_fast ? ntq : ntp;
  a.rect = (nslow % 8 == 0) && a.nout >= 8;
  a.nwg = a.ntiles < cus ? a.ntiles : cus;
  if (splits > 1 && a.ntiles <= cus) {
    a.rect = 0;
    a.ipx = (a.ntiles + 7) / 8;
    a.nwg = 8 * a.ipx;
  }
  if (a.rect) a.nwg &= ~7;
  if (a.nwg <= 0) return TFB_ERR_SHAPE;
  a.R = a.rect ? nslow / 8 : 1;
  // panel width: GW * R ~ the 32 workgroups an XCD runs together; a narrow fast operand (<= 4 tiles) is walked whole, so
  // that the tiles sharing a row block of the slow operand run together
  int gw = a.R >= 32 ? 1 : (32 + a.R - 1) / a.R;
  if (a.R > 8 && a.R < 32) gw = 32 / a.R > 0 ? 32 / a.R : 1;
  if (gw > a.nfast || a.nfast <= 4) gw = a.nfast;
  a.GW = gw;
  a.panel = a.GW * a.R;
  a.gw_last = a.nfast % a.GW ? a.nfast % a.GW : a.GW;
  a.d_nfast = fastdiv_make(a.nfast);
  a.d_panel = fastdiv_make(a.panel);
  a.d_gw = fastdiv_make(a.GW);
  a.d_gw_last = fastdiv_make(a.gw_last);
  a.d_nout = fastdiv_make(a.nout);
  hipLaunchKernelGGL((gemm_pp_kernel<ES, FMTP, FMTQ, LAYP, LAYQ, Epi>), dim3(a.nwg), dim3(512), 0, stream, a, epi);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// k ranges for a long contraction (nkt k-tiles) over fewer than 64 output tiles of 256 x 256, one work item per workgroup:
// up to 32 tiles, as many ranges per XCD as its CUs have room for tiles (an XCD's workgroups then read one k range of the
// operands together: 27 tiles -> 8 ranges, 9 tiles -> 24); beyond, the count that fills the CUs. 0: not worth it (less
// than 80 % of the CUs busy, fewer than 16 k-tiles per item, or the partial tiles do not fit the workspace).
static inline int gemm_pp_fewtile_splits(long t256, long nkt, long out_elems, long ws_bytes) {
  const long cus = tfb_resident_slots(1);
  if (t256 <= 0 || t256 >= 64) return 0;
  int c = t256 * 8 <= cus ? 8 * (int)(cus / 8 / t256) : (int)(cus / t256);
  while (c > 1 && (nkt / c < 16 || (long)c * out_elems * 4 > ws_bytes)) --c;
  return (c > 1 && (double)(t256 * c) >= 0.8 * (double)cus) ? c : 0;
}

// both operands k-contiguous, no k-split
template <int ES, int FMTP, int FMTQ, class Epi>
static int gemm_pp_launch(GemmOperand P, GemmOperand Q, int np, int nq, long kbytes, Epi epi, hipStream_t stream) {
  if (kbytes < 256) return TFB_ERR_SHAPE;
  return gemm_pp_launch_lay<ES, FMTP, FMTQ, TFB_K_CONTIG, TFB_K_CONTIG>(P, Q, np, nq, kbytes, 1, epi, stream);
}

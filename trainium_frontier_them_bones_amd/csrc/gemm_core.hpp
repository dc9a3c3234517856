// MFMA GEMM core for gfx950: D[p][q] = sum_k P[p][k] * Q[q][k], fp32 accumulation.
//
// One workgroup of WP x WQ wavefronts owns a BP x BQ output tile; a wavefront owns TP x TQ MFMA tiles of 32 x 32.
// Operand tiles (128 bytes of k per row: 64 bf16 or 128 fp8) go from global memory straight into LDS with
// global_load_lds_dwordx4 (no staging registers, no VALU work): one instruction moves 1 KB, lane l filling bytes
// 16 l .. 16 l + 15, so the LDS layout is chosen by which 16-byte global chunk each lane fetches:
//   K_CONTIG  [rows][K]:  LDS row = 128 bytes of k, chunk c of row r at slot c ^ (4 ((r >> 1) & 1) | ((r >> 2) & 3))
//             (tfb_kc_swz): the 128-bit fragment reads of a wavefront (32 rows x 2 chunks) then count no bank
//             conflicts (LDS here has 64 banks of 4 bytes).
//   K_STRIDED [K][rows]:  LDS row = one k with the tile's rows contiguous. bf16: 16-byte chunk c of k-row k at slot
//             c ^ (4 (k & 3)); fragments are fetched with ds_read_b64_tr_b16, whose 16-lane transpose hands lane i
//             four consecutive k of row i when lane j points at (k0 + j / 4, row0 + 4 (j % 4)). fp8 (128-row tiles):
//             slot c ^ (2 ((k >> 1) & 3)) and ds_read_b64_tr_b8 (lane j at (k0 + j / 2, row0 + 8 (j % 2)) gives lane i
//             eight consecutive k of row i).
// Two LDS buffers (separate __shared__ objects, so the compiler can tell a fragment read of one from the loads in
// flight into the other and does not wait for them), loads of k-tile t+1 in flight during the MFMAs of tile t, one
// barrier per k-tile, fragments of k-step s+1 requested between the MFMAs of step s.
// The P tile feeds the MFMA A operand (rows), the Q tile the B operand (columns), so a lane ends up holding
// D[p .. p+3][q] for four consecutive p: callers put the dimension that is contiguous in the output on the P side.
//
// Epilogues: "staged" (default) - each wavefront passes its accumulators through its own LDS slice, 32 output rows
// at a time, and every lane then owns 8 consecutive p of one q, so global reads/writes of the epilogue are 128-bit
// and coalesced along the output rows; or "tile" (kTileEpilogue) - the functor gets the raw accumulator registers
// (used when the epilogue reduces along p in registers).
//
// Element types: bf16 (v_mfma_f32_32x32x16_bf16) or OCP fp8 (v_mfma_scale_f32_32x32x64_f8f6f4 with unit scales,
// e4m3/e5m2 per side).
#pragma once
#include <type_traits>

#include "common.hpp"

// slot swizzle of the K_CONTIG layout: chunk c of row r sits at slot c ^ tfb_kc_swz(r). With this map the 128-bit fragment
// reads count no bank conflicts (SQ_LDS_BANK_CONFLICT 0); the earlier map (r + r / 8) & 7 cost every such read 4 cycles.
__device__ __forceinline__ int tfb_kc_swz(int r) { return (4 * ((r >> 1) & 1)) | ((r >> 2) & 3); }
#define TFB_K_CONTIG 0
#define TFB_K_STRIDED 1

struct GemmOperand {
  const uint8_t* base;
  long ld;  // bytes between consecutive rows (K_CONTIG) or consecutive k (K_STRIDED)
};

// n / d for 0 <= n < 2^31 as one 64-bit multiply and a shift: m = ceil(2^(31 + s) / d) with s = ceil(log2 d) (exact for
// every such n because m d - 2^(31 + s) <= 2^s). The host builds it once per launch; in the kernel a division by a launch
// parameter would otherwise be ~25 dependent instructions per wavefront (~200 for a 64-bit one) before the first load.
struct FastDiv {
  uint32_t m, sh;
};
static inline FastDiv fastdiv_make(uint32_t d) {
  if (d == 0) d = 1;
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;
  FastDiv f;
  f.m = (uint32_t)(((1ull << (31 + s)) + d - 1) / d);
  f.sh = 31 + s;
  return f;
}
__device__ __forceinline__ int fastdiv(int n, FastDiv f) { return (int)(((uint64_t)(uint32_t)n * f.m) >> f.sh); }

struct GemmArgs {
  GemmOperand P, Q;
  int np, nq;   // output extent (multiples of BP / BQ)
  int nkt;      // k-tiles (128 bytes of k each) in all; split z of `splits` takes tiles [z nkt / Z, (z + 1) nkt / Z)
  int splits;   // k-splits: gridDim.x = output tiles * splits
  int gblock;   // tiles of the smaller operand per traversal block (see the kernel); 0: plain row-major traversal
  int ntp;      // tiles along p
  int slots;    // workgroups resident at once (2 per CU): the first round of the launch, when it is to be staggered
                //   (see the kernel; 0: no stagger)
  int sleeps;   // length of that stagger in s_sleep(127) units
  // Grouped (ragged) launches, both optional:
  const int* q_group;    // group id of each q tile (-1: the tile is beyond the ragged extent, the workgroup exits);
  long p_group_stride;   //   the P operand of group g starts p_group_stride bytes * g further (per-expert weights)
  const int* k_seg;      // [groups + 1] k offsets in elements: group = blockIdx.y contracts over k_seg[g] .. k_seg[g+1]
  // Filled by gemm_launch_args from the fields above (the workgroup -> tile map, with its divisions prepared):
  int ntiles;   // output tiles
  int per;      // ntiles / 8 when ntiles is a multiple of 8 (an XCD's run of tiles), else 0: no re-dealing of ids
  int nfast;    // tiles of the operand the traversal walks fastest
  int p_fast;   // that operand is P
  int rows;     // block traversal: rows of tiles of the other operand in one XCD's run (0: plain traversal)
  int blk;      // gblock * rows
  FastDiv d_ntiles, d_per, d_nfast, d_blk, d_gblock, d_splits, d_split8;  // d_split8: by splits / 8
};

// Operand pre-operation, applied to a fragment (8 bf16 along k of one row) on its way into the MFMA.
struct LoadIdentity {
  template <class T>
  __device__ __forceinline__ T operator()(T v) const { return v; }
};

typedef __attribute__((address_space(3))) void tfb_lds_void_t;
typedef const __attribute__((address_space(1))) void tfb_glb_void_t;
typedef short tfb_s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) tfb_s16x4 tfb_lds_s16x4_t;

template <int BP_, int BQ_, int WP_, int WQ_, int ES_, int LAYP_, int LAYQ_, int FMTP_ = 0, int FMTQ_ = 0, int OCC_ = 0,
          int NSTAGE_ = 2>
struct GemmCfg {
  static constexpr int NSTAGE = NSTAGE_;  // LDS stages: 2 (one k-tile of loads in flight)
  static constexpr int BP = BP_, BQ = BQ_, WP = WP_, WQ = WQ_, ES = ES_;
  static constexpr int LAYP = LAYP_, LAYQ = LAYQ_, FMTP = FMTP_, FMTQ = FMTQ_;
  static constexpr int NW = WP * WQ, NT = NW * 64;
  static constexpr int TP = BP / WP / 32, TQ = BQ / WQ / 32;
  static constexpr int BK = 128 / ES;                  // elements of k per tile
  static constexpr int STAGE_BYTES = (BP + BQ) * 128;  // one k-tile of both operands
  // epilogue staging: a wavefront's slice is 32 rows x (ETP * 32) floats (+ 4 of pad); ETP of the TP tiles per pass
  static constexpr int EPI_LIMIT = 72 * 1024;
  static constexpr int ETP = (TP >= 2 && NW * 32 * (TP * 32 + 4) * 4 > EPI_LIMIT) ? TP / 2 : TP;
  static constexpr int STAGE_LD = ETP * 32 + 4;
  static constexpr int EPI_BYTES = NW * 32 * STAGE_LD * 4;
  static constexpr int BUF0_BYTES = STAGE_BYTES > EPI_BYTES ? STAGE_BYTES : EPI_BYTES;
  static constexpr int LDS_BYTES = BUF0_BYTES + (NSTAGE - 1) * STAGE_BYTES;
  // wavefronts per SIMD the kernel is compiled for: two workgroups per CU when registers and LDS allow it
  static constexpr int OCC = OCC_ > 0 ? OCC_ : ((NT <= 256 && 2 * LDS_BYTES <= 160 * 1024 && TP * TQ <= 4) ? 2 : 1);
  static_assert(ES == 1 || ES == 2, "fp8 or bf16");
  static_assert(NW >= 4 && (NW & (NW - 1)) == 0, "4, 8 or 16 wavefronts");
  static_assert((BP / 8) % NW == 0 && (BQ / 8) % NW == 0, "1 KB load instructions vs wavefronts");
  static_assert(LAYP == TFB_K_CONTIG || BP == 128 || BP == 256, "K_STRIDED tiles are 128 or 256 rows");
  static_assert(LAYQ == TFB_K_CONTIG || BQ == 128 || BQ == 256, "K_STRIDED tiles are 128 or 256 rows");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS");
  static_assert(NSTAGE == 2, "two LDS stages (a three-stage loop was measured no faster and removed)");
};

// ---- global -> LDS (one operand tile, this wavefront's share) ---------------------------------------------------
template <int ROWS, int NW, int LAY, int ES = 2>
struct TileDma;

template <int ROWS, int NW, int ES>
struct TileDma<ROWS, NW, TFB_K_CONTIG, ES> {
  static constexpr int NI = ROWS / 8 / NW;            // instructions per wavefront: 8 rows x 128 bytes each
  static constexpr int NV = NW >= 8 ? 1 : 8 / NW;     // distinct per-lane offsets over the instructions
  const uint8_t* base;  // wavefront-uniform
  long step;            // bytes between this wavefront's consecutive instructions
  uint32_t voff[NV];
  __device__ __forceinline__ void init(const GemmOperand& o, long row0, long k0_bytes, int wave, int lane) {
    const int lrow = lane >> 3;
    base = o.base + (row0 + wave * 8) * o.ld + k0_bytes;
    step = 8L * NW * o.ld;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      // rows 8 g .. 8 g + 7 with g = i * NW + wave; slot (lane & 7) of row r holds chunk slot ^ tfb_kc_swz(r), which
      // depends on g through its parity only (NW is even), so NV offsets serve all instructions
      const int ch = (lane & 7) ^ tfb_kc_swz(lrow + 8 * (v * NW + wave));
      voff[v] = (uint32_t)(lrow * o.ld + ch * 16);
    }
  }
  // k-tile t of the split (128 bytes of k further per tile)
  __device__ __forceinline__ void issue(uint8_t* lds, int t, int wave) const {
#pragma unroll
    for (int i = 0; i < NI; ++i)
      __builtin_amdgcn_global_load_lds((tfb_glb_void_t*)(base + i * step + (long)t * 128 + (size_t)voff[i % NV]),
                                       (tfb_lds_void_t*)(lds + (i * NW + wave) * 1024), 16, 0, 0);
  }
};

template <int ROWS, int NW, int ES>
struct TileDma<ROWS, NW, TFB_K_STRIDED, ES> {
  static constexpr int LPR = ROWS * ES / 16;   // lanes (16-byte chunks) per k-row
  static constexpr int RPI = 64 / LPR;         // k-rows per instruction
  static constexpr int KROWS = 128 / ES;       // k-rows per tile
  static constexpr int NI = KROWS / RPI / NW;  // = ROWS / 8 / NW
  // the swizzle term (k & 3 for bf16, (k >> 1) & 3 for fp8) must not depend on the instruction index
  static_assert((NW * RPI) % (ES == 2 ? 4 : 8) == 0, "swizzle phase vs instruction index");
  static_assert(ES == 2 || ROWS == 128, "fp8 K_STRIDED tiles are 128 rows");
  const uint8_t* base;
  long step, tstep;
  uint32_t voff;
  __device__ __forceinline__ void init(const GemmOperand& o, long row0, long k0_bytes, int wave, int lane) {
    const int kl = lane / LPR, slot = lane % LPR;
    const long k0 = k0_bytes / ES;  // elements
    base = o.base + (k0 + (long)wave * RPI) * o.ld + row0 * ES;
    step = (long)NW * RPI * o.ld;
    tstep = (long)KROWS * o.ld;
    const int k = wave * RPI + kl;  // the swizzle phase of the k-row this lane fills, the same for every instruction
    const int sw = ES == 2 ? 4 * (k & 3) : 2 * ((k >> 1) & 3);
    voff = (uint32_t)(kl * o.ld + ((slot ^ sw) * 16));
  }
  __device__ __forceinline__ void issue(uint8_t* lds, int t, int wave) const {
#pragma unroll
    for (int i = 0; i < NI; ++i)
      __builtin_amdgcn_global_load_lds((tfb_glb_void_t*)(base + i * step + t * tstep + (size_t)voff),
                                       (tfb_lds_void_t*)(lds + (i * NW + wave) * 1024), 16, 0, 0);
  }
};

// ---- LDS -> MFMA fragments ---------------------------------------------------------------------------------------
// Per-lane addressing of one operand: off(i, s) = byte offset of the lane's fragment of MFMA tile i, k-step s.
template <int ROWS, int ES, int LAY>
struct FragReader;

template <int ROWS>
struct FragReader<ROWS, 2, TFB_K_CONTIG> {
  static constexpr int KSTEPS = 4;
  typedef bf16x8 frag_t;
  int row, lh;
  __device__ __forceinline__ void init(int wave_row0, int lane) { row = wave_row0 + (lane & 31); lh = lane >> 5; }
  __device__ __forceinline__ frag_t read(const uint8_t* lds, int i, int s) const {
    const int r = row + 32 * i;
    return *(const bf16x8*)(lds + r * 128 + ((((2 * s + lh) ^ tfb_kc_swz(r)) & 7) << 4));
  }
};
template <int ROWS>
struct FragReader<ROWS, 1, TFB_K_CONTIG> {
  static constexpr int KSTEPS = 2;
  typedef i32x8 frag_t;
  int row, lh;
  __device__ __forceinline__ void init(int wave_row0, int lane) { row = wave_row0 + (lane & 31); lh = lane >> 5; }
  __device__ __forceinline__ frag_t read(const uint8_t* lds, int i, int s) const {
    const int r = row + 32 * i, f = tfb_kc_swz(r);
    const i32x4 a = *(const i32x4*)(lds + r * 128 + ((((4 * s + 2 * lh) ^ f) & 7) << 4));
    const i32x4 b = *(const i32x4*)(lds + r * 128 + ((((4 * s + 2 * lh + 1) ^ f) & 7) << 4));
    return i32x8{a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
  }
};
template <int ROWS>
struct FragReader<ROWS, 2, TFB_K_STRIDED> {
  static constexpr int KSTEPS = 4;
  typedef bf16x8 frag_t;
  static constexpr int PITCH = ROWS * 2;
  int wave_row0, lane;
  __device__ __forceinline__ void init(int wave_row0_, int lane_) { wave_row0 = wave_row0_; lane = lane_; }
  __device__ __forceinline__ frag_t read(const uint8_t* lds, int i, int s) const {
    // 16-lane group g4: rows 16 (g4 & 1) .. + 15 of the MFMA tile, k-group g4 >> 1; lane j of the group points at
    // k-row j / 4 (of four consecutive k), rows 4 (j % 4) .. + 3
    const int g4 = lane >> 4, j = lane & 15;
    const int p = wave_row0 + 32 * i + 16 * (g4 & 1) + 4 * (j & 3);
    const int kq = j >> 2;  // = k & 3
    const int k = 16 * s + 8 * (g4 >> 1) + kq;
    const int off = k * PITCH + ((((p >> 3) ^ (4 * kq)) << 4) | ((p & 4) << 1));
    const tfb_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tfb_lds_s16x4_t*)(lds + off));
    const tfb_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tfb_lds_s16x4_t*)(lds + off + 4 * PITCH));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    const s16x8 v = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    return __builtin_bit_cast(bf16x8, v);
  }
};

// fp8, one k per LDS row of ROWS bytes: ds_read_b64_tr_b8 hands lane i of a 16-lane group the bytes
// src[2 e + (i >> 3)][i & 7], e = 0..7, of the 16 x 8 bytes its lanes point at; with lane j pointing at
// (k0 + j / 2, row0 + 8 (j % 2)) lane i receives 8 consecutive k of row row0 + i. 16-byte chunk c of k-row k sits at
// slot c ^ (2 ((k >> 1) & 3)): the 8 k-rows x 2 chunks that 32 lanes read together then cover all 64 banks once.
template <int ROWS>
struct FragReader<ROWS, 1, TFB_K_STRIDED> {
  static constexpr int KSTEPS = 2;
  typedef i32x8 frag_t;
  static constexpr int PITCH = ROWS;
  int wave_row0, lane;
  __device__ __forceinline__ void init(int wave_row0_, int lane_) { wave_row0 = wave_row0_; lane = lane_; }
  __device__ __forceinline__ frag_t read(const uint8_t* lds, int i, int s) const {
    typedef int tfb_i32x2 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(3))) tfb_i32x2 tfb_lds_i32x2_t;
    const int g4 = lane >> 4, j = lane & 15;
    const int p = wave_row0 + 32 * i + 16 * (g4 & 1) + 8 * (j & 1);  // first of this lane's 8 source rows
    const int kq = j >> 1;                                           // k offset of the source lane, 0..7
    const int k = 64 * s + 32 * (g4 >> 1) + kq;
    const int off = k * PITCH + ((((p >> 4) ^ (2 * ((kq >> 1) & 3))) << 4) | (p & 8));
    frag_t v;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const tfb_i32x2 t = __builtin_amdgcn_ds_read_tr8_b64_v2i32((tfb_lds_i32x2_t*)(lds + off + 8 * q * PITCH));
      v[2 * q] = t.x;
      v[2 * q + 1] = t.y;
    }
    return v;
  }
};

template <int ES, int FMTP, int FMTQ, class FA, class FB>
__device__ __forceinline__ f32x16 mfma32(const FA& a, const FB& b, f32x16 c) {
  if constexpr (ES == 2) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  } else {
    // formats: 0 = e4m3, 1 = e5m2; E8M0 scale byte 127 = 2^0
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, FMTP, FMTQ, 0, 127, 0, 127);
  }
}

template <class T, class = void>
struct has_for_group : std::false_type {};
template <class T>
struct has_for_group<T, std::void_t<decltype(std::declval<const T&>().for_group(0))>> : std::true_type {};
// An epilogue with per-group state (scale row, output slab) provides  Epi for_group(int g) const.
template <class Epi>
__device__ __forceinline__ Epi epi_for_group(const Epi& e, int g) {
  if constexpr (has_for_group<Epi>::value) return e.for_group(g);
  else return e;
}

// An epilogue that reads device scalars (scale rows) provides  Epi prepare() const, called once before the k-loop: it
// returns the functor with those values held in registers. Read inside operator() they would be re-loaded after every
// store (the stores may alias them), and each re-load's wait also waits for every store still in flight: an epilogue of
// eight chunks then costs eight store round trips (measured: twice its GEMM's k-loop).
template <class T, class = void>
struct has_prepare : std::false_type {};
template <class T>
struct has_prepare<T, std::void_t<decltype(std::declval<const T&>().prepare())>> : std::true_type {};
template <class Epi>
__device__ __forceinline__ Epi epi_prepare(const Epi& e) {
  if constexpr (has_prepare<Epi>::value) return e.prepare();
  else return e;
}

// A staged epilogue with the static member kPartner32 also receives the 8 values 32 output columns away (p ^ 32: the
// other half of a 64-wide head, for rotary embeddings): operator()(p, q, v, v_partner, split). Needs a wavefront slice
// of exactly 64 staged columns.
template <class T, class = void>
struct has_partner32 : std::false_type {};
template <class T>
struct has_partner32<T, std::void_t<decltype(T::kPartner32)>> : std::true_type {};

template <class T, class = void>
struct has_tile_epilogue : std::false_type {};
template <class T>
struct has_tile_epilogue<T, std::void_t<decltype(T::kTileEpilogue)>> : std::true_type {};

// the residual a projection's store adds is read once by that kernel (output projection with the hint: 0.72 -> 0.70 ms per step)
#ifndef TFB_NT_RES
#define TFB_NT_RES 1
#endif
#ifndef TFB_STAGGER_SLEEPS
#define TFB_STAGGER_SLEEPS 2
#endif
#ifndef TFB_STAGGER_SHORT_ROUNDS
#define TFB_STAGGER_SHORT_ROUNDS 4
#endif
#ifndef TFB_STAGGER_SPLITK
#define TFB_STAGGER_SPLITK 0
#endif
template <class T, class = void>
struct stagger_sleeps : std::integral_constant<int, TFB_STAGGER_SLEEPS> {};
template <class T>
struct stagger_sleeps<T, std::void_t<decltype(T::kStaggerSleeps)>> : std::integral_constant<int, T::kStaggerSleeps> {};

// A staged epilogue that reads an operand of its own (the saved activation of the fp8 MLP's backward) declares
//   typedef ... pre_t;  pre_t prefetch(int p, int q) const;  void operator()(p, q, v, const pre_t&, split) const;
// prefetch is called for every 8-element chunk the lane will finish BEFORE the k-loop, so those loads are in flight
// under the MFMAs instead of being eight dependent load-use chains at the end of the tile.
template <class T, class = void>
struct has_prefetch : std::false_type {};
template <class T>
struct has_prefetch<T, std::void_t<typename T::pre_t>> : std::true_type {};
template <class T, bool = has_prefetch<T>::value>
struct prefetch_type { typedef int type; };
template <class T>
struct prefetch_type<T, true> { typedef typename T::pre_t type; };

// Epi: either  __device__ void operator()(int p, int q, const float (&v)[8], int split)  with v = D[p..p+7][q], p % 8 == 0,
// or (with a static member kTileEpilogue)  __device__ void tile(acc, pw, qw, lr, lh, tile_id, split).
template <class Cfg, class PreP, class PreQ, class Epi>
__global__ __launch_bounds__(Cfg::NT, Cfg::OCC) void gemm_kernel(GemmArgs a, PreP prep, PreQ preq, Epi epi_in) {
  constexpr int BP = Cfg::BP, BQ = Cfg::BQ, NW = Cfg::NW, TP = Cfg::TP, TQ = Cfg::TQ, ES = Cfg::ES;
  __shared__ __attribute__((aligned(1024))) uint8_t buf0[Cfg::BUF0_BYTES];
  __shared__ __attribute__((aligned(1024))) uint8_t buf1[Cfg::STAGE_BYTES];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  // Two workgroups share a CU. Launched together they run in lockstep: both in the k-loop (each at half the MFMA rate),
  // then both in the epilogue (MFMA idle, memory busy). The one that landed in an odd wavefront slot (HW_ID.wave_id
  // bit 0) therefore starts ~7 us late, once, in the first round of workgroups: from then on one's epilogue runs
  // under the other's MFMAs (measured -0.5 to -1.3 ms per training step; delaying both costs +0.65 ms, none is the
  // old behaviour). Only where there is a second round to overlap with and no k-split (long k-loops, small epilogues).
  constexpr int kSleeps = stagger_sleeps<Epi>::value;  // an epilogue may name its own count (static kStaggerSleeps)
  // All launch parameters the tile map and the first loads need are asked for here, in one batch: left to the compiler
  // they are fetched where first used, four or five dependent round trips to the scalar cache in front of every tile.
  asm volatile("" ::"s"(a.P.base), "s"(a.P.ld), "s"(a.Q.base), "s"(a.Q.ld), "s"(a.nkt), "s"(a.splits), "s"(a.gblock),
               "s"(a.slots), "s"(a.q_group), "s"(a.p_group_stride), "s"(a.k_seg), "s"(a.ntiles), "s"(a.per), "s"(a.nfast),
               "s"(a.p_fast), "s"(a.rows), "s"(a.blk), "s"(a.d_per.m), "s"(a.d_per.sh), "s"(a.d_nfast.m), "s"(a.d_nfast.sh),
               "s"(a.d_blk.m), "s"(a.d_blk.sh), "s"(a.d_gblock.m), "s"(a.d_gblock.sh), "s"(a.d_splits.m), "s"(a.d_splits.sh),
               "s"(a.sleeps));
  if (Cfg::OCC == 2 && kSleeps > 0 && (int)blockIdx.x < a.slots) {
    if (__builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 4) & 1)  // getreg(size 4, offset 0, HW_REG_HW_ID): wave_id
      for (int i = 0; i < a.sleeps; ++i) __builtin_amdgcn_s_sleep(127);  // 127 x 64 clocks each
  }
  const int wp = wave % Cfg::WP, wq = wave / Cfg::WP;
  const int lr = lane & 31, lh = lane >> 5;

  // Workgroup -> (output tile, k-split). Consecutive workgroup ids sit on consecutive XCDs. With a multiple of 8 splits a
  // split stays on ONE XCD: the k-range of both operands it contracts over is then fetched into that XCD's L2 once and
  // shared by all its output tiles, instead of every XCD streaming most of both operands. Without splits, ids are
  // re-dealt so that one XCD gets a contiguous run of tiles. (Everything up to the first operand load below is serial
  // scalar work in front of every tile: the divisions are multiplications prepared by the host.)
  auto xcd_run = [&](int pid) { return a.per ? (pid & 7) * a.per + (pid >> 3) : pid; };
  int lid, split;
  {
    const int L = blockIdx.x;
    if (a.splits == 1) {
      split = 0;
      lid = xcd_run(L);
    } else if ((a.splits & 7) == 0) {
      const int j = L >> 3;
      lid = fastdiv(j, a.d_split8);
      split = (L & 7) + 8 * (j - lid * (a.splits >> 3));
    } else {
      split = fastdiv(L, a.d_ntiles);
      lid = xcd_run(L - split * a.ntiles);
    }
  }
  // An XCD's run of tiles walks the smaller operand's tiles fastest: the run then shares few rows of the larger
  // operand (which is thereby partitioned over the XCDs' L2s) and re-reads the smaller one. When the smaller operand
  // does not fit the L2 beside the streaming larger one (a 3.5 MB weight against a 4 MB L2), the run is walked in
  // blocks of `gblock` of its tiles: block 0 against all of the run's rows of the larger operand, then block 1, ...
  // so the smaller operand is fetched once per XCD instead of once per row of tiles.
  int tile_p, tile_q;
  {
    int fast, slow;
    if (a.rows > 0) {
      const int xcd = fastdiv(lid, a.d_per), idx = lid - xcd * a.per;
      const int b = fastdiv(idx, a.d_blk), rem = idx - b * a.blk;
      const int rg = fastdiv(rem, a.d_gblock);
      fast = b * a.gblock + rem - rg * a.gblock;
      slow = xcd * a.rows + rg;
    } else {
      slow = fastdiv(lid, a.d_nfast);
      fast = lid - slow * a.nfast;
    }
    tile_p = a.p_fast ? fast : slow;
    tile_q = a.p_fast ? slow : fast;
  }
  const long p0 = (long)tile_p * BP, q0 = (long)tile_q * BQ;
  int kt0 = 0;
  if (a.splits > 1) {
    kt0 = fastdiv(split * a.nkt, a.d_splits);
    a.nkt = fastdiv((split + 1) * a.nkt, a.d_splits) - kt0;
  }
  int group = 0;
  if (a.q_group) {
    group = a.q_group[tile_q];
    if (group < 0) return;  // the whole workgroup leaves before any barrier
    a.P.base += (long)group * a.p_group_stride;
  }
  if (a.k_seg) {
    group = blockIdx.y;
    const int k0 = a.k_seg[group], k1 = a.k_seg[group + 1];
    kt0 = k0 * ES / 128;
    a.nkt = (k1 - k0) * ES / 128;  // may be 0: the accumulators stay zero and are still written
  }
  const int nkt = a.nkt;

  // the first k-tile's loads leave before anything else is set up
  TileDma<BP, NW, Cfg::LAYP, ES> dp;
  TileDma<BQ, NW, Cfg::LAYQ, ES> dq;
  dp.init(a.P, p0, (long)kt0 * 128, wave, lane);
  dq.init(a.Q, q0, (long)kt0 * 128, wave, lane);
  auto issue = [&](uint8_t* buf, int t) {
    dp.issue(buf, t, wave);
    dq.issue(buf + BP * 128, t, wave);
  };
  if (nkt > 0) issue(buf0, 0);

  const Epi epi = epi_prepare(epi_for_group(epi_in, group));
  typedef FragReader<BP, ES, Cfg::LAYP> RP;
  typedef FragReader<BQ, ES, Cfg::LAYQ> RQ;
  RP rp;
  RQ rq;
  rp.init(wp * (TP * 32), lane);
  rq.init(wq * (TQ * 32), lane);

  f32x16 acc[TP][TQ];
#pragma unroll
  for (int i = 0; i < TP; ++i)
#pragma unroll
    for (int j = 0; j < TQ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // the staged epilogue's chunk of pass k, column block j: row and first column inside the wavefront's 32-row slice
  constexpr bool kPrefetch = has_prefetch<Epi>::value && !has_tile_epilogue<Epi>::value && Cfg::ETP == TP;
  constexpr int EPI_CPR = Cfg::ETP * 4, EPI_NK = 32 * EPI_CPR / 64;
  auto chunk_row = [&](int k) { return 2 * (((lane >> 3) + k * 8) / (EPI_CPR / 4)) + ((lane >> 2) & 1); };
  auto chunk_col = [&](int k) { return (4 * (((lane >> 3) + k * 8) % (EPI_CPR / 4)) + (lane & 3)) * 8; };
  [[maybe_unused]] typename prefetch_type<Epi>::type pre[TQ][EPI_NK];
  auto prefetch_epilogue = [&]() {
    if constexpr (kPrefetch) {
#pragma unroll
      for (int j = 0; j < TQ; ++j)
#pragma unroll
        for (int k = 0; k < EPI_NK; ++k)
          pre[j][k] = epi.prefetch((int)p0 + wp * (TP * 32) + chunk_col(k), (int)q0 + wq * (TQ * 32) + j * 32 + chunk_row(k));
    }
  };
#ifndef TFB_PREFETCH_AFTER_FIRST
#define TFB_PREFETCH_AFTER_FIRST 1
#endif
  if (!TFB_PREFETCH_AFTER_FIRST) prefetch_epilogue();

  auto compute = [&](const uint8_t* buf) {
    const uint8_t* sp = buf;
    const uint8_t* sq = buf + BP * 128;
    constexpr int KS = RP::KSTEPS;
    constexpr int NR = TP + TQ, NM = TP * TQ;
    typename RP::frag_t fa[2][TP];
    typename RQ::frag_t fb[2][TQ];
    // fragments are requested in the order the MFMAs below first need them: P tile 0, all Q tiles, P tiles 1..
    auto rd = [&](int nb, int s, int r) {
      if (r == 0) fa[nb][0] = prep(rp.read(sp, 0, s));
      else if (r <= TQ) fb[nb][r - 1] = preq(rq.read(sq, r - 1, s));
      else fa[nb][r - TQ] = prep(rp.read(sp, r - TQ, s));
    };
#pragma unroll
    for (int r = 0; r < NR; ++r) rd(0, 0, r);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      int m = 0, r = 0;
#pragma unroll
      for (int i = 0; i < TP; ++i)
#pragma unroll
        for (int j = 0; j < TQ; ++j) {
          acc[i][j] = mfma32<ES, Cfg::FMTP, Cfg::FMTQ>(fa[s & 1][i], fb[s & 1][j], acc[i][j]);
          ++m;
          if (s + 1 < KS) {
            // the next k-step's fragment reads are spread evenly between this step's MFMAs
            while (r < NR && r * NM < m * NR) {
              rd((s + 1) & 1, s + 1, r);
              ++r;
              __builtin_amdgcn_sched_barrier(0);
            }
          }
        }
    }
  };

  {
    __syncthreads();
    // The epilogue's operands are requested here, behind the first k-tile's barrier: vector loads return in order, so
    // asked for before it they made that barrier wait for a stream from HBM; now they fly under the first k-tile's MFMAs.
    if (TFB_PREFETCH_AFTER_FIRST) prefetch_epilogue();
    for (int t = 0; t + 2 <= nkt; t += 2) {
      issue(buf1, t + 1);
      compute(buf0);
      __syncthreads();
      issue(buf0, t + 2 < nkt ? t + 2 : nkt - 1);  // (the last pair re-fetches a tile nobody reads: no branch in the loop)
      compute(buf1);
      __syncthreads();
    }
    if (nkt & 1) compute(buf0);
    __syncthreads();
  }

  const int pw = wp * (TP * 32), qw = wq * (TQ * 32);  // wavefront's origin inside the tile
  if constexpr (has_tile_epilogue<Epi>::value) {
    // whole-accumulator epilogue: acc[i][j][4*jj + e] = D[pw + 32 i + 8 jj + 4 lh + e][qw + 32 j + lr]
    epi.tile(acc, (int)p0 + pw, (int)q0 + qw, lr, lh, lid, split);
  } else {
    // (the barrier above has passed: every wavefront is done reading the operand tiles.) Each wavefront stages
    // 32 output rows at a time through its own LDS slice (no workgroup barrier: LDS operations of one wavefront
    // execute in order) and then finishes them as 8-element chunks, a row's chunks on consecutive lanes.
    constexpr int SLD = Cfg::STAGE_LD, ETP = Cfg::ETP;
    float* stage = (float*)buf0 + wave * (32 * SLD);
    constexpr int CPR = EPI_CPR;  // 8-element chunks per staged row
#pragma unroll
    for (int j = 0; j < TQ; ++j) {
#pragma unroll
      for (int i0 = 0; i0 < TP; i0 += ETP) {
#pragma unroll
        for (int i = 0; i < ETP; ++i)
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
            f32x4 v = {acc[i0 + i][j][jj * 4 + 0], acc[i0 + i][j][jj * 4 + 1], acc[i0 + i][j][jj * 4 + 2],
                       acc[i0 + i][j][jj * 4 + 3]};
            *(f32x4*)(stage + lr * SLD + i * 32 + jj * 8 + lh * 4) = v;
          }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int k = 0; k < 32 * CPR / 64; ++k) {
          // 8 consecutive lanes take 4 chunks of each of two rows: their 128-bit reads fall on 8 different bank groups
          const int row = chunk_row(k), pc = chunk_col(k);
          f32x4 lo = *(const f32x4*)(stage + row * SLD + pc);
          f32x4 hi = *(const f32x4*)(stage + row * SLD + pc + 4);
          const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          if constexpr (has_partner32<Epi>::value) {
            static_assert(ETP == 2 && TP == 2, "partner epilogue: 64 staged columns per wavefront");
            f32x4 plo = *(const f32x4*)(stage + row * SLD + (pc ^ 32));
            f32x4 phi = *(const f32x4*)(stage + row * SLD + (pc ^ 32) + 4);
            const float vp[8] = {plo[0], plo[1], plo[2], plo[3], phi[0], phi[1], phi[2], phi[3]};
            if constexpr (kPrefetch) epi((int)p0 + pw + pc, (int)q0 + qw + j * 32 + row, v, vp, pre[j][k], split);
            else epi((int)p0 + pw + pc, (int)q0 + qw + j * 32 + row, v, vp, split);
          } else if constexpr (kPrefetch) {
            epi((int)p0 + pw + pc, (int)q0 + qw + j * 32 + row, v, pre[j][k], split);
          } else {
            epi((int)p0 + pw + i0 * 32 + pc, (int)q0 + qw + j * 32 + row, v, split);
          }
        }
        __builtin_amdgcn_wave_barrier();
      }
    }
  }
}

template <class Cfg, class PreP, class PreQ, class Epi>
static int gemm_launch_args(GemmArgs a, int groups_y, int splits, PreP prep, PreQ preq, Epi epi, hipStream_t stream);

// Host-side launch: np, nq multiples of the tile; kbytes a multiple of 128; the k-tiles are dealt to the splits evenly
// to within one tile.
template <class Cfg, class PreP, class PreQ, class Epi>
static int gemm_launch(GemmOperand P, GemmOperand Q, int np, int nq, long kbytes, int splits, PreP prep, PreQ preq,
                       Epi epi, hipStream_t stream) {
  if (np <= 0 || nq <= 0 || kbytes <= 0 || splits <= 0) return TFB_ERR_SHAPE;
  if (np % Cfg::BP || nq % Cfg::BQ || kbytes % 128 || splits > kbytes / 128) return TFB_ERR_SHAPE;
  GemmArgs a;
  a.P = P;
  a.Q = Q;
  a.np = np;
  a.nq = nq;
  a.nkt = (int)(kbytes / 128);
  a.ntp = np / Cfg::BP;
  a.q_group = nullptr;
  a.p_group_stride = 0;
  a.k_seg = nullptr;
  return gemm_launch_args<Cfg>(a, 1, splits, prep, preq, epi, stream);
}

// Launch with prepared arguments; groups_y > 1 only with a.k_seg.
template <class Cfg, class PreP, class PreQ, class Epi>
static int gemm_launch_args(GemmArgs a, int groups_y, int splits, PreP prep, PreQ preq, Epi epi, hipStream_t stream) {
  // the per-lane part of a load address is a 32-bit offset: 8 rows (K_CONTIG) or 8 k-rows (K_STRIDED) of the operand
  if (a.P.ld <= 0 || a.Q.ld <= 0 || a.P.ld > (1L << 28) || a.Q.ld > (1L << 28)) return TFB_ERR_SHAPE;
  if (((uintptr_t)a.P.base | (uintptr_t)a.Q.base | (uintptr_t)a.P.ld | (uintptr_t)a.Q.ld) & 15) return TFB_ERR_ARG;
  if ((long)splits * a.nkt >= (1L << 31)) return TFB_ERR_SHAPE;
  a.splits = splits;
  const int ntq = a.nq / Cfg::BQ;
  if ((long)a.ntp * ntq * splits >= (1L << 31)) return TFB_ERR_SHAPE;
  a.ntiles = a.ntp * ntq;
  // the stagger of the first round: only where there is a second round to overlap with and no k-split
  a.slots = tfb_resident_slots(2);
  if (!((splits == 1 || TFB_STAGGER_SPLITK) && (long)a.ntiles * splits >= 2L * a.slots)) a.slots = 0;
  // a launch of few rounds has less to gain from the offset and pays the same for it (measured on the 1536-tile GEMMs of
  // the step, three rounds: 0.730 / 0.755 ms per step with one / two units; on the 4608- and 6144-tile ones two is better)
  a.sleeps = a.slots > 0 && (long)a.ntiles * splits <= TFB_STAGGER_SHORT_ROUNDS * (long)a.slots ? 1 : stagger_sleeps<Epi>::value;
  a.per = (a.ntiles & 7) == 0 ? a.ntiles >> 3 : 0;
  a.p_fast = a.np <= a.nq || a.q_group;
  a.nfast = a.p_fast ? a.ntp : ntq;
  // traversal blocks: the largest divisor of the smaller operand's tile count whose tiles (all of k) stay under ~1.6 MB;
  // none when the whole smaller operand is that small, or when a single tile of it is already larger
  a.gblock = 0;
  if (splits == 1 && !a.q_group && !a.k_seg) {
    const long tile_bytes = (long)(a.p_fast ? Cfg::BP : Cfg::BQ) * a.nkt * 128;
    const long budget = 1600 * 1024;
    if (tile_bytes * a.nfast > budget && tile_bytes <= budget) {
      for (int g = 1; g <= a.nfast; ++g)
        if (a.nfast % g == 0 && tile_bytes * g <= budget) a.gblock = g;
    }
  }
  a.rows = (a.gblock > 0 && a.per > 0 && a.per % a.nfast == 0) ? a.per / a.nfast : 0;
  a.blk = a.gblock * a.rows;
  a.d_ntiles = fastdiv_make(a.ntiles);
  a.d_per = fastdiv_make(a.per);
  a.d_nfast = fastdiv_make(a.nfast);
  a.d_blk = fastdiv_make(a.blk);
  a.d_gblock = fastdiv_make(a.gblock);
  a.d_splits = fastdiv_make(splits);
  a.d_split8 = fastdiv_make(splits >> 3);
  dim3 grid(a.ntp * (a.nq / Cfg::BQ) * splits, groups_y, 1);
  hipLaunchKernelGGL((gemm_kernel<Cfg, PreP, PreQ, Epi>), grid, dim3(Cfg::NT), 0, stream, a, prep, preq, epi);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}
// ---- shared epilogue helpers -----------------------------------------------------------------

// out = bf16(res + bf16(D)): the residual add that follows a projection, made where the product leaves the accumulators
// (two roundings, as the separate add of the bf16 product makes them). The residual chunk is requested before the k-loop.
struct EpiStoreRes {
  bf16_t* out;
  const bf16_t* res;
  long ld;  // elements, of both
  using pre_t = u32x4;
  __device__ __forceinline__ pre_t prefetch(int p, int q) const { return tfb_load_nt((const u32x4*)(res + (long)q * ld + p), TFB_NT_RES); }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], const pre_t& r, int) const {
    float a[8], b[8];
    unpack8bf(pack8bf(v), a);
    unpack8bf(r, b);
#pragma unroll
    for (int k = 0; k < 8; ++k) a[k] += b[k];
    *(u32x4*)(out + (long)q * ld + p) = pack8bf(a);
  }
  // the same from the rounded product (the 256 x 256 kernel's epilogue protocol: pre() before the rounding, chunk() after)
  __device__ __forceinline__ float pre(float x) const { return x; }
  __device__ __forceinline__ void chunk(int p, int q, const u32x4& v, const pre_t& r) const {
    float a[8], b[8];
    unpack8bf(v, a);
    unpack8bf(r, b);
#pragma unroll
    for (int k = 0; k < 8; ++k) a[k] += b[k];
    *(u32x4*)(out + (long)q * ld + p) = pack8bf(a);
  }
};

// out (bf16 or fp32) [nq][ld] (+)= D
struct EpiStore {
  void* out;
  long ld;  // elements
  int f32;
  int accumulate;
  const float* alpha = nullptr;  // optional device scalar the product is multiplied by before the (one) rounding
  float a = 1.0f;                // *alpha, read once by prepare()
  __device__ __forceinline__ EpiStore prepare() const {
    EpiStore e = *this;
    e.a = alpha ? *alpha : 1.0f;
    return e;
  }
  // the 256 x 256 kernel's protocol, for a plain bf16 output (no accumulation)
  __device__ __forceinline__ float pre(float x) const { return x * a; }
  __device__ __forceinline__ void chunk(int p, int q, const u32x4& v) const { *(u32x4*)((bf16_t*)out + (long)q * ld + p) = v; }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], int) const {
    float r[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) r[k] = v[k] * a;
    if (f32) {
      float* o = (float*)out + (long)q * ld + p;
      if (accumulate) {
        f32x4 c0 = *(const f32x4*)o, c1 = *(const f32x4*)(o + 4);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          r[k] += c0[k];
          r[4 + k] += c1[k];
        }
      }
      *(f32x4*)o = f32x4{r[0], r[1], r[2], r[3]};
      *(f32x4*)(o + 4) = f32x4{r[4], r[5], r[6], r[7]};
    } else {
      bf16_t* o = (bf16_t*)out + (long)q * ld + p;
      if (accumulate) {
        float c[8];
        unpack8bf(*(const u32x4*)o, c);
#pragma unroll
        for (int k = 0; k < 8; ++k) r[k] += c[k];
      }
      *(u32x4*)o = pack8bf(r);
    }
  }
};

// Per-group output slabs (grouped launches): group g writes out + g * slab elements.
struct EpiStoreGrouped {
  EpiStore base;
  long slab;  // elements per group
  __device__ __forceinline__ EpiStoreGrouped for_group(int g) const {
    EpiStoreGrouped e = *this;
    e.base.out = base.f32 ? (void*)((float*)base.out + (long)g * slab) : (void*)((bf16_t*)base.out + (long)g * slab);
    return e;
  }
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], int s) const { base(p, q, v, s); }
};

// fp32 partial of one k-split: ws [splits][nq][ld]
struct EpiSplit {
  static constexpr bool kSplitF32 = true;  // (the 256 x 256 kernel hands this epilogue the raw fp32 accumulators)
  float* ws;
  long ld, slab;  // slab = nq * ld
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], int split) const {
    float* o = ws + (long)split * slab + (long)q * ld + p;
    *(f32x4*)o = f32x4{v[0], v[1], v[2], v[3]};
    *(f32x4*)(o + 4) = f32x4{v[4], v[5], v[6], v[7]};
  }
};

// out (+)= scale * (sum over splits of ws), rounded once; scale = imm / (*sa * *sb) (absent factors are 1: the fp8
// GEMMs' power-of-two descale, exact), times *alpha when given
static __global__ void splitk_reduce_kernel(const float* __restrict__ ws, void* out, long n, int splits, int f32,
                                            int accumulate, const float* sa, const float* sb, float imm,
                                            const float* alpha) {
  long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= n) return;
  f32x4 s = *(const f32x4*)(ws + i);
  for (int k = 1; k < splits; ++k) s += *(const f32x4*)(ws + (long)k * n + i);
  if (sa || sb || imm != 1.0f) {
    float d = 1.0f;
    if (sa) d *= *sa;
    if (sb) d *= *sb;
    s *= imm / d;
  }
  if (alpha) s *= *alpha;
  if (f32) {
    float* o = (float*)out + i;
    if (accumulate) s += *(const f32x4*)o;
    *(f32x4*)o = s;
  } else {
    bf16_t* o = (bf16_t*)out + i;
    if (accumulate) {
      u32x2 c = *(const u32x2*)o;
      s[0] += bflo(c.x);
      s[1] += bfhi(c.x);
      s[2] += bflo(c.y);
      s[3] += bfhi(c.y);
    }
    u32x2 r = {pack2bf(s[0], s[1]), pack2bf(s[2], s[3])};
    *(u32x2*)o = r;
  }
}

static inline int splitk_reduce(const float* ws, void* out, long n, int splits, int f32, int accumulate, hipStream_t s,
                                const float* sa = nullptr, const float* sb = nullptr, float imm = 1.0f,
                                const float* alpha = nullptr) {
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, s, ws, out, n, splits, f32,
                     accumulate, sa, sb, imm, alpha);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// How many k-splits a token-contraction GEMM with `tiles` output tiles and `nkt` k-tiles should use.
// 8 splits (one per XCD: each XCD then fetches only its own k-range of both operands; measured 8-20 % faster than the
// best other count at equal occupancy) when that fills at least 80 % of whole rounds of the resident workgroup slots
// (2 per CU: 512 on the 256 CUs of an MI355X) or fits one round. Otherwise a cost model in units of one k-tile of one workgroup:
// rounds x (k-tiles per split + 10 for prologue and epilogue) + the fp32 partials' round trip through memory (8 bytes
// per output element and split at ~4 TB/s, one k-tile ~0.7 us).
static inline int choose_splits(long tiles, int nkt, long out_elems, long ws_bytes) {
  const long slots = tfb_resident_slots(2);
  if (tiles >= 2 * slots || nkt < 32) return 1;
  if (nkt >= 8 * 16 && 8 * out_elems * 4 <= ws_bytes) {
    const long wgs = tiles * 8, rounds = (wgs + slots - 1) / slots;
    if (rounds == 1 || (double)wgs >= 0.8 * (double)(rounds * slots)) return 8;
  }
  int best = 1;
  double best_cost = 1e30;
  for (int sp = 1; sp <= 32; ++sp) {
    if (sp > 1 && (nkt / sp < 16 || (long)sp * out_elems * 4 > ws_bytes)) break;
    const long rounds = (tiles * sp + slots - 1) / slots;
    const double cost = (double)rounds * ((double)nkt / sp + 10.0) + (sp > 1 ? sp * (double)out_elems * 2e-6 / 0.7 : 0.0);
    if (cost < best_cost) {
      best_cost = cost;
      best = sp;
    }
  }
  return best;
}

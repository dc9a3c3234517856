// MFMA GEMM core for gfx950: D[p][q] = sum_k P[p][k] * Q[q][k], fp32 accumulation.
//
// One workgroup of WP x WQ wavefronts owns a BP x BQ output tile. Both operand tiles are
// staged in LDS as [row][128 bytes of k + 16 bytes of pad], the eight 16-byte chunks of a row
// XOR-swizzled by (row / 8) mod 8. With the measured bank behaviour of gfx950's LDS (32 banks
// of 4 bytes; 128-bit accesses resolved per 8 consecutive lanes, 64-bit accesses per 16) the
// 144-byte stride makes the 128-bit fragment reads (8 consecutive rows, one chunk) conflict-free,
// and the swizzle does the same for the 64-bit transposing writes (8 rows that are 8 apart times
// two adjacent k-groups per 16 lanes) while global loads stay 128-byte coalesced. Staging is
// double-buffered (NBUF 2: the
// next k-tile's global loads are in flight while the MFMAs of the current one run, one barrier
// per k-tile) or single-buffered (NBUF 1: half the LDS, two barriers, more workgroups per CU).
// The P tile feeds the MFMA A operand (rows), the Q tile the B operand (columns), so a lane
// ends up holding D[p .. p+3][q] for four consecutive p: callers put the dimension that is
// contiguous in the output on the P side.
//
// Epilogues: "staged" (default) - each wavefront passes its accumulators through its own LDS
// slice, 32 output rows at a time, and every lane then owns 8 consecutive p of one q, so global
// reads/writes of the epilogue are 128-bit and coalesced along the output rows; or "tile" (kTileEpilogue) - the functor gets the raw
// accumulator registers (used when the epilogue reduces along p in registers).
//
// Element types: bf16 (v_mfma_f32_32x32x16_bf16, 64 k per tile) or OCP fp8
// (v_mfma_scale_f32_32x32x64_f8f6f4 with unit scales, 128 k per tile, e4m3/e5m2 per side).
// Operand layouts: K_CONTIG = [rows][K] (k contiguous); K_STRIDED = [K][rows] (bf16 only,
// transposed on the way into LDS through 4k x 8row register micro-blocks), which is what
// the weight-gradient GEMMs (contraction over tokens) read.
#pragma once
#include <type_traits>

#include "common.hpp"

#define TFB_K_CONTIG 0
#define TFB_K_STRIDED 1
#define TFB_LDS_ROW 144  // 128 bytes of k + 16 bytes of pad

struct GemmOperand {
  const uint8_t* base;
  long ld;  // bytes between consecutive rows (K_CONTIG) or consecutive k (K_STRIDED)
};

struct GemmArgs {
  GemmOperand P, Q;
  int np, nq;   // output extent (multiples of BP / BQ)
  int nkt;      // k-tiles (128 bytes of k each) per split
  int ntp;      // tiles along p
  // Grouped (ragged) launches, both optional:
  const int* q_group;    // group id of each q tile (-1: the tile is beyond the ragged extent, the workgroup exits);
  long p_group_stride;   //   the P operand of group g starts p_group_stride bytes * g further (per-expert weights)
  const int* k_seg;      // [groups + 1] k offsets in elements: group = blockIdx.y contracts over k_seg[g] .. k_seg[g+1]
};

struct LoadIdentity {
  __device__ __forceinline__ u32x4 operator()(u32x4 v) const { return v; }
};

// Byte offset of 16-byte chunk `chunk` of row `row` in a staged tile.
__device__ __forceinline__ int lds_off(int row, int chunk) {
  return row * TFB_LDS_ROW + (((chunk ^ (row >> 3)) & 7) << 4);
}

template <int BP_, int BQ_, int WP_, int WQ_, int ES_, int LAYP_, int LAYQ_, int FMTP_ = 0, int FMTQ_ = 0, int NBUF_ = 2>
struct GemmCfg {
  static constexpr int BP = BP_, BQ = BQ_, WP = WP_, WQ = WQ_, ES = ES_, NBUF = NBUF_;
  static constexpr int LAYP = LAYP_, LAYQ = LAYQ_, FMTP = FMTP_, FMTQ = FMTQ_;
  static constexpr int NT = WP * WQ * 64;
  static constexpr int TP = BP / WP / 32, TQ = BQ / WQ / 32;
  static constexpr int BK = 128 / ES;  // elements of k per tile
  static constexpr int TILE_BYTES = (BP + BQ) * TFB_LDS_ROW;
  static constexpr int STAGE_LD = TP * 32 + 4;  // floats per staged row: a wavefront's 32 x (TP*32) slice
  static constexpr int STAGE_BYTES = WP * WQ * 32 * STAGE_LD * 4;
  static constexpr int LDS_BYTES = NBUF * TILE_BYTES > STAGE_BYTES ? NBUF * TILE_BYTES : STAGE_BYTES;
  static_assert(ES == 1 || ES == 2, "fp8 or bf16");
  static_assert(NBUF == 1 || NBUF == 2, "single or double buffering");
  static_assert(ES == 2 || (LAYP == TFB_K_CONTIG && LAYQ == TFB_K_CONTIG), "fp8 operands are k-contiguous");
  static_assert((BP * 8) % NT == 0 && (BQ * 8) % NT == 0, "tile rows vs threads");
};

// ---- global -> register -> LDS staging of one operand tile ---------------------------------
template <int ROWS, int NT, int LAY>
struct TileLoader;

template <int ROWS, int NT>
struct TileLoader<ROWS, NT, TFB_K_CONTIG> {
  static constexpr int N = ROWS * 8 / NT;
  u32x4 g[N];
  __device__ __forceinline__ void load(const GemmOperand& o, long row0, long kbyte0, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      int c = tid + i * NT;
      int row = c >> 3, cc = c & 7;
      g[i] = *(const u32x4*)(o.base + (row0 + row) * o.ld + kbyte0 + cc * 16);
    }
  }
  template <class Pre>
  __device__ __forceinline__ void store(uint8_t* lds, int tid, const Pre& pre) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      int c = tid + i * NT;
      int row = c >> 3, cc = c & 7;
      *(u32x4*)(lds + lds_off(row, cc)) = pre(g[i]);
    }
  }
};

template <int ROWS, int NT>
struct TileLoader<ROWS, NT, TFB_K_STRIDED> {
  // bf16 only: 64 k x ROWS tile, micro-blocks of 4 k x 8 rows
  static constexpr int N = ROWS * 2 / NT;
  static_assert((ROWS * 2) % NT == 0 && N >= 1 && ROWS % 64 == 0, "K_STRIDED tile rows vs threads");
  u32x4 g[N][4];
  __device__ __forceinline__ void load(const GemmOperand& o, long row0, long kbyte0, int tid) {
    const long k0 = kbyte0 >> 1;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      int mb = tid + i * NT;
      // 16 consecutive lanes = 8 row groups x 2 adjacent k groups: 128-byte coalesced loads, conflict-free writes
      int hi = mb >> 4;
      int rg = (mb & 7) + 8 * (hi % (ROWS / 64)), kg = ((mb >> 3) & 1) + 2 * (hi / (ROWS / 64));
#pragma unroll
      for (int j = 0; j < 4; ++j)
        g[i][j] = *(const u32x4*)(o.base + (k0 + 4 * kg + j) * o.ld + (row0 + 8 * rg) * 2);
    }
  }
  template <class Pre>
  __device__ __forceinline__ void store(uint8_t* lds, int tid, const Pre& pre) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      int mb = tid + i * NT;
      int hi = mb >> 4;
      int rg = (mb & 7) + 8 * (hi % (ROWS / 64)), kg = ((mb >> 3) & 1) + 2 * (hi / (ROWS / 64));
      u32x4 v0 = pre(g[i][0]), v1 = pre(g[i][1]), v2 = pre(g[i][2]), v3 = pre(g[i][3]);
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        // rows 2w (low halves) and 2w+1 (high halves) of the micro-block: 4 consecutive k each
        u32x2 lo, hi;
        lo.x = __builtin_amdgcn_perm(v1[w], v0[w], 0x05040100u);
        lo.y = __builtin_amdgcn_perm(v3[w], v2[w], 0x05040100u);
        hi.x = __builtin_amdgcn_perm(v1[w], v0[w], 0x07060302u);
        hi.y = __builtin_amdgcn_perm(v3[w], v2[w], 0x07060302u);
        const int r0 = 8 * rg + 2 * w;
        *(u32x2*)(lds + lds_off(r0, kg >> 1) + (kg & 1) * 8) = lo;
        *(u32x2*)(lds + lds_off(r0 + 1, kg >> 1) + (kg & 1) * 8) = hi;
      }
    }
  }
};

// ---- MFMA fragments ------------------------------------------------------------------------
template <int ES>
struct Frag;
template <>
struct Frag<2> {
  bf16x8 v;
  static constexpr int KSTEPS = 4;  // 4 x 16 bf16 per 128-byte tile row
  __device__ __forceinline__ void read(const uint8_t* lds, int row, int s, int h) {
    v = *(const bf16x8*)(lds + lds_off(row, 2 * s + h));
  }
};
template <>
struct Frag<1> {
  i32x8 v;
  static constexpr int KSTEPS = 2;  // 2 x 64 fp8 per 128-byte tile row
  __device__ __forceinline__ void read(const uint8_t* lds, int row, int s, int h) {
    i32x4 a = *(const i32x4*)(lds + lds_off(row, 4 * s + 2 * h));
    i32x4 b = *(const i32x4*)(lds + lds_off(row, 4 * s + 2 * h + 1));
    v = i32x8{a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
  }
};

template <int ES, int FMTP, int FMTQ>
__device__ __forceinline__ f32x16 mfma32(const Frag<ES>& a, const Frag<ES>& b, f32x16 c) {
  if constexpr (ES == 2) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c, 0, 0, 0);
  } else {
    // formats: 0 = e4m3, 1 = e5m2; E8M0 scale byte 127 = 2^0
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a.v, b.v, c, FMTP, FMTQ, 0, 127, 0, 127);
  }
}

// The workgroup's (tile_p, tile_q): consecutive workgroup ids are dealt round-robin to the
// 8 XCDs (each with its own L2), so ids are re-dealt so that one XCD gets a contiguous run
// of tiles; p runs fastest, so a run shares its Q rows through that XCD's L2.
__device__ __forceinline__ int xcd_remap(int pid, int nb) {
  return (nb & 7) == 0 ? (pid & 7) * (nb >> 3) + (pid >> 3) : pid;
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

template <class T, class = void>
struct has_tile_epilogue : std::false_type {};
template <class T>
struct has_tile_epilogue<T, std::void_t<decltype(T::kTileEpilogue)>> : std::true_type {};

// Epi: either  __device__ void operator()(int p, int q, const float (&v)[8], int split)  with v = D[p..p+7][q], p % 8 == 0,
// or (with a static member kTileEpilogue)  __device__ void tile(acc, pw, qw, lr, lh, tile_id, split).
template <class Cfg, class PreP, class PreQ, class Epi>
__global__ __launch_bounds__(Cfg::NT) void gemm_kernel(GemmArgs a, PreP prep, PreQ preq, Epi epi_in) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int BP = Cfg::BP, BQ = Cfg::BQ, NT = Cfg::NT, TP = Cfg::TP, TQ = Cfg::TQ, ES = Cfg::ES;
  constexpr int BUF = Cfg::TILE_BYTES;
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int wp = wave % Cfg::WP, wq = wave / Cfg::WP;
  const int lr = lane & 31, lh = lane >> 5;

  const int lid = xcd_remap(blockIdx.x, gridDim.x);
  const int tile_p = lid % a.ntp, tile_q = lid / a.ntp;
  const long p0 = (long)tile_p * BP, q0 = (long)tile_q * BQ;
  long kt0 = (long)blockIdx.z * a.nkt;
  int group = 0;
  if (a.q_group) {
    group = a.q_group[tile_q];
    if (group < 0) return;  // the whole workgroup leaves before any barrier
    a.P.base += (long)group * a.p_group_stride;
  }
  if (a.k_seg) {
    group = blockIdx.y;
    const long k0 = a.k_seg[group], k1 = a.k_seg[group + 1];
    kt0 = k0 * ES / 128;
    a.nkt = (int)((k1 - k0) * ES / 128);  // may be 0: the accumulators stay zero and are still written
  }
  const Epi epi = epi_for_group(epi_in, group);

  TileLoader<BP, NT, Cfg::LAYP> lp;
  TileLoader<BQ, NT, Cfg::LAYQ> lq;

  f32x16 acc[TP][TQ];
#pragma unroll
  for (int i = 0; i < TP; ++i)
#pragma unroll
    for (int j = 0; j < TQ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  if (a.nkt > 0) {
    lp.load(a.P, p0, kt0 * 128, tid);
    lq.load(a.Q, q0, kt0 * 128, tid);
    lp.store(smem, tid, prep);
    lq.store(smem + BP * TFB_LDS_ROW, tid, preq);
  }
  __syncthreads();

  for (int t = 0; t < a.nkt; ++t) {
    const uint8_t* sp = smem + (Cfg::NBUF == 2 ? (t & 1) * BUF : 0);
    const uint8_t* sq = sp + BP * TFB_LDS_ROW;
    const bool more = (t + 1 < a.nkt);
    if (more) {
      lp.load(a.P, p0, (kt0 + t + 1) * 128, tid);
      lq.load(a.Q, q0, (kt0 + t + 1) * 128, tid);
    }
    {
      // fragments of k-step s+1 are requested before the MFMAs of step s are issued
      constexpr int KS = Frag<ES>::KSTEPS;
      Frag<ES> fa[2][TP], fb[2][TQ];
#pragma unroll
      for (int i = 0; i < TP; ++i) fa[0][i].read(sp, wp * (TP * 32) + i * 32 + lr, 0, lh);
#pragma unroll
      for (int j = 0; j < TQ; ++j) fb[0][j].read(sq, wq * (TQ * 32) + j * 32 + lr, 0, lh);
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        if (s + 1 < KS) {
#pragma unroll
          for (int i = 0; i < TP; ++i) fa[(s + 1) & 1][i].read(sp, wp * (TP * 32) + i * 32 + lr, s + 1, lh);
#pragma unroll
          for (int j = 0; j < TQ; ++j) fb[(s + 1) & 1][j].read(sq, wq * (TQ * 32) + j * 32 + lr, s + 1, lh);
        }
#pragma unroll
        for (int i = 0; i < TP; ++i)
#pragma unroll
          for (int j = 0; j < TQ; ++j)
            acc[i][j] = mfma32<ES, Cfg::FMTP, Cfg::FMTQ>(fa[s & 1][i], fb[s & 1][j], acc[i][j]);
      }
    }
    if (Cfg::NBUF == 1) __syncthreads();
    if (more) {
      uint8_t* np_ = smem + (Cfg::NBUF == 2 ? ((t + 1) & 1) * BUF : 0);
      lp.store(np_, tid, prep);
      lq.store(np_ + BP * TFB_LDS_ROW, tid, preq);
    }
    __syncthreads();
  }

  const int pw = wp * (TP * 32), qw = wq * (TQ * 32);  // wavefront's origin inside the tile
  if constexpr (has_tile_epilogue<Epi>::value) {
    // whole-accumulator epilogue: acc[i][j][4*jj + e] = D[pw + 32 i + 8 jj + 4 lh + e][qw + 32 j + lr]
    epi.tile(acc, (int)p0 + pw, (int)q0 + qw, lr, lh, lid, (int)blockIdx.z);
  } else {
    // (the loop's last barrier has passed: every wavefront is done reading the operand tiles.) Each wavefront stages
    // 32 output rows at a time through its own LDS slice (no workgroup barrier: LDS operations of one wavefront
    // execute in order) and then finishes them as 8-element chunks, a row's chunks on consecutive lanes.
    constexpr int SLD = Cfg::STAGE_LD;
    float* stage = (float*)smem + wave * (32 * SLD);
    constexpr int CPR = TP * 4;  // 8-element chunks per staged row
#pragma unroll
    for (int j = 0; j < TQ; ++j) {
#pragma unroll
      for (int i = 0; i < TP; ++i)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          f32x4 v = {acc[i][j][jj * 4 + 0], acc[i][j][jj * 4 + 1], acc[i][j][jj * 4 + 2], acc[i][j][jj * 4 + 3]};
          *(f32x4*)(stage + lr * SLD + i * 32 + jj * 8 + lh * 4) = v;
        }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int k = 0; k < 32 * CPR / 64; ++k) {
        // 8 consecutive lanes take 4 chunks of each of two rows: their 128-bit reads fall on 8 different bank groups
        const int rest = (lane >> 3) + k * 8;
        const int row = 2 * (rest / (CPR / 4)) + ((lane >> 2) & 1);
        const int pc = (4 * (rest % (CPR / 4)) + (lane & 3)) * 8;
        f32x4 lo = *(const f32x4*)(stage + row * SLD + pc);
        f32x4 hi = *(const f32x4*)(stage + row * SLD + pc + 4);
        const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        epi((int)p0 + pw + pc, (int)q0 + qw + j * 32 + row, v, (int)blockIdx.z);
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
}

template <class Cfg, class PreP, class PreQ, class Epi>
static int gemm_launch_args(GemmArgs a, int groups_y, int splits, PreP prep, PreQ preq, Epi epi, hipStream_t stream);

// Host-side launch: np, nq multiples of the tile; kbytes a multiple of 128 * splits.
template <class Cfg, class PreP, class PreQ, class Epi>
static int gemm_launch(GemmOperand P, GemmOperand Q, int np, int nq, long kbytes, int splits, PreP prep, PreQ preq,
                       Epi epi, hipStream_t stream) {
  if (np <= 0 || nq <= 0 || kbytes <= 0 || splits <= 0) return TFB_ERR_SHAPE;
  if (np % Cfg::BP || nq % Cfg::BQ || kbytes % (128L * splits)) return TFB_ERR_SHAPE;
  GemmArgs a;
  a.P = P;
  a.Q = Q;
  a.np = np;
  a.nq = nq;
  a.nkt = (int)(kbytes / 128 / splits);
  a.ntp = np / Cfg::BP;
  a.q_group = nullptr;
  a.p_group_stride = 0;
  a.k_seg = nullptr;
  return gemm_launch_args<Cfg>(a, 1, splits, prep, preq, epi, stream);
}

// Launch with prepared arguments; groups_y > 1 only with a.k_seg.
template <class Cfg, class PreP, class PreQ, class Epi>
static int gemm_launch_args(GemmArgs a, int groups_y, int splits, PreP prep, PreQ preq, Epi epi, hipStream_t stream) {
  auto kern = gemm_kernel<Cfg, PreP, PreQ, Epi>;
  static bool attr_set = false;  // per template instantiation
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES) != hipSuccess)
      return TFB_ERR_LAUNCH;
    attr_set = true;
  }
  dim3 grid(a.ntp * (a.nq / Cfg::BQ), groups_y, splits);
  hipLaunchKernelGGL(kern, grid, dim3(Cfg::NT), Cfg::LDS_BYTES, stream, a, prep, preq, epi);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// ---- shared epilogue helpers -----------------------------------------------------------------
__device__ __forceinline__ u32x4 pack8bf(const float (&v)[8]) {
  u32x4 o = {pack2bf(v[0], v[1]), pack2bf(v[2], v[3]), pack2bf(v[4], v[5]), pack2bf(v[6], v[7])};
  return o;
}
__device__ __forceinline__ void unpack8bf(u32x4 u, float (&v)[8]) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    v[2 * k] = bflo(u[k]);
    v[2 * k + 1] = bfhi(u[k]);
  }
}

// out (bf16 or fp32) [nq][ld] (+)= D
struct EpiStore {
  void* out;
  long ld;  // elements
  int f32;
  int accumulate;
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], int) const {
    float r[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) r[k] = v[k];
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
  float* ws;
  long ld, slab;  // slab = nq * ld
  __device__ __forceinline__ void operator()(int p, int q, const float (&v)[8], int split) const {
    float* o = ws + (long)split * slab + (long)q * ld + p;
    *(f32x4*)o = f32x4{v[0], v[1], v[2], v[3]};
    *(f32x4*)(o + 4) = f32x4{v[4], v[5], v[6], v[7]};
  }
};

// out (+)= sum over splits of ws, rounded once
static __global__ void splitk_reduce_kernel(const float* __restrict__ ws, void* out, long n, int splits, int f32,
                                            int accumulate) {
  long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= n) return;
  f32x4 s = *(const f32x4*)(ws + i);
  for (int k = 1; k < splits; ++k) s += *(const f32x4*)(ws + (long)k * n + i);
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

static inline int splitk_reduce(const float* ws, void* out, long n, int splits, int f32, int accumulate, hipStream_t s) {
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, s, ws, out, n, splits, f32,
                     accumulate);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// How many k-splits a token-contraction GEMM with `tiles` output tiles and `nkt` k-tiles should use.
static inline int choose_splits(long tiles, int nkt, long out_elems, long ws_bytes) {
  if (tiles >= 512 || nkt < 32) return 1;
  int splits = (int)((768 + tiles - 1) / tiles);
  while (splits > 1 && (nkt % splits != 0 || nkt / splits < 8)) --splits;
  if ((long)splits * out_elems * 4 > ws_bytes) splits = 1;
  return splits;
}

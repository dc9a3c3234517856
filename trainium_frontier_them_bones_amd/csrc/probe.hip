// Hardware probes behind the design of the GEMM and attention data paths (diagnostics, not on the training path):
//   tfb_probe_load_issue  what one 1 KB vector load costs the wavefront that issues it, by destination (registers or LDS)
//                         and by the number of wavefronts of a CU that issue at once, from an L2-resident region;
//   tfb_probe_lds_mix     how much the fragment reads of four wavefronts slow down while four others stream operands into
//                         the same CU by global -> LDS DMA, by global -> VGPR -> ds_write_b128, or into registers only;
//   tfb_probe_gemm_phases where a workgroup of the bf16 GEMM (the library's own kernel and launch, with an epilogue that
//                         also reports cycle counts) spends its time: start-up, first k-tile, k-loop, epilogue.
// Each wavefront reports its own cycle count (s_memtime); the host turns them into cycles per instruction and bytes per
// clock per CU. One workgroup per CU in the first two.
#include "gemm_core.hpp"

namespace {

typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void glb_void_t;

constexpr unsigned kPitch = 1536;  // the row pitch of a K = 768 bf16 operand: one instruction = 8 rows x 128 bytes

// TO_LDS: global_load_lds_dwordx4 (the operand DMA of the GEMM and attention kernels); else global_load_dwordx4.
template <bool TO_LDS, int NT>
__global__ __launch_bounds__(NT, 1) void load_issue_kernel(const uint8_t* __restrict__ src, unsigned region,
                                                          unsigned long long* __restrict__ cycles, int iters) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[NT / 64 * 8 * 1024];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const unsigned lane_off = (unsigned)(lane >> 3) * kPitch + (lane & 7) * 16;
  const unsigned rows = region / kPitch;
  const unsigned row0 = (blockIdx.x * (NT / 64) + wave) * 64;
  uint8_t* my = lds + wave * 8 * 1024;
  u32x4 acc = {0, 0, 0, 0};
  u32x4 prev[8] = {};
  const unsigned long long c0 = __builtin_readcyclecounter();
  for (int it = 0; it < iters; ++it) {
    const unsigned r = (row0 + (unsigned)it * 64 * 977) % (rows - 64);
    const uint8_t* g = src + r * kPitch + (unsigned)(it % 12) * 128 + lane_off;
    if (TO_LDS) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        __builtin_amdgcn_global_load_lds((glb_void_t*)(g + j * 8 * kPitch), (lds_void_t*)(my + j * 1024), 16, 0, 0);
    } else {
      // the values of one iteration are consumed in the next, so the loop waits for data one iteration old
      u32x4 v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = *(const u32x4*)(g + j * 8 * kPitch);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        acc ^= prev[j];
        prev[j] = v[j];
      }
    }
  }
  const unsigned long long c1 = __builtin_readcyclecounter();
  if (lane == 0) cycles[blockIdx.x * 16 + wave] = c1 - c0;
  __syncthreads();
  if (TO_LDS) acc = *(const u32x4*)(my + lane * 16);
  else
    for (int j = 0; j < 8; ++j) acc ^= prev[j];
  if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) cycles[blockIdx.x * 16 + 15] = acc.z;  // keeps the loads alive
}

// MODE 0: readers only. 1: + DMA. 2: + global -> VGPR -> ds_write_b128. 3: + global -> VGPR only.
template <int MODE>
__global__ __launch_bounds__(512, 1) void lds_mix_kernel(const uint8_t* __restrict__ src, unsigned region,
                                                        unsigned long long* __restrict__ cycles, int riters, int liters) {
  __shared__ __attribute__((aligned(1024))) uint8_t rbuf[4 * 20 * 1024];
  __shared__ __attribute__((aligned(1024))) uint8_t wbuf[4 * 8 * 1024];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  for (int i = threadIdx.x; i < (int)sizeof(rbuf) / 4; i += 512) ((uint32_t*)rbuf)[i] = i;
  __syncthreads();
  u32x4 acc = {0, 0, 0, 0};
  if (wave < 4) {
    // 16 conflict-free 128-bit reads in flight per wavefront; the window moves with the iteration so that nothing is
    // loop-invariant
    const uint8_t* base = rbuf + wave * (20 * 1024) + lane * 16;
    const unsigned long long c0 = __builtin_readcyclecounter();
    for (int it = 0; it < riters; ++it) {
      const uint8_t* b = base + (it & 3) * 1024;
      u32x4 v[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) v[j] = *(const u32x4*)(b + j * 1024);
#pragma unroll
      for (int j = 0; j < 16; ++j) acc ^= v[j];
    }
    const unsigned long long c1 = __builtin_readcyclecounter();
    if (lane == 0) cycles[blockIdx.x * 16 + wave] = c1 - c0;
  } else if (MODE != 0) {
    const int lw = wave - 4;
    const unsigned lane_off = (unsigned)(lane >> 3) * kPitch + (lane & 7) * 16;
    const unsigned rows = region / kPitch;
    const unsigned row0 = (blockIdx.x * 4 + lw) * 64;
    uint8_t* my = wbuf + lw * 8 * 1024;
    const unsigned long long c0 = __builtin_readcyclecounter();
    for (int it = 0; it < liters; ++it) {
      const unsigned r = (row0 + (unsigned)it * 64 * 977) % (rows - 64);
      const uint8_t* g = src + r * kPitch + (unsigned)(it % 12) * 128 + lane_off;
      if (MODE == 1) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          __builtin_amdgcn_global_load_lds((glb_void_t*)(g + j * 8 * kPitch), (lds_void_t*)(my + j * 1024), 16, 0, 0);
      } else {
        u32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = *(const u32x4*)(g + j * 8 * kPitch);
        if (MODE == 2) {
#pragma unroll
          for (int j = 0; j < 8; ++j) *(u32x4*)(my + j * 1024 + lane * 16) = v[j];
          acc.x ^= *(const uint32_t*)(my + ((it & 7) * 1024) + lane * 4);  // the stores are read: none of them is dead
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) acc ^= v[j];
        }
      }
    }
    const unsigned long long c1 = __builtin_readcyclecounter();
    if (lane == 0) cycles[blockIdx.x * 16 + wave] = c1 - c0;
  }
  __syncthreads();
  if (MODE == 1 && wave >= 4) acc = *(const u32x4*)(wbuf + (wave - 4) * 8 * 1024 + lane * 16);
  if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) cycles[blockIdx.x * 16 + 15] = acc.z;
}

// EpiStore with the phase report switched on (see has_phase_probe)
struct EpiStoreProbe : EpiStore {
  unsigned long long* phase_cycles;
};

}  // namespace

// cycles: uint64 [CUs][16], entry [cu][w] = cycles wavefront w spent issuing iters x 8 loads of 1 KB each (8 rows x 128 bytes
// at a pitch of 1536 bytes) from the first `region` bytes of src. to_lds 1: global -> LDS DMA, 0: into registers.
// waves: 1, 4 or 8 per CU. region >= 128 KB, < 4 GB. The caller zero-fills cycles and reads it after the stream is done.
extern "C" int tfb_probe_load_issue(const void* src, long region, int to_lds, int waves, int iters, void* cycles, void* stream) {
  if (!src || !cycles) return TFB_ERR_ARG;
  if (region < (128 << 10) || region >= (1L << 32) || iters <= 0 || (waves != 1 && waves != 4 && waves != 8)) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const int cus = tfb_resident_slots(1);
  const uint8_t* p = (const uint8_t*)src;
  unsigned long long* c = (unsigned long long*)cycles;
  const unsigned rg = (unsigned)region;
#define TFB_PROBE_LAUNCH(LDS_, NT_) hipLaunchKernelGGL((load_issue_kernel<LDS_, NT_>), dim3(cus), dim3(NT_), 0, s, p, rg, c, iters)
  if (to_lds) {
    if (waves == 1) TFB_PROBE_LAUNCH(true, 64);
    else if (waves == 4) TFB_PROBE_LAUNCH(true, 256);
    else TFB_PROBE_LAUNCH(true, 512);
  } else {
    if (waves == 1) TFB_PROBE_LAUNCH(false, 64);
    else if (waves == 4) TFB_PROBE_LAUNCH(false, 256);
    else TFB_PROBE_LAUNCH(false, 512);
  }
#undef TFB_PROBE_LAUNCH
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// cycles: uint64 [CUs][16]: entries 0..3 the four reading wavefronts (riters x 16 ds_read_b128 of 1 KB each), 4..7 the four
// streaming ones (liters x 8 loads of 1 KB; zero in mode 0). mode 0: readers alone; 1: + global -> LDS DMA; 2: + global ->
// VGPR -> ds_write_b128; 3: + global -> VGPR only. Give the streaming wavefronts enough iterations to outlast the readers.
extern "C" int tfb_probe_lds_mix(const void* src, long region, int mode, int riters, int liters, void* cycles, void* stream) {
  if (!src || !cycles) return TFB_ERR_ARG;
  if (region < (128 << 10) || region >= (1L << 32) || riters <= 0 || liters < 0 || mode < 0 || mode > 3) return TFB_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const int cus = tfb_resident_slots(1);
  const uint8_t* p = (const uint8_t*)src;
  unsigned long long* c = (unsigned long long*)cycles;
  const unsigned rg = (unsigned)region;
  if (mode == 0) hipLaunchKernelGGL(lds_mix_kernel<0>, dim3(cus), dim3(512), 0, s, p, rg, c, riters, liters);
  else if (mode == 1) hipLaunchKernelGGL(lds_mix_kernel<1>, dim3(cus), dim3(512), 0, s, p, rg, c, riters, liters);
  else if (mode == 2) hipLaunchKernelGGL(lds_mix_kernel<2>, dim3(cus), dim3(512), 0, s, p, rg, c, riters, liters);
  else hipLaunchKernelGGL(lds_mix_kernel<3>, dim3(cus), dim3(512), 0, s, p, rg, c, riters, liters);
  TFB_LAUNCH_CHECK();
  return TFB_OK;
}

// c [M][N] bf16 = a [M][K] b[N][K]^T (bf16, M, N multiples of 128, K of 64) through the library's bf16 GEMM kernel, tile
// traversal and launch path, with the phases of every workgroup written to cycles: uint64 [(M / 128) (N / 128)][4] =
// cycles from kernel entry to the first operand load's issue, to the first k-tile's arrival, in the k-loop, in the epilogue.
extern "C" int tfb_probe_gemm_phases(const void* a, const void* b, void* c, long M, long N, long K, void* cycles, void* stream) {
  if (!a || !b || !c || !cycles) return TFB_ERR_ARG;
  if (M <= 0 || N <= 0 || K <= 0 || M % 128 || N % 128 || K % 64 || M > (1L << 30) || N > (1L << 30)) return TFB_ERR_SHAPE;
  using Cfg = GemmCfg<128, 128, 2, 2, 2, TFB_K_CONTIG, TFB_K_CONTIG>;
  EpiStoreProbe e;
  e.out = c;
  e.ld = N;
  e.f32 = 0;
  e.accumulate = 0;
  e.phase_cycles = (unsigned long long*)cycles;
  return gemm_launch<Cfg>(GemmOperand{(const uint8_t*)b, K * 2}, GemmOperand{(const uint8_t*)a, K * 2}, (int)N, (int)M, K * 2, 1,
                          LoadIdentity{}, LoadIdentity{}, e, (hipStream_t)stream);
}

// Measurement only, not part of the operator: what the matrix pipes of this GPU
// sustain on the scaled FP4 MFMA alone, with no memory traffic at all.  Built as
// its own small library (libwave_probe.so) so that the operator's C ABI stays what
// include/wave_mxfp4.h declares; `bench.py --workload mfma_ceiling` is its caller.
//
// Every wave loads the operand fragments of its wave tile once (2 K steps x (4 + 4)
// fragments of a 128 x 128 tile, or 4 K steps x (2 + 4) of a 64 x 128 tile) and then
// issues, `iters` times, the 32 v_mfma_scale_f32_32x32x64_f8f6f4 they feed, in the
// order the GEMM kernels use (K step outermost, every accumulator once per step).  With random operand bytes the
// chip draws more power per instruction than with zeros and clocks lower: the two
// rates bracket what any GEMM kernel on that data can reach.  The reference prices
// its kernels against the instruction's issue cost the same way
// (benchmark/wave_att_analyzer.py:35-36: 32 cycles for 32x32x64).
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

// NT = 256: 4 waves per workgroup, each a 128 x 128 wave tile (4 x 4 MFMA tiles, 16 accumulators).
// NT = 512: 8 waves, each 64 x 128 (2 x 4 MFMA tiles), the shape of the 8-wave GEMM kernels: two waves per SIMD
// have 256 registers each.
// GAP: s_sleep 1 instructions (64 cycles each) after the 32 MFMAs of an iteration: with GAP = 8 a wave's matrix
// pipe idles a third of the time, about the duty cycle of the GEMM kernels (their rate on all-zero operands is
// 72-74 % of this loop's).  What that loop sustains on random operands is what the GEMM's stalls alone would
// leave of the MFMA-alone rate; what the GEMM loses beyond that is the energy of its data movement.
template <int NT, int GAP>
__global__ void __launch_bounds__(NT) mfma_probe_kernel(const v4i *__restrict__ src, float *__restrict__ out,
                                                        unsigned long long *__restrict__ ticks, int iters, int scale) {
  constexpr int MI = NT == 256 ? 4 : 2, MJ = 4, KT = NT == 256 ? 2 : 4;  // 32 MFMAs per wave and iteration
  v16f acc[MI * MJ];
#pragma unroll
  for (int i = 0; i < MI * MJ; ++i)
#pragma unroll
    for (int g = 0; g < 16; ++g) acc[i][g] = 0.f;
  v4i fa[KT][MI], fb[KT][MJ];
#pragma unroll
  for (int t = 0; t < KT; ++t) {
#pragma unroll
    for (int i = 0; i < MI; ++i) fa[t][i] = src[(((size_t)blockIdx.x * 4 + t) * 8 + i) * NT + threadIdx.x];
#pragma unroll
    for (int j = 0; j < MJ; ++j) fb[t][j] = src[(((size_t)blockIdx.x * 4 + t) * 8 + 4 + j) * NT + threadIdx.x];
  }
  const unsigned long long t0 = __builtin_amdgcn_s_memtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int t = 0; t < KT; ++t)
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < MJ; ++j) {
          const v8i a = {fa[t][i].x, fa[t][i].y, fa[t][i].z, fa[t][i].w, 0, 0, 0, 0};
          const v8i b = {fb[t][j].x, fb[t][j].y, fb[t][j].z, fb[t][j].w, 0, 0, 0, 0};
          acc[i * MJ + j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[i * MJ + j], 4, 4, 0, scale, 0, scale);
        }
#pragma unroll
    for (int g = 0; g < GAP; ++g) __builtin_amdgcn_s_sleep(1);
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memtime();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < MI * MJ; ++i)
#pragma unroll
    for (int g = 0; g < 16; ++g) s += acc[i][g];
  out[(size_t)blockIdx.x * NT + threadIdx.x] = s;
  if (threadIdx.x == 0) ticks[blockIdx.x] = t1 - t0;
}

// Second probe: what the L2 (and, with a footprint beyond it, the Infinity Cache) delivers to a CU's LDS through the
// GEMM kernels' operand DMA, with nothing else going on.  A region is a panel of 256 rows x 4096 bytes (1 MB, the
// A or B panel of a 256-row tile at K = 8192); a workgroup of 8 waves walks its panel's 32 K tiles of 128 bytes
// per row `iters` times, one wave instruction = 8 rows x 128 bytes (buffer_load_dwordx4 ... lds), counted waits.
// Workgroup w reads panel w % panels: with 12 panels an XCD's workgroups share 3 (L2 resident), with 96 they walk
// 12 MB per XCD, three times its L2.
#define WAVE_PROBE_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))
__global__ void __launch_bounds__(512) dma_probe_kernel(const uint8_t *__restrict__ src, int panels, int iters) {
  __shared__ __attribute__((aligned(1024))) uint8_t ring[2 * 32 * 1024];
  constexpr int NW = 8, PITCH = 4096, ND = 256 / 8 / NW;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint8_t *base = src + (size_t)(blockIdx.x % panels) * (256 * PITCH);
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(base), 0, 256 * PITCH, 0x00020000);
  const int voff = (lane >> 3) * PITCH + (lane & 7) * 16;
  for (int it = 0; it < iters; ++it) {
    for (int kt = 0; kt < 32; ++kt) {
#pragma unroll
      for (int d = 0; d < ND; ++d)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, WAVE_PROBE_LDS_PTR(ring + ((kt & 1) * 32 + d * NW + wave) * 1024), 16, voff,
                                                 ((d * NW + wave) * 8) * PITCH + kt * 128, 0, 0);
      __builtin_amdgcn_s_waitcnt((12 & 15) | (7 << 4) | (15 << 8));  // vmcnt(12): three K tiles in flight per wave
    }
  }
  __builtin_amdgcn_s_waitcnt(0);
}

// Third probe: a read-once stream with nothing else going on, in the access pattern of the decode kernels' B
// operand: strips of 128 rows x 4096 bytes in 16-row blocks of contiguous rows (b_preshuffle order), one workgroup of
// four waves per strip, a wave instruction = two 512-byte pieces of one K step into registers (non-temporal), four K
// tiles in flight per wave, every workgroup starting at a K tile of its own.  Launched over operand sets that
// together exceed the Infinity Cache it streams from HBM; over one set of 117 MB, from the Infinity Cache.
__global__ void __launch_bounds__(256) stream_probe_kernel(const uint8_t *__restrict__ b, int nkt, int *sink) {
  constexpr int KP = 4096, SETS = 4;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint8_t *base = b + (size_t)blockIdx.x * 128 * KP;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(base), 0, 128 * KP, 0x00020000);
  const int fr = lane & 31, fg = lane >> 5;
  const int goff = wave * 32 * KP + (fr >> 4) * 16 * KP + fg * 256 + (fr & 15) * 16;
  int kt = (int)(blockIdx.x / 8) % nkt;
  v4i r[SETS][4];
  v4i acc = {0, 0, 0, 0};
#pragma unroll
  for (int s = 0; s < SETS; ++s) {
#pragma unroll
    for (int t = 0; t < 4; ++t) r[s][t] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, goff, (kt * 4 + t) * 512, 2);
    kt = kt + 1 == nkt ? 0 : kt + 1;
  }
  for (int j = SETS; j < nkt; j += SETS) {
#pragma unroll
    for (int s = 0; s < SETS; ++s) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        acc += r[s][t];
        r[s][t] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, goff, (kt * 4 + t) * 512, 2);
      }
      kt = kt + 1 == nkt ? 0 : kt + 1;
    }
  }
#pragma unroll
  for (int s = 0; s < SETS; ++s)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc += r[s][t];
  if (acc.x == 0x12345678) sink[0] = acc.y + acc.z + acc.w;  // (keeps the loads)
}

}  // namespace

extern "C" {

// One launch of the stream probe over `strips` strips of 128 x 4096 bytes at `b` (K = 8192: 32 K tiles).
int wave_probe_read_once(const void *b, int strips, int *sink, void *hip_stream) {
  if (!b || !sink || strips < 1) return -1;
  stream_probe_kernel<<<strips, 256, 0, (hipStream_t)hip_stream>>>((const uint8_t *)b, 32, sink);
  return (int)hipGetLastError();
}


// One launch of the DMA probe: `workgroups` workgroups of 8 waves, each `iters` x 1 MB from panel (id % panels) of
// `src` (panels x 1 MB) into its LDS.  Returns 0, -1 for a bad argument, or the hipError_t of the launch.
int wave_probe_l2_dma(const void *src, int panels, int iters, int workgroups, void *hip_stream) {
  if (!src || panels < 1 || iters < 1 || workgroups < 1) return -1;
  dma_probe_kernel<<<workgroups, 512, 0, (hipStream_t)hip_stream>>>((const uint8_t *)src, panels, iters);
  return (int)hipGetLastError();
}


// Bytes of `operands` one launch reads: 32 fragments of 16 bytes per thread.
size_t wave_probe_operand_bytes(int workgroups, int waves_per_workgroup) {
  return (size_t)workgroups * 32 * (size_t)(waves_per_workgroup * 64) * 16;
}

// One launch: `workgroups` workgroups of 4 or 8 waves, each wave `iters` x 32 MFMAs of 2 * 32 * 32 * 64 flop.
// out: workgroups * waves * 64 floats; ticks: workgroups 64-bit counts of the constant 100 MHz counter.
// The sums are never rescaled (that would move all accumulators through the vector registers): pick scale_byte
// so that iters * 32 products of at most 36 * 2^(2 * (scale_byte - 127)) stay finite, e.g. 110.
// Returns 0, or -1 for a bad argument, or the hipError_t of the launch.
// idle_sleeps: 0, 4, 8 or 16 s_sleep 1 instructions (64 cycles each) after every 32 MFMAs (1024 busy cycles of a
// wave that has its SIMD to itself): the duty cycle of the matrix pipes as a knob.
int wave_probe_mfma_fp4_duty(const void *operands, float *out, unsigned long long *ticks, int iters, int scale_byte,
                             int workgroups, int waves_per_workgroup, int idle_sleeps, void *hip_stream) {
  if (!operands || !out || !ticks || iters < 1 || workgroups < 1 || scale_byte < 0 || scale_byte > 254) return -1;
  hipStream_t stream = (hipStream_t)hip_stream;
  const int s = scale_byte | (scale_byte << 8) | (scale_byte << 16) | (scale_byte << 24);
#define WAVE_PROBE_LAUNCH(NT, GAP) \
  mfma_probe_kernel<NT, GAP><<<workgroups, NT, 0, stream>>>((const v4i *)operands, out, ticks, iters, s)
  if (waves_per_workgroup == 4) {
    switch (idle_sleeps) {
      case 0: WAVE_PROBE_LAUNCH(256, 0); break;
      case 4: WAVE_PROBE_LAUNCH(256, 4); break;
      case 8: WAVE_PROBE_LAUNCH(256, 8); break;
      case 16: WAVE_PROBE_LAUNCH(256, 16); break;
      default: return -1;
    }
  } else if (waves_per_workgroup == 8) {
    switch (idle_sleeps) {
      case 0: WAVE_PROBE_LAUNCH(512, 0); break;
      case 4: WAVE_PROBE_LAUNCH(512, 4); break;
      case 8: WAVE_PROBE_LAUNCH(512, 8); break;
      case 16: WAVE_PROBE_LAUNCH(512, 16); break;
      default: return -1;
    }
  } else {
    return -1;
  }
#undef WAVE_PROBE_LAUNCH
  return (int)hipGetLastError();
}

int wave_probe_mfma_fp4(const void *operands, float *out, unsigned long long *ticks, int iters, int scale_byte,
                        int workgroups, int waves_per_workgroup, void *hip_stream) {
  return wave_probe_mfma_fp4_duty(operands, out, ticks, iters, scale_byte, workgroups, waves_per_workgroup, 0, hip_stream);
}

}  // extern "C"

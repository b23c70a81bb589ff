// Pieces shared by the tile kernels of the MXFP4 GEMM (gfx950): tile
// configuration, workgroup -> tile mapping, buffer descriptors, wait counts.
#ifndef WAVE_MXFP4_TILE_COMMON_H_
#define WAVE_MXFP4_TILE_COMMON_H_

#include "mxfp4_common.h"

namespace wave_mxfp4 {

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_>
struct TileCfg {
  static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr int NWAVES = WAVES_M * WAVES_N;
  static constexpr int NT = NWAVES * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // per-wave tile
  static constexpr int MT_M = WM / 32, MT_N = WN / 32;        // 32x32 MFMA tiles per wave
  static constexpr int A_BYTES = BM * kTileKBytes, B_BYTES = BN * kTileKBytes;
  static constexpr int RING_SLOTS = 5;
  static constexpr int SLOT_BYTES = A_BYTES > B_BYTES ? A_BYTES : B_BYTES;
  static constexpr int LDS_BYTES = RING_SLOTS * SLOT_BYTES;
  // One DMA instruction of a wave fills 8 LDS rows (64 lanes x 16 B).
  static constexpr int A_LD = BM / 8 / NWAVES, B_LD = BN / 8 / NWAVES;
  static_assert(BM % (8 * NWAVES) == 0 && BN % (8 * NWAVES) == 0, "operand tiles must split over the waves' DMA instructions");
  static_assert(LDS_BYTES <= 160 * 1024, "ring does not fit LDS");
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be MFMA aligned");
};

// Workgroup id -> (tile_m, tile_n).  The hardware deals consecutive workgroup
// ids round-robin over the 8 XCDs, each with its own L2.  Ids are first
// regrouped so every XCD owns one contiguous run of the tile sequence, then the
// sequence walks bands of kGroupM tile rows column by column, so the ~32 tiles
// an XCD runs at once share A rows and B rows in its L2.  Returns false for
// padding ids.
constexpr int kNumXcd = 8;
constexpr int kGroupM = 8;

__device__ __forceinline__ bool map_tile(int pid, int tiles_m, int tiles_n, int &tm, int &tn) {
  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + kNumXcd - 1) / kNumXcd;
  const int seq = (pid % kNumXcd) * per_xcd + pid / kNumXcd;
  if (seq >= total) return false;
  const int band_tiles = kGroupM * tiles_n;
  const int band = seq / band_tiles;
  const int in_band = seq - band * band_tiles;
  const int rows = min(kGroupM, tiles_m - band * kGroupM);
  tm = band * kGroupM + in_band % rows;
  tn = in_band / rows;
  return true;
}

// Raw (stride 0) buffer descriptor over [base, base + bytes): loads take a 32-bit
// per-lane offset plus a scalar offset, so no 64-bit address math is issued
// between the MFMAs; accesses past the end read zeros and drop their stores,
// which is how the kernels handle a last tile row that runs past M (and a slip
// in an index) without per-lane clamps or guards.  Every descriptor in the
// library ends with its tensor.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc_n(const void *base, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}

// Bytes of a scale tensor of `rows` rows in `layout` (row-major: rows * ks; the blocked layouts are padded to
// whole 32-row blocks of ksp = ceil(ks / 8) * 8 groups), and a descriptor size clipped to what one holds.
__device__ __forceinline__ int64_t scale_tensor_bytes(int layout, int64_t rows, int64_t ks, int64_t ksp) {
  return layout == WAVE_MXFP4_SCALE_ROW_MAJOR ? rows * ks : ((rows + 31) >> 5) * 32 * ksp;
}
__device__ __forceinline__ int rsrc_bytes(int64_t bytes) {
  return (int)(bytes < 0 ? 0 : bytes > 0x7FFFFFFF ? 0x7FFFFFFF : bytes);
}

// s_waitcnt immediate that waits for vmcnt <= n and lgkmcnt == 0 (gfx9
// encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14).
__host__ __device__ constexpr int waitcnt_vm_lgkm0(int n) { return (n & 15) | (7 << 4) | ((n >> 4) << 14); }

}  // namespace wave_mxfp4
#endif  // WAVE_MXFP4_TILE_COMMON_H_

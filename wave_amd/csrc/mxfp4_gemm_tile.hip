// Tiled MXFP4 block-scaled GEMM for gfx950 (MI355X).
//
// One workgroup computes a BM x BN tile of C = dequant(A) . dequant(B)^T with
// v_mfma_scale_f32_32x32x64_f8f6f4 (e2m1 operands, cbsz = blgp = 4).  It is
// the hand-written counterpart of the kernels the reference generates from
// wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:38-145 (plain),
// :334-403 (preshuffled scales / B) and :611-816 (split-K).
//
// Data flow per K tile of 256 elements (128 packed bytes per row):
//   global --(global_load_lds_dwordx4, 16 B per lane)--> LDS ring slot
//   LDS --(ds_read_b128)--> one 16 B MFMA operand fragment per lane
//   scales: global -> VGPR one K tile ahead, one byte per lane per MFMA
//
// What bounds the design (measured on MI355X):
// * A wave's DMA instruction moves 8 rows x 128 B = 8 full cache lines; the
//   vector L1 retires about one line per 2 clocks whatever part of the line is
//   used, so rows are always fetched as whole 128-byte lines (K tile = 256).
// * At full MFMA rate a 256x256 tile needs 32 B/clk/CU of the ~55 B/clk/CU the
//   DMA path sustains.  A burst of DMA instructions blocks the issuing wave
//   (and the MFMAs queued behind it), so the DMA instructions are spread
//   evenly: one half operand tile per 64-wide K step.
// * That needs more than two buffers in flight.  LDS (160 KB) is used as a
//   ring of five operand-tile slots A(j) B(j) A(j+1) B(j+1) A(j+2): slot of
//   operand tile h = 2*j + (0 for A, 1 for B) is h % 5.
// * Scale bytes are read as dwords.  In the e8m0_shuffle tile order a wave's
//   load touches one cache line; in row-major order it touches 32, which costs
//   more L1 time than the operand data, so row-major scales are reshuffled by a
//   pre-pass (see the C ABI) and only fall back to direct reads without scratch.
//
// LDS rows are 128 B; 16-byte chunk c of row r is stored at chunk position
// c ^ ((r / 2) % 8), which keeps the 16 lanes ds_read_b128 serves together on
// 16 different 16-byte bank groups (no conflicts measured).  The DMA writes
// LDS linearly, so the XOR is applied to the global source address and undone
// by the fragment reader.
//
// MFMA operand order is swapped (B rows feed the "A" port) so that a lane's
// accumulator holds runs of four consecutive N columns of one M row, each
// stored with one 16-byte (f32) or 8-byte (bf16) store.
#include <type_traits>

#include "mxfp4_tile_common.h"

namespace wave_mxfp4 {

// Byte `idx` (0..7) of the 8 bytes {hi, lo}: v_perm_b32 takes its selector
// bytes from the third operand; selector values 0..3 pick from the second
// operand (low dword), 4..7 from the first (high dword).
__device__ __forceinline__ uint32_t perm_bytes(uint32_t hi, uint32_t lo, uint32_t sel) {
  return __builtin_amdgcn_perm(hi, lo, sel);
}

// How one operand's scales are addressed by the kernel.  Per 32-row tile and K
// tile a lane needs four bytes: the scales of (row, group 2t + fg), t = 0..3.
//   MFMA32    : they are one dword, at block(r/32, kt)*256 + lane*4 (one load,
//               one cache line per wave instruction, no byte shuffling).
//   otherwise : two dwords at `off + kt*kt_stride` and that plus `delta`, then
//               v_perm with `sel`:
//     row-major : off = row*ks, kt_stride = 8, delta = 4; the row's bytes 0..7 are
//                 groups 0..7                                  -> sel 0x06040200 / 0x07050301
//     shuffled  : group g of row r sits at tile(r/32, kt)*256 + (g%4)*64 + (r%16)*4 +
//                 (g/4)*2 + (r/16)%2.  off = tile row + fg*64 + (r%16)*4, kt_stride = 256,
//                 delta = 128; dword0 = groups {fg, 4+fg}, dword1 = groups {2+fg, 6+fg},
//                 each for both 16-row halves                  -> sel 0x06020400 / 0x07030501
struct ScaleAddr {
  int kt_stride;
  int delta;
};

__device__ __forceinline__ ScaleAddr scale_addr(int layout) {
  if (layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE) return ScaleAddr{256, 128};
  if (layout == WAVE_MXFP4_SCALE_MFMA32) return ScaleAddr{256, 0};
  return ScaleAddr{8, 4};
}

// `row` is the absolute row, `row0` the first row of the workgroup's tile; the
// offset is relative to scale_tile_base(row0).
__device__ __forceinline__ void scale_lane_setup(int layout, int row, int row0, int fg, int ks, int ksp,
                                                 uint32_t &off, uint32_t &sel) {
  if (layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE) {
    off = (uint32_t)(((row >> 5) - (row0 >> 5)) * ((ksp >> 3) * 256) + fg * 64 + (row & 15) * 4);
    sel = ((row >> 4) & 1) ? 0x07030501u : 0x06020400u;
  } else if (layout == WAVE_MXFP4_SCALE_MFMA32) {
    off = (uint32_t)(((row >> 5) - (row0 >> 5)) * ((ksp >> 3) * 256) + (fg * 32 + (row & 31)) * 4);
    sel = 0x03020100u;  // identity on the low dword
  } else {
    off = (uint32_t)((row - row0) * ks);
    sel = fg ? 0x07050301u : 0x06040200u;
  }
}

__device__ __forceinline__ const uint8_t *scale_tile_base(const uint8_t *base, int layout, int row0, int ks,
                                                          int ksp) {
  return layout == WAVE_MXFP4_SCALE_ROW_MAJOR ? base + (int64_t)row0 * ks
                                              : base + (int64_t)(row0 >> 5) * ((ksp >> 3) * 256);
}

// The kernel body lives in a __device__ function so that only the device pass
// sees the gfx950 buffer-resource types and builtins.
// MODE: kDirect reads the scales in whatever layout they come in (two dwords
// and a v_perm per 32-row tile); kNative requires both scale tensors in MFMA32
// order (one dword); kGenericK is kDirect plus a partial last K tile and scale
// rows that are not 8-byte multiples (K % 256 != 0).  kDirectLds is kDirect for
// row-major scales of a short K range (at most 16 K tiles per workgroup): the
// workgroup copies the scale rows of its tile into LDS once, in whole runs of
// each row, and the waves read their eight bytes per K tile from there - a
// row-major dword load touches 32 cache lines per wave instruction, which made
// kDirect 2.5 times slower per K tile than kNative (1.30 against 0.51 us at
// 1024 x 1024).  Needs LDS behind the ring, so only the 128x128 tile has it.
enum TileMode { kDirect = 0, kNative = 1, kGenericK = 2, kDirectLds = 3 };
constexpr int kSlabMaxKTiles = 16;
constexpr int kSlabMaxPitch = (kSlabMaxKTiles + 2) * 8;  // bytes per row: the K tiles' 8 bytes each, padded to an odd
                                                         // number of 8-byte units (conflict-free 8-byte reads)

// FMT is the element format code of the scaled MFMA: 4 = e2m1 (MXFP4, everything
// described above), 0 = e4m3, 1 = e5m2 (MXFP8: tkl.f8e5m2 operands through the
// same instruction, tests/kernel/wave_gemm_mxfp_test.py:416-501).  An MXFP8 row
// holds one byte per element, so the same 128-byte K tile is 128 elements = two
// 64-wide K steps of 32 bytes per lane = four scale groups; the byte geometry of
// the ring, the DMA and the swizzle is unchanged.  MXFP8 takes row-major B and
// scales that are row-major (kDirect) or MFMA32-ordered (kNative: an MFMA32 block
// covers 8 groups = two MXFP8 K tiles, the odd one's bytes sit in the upper half
// of the lane's dword).
// FMT is A's format, FMT_B B's (MXFP8 operands may differ: e4m3 activations against e5m2 weights or the other
// way round, cbsz / blgp 0 / 1 of the instruction).  An 8-bit A may also meet a 4-bit B (FMT_B = 4: MXFP8
// activations against MXFP4 weights, B [N, K/2] packed): the K tile is A's, 128 elements, of which a row of B
// holds 64 bytes - the lower four chunks of its LDS row, the other four are neither fetched nor read - and a
// K step takes one 16-byte chunk of B per lane, as in MXFP4.
template <class Cfg, int MODE, int FMT = 4, int FMT_B = FMT>
__device__ __forceinline__ void tile_gemm_body(const GemmParams &p) {
  constexpr bool GENERIC_K = MODE == kGenericK;
  constexpr bool NATIVE = MODE == kNative;
  constexpr bool SC_LDS = MODE == kDirectLds;
  constexpr bool FP8 = FMT != 4 || FMT_B != 4;
  constexpr bool B4 = FP8 && FMT_B == 4;  // 8-bit A against 4-bit B
  constexpr bool A4 = FP8 && FMT == 4;    // 4-bit A against 8-bit B
  static_assert(!SC_LDS || (!FP8 && Cfg::LDS_BYTES + (Cfg::BM + Cfg::BN) * kSlabMaxPitch <= 160 * 1024),
                "scale rows in LDS: MXFP4 on a tile whose ring leaves room");
  static_assert(!FP8 || MODE != kGenericK, "MXFP8 needs whole K tiles");
  constexpr int BM = Cfg::BM, BN = Cfg::BN, MT_M = Cfg::MT_M, MT_N = Cfg::MT_N;
  constexpr int NWAVES = Cfg::NWAVES, A_LD = Cfg::A_LD, B_LD = Cfg::B_LD;
  constexpr int SLOT = Cfg::SLOT_BYTES, RING = Cfg::RING_SLOTS;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wave_m = wave / Cfg::WAVES_N, wave_n = wave % Cfg::WAVES_N;

  // ---------------- which tile ----------------
  int tm, tn;
  if (!map_tile(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn)) return;
  const int split = blockIdx.y;

  int row_begin = 0, row_end = p.m;
  const uint8_t *b_ptr = p.b;
  const uint8_t *bs_ptr = p.b_scale;
  if (p.num_groups > 0) {
    // tm counts BM-row tiles over all groups; find the group it falls in.
    int e = 0, first = 0, lo = 0, hi = 0;
    bool found = false;
    for (; e < p.num_groups; ++e) {
      // (clamped, not validated: a group's range is cut to [0, M] with end >= begin)
      lo = min(max(p.offsets[e], 0), p.m);
      hi = min(max(p.offsets[e + 1], lo), p.m);
      const int t = (hi - lo + BM - 1) / BM;
      if (tm < first + t) {
        found = true;
        break;
      }
      first += t;
    }
    if (!found) return;
    row_begin = lo + (tm - first) * BM;
    row_end = hi;
    b_ptr += (int64_t)e * p.b_group_stride;
    bs_ptr += (int64_t)e * p.b_scale_group_stride;
  } else {
    row_begin = tm * BM;
  }
  const int m0 = row_begin;
  const int n0 = tn * BN;

  const int kt_begin = split * p.tiles_per_split;
  const int kt_end = min(p.k_tiles, kt_begin + p.tiles_per_split);
  const int nkt = kt_end - kt_begin;
  if (nkt <= 0) return;

  // ---------------- global -> LDS addressing ----------------
  // DMA instruction d of this wave fills LDS rows (d*NWAVES + wave)*8 .. +7 of
  // an operand tile; lane t lands at row t/8, chunk position t%8, which must
  // hold logical chunk (t%8) ^ swz(row), swz(row) = (row/2) % 8.  Consecutive d
  // are 8*NWAVES rows apart (a multiple of 16), so the chunk does not depend on d.
  const int kp = p.kp;
  const int kpb = B4 ? kp >> 1 : kp;  // bytes of a row of B
  const int kpa = A4 ? kp >> 1 : kp;  // ... of A
  // (every descriptor ends with its tensor, or its expert's part of it: an access past it reads zeros instead of
  // a neighbour's memory)
  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc_n(p.a + (int64_t)m0 * kpa, rsrc_bytes(((int64_t)p.m - m0) * kpa));
  // preshuffle keeps 16-row blocks contiguous
  const __amdgpu_buffer_rsrc_t b_rsrc = make_rsrc_n(b_ptr + (int64_t)n0 * kpb, rsrc_bytes(((int64_t)p.n - n0) * kpb));
  const int ld_row0 = wave * 8 + (lane >> 3);
  const int ld_chunk = (lane & 7) ^ ((ld_row0 >> 1) & 7);
  const int a_row_lim = p.m - 1 - m0, b_row_lim = p.n - 1 - n0;  // clamp to allocated rows
  // Per-lane byte offsets inside the operand tile at K tile 0, one per DMA
  // instruction; K tile kt adds a scalar kt*128 (kt*2048 for preshuffled B).
  //   row-major  : r*kp + c*16
  //   preshuffle : (r/16)*16*kp + (c/2)*512 + (c%2)*256 + (r%16)*16
  int a_goff[A_LD], b_goff[B_LD];
#pragma unroll
  for (int d = 0; d < A_LD; ++d) {
    a_goff[d] = min(ld_row0 + d * NWAVES * 8, a_row_lim) * kpa + ld_chunk * 16;
    if (A4 && ld_chunk >= 4) a_goff[d] = (int)0x80000000;  // the upper half of the LDS row: no request, zeros
  }
#pragma unroll
  for (int d = 0; d < B_LD; ++d) {
    const int r = min(ld_row0 + d * NWAVES * 8, b_row_lim);
    b_goff[d] = p.b_preshuffled
                    ? (r >> 4) * 16 * kp + (r & 15) * 16 + (ld_chunk >> 1) * 512 + (ld_chunk & 1) * 256
                    : r * kpb + ld_chunk * 16;
    if (B4 && ld_chunk >= 4) b_goff[d] = (int)0x80000000;  // the upper half of the LDS row: no request, zeros
  }
  const int b_kt_stride = p.b_preshuffled ? 2048 : B4 ? kTileKBytes / 2 : kTileKBytes;
  const int tail_chunks = GENERIC_K ? ((p.k & (kTileK - 1)) >> 5) : 0;  // valid chunks of a partial last tile
  // kNative with a partial last K tile (MXFP4 only): the lanes whose chunk lies past the end of K fetch from
  // beyond the descriptor instead, which lands zeros in LDS: the same instructions as for a whole tile, so the
  // counted waits hold.  (The padded scale groups of the MFMA32 buffer are finite and meet those zeros.)
  // The per-lane offsets are redirected in place just before the last K tile is issued, nothing is selected
  // per instruction: part 0 = A and the first half of B, part 1 = the second half of B (issued a K tile later).
  const int native_tail = NATIVE && !FP8 ? ((p.k & (kTileK - 1)) >> 5) : 0;
  const bool tail_lane = native_tail != 0 && ld_chunk >= native_tail;
  auto arm_tail = [&](int part) {
    if (!NATIVE || FP8) return;
    if (part == 0) {
#pragma unroll
      for (int d = 0; d < A_LD; ++d) a_goff[d] = tail_lane ? (int)0x80000000 : a_goff[d];
#pragma unroll
      for (int d = 0; d < B_LD / 2; ++d) b_goff[d] = tail_lane ? (int)0x80000000 : b_goff[d];
    } else {
#pragma unroll
      for (int d = B_LD / 2; d < B_LD; ++d) b_goff[d] = tail_lane ? (int)0x80000000 : b_goff[d];
    }
  };

  // DMA instructions [d0, d1) of operand tile `op` (0 = A, 1 = B) of K tile
  // `kt` into ring slot `slot`.
  auto issue_g2l = [&](int op, int kt, int slot, int d0, int d1) {
    uint8_t *dst_tile = smem + slot * SLOT;
    // Partial last K tile: chunks at or past the end of K are written as zeros
    // (fp4 +0.0), so they add nothing whatever their scale.
    const bool tail = GENERIC_K && tail_chunks != 0 && kt == p.k_tiles - 1;
    const v4i zero = {0, 0, 0, 0};
    const int soff = op == 0 ? kt * (A4 ? kTileKBytes / 2 : kTileKBytes) : kt * b_kt_stride;
#pragma unroll
    for (int d = d0; d < d1; ++d) {
      uint8_t *dst = dst_tile + (d * NWAVES + wave) * 1024;
      if (!tail || ld_chunk < tail_chunks) {
        if (op == 0)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, WAVE_LDS_PTR(dst), 16, a_goff[d], soff, 0, 0);
        else
          __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, WAVE_LDS_PTR(dst), 16, b_goff[d], soff, 0, 0);
      } else {
        *(v4i *)(dst + lane * 16) = zero;
      }
    }
  };

  // ---------------- fragment addressing ----------------
  // 32x32x64 MFMA operand lane l: row l%32 of the 32-row tile, 32 elements
  // (16 B) at K block l/32 of the 64-wide K step t, i.e. logical chunk
  // t*2 + l/32 of the LDS row.  Wave and tile row bases are multiples of 32,
  // so swz(row) only depends on the lane.
  const int fr = lane & 31, fg = lane >> 5;
  // (MXFP8: K step s takes 32 bytes per lane in two halves, like the two 32-deep passes the instruction makes:
  //  registers 0-3 hold K 16*(l/32) .. +15 of the step, registers 4-7 K 32 + 16*(l/32) .. +15, i.e. chunks
  //  4s + l/32 and 4s + 2 + l/32; foff[2s + h] is half h.  The scale of lane l still belongs to the 32-block l/32.)
  uint32_t foff[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int chunk = FP8 ? (t >> 1) * 4 + (t & 1) * 2 + fg : t * 2 + fg;
    foff[t] = (uint32_t)(fr * kTileKBytes + ((chunk ^ ((fr >> 1) & 7)) << 4));
  }
  const uint32_t a_fbase = (uint32_t)(wave_m * Cfg::WM * kTileKBytes);
  const uint32_t b_fbase = (uint32_t)(wave_n * Cfg::WN * kTileKBytes);

  typedef typename std::conditional<FP8 && !A4, v8i, v4i>::type Frag;
  typedef typename std::conditional<FP8 && !B4, v8i, v4i>::type FragB;
  // (a 4-bit operand against an 8-bit one: its K step s is the chunk 2s + fg of the row's lower half)
  uint32_t foff_b4[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) foff_b4[t] = (uint32_t)(fr * kTileKBytes + (((t * 2 + fg) ^ ((fr >> 1) & 7)) << 4));
  auto read_frags = [&](int slot_a, int slot_b, int t, Frag(&fa)[MT_M], FragB(&fb)[MT_N]) {
    if constexpr (FP8) {
      const uint8_t *ta = smem + slot_a * SLOT + a_fbase, *tb = smem + slot_b * SLOT + b_fbase;
#pragma unroll
      for (int i = 0; i < MT_M; ++i) {
        if constexpr (A4) {
          fa[i] = *(const v4i *)(ta + foff_b4[t] + i * 32 * kTileKBytes);
        } else {
          const v4i lo = *(const v4i *)(ta + foff[2 * t] + i * 32 * kTileKBytes);
          const v4i hi = *(const v4i *)(ta + foff[2 * t + 1] + i * 32 * kTileKBytes);
          fa[i] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
      }
#pragma unroll
      for (int j = 0; j < MT_N; ++j) {
        if constexpr (B4) {
          fb[j] = *(const v4i *)(tb + foff_b4[t] + j * 32 * kTileKBytes);
        } else {
          const v4i lo = *(const v4i *)(tb + foff[2 * t] + j * 32 * kTileKBytes);
          const v4i hi = *(const v4i *)(tb + foff[2 * t + 1] + j * 32 * kTileKBytes);
          fb[j] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
      }
    } else {
      const uint8_t *ba = smem + slot_a * SLOT + a_fbase + foff[t];
      const uint8_t *bb = smem + slot_b * SLOT + b_fbase + foff[t];
#pragma unroll
      for (int i = 0; i < MT_M; ++i) fa[i] = *(const v4i *)(ba + i * 32 * kTileKBytes);
#pragma unroll
      for (int j = 0; j < MT_N; ++j) fb[j] = *(const v4i *)(bb + j * 32 * kTileKBytes);
    }
  };

  // ---------------- scales ----------------
  // Per 32-row tile and K tile a lane ends up with one VGPR whose byte t is its
  // scale for K step t (selected with op_sel): the scale of (row, group 2t + fg)
  // with groups numbered 0..7 inside the K tile.
  uint32_t a_soff[MT_M], a_ssel[MT_M], b_soff[MT_N], b_ssel[MT_N];
#pragma unroll
  for (int i = 0; i < MT_M; ++i)
    scale_lane_setup(p.a_scale_layout, min(m0 + wave_m * Cfg::WM + i * 32 + fr, p.m - 1), m0, fg, p.ks, p.ksp,
                     a_soff[i], a_ssel[i]);
#pragma unroll
  for (int j = 0; j < MT_N; ++j)
    scale_lane_setup(p.b_scale_layout, min(n0 + wave_n * Cfg::WN + j * 32 + fr, p.n - 1), n0, fg, p.ks, p.ksp,
                     b_soff[j], b_ssel[j]);
  if constexpr (FP8 && !NATIVE) {
    // row-major [R, K/32]: the K tile's four groups are one dword of the row; byte s of the canonical
    // register is group 2s + fg
#pragma unroll
    for (int i = 0; i < MT_M; ++i) a_ssel[i] = fg ? 0x0c0c0301u : 0x0c0c0200u;
#pragma unroll
    for (int j = 0; j < MT_N; ++j) b_ssel[j] = fg ? 0x0c0c0301u : 0x0c0c0200u;
  }
  const ScaleAddr a_sa = FP8 && !NATIVE ? ScaleAddr{4, 0} : scale_addr(p.a_scale_layout);
  const ScaleAddr b_sa = FP8 && !NATIVE ? ScaleAddr{4, 0} : scale_addr(p.b_scale_layout);
  const uint8_t *as_base = scale_tile_base(p.a_scale, p.a_scale_layout, m0, p.ks, p.ksp);
  const uint8_t *bs_base = scale_tile_base(bs_ptr, p.b_scale_layout, n0, p.ks, p.ksp);
  const __amdgpu_buffer_rsrc_t as_rsrc =
      make_rsrc_n(as_base, rsrc_bytes(scale_tensor_bytes(p.a_scale_layout, p.m, p.ks, p.ksp) - (as_base - p.a_scale)));
  const __amdgpu_buffer_rsrc_t bs_rsrc =
      make_rsrc_n(bs_base, rsrc_bytes(scale_tensor_bytes(p.b_scale_layout, p.n, p.ks, p.ksp) - (bs_base - bs_ptr)));

  // kDirectLds: rows 0..BM-1 of the slab are A's tile rows, BM..BM+BN-1 B's; row r holds the 8 bytes of each of
  // the workgroup's K tiles (rows past the tensor repeat its last row, like the clamped loads of kDirect).
  uint8_t *slab = smem + Cfg::LDS_BYTES;
  const uint32_t slab_pitch = (uint32_t)((nkt + 1 + (nkt & 1)) * 8);
  uint32_t a_loff[MT_M], b_loff[MT_N];
#pragma unroll
  for (int i = 0; i < MT_M; ++i) a_loff[i] = (uint32_t)(wave_m * Cfg::WM + i * 32 + fr) * slab_pitch;
#pragma unroll
  for (int j = 0; j < MT_N; ++j) b_loff[j] = (uint32_t)(BM + wave_n * Cfg::WN + j * 32 + fr) * slab_pitch;
  constexpr int kSlabIters = SC_LDS ? (BM > BN ? BM : BN) * kSlabMaxKTiles / Cfg::NT : 1;
  uint2 slab_a[kSlabIters], slab_b[kSlabIters];
  auto slab_load = [&]() {  // unit u = 8 bytes: K tile u % nkt of row u / nkt
#pragma unroll
    for (int it = 0; it < kSlabIters; ++it) {
      const int u = it * Cfg::NT + (int)threadIdx.x;
      const int r = u / nkt, c = u - r * nkt;
      slab_a[it] = slab_b[it] = uint2{0x7F7F7F7Fu, 0x7F7F7F7Fu};
      if (r < BM)
        slab_a[it] = *(const uint2 *)(p.a_scale + (int64_t)min(m0 + r, p.m - 1) * p.ks + (kt_begin + c) * 8);
      if (r < BN)
        slab_b[it] = *(const uint2 *)(bs_ptr + (int64_t)min(n0 + r, p.n - 1) * p.ks + (kt_begin + c) * 8);
    }
  };
  auto slab_store = [&]() {
#pragma unroll
    for (int it = 0; it < kSlabIters; ++it) {
      const int u = it * Cfg::NT + (int)threadIdx.x;
      const int r = u / nkt, c = u - r * nkt;
      if (r < BM) *(uint2 *)(slab + (uint32_t)r * slab_pitch + c * 8) = slab_a[it];
      if (r < BN) *(uint2 *)(slab + (uint32_t)(BM + r) * slab_pitch + c * 8) = slab_b[it];
    }
  };

  uint32_t raw_a[MT_M][2], raw_b[MT_N][2];
  uint32_t sc_a[MT_M], sc_b[MT_N];
  auto load_scales = [&](int kt) {
    if (GENERIC_K && (p.ks & 7) != 0) {
      // Row-major rows are not 8-byte multiples: four guarded byte loads per
      // row, assembled directly in canonical order (groups past the end of K
      // multiply zeros; 127 = 1.0 keeps them finite).
#pragma unroll
      for (int i = 0; i < MT_M + MT_N; ++i) {
        const bool is_a = i < MT_M;
        const bool shuffled = (is_a ? p.a_scale_layout : p.b_scale_layout) != WAVE_MXFP4_SCALE_ROW_MAJOR;
        const uint8_t *base = is_a ? as_base : bs_base;
        const uint32_t off = is_a ? a_soff[i] : b_soff[i - MT_M];
        const ScaleAddr sa = is_a ? a_sa : b_sa;
        uint32_t(&raw)[2] = is_a ? raw_a[i] : raw_b[i - MT_M];
        if (shuffled) {  // the padded shuffled buffer is always dword addressable
          raw[0] = *(const uint32_t *)(base + off + (int64_t)kt * sa.kt_stride);
          raw[1] = *(const uint32_t *)(base + off + (int64_t)kt * sa.kt_stride + sa.delta);
        } else {
          uint32_t v = 0;
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int g = kt * 8 + 2 * t + fg;
            v |= (g < p.ks ? (uint32_t)base[off + g] : 127u) << (8 * t);
          }
          raw[0] = v;
          raw[1] = 0;
        }
      }
      return;
    }
    if constexpr (SC_LDS) {
      const uint32_t ko = (uint32_t)(kt - kt_begin) * 8;
#pragma unroll
      for (int i = 0; i < MT_M; ++i) {
        const uint2 v = *(const uint2 *)(slab + a_loff[i] + ko);
        raw_a[i][0] = v.x, raw_a[i][1] = v.y;
      }
#pragma unroll
      for (int j = 0; j < MT_N; ++j) {
        const uint2 v = *(const uint2 *)(slab + b_loff[j] + ko);
        raw_b[j][0] = v.x, raw_b[j][1] = v.y;
      }
      return;
    }
    const int blk = FP8 && NATIVE ? kt >> 1 : kt;  // MXFP8: one MFMA32 block serves two K tiles
    const int ao = blk * a_sa.kt_stride, bo = blk * b_sa.kt_stride;
#pragma unroll
    for (int i = 0; i < MT_M; ++i) {
      raw_a[i][0] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(as_rsrc, (int)a_soff[i], ao, 0);
      if (!NATIVE && !FP8)
        raw_a[i][1] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(as_rsrc, (int)a_soff[i], ao + a_sa.delta, 0);
    }
#pragma unroll
    for (int j = 0; j < MT_N; ++j) {
      raw_b[j][0] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(bs_rsrc, (int)b_soff[j], bo, 0);
      if (!NATIVE && !FP8)
        raw_b[j][1] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(bs_rsrc, (int)b_soff[j], bo + b_sa.delta, 0);
    }
  };
  auto canon_scales = [&](int kt) {
    if constexpr (FP8 && NATIVE) {
      // bytes 0, 1 of the canonical register: the tile's K steps; they are bytes 2, 3 of the block's dword for
      // the odd tile of a pair.  A pinned instruction, for the reason given below.
      const int shift = (kt & 1) * 16;
#pragma unroll
      for (int i = 0; i < MT_M; ++i) asm volatile("v_lshrrev_b32 %0, %1, %2" : "=v"(sc_a[i]) : "s"(shift), "v"(raw_a[i][0]));
#pragma unroll
      for (int j = 0; j < MT_N; ++j) asm volatile("v_lshrrev_b32 %0, %1, %2" : "=v"(sc_b[j]) : "s"(shift), "v"(raw_b[j][0]));
      return;
    }
    const bool a_bytes = GENERIC_K && (p.ks & 7) != 0 && p.a_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR;
    const bool b_bytes = GENERIC_K && (p.ks & 7) != 0 && p.b_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR;
    if (NATIVE) {
      // A real register move, pinned here: if the copy were left to the
      // compiler it would be folded into the loop's phi, the next scale load
      // (issued right after) could then not reuse this register, and the copy
      // it needs instead would wait for that load at the top of every iteration.
#pragma unroll
      for (int i = 0; i < MT_M; ++i) asm volatile("v_mov_b32 %0, %1" : "=v"(sc_a[i]) : "v"(raw_a[i][0]));
#pragma unroll
      for (int j = 0; j < MT_N; ++j) asm volatile("v_mov_b32 %0, %1" : "=v"(sc_b[j]) : "v"(raw_b[j][0]));
      return;
    }
#pragma unroll
    for (int i = 0; i < MT_M; ++i)
      sc_a[i] = a_bytes ? raw_a[i][0] : perm_bytes(FP8 ? 0u : raw_a[i][1], raw_a[i][0], a_ssel[i]);
#pragma unroll
    for (int j = 0; j < MT_N; ++j)
      sc_b[j] = b_bytes ? raw_b[j][0] : perm_bytes(FP8 ? 0u : raw_b[j][1], raw_b[j][0], b_ssel[j]);
  };

  // ---------------- accumulators ----------------
  v16f acc[MT_M][MT_N];
#pragma unroll
  for (int i = 0; i < MT_M; ++i)
#pragma unroll
    for (int j = 0; j < MT_N; ++j)
#pragma unroll
      for (int g = 0; g < 16; ++g) acc[i][j][g] = 0.f;

  auto mfma_block = [&](const Frag(&fa)[MT_M], const FragB(&fb)[MT_N], auto t_tag) {
    constexpr int T = decltype(t_tag)::value;
#pragma unroll
    for (int i = 0; i < MT_M; ++i) {
      v8i va;
      if constexpr (FP8 && !A4) va = fa[i];
      else va = v8i{fa[i].x, fa[i].y, fa[i].z, fa[i].w, 0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < MT_N; ++j) {
        v8i vb;
        if constexpr (FP8 && !B4) vb = fb[j];
        else vb = v8i{fb[j].x, fb[j].y, fb[j].z, fb[j].w, 0, 0, 0, 0};
        // first port = B rows (N index), second port = A rows (M index)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vb, va, acc[i][j], FMT_B, FMT, T,
                                                                     (int)sc_b[j], T, (int)sc_a[i]);
      }
    }
  };
  typedef std::integral_constant<int, 0> T0;
  typedef std::integral_constant<int, 1> T1;
  typedef std::integral_constant<int, 2> T2;
  typedef std::integral_constant<int, 3> T3;

  // Issue order inside a phase (16 MFMAs of a 4-wave 256x256 tile): the LDS
  // reads of the next K step go out behind the first MFMAs, the DMA
  // instructions are spread one per group.  Masks: 0x008 MFMA, 0x100 LDS read,
  // 0x020 VMEM read.
  constexpr int HALF_LD = (A_LD < B_LD ? A_LD : B_LD) / 2;  // DMA instructions per phase
  constexpr int NGROUP = HALF_LD < 1 ? 1 : HALF_LD;
  auto order_phase = [&]() {
    constexpr int R = MT_M + MT_N, Q = MT_M * MT_N;
    constexpr int RG = (R + NGROUP - 1) / NGROUP, QG = Q / NGROUP;
#pragma unroll
    for (int g = 0; g < NGROUP; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, RG, 0);
      if (QG > 1) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      if (QG > 2) __builtin_amdgcn_sched_group_barrier(0x008, QG - 2, 0);
    }
  };

  // ---------------- main loop ----------------
  // Ring slots: operand tile h = 2*j + op lives in slot h % 5.  While K tile j
  // is multiplied (phases P0..P3 = its four 64-wide K steps):
  //   P0: second half of B(j+1)      P1: first half of A(j+2)
  //   P2: second half of A(j+2)      P3: barrier, then first half of B(j+2)
  // The barrier at P3 needs this wave's part of A(j+1), B(j+1) landed: every DMA
  // issued after B(j+1) is the A_LD instructions of A(j+2), hence vmcnt(A_LD).
  // After it all waves have finished reading tile j, which frees the slots of
  // A(j) (-> B(j+2), issued from P3 on) and B(j) (-> A(j+3)).
  // Fragments are double-buffered in registers across the K steps.
  Frag fa0[MT_M], fa1[MT_M];
  FragB fb0[MT_N], fb1[MT_N];
  constexpr int kWaitSteady = GENERIC_K ? 0 : A_LD;
  constexpr int kWaitPrologue = GENERIC_K ? 0 : A_LD + B_LD / 2;

  // (the last K tile of the problem is the last of the last split only)
  const bool has_tail = native_tail != 0 && kt_end == p.k_tiles;
  if (has_tail && nkt == 1) arm_tail(0), arm_tail(1);
  if constexpr (SC_LDS) slab_load();
  issue_g2l(0, kt_begin, 0, 0, A_LD);
  issue_g2l(1, kt_begin, 1, 0, B_LD);
  if constexpr (!SC_LDS) load_scales(kt_begin);
  if (nkt > 1) {
    if (has_tail && nkt == 2) arm_tail(0);
    issue_g2l(0, kt_begin + 1, 2, 0, A_LD);
    issue_g2l(1, kt_begin + 1, 3, 0, B_LD / 2);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(kWaitPrologue));
  } else {
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  }
  if constexpr (SC_LDS) {
    slab_store();  // (waits for the slab loads; the operand DMA issued behind them stays in flight)
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(63));
  }
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  if constexpr (SC_LDS) load_scales(kt_begin);
  canon_scales(kt_begin);
  if (nkt > 1) load_scales(kt_begin + 1);
  read_frags(0, 1, 0, fa0, fb0);
  __builtin_amdgcn_sched_barrier(0);

  // One K tile.  sa/sb: ring slots of A(j), B(j).  HAS1: tile j+1 exists;
  // HAS2: tile j+2 exists.  The sched_barriers pin the phase order.
  auto k_tile = [&](int j, int sa, int sb, auto has1_tag, auto has2_tag) {
    constexpr bool HAS1 = decltype(has1_tag)::value, HAS2 = decltype(has2_tag)::value;
    const int kt = kt_begin + j;
    // slots: A(j+1) = sa+2, B(j+1) = sa+3, A(j+2) = sa+4, B(j+2) = sa (mod 5)
    const int sa1 = sa + 2 >= RING ? sa + 2 - RING : sa + 2;
    const int sb1 = sa + 3 >= RING ? sa + 3 - RING : sa + 3;
    const int sa2 = sa + 4 >= RING ? sa + 4 - RING : sa + 4;
    if constexpr (FP8) {
      // two K steps per tile: the same DMA sequence folded into two phases
      read_frags(sa, sb, 1, fa1, fb1);
      mfma_block(fa0, fb0, T0{});
      if (HAS1) issue_g2l(1, kt + 1, sb1, B_LD / 2, B_LD);
      if (HAS2) issue_g2l(0, kt + 2, sa2, 0, A_LD);
      __builtin_amdgcn_sched_barrier(0);
      if (HAS1) {
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(HAS2 ? kWaitSteady : 0));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        read_frags(sa1, sb1, 0, fa0, fb0);
      }
      mfma_block(fa1, fb1, T1{});
      if (HAS2) issue_g2l(1, kt + 2, sa, 0, B_LD / 2);
      __builtin_amdgcn_sched_barrier(0);
      if (HAS1) canon_scales(kt + 1);
      if (HAS2) load_scales(kt + 2);
      __builtin_amdgcn_sched_barrier(0);
      return;
    }
    read_frags(sa, sb, 1, fa1, fb1);
    mfma_block(fa0, fb0, T0{});
    if (HAS1) issue_g2l(1, kt + 1, sb1, B_LD / 2, B_LD);
    order_phase();
    __builtin_amdgcn_sched_barrier(0);
    read_frags(sa, sb, 2, fa0, fb0);
    mfma_block(fa1, fb1, T1{});
    if (HAS2) issue_g2l(0, kt + 2, sa2, 0, A_LD / 2);
    order_phase();
    __builtin_amdgcn_sched_barrier(0);
    read_frags(sa, sb, 3, fa1, fb1);
    mfma_block(fa0, fb0, T2{});
    if (HAS2) issue_g2l(0, kt + 2, sa2, A_LD / 2, A_LD);
    order_phase();
    __builtin_amdgcn_sched_barrier(0);
    if (HAS1) {
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(HAS2 ? kWaitSteady : 0));
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      read_frags(sa1, sb1, 0, fa0, fb0);
    }
    mfma_block(fa1, fb1, T3{});
    if (HAS2) issue_g2l(1, kt + 2, sa, 0, B_LD / 2);
    order_phase();
    __builtin_amdgcn_sched_barrier(0);
    if (HAS1) canon_scales(kt + 1);
    if (HAS2) load_scales(kt + 2);
    __builtin_amdgcn_sched_barrier(0);
  };
  int j = 0, sa = 0;
  for (; j < nkt - 3; ++j) {
    const int sb = sa + 1 >= RING ? 0 : sa + 1;
    k_tile(j, sa, sb, std::true_type{}, std::true_type{});
    sa = sa + 2 >= RING ? sa + 2 - RING : sa + 2;
  }
  if (j < nkt - 2) {  // K tile nkt - 3 issues A and the first half of B of the last K tile
    if (has_tail) arm_tail(0);
    const int sb = sa + 1 >= RING ? 0 : sa + 1;
    k_tile(j, sa, sb, std::true_type{}, std::true_type{});
    sa = sa + 2 >= RING ? sa + 2 - RING : sa + 2;
    ++j;
  }
  if (has_tail && nkt >= 2) arm_tail(1);  // K tile nkt - 2 issues the second half of B of the last K tile
  if (j < nkt - 1) {
    const int sb = sa + 1 >= RING ? 0 : sa + 1;
    k_tile(j, sa, sb, std::true_type{}, std::false_type{});
    sa = sa + 2 >= RING ? sa + 2 - RING : sa + 2;
    ++j;
  }
  {
    const int sb = sa + 1 >= RING ? 0 : sa + 1;
    k_tile(j, sa, sb, std::false_type{}, std::false_type{});
  }

  // ---------------- epilogue ----------------
  // acc[i][jn][4q + e]: M row = lane%32, N column = 8q + 4*(lane/32) + e of the
  // 32x32 tile (i, jn).  Storing that directly would touch 32 cache lines per
  // store instruction with 8-16 bytes each; instead every wave transposes its
  // sub-tile through its own share of LDS (the ring is no longer needed) and
  // writes whole rows: 16 bytes per lane, full 128-byte lines.
  const int64_t ldc = p.n;
  const bool to_partial = p.partial != nullptr;
  const bool out_bf16 = !to_partial && p.out_bf16;
  const int wm0 = m0 + wave_m * Cfg::WM, wn0 = n0 + wave_n * Cfg::WN;
  const int align_elems = out_bf16 ? 8 : 4;
  if ((p.n % align_elems) == 0) {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
    __builtin_amdgcn_s_barrier();  // every wave is done reading the ring
    asm volatile("" ::: "memory");
    uint8_t *stage = smem + wave * (Cfg::LDS_BYTES / NWAVES);
    if (out_bf16) {
      // [WM rows][WN bf16] with rows padded by 8 bytes (bank spread of the b64 writes)
      constexpr int ROWB = Cfg::WN * 2 + 8;
      static_assert(Cfg::WM * ROWB <= Cfg::LDS_BYTES / NWAVES, "bf16 staging does not fit");
      typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int i = 0; i < MT_M; ++i)
#pragma unroll
        for (int jn = 0; jn < MT_N; ++jn)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const bf4 h = {(__bf16)acc[i][jn][4 * q], (__bf16)acc[i][jn][4 * q + 1], (__bf16)acc[i][jn][4 * q + 2],
                           (__bf16)acc[i][jn][4 * q + 3]};
            *(bf4 *)(stage + (i * 32 + fr) * ROWB + (jn * 32 + q * 8 + fg * 4) * 2) = h;
          }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(63));
      constexpr int LPR = Cfg::WN * 2 / 16;  // lanes per row
      constexpr int RPI = 64 / LPR;          // rows per store instruction
      const int lr = lane / LPR, lc = lane % LPR;
      __bf16 *cbase = (__bf16 *)p.c;
#pragma unroll
      for (int r0 = 0; r0 < Cfg::WM; r0 += RPI) {
        const int r = r0 + lr, m = wm0 + r, n = wn0 + lc * 8;
        const v4i v = *(const v4i *)(stage + r * ROWB + lc * 16);
        if (m < row_end && n < p.n) *(v4i *)(cbase + (int64_t)m * ldc + n) = v;
      }
    } else {
      // f32: two passes of WM/2 rows, [WM/2 rows][WN f32] padded by 16 bytes
      constexpr int ROWB = Cfg::WN * 4 + 16;
      constexpr int HALF_M = MT_M > 1 ? MT_M / 2 : 1;
      constexpr int PASSES = MT_M / HALF_M;
      static_assert(HALF_M * 32 * ROWB <= Cfg::LDS_BYTES / NWAVES, "f32 staging does not fit");
      float *cbase = to_partial ? p.partial + (int64_t)split * p.m * ldc : (float *)p.c;
      constexpr int LPR = Cfg::WN * 4 / 16;
      constexpr int RPI = 64 / LPR;
      const int lr = lane / LPR, lc = lane % LPR;
#pragma unroll
      for (int ps = 0; ps < PASSES; ++ps) {
        if (ps > 0) {
          asm volatile("" ::: "memory");
          __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(63));  // previous pass's LDS reads are done
        }
#pragma unroll
        for (int ih = 0; ih < HALF_M; ++ih)
#pragma unroll
          for (int jn = 0; jn < MT_N; ++jn)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int i = ps * HALF_M + ih;
              const v4f v = {acc[i][jn][4 * q], acc[i][jn][4 * q + 1], acc[i][jn][4 * q + 2], acc[i][jn][4 * q + 3]};
              *(v4f *)(stage + (ih * 32 + fr) * ROWB + (jn * 32 + q * 8 + fg * 4) * 4) = v;
            }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(63));
#pragma unroll
        for (int r0 = 0; r0 < HALF_M * 32; r0 += RPI) {
          const int r = r0 + lr, m = wm0 + ps * HALF_M * 32 + r, n = wn0 + lc * 4;
          const v4f v = *(const v4f *)(stage + r * ROWB + lc * 16);
          if (m < row_end && n < p.n) *(v4f *)(cbase + (int64_t)m * ldc + n) = v;
        }
      }
    }
    return;
  }
  // N not a multiple of the vector width: element-wise stores straight from
  // the accumulators.
#pragma unroll
  for (int i = 0; i < MT_M; ++i) {
    const int m = wm0 + i * 32 + fr;
    if (m >= row_end) continue;
#pragma unroll
    for (int jn = 0; jn < MT_N; ++jn) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = wn0 + jn * 32 + q * 8 + fg * 4;
        if (n >= p.n) continue;
        const int64_t idx = (int64_t)m * ldc + n;
        for (int r = 0; r < 4 && n + r < p.n; ++r) {
          const float v = acc[i][jn][4 * q + r];
          if (to_partial)
            p.partial[(int64_t)split * p.m * ldc + idx + r] = v;
          else if (out_bf16)
            ((__bf16 *)p.c)[idx + r] = (__bf16)v;
          else
            ((float *)p.c)[idx + r] = v;
        }
      }
    }
  }
}

template <class Cfg, int MODE, int FMT, int FMT_B>
__global__ void __launch_bounds__(Cfg::NT, 1) tile_gemm_kernel(const GemmParams p) {
  tile_gemm_body<Cfg, MODE, FMT, FMT_B>(p);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
typedef TileCfg<256, 256, 2, 2> Cfg256x256w4;
typedef TileCfg<256, 256, 4, 2> Cfg256x256w8;
typedef TileCfg<128, 128, 2, 2> Cfg128x128w4;
typedef TileCfg<128, 256, 2, 2> Cfg128x256w4;

void tile_variant_shape(int variant, int *bm, int *bn) {
  switch (variant) {
    case WAVE_MXFP4_VARIANT_T256x256_W2x2:
    case WAVE_MXFP4_VARIANT_T256x256_W1x4_BDIRECT:
    case WAVE_MXFP4_VARIANT_T256x256_W4x2: *bm = 256; *bn = 256; break;
    case WAVE_MXFP4_VARIANT_T128x128_W2x2: *bm = 128; *bn = 128; break;
    case WAVE_MXFP4_VARIANT_T128x256_W2x2: *bm = 128; *bn = 256; break;
    case WAVE_MXFP4_VARIANT_T256x192_W4x2: *bm = 256; *bn = 192; break;  // (persistent kernel only)
    default: *bm = 0; *bn = 0; break;
  }
}

template <class Cfg, int MODE, int FMT = 4, int FMT_B = FMT>
static hipError_t launch_cfg(const GemmParams &p, hipStream_t stream) {
  // (kDirectLds: the scale rows of the tile behind the ring)
  constexpr int kLds = Cfg::LDS_BYTES + (MODE == kDirectLds ? (Cfg::BM + Cfg::BN) * kSlabMaxPitch : 0);
  static LdsAttrOnce once;
  const hipError_t e = allow_dynamic_lds(once, (const void *)tile_gemm_kernel<Cfg, MODE, FMT, FMT_B>, kLds);
  if (e != hipSuccess) return e;
  const int total = p.tiles_m * p.tiles_n;
  const int per_xcd = (total + kNumXcd - 1) / kNumXcd;
  dim3 grid(per_xcd * kNumXcd, p.splits, 1);
  tile_gemm_kernel<Cfg, MODE, FMT, FMT_B><<<grid, dim3(Cfg::NT), kLds, stream>>>(p);
  return hipGetLastError();
}

template <class Cfg>
static hipError_t launch_by_scales(const GemmParams &p, hipStream_t stream) {
  const bool native =
      p.a_scale_layout == WAVE_MXFP4_SCALE_MFMA32 && p.b_scale_layout == WAVE_MXFP4_SCALE_MFMA32;
  if constexpr (Cfg::LDS_BYTES + (Cfg::BM + Cfg::BN) * kSlabMaxPitch <= 160 * 1024) {
    // row-major scales of a short K range go through LDS (8-byte aligned rows: K % 256 == 0 here)
    const bool rows_ok = p.a_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR && p.b_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR &&
                         ((uintptr_t)p.a_scale & 7) == 0 && ((uintptr_t)p.b_scale & 7) == 0 && (p.ks & 7) == 0 &&
                         (p.b_scale_group_stride & 7) == 0;
    if (rows_ok && p.tiles_per_split <= kSlabMaxKTiles) return launch_cfg<Cfg, kDirectLds>(p, stream);
  }
  return native ? launch_cfg<Cfg, kNative>(p, stream) : launch_cfg<Cfg, kDirect>(p, stream);
}

// K % 256 != 0 (partial last K tile, scale rows that are not 8-byte multiples)
// with scales that are not in MFMA32 order is served by one extra instantiation
// of the 128x128 kernel; the caller sizes its grid for 128x128 tiles then.
hipError_t launch_tile_gemm(const GemmParams &p, int variant, hipStream_t stream) {
  const bool native =
      p.a_scale_layout == WAVE_MXFP4_SCALE_MFMA32 && p.b_scale_layout == WAVE_MXFP4_SCALE_MFMA32;
  // (with both scale tensors in MFMA32 order every tile kernel takes a partial last K tile)
  if ((p.k & (kTileK - 1)) != 0 && !native) return launch_cfg<Cfg128x128w4, kGenericK>(p, stream);
  switch (variant) {
    case WAVE_MXFP4_VARIANT_T256x256_W2x2: return launch_by_scales<Cfg256x256w4>(p, stream);
    case WAVE_MXFP4_VARIANT_T256x256_W4x2: return launch_by_scales<Cfg256x256w8>(p, stream);
    case WAVE_MXFP4_VARIANT_T128x128_W2x2: return launch_by_scales<Cfg128x128w4>(p, stream);
    case WAVE_MXFP4_VARIANT_T128x256_W2x2: return launch_by_scales<Cfg128x256w4>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

// MXFP8: `p` describes the byte geometry (kp = K bytes per row, ks = K/32, k_tiles = K/128).
template <class Cfg, int FMT_A, int FMT_B>
static hipError_t launch_fp8_by_scales(const GemmParams &p, hipStream_t stream) {
  const bool native =
      p.a_scale_layout == WAVE_MXFP4_SCALE_MFMA32 && p.b_scale_layout == WAVE_MXFP4_SCALE_MFMA32;
  return native ? launch_cfg<Cfg, kNative, FMT_A, FMT_B>(p, stream) : launch_cfg<Cfg, kDirect, FMT_A, FMT_B>(p, stream);
}

// a_fmt, b_fmt: 0 = e4m3, 1 = e5m2, 2 = e2m1 (packed, two per byte; one operand at most)
template <class Cfg>
static hipError_t launch_fp8_formats(const GemmParams &p, int a_fmt, int b_fmt, hipStream_t stream) {
  if (a_fmt == 2 && b_fmt == 2) return hipErrorInvalidValue;  // (both 4-bit: the MXFP4 entry point)
  if (a_fmt == 2) return b_fmt ? launch_fp8_by_scales<Cfg, 4, 1>(p, stream) : launch_fp8_by_scales<Cfg, 4, 0>(p, stream);
  const int a_e5m2 = a_fmt;
  if (b_fmt == 2) return a_e5m2 ? launch_fp8_by_scales<Cfg, 1, 4>(p, stream) : launch_fp8_by_scales<Cfg, 0, 4>(p, stream);
  if (a_e5m2) return b_fmt ? launch_fp8_by_scales<Cfg, 1, 1>(p, stream) : launch_fp8_by_scales<Cfg, 1, 0>(p, stream);
  return b_fmt ? launch_fp8_by_scales<Cfg, 0, 1>(p, stream) : launch_fp8_by_scales<Cfg, 0, 0>(p, stream);
}

// MXFP8: `p` describes the byte geometry (kp = K bytes per row, ks = K/32, k_tiles = K/128).
hipError_t launch_tile_gemm_fp8(const GemmParams &p, int variant, int a_fmt, int b_fmt, hipStream_t stream) {
  if (variant == WAVE_MXFP4_VARIANT_T256x256_W2x2) return launch_fp8_formats<Cfg256x256w4>(p, a_fmt, b_fmt, stream);
  if (variant == WAVE_MXFP4_VARIANT_T256x256_W4x2) return launch_fp8_formats<Cfg256x256w8>(p, a_fmt, b_fmt, stream);
  if (variant == WAVE_MXFP4_VARIANT_T128x128_W2x2) return launch_fp8_formats<Cfg128x128w4>(p, a_fmt, b_fmt, stream);
  return hipErrorInvalidValue;
}

}  // namespace wave_mxfp4

// Tiled MXFP4 block-scaled GEMM for gfx950 (MI355X).
//
// One workgroup computes a BM x BN tile of C = dequant(A) . dequant(B)^T with
// v_mfma_scale_f32_32x32x64_f8f6f4 (e2m1 operands, cbsz = blgp = 4).  It is
// the hand-written counterpart of the kernels the reference generates from
// wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:38-145 (plain),
// :334-403 (preshuffled scales / B) and :611-816 (split-K).
//
// Data flow per K tile of 256 elements (128 packed bytes per row):
//   global --(global_load_lds_dwordx4, 16 B per lane)--> LDS stage (2 stages)
//   LDS --(ds_read_b128)--> one 16 B MFMA operand fragment per lane
//   scales: global -> VGPR (one iteration ahead), one byte per lane per MFMA
// LDS rows are 128 B; 16-byte chunk c of row r is stored at chunk position
// c ^ ((r / 2) % 8), which keeps the 16 lanes ds_read_b128 serves together on
// 16 different 16-byte bank groups.  The DMA writes LDS linearly, so the XOR is applied to the
// global source address, and undone by the fragment reader.
//
// MFMA operand order is swapped (B rows feed the "A" port) so that a lane's
// accumulator holds runs of four consecutive N columns of one M row, each
// stored with one 16-byte (f32) or 8-byte (bf16) store.
#include <type_traits>

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
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  // One DMA instruction of a wave fills 8 LDS rows (64 lanes x 16 B).
  static constexpr int A_LD = BM / 8 / NWAVES, B_LD = BN / 8 / NWAVES;
  static_assert(BM % (8 * NWAVES) == 0 && BN % (8 * NWAVES) == 0, "tile rows must split over waves");
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

// Byte `idx` (0..7) of the 8 bytes {hi, lo}: v_perm_b32 takes its selector
// bytes from the third operand; selector values 0..3 pick from the second
// operand (low dword), 4..7 from the first (high dword).
__device__ __forceinline__ uint32_t perm_bytes(uint32_t hi, uint32_t lo, uint32_t sel) {
  return __builtin_amdgcn_perm(hi, lo, sel);
}

// How one operand's scales are addressed by the kernel, whatever their layout:
// per 32-row tile a lane reads two dwords at `off + kt*kt_stride` and that plus
// `delta`, then picks its four bytes (K steps 0..3) with v_perm and `sel`.
//   row-major : off = row*ks, kt_stride = 8, delta = 4; the row's bytes 0..7 are
//               groups 0..7, the lane needs 2t + fg            -> sel 0x06040200 / 0x07050301
//   shuffled  : group g of row r sits at tile(r/32, kt)*256 + (g%4)*64 + (r%16)*4 +
//               (g/4)*2 + (r/16)%2.  off = tile row + fg*64 + (r%16)*4, kt_stride = 256,
//               delta = 128; dword0 = groups {fg, 4+fg}, dword1 = groups {2+fg, 6+fg},
//               each for both 16-row halves                    -> sel 0x06020400 / 0x07030501
struct ScaleAddr {
  int kt_stride;
  int delta;
};

__device__ __forceinline__ void scale_lane_setup(bool shuffled, int row, int fg, int ks, int ksp,
                                                 uint32_t &off, uint32_t &sel) {
  if (shuffled) {
    off = (uint32_t)((row >> 5) * ((ksp >> 3) * 256) + fg * 64 + (row & 15) * 4);
    sel = ((row >> 4) & 1) ? 0x07030501u : 0x06020400u;
  } else {
    off = (uint32_t)(row * ks);
    sel = fg ? 0x07050301u : 0x06040200u;
  }
}

template <class Cfg, bool GENERIC_K>
__global__ void __launch_bounds__(Cfg::NT, 1) tile_gemm_kernel(const GemmParams p) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, MT_M = Cfg::MT_M, MT_N = Cfg::MT_N;
  constexpr int NWAVES = Cfg::NWAVES, A_LD = Cfg::A_LD, B_LD = Cfg::B_LD;
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
      lo = p.offsets[e];
      hi = p.offsets[e + 1];
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
  // DMA instruction d of this wave fills LDS rows (d*NWAVES + wave)*8 .. +7;
  // lane t lands at row t/8, chunk position t%8, which must hold logical
  // chunk (t%8) ^ swz(row), swz(row) = (row/2) % 8.  Consecutive d are 8*NWAVES
  // rows apart (a multiple of 16), so the chunk does not depend on d.
  const int kp = p.kp;
  const uint8_t *a_tile = p.a + (int64_t)m0 * kp;
  const uint8_t *b_tile = b_ptr + (int64_t)n0 * kp;  // preshuffle keeps 16-row blocks contiguous
  const int ld_row0 = wave * 8 + (lane >> 3);
  const int ld_chunk = (lane & 7) ^ ((ld_row0 >> 1) & 7);
  const int a_row_lim = p.m - 1 - m0, b_row_lim = p.n - 1 - n0;  // clamp to allocated rows
  // B offset of (row r, chunk c) inside the tile, K tile 0:
  //   row-major  : r*kp + c*16
  //   preshuffle : (r/16)*16*kp + (c/2)*512 + (c%2)*256 + (r%16)*16
  const int b_row_shift = p.b_preshuffled ? 4 : 0;
  const int b_row_mask = p.b_preshuffled ? 15 : 0;
  const int b_blk_stride = p.b_preshuffled ? 16 * kp : kp;
  const int b_chunk_off = p.b_preshuffled ? (ld_chunk >> 1) * 512 + (ld_chunk & 1) * 256 : ld_chunk * 16;
  const int b_kt_stride = p.b_preshuffled ? 2048 : kTileKBytes;
  const int tail_chunks = GENERIC_K ? ((p.k & (kTileK - 1)) >> 5) : 0;  // valid chunks of a partial last tile

  auto issue_g2l = [&](int kt, int stage) {
    uint8_t *sa = smem + stage * Cfg::STAGE_BYTES;
    uint8_t *sb = sa + Cfg::A_BYTES;
    const uint8_t *ga = a_tile + (int64_t)kt * kTileKBytes;
    const uint8_t *gb = b_tile + (int64_t)kt * b_kt_stride;
    // The row offsets are recomputed per K tile (a handful of VALU ops hidden
    // under the MFMAs) rather than kept in 2*(A_LD+B_LD) registers.
    int lr = ld_row0;
    asm volatile("" : "+v"(lr));
    // Partial last K tile: chunks at or past the end of K are written as zeros
    // (fp4 +0.0), so they add nothing whatever their scale.
    const bool tail = GENERIC_K && tail_chunks != 0 && kt == p.k_tiles - 1;
    const v4i zero = {0, 0, 0, 0};
#pragma unroll
    for (int d = 0; d < A_LD; ++d) {
      const int r = min(lr + d * NWAVES * 8, a_row_lim);
      const uint32_t off = (uint32_t)(r * kp + ld_chunk * 16);
      uint8_t *dst = sa + (d * NWAVES + wave) * 1024;
      if (!tail || ld_chunk < tail_chunks)
        __builtin_amdgcn_global_load_lds(WAVE_GLOBAL_PTR(ga + off), WAVE_LDS_PTR(dst), 16, 0, 0);
      else
        *(v4i *)(dst + lane * 16) = zero;
    }
#pragma unroll
    for (int d = 0; d < B_LD; ++d) {
      const int r = min(lr + d * NWAVES * 8, b_row_lim);
      const uint32_t off = (uint32_t)((r >> b_row_shift) * b_blk_stride + (r & b_row_mask) * 16 + b_chunk_off);
      uint8_t *dst = sb + (d * NWAVES + wave) * 1024;
      if (!tail || ld_chunk < tail_chunks)
        __builtin_amdgcn_global_load_lds(WAVE_GLOBAL_PTR(gb + off), WAVE_LDS_PTR(dst), 16, 0, 0);
      else
        *(v4i *)(dst + lane * 16) = zero;
    }
  };

  // ---------------- fragment addressing ----------------
  // 32x32x64 MFMA operand lane l: row l%32 of the 32-row tile, 32 elements
  // (16 B) at K block l/32 of the 64-wide K step t, i.e. logical chunk
  // t*2 + l/32 of the LDS row.  Wave and tile row bases are multiples of 32,
  // so swz(row) only depends on the lane.
  const int fr = lane & 31, fg = lane >> 5;
  uint32_t foff[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) foff[t] = (uint32_t)(fr * kTileKBytes + (((t * 2 + fg) ^ ((fr >> 1) & 7)) << 4));
  const uint32_t a_fbase = (uint32_t)(wave_m * Cfg::WM * kTileKBytes);
  const uint32_t b_fbase = (uint32_t)(Cfg::A_BYTES + wave_n * Cfg::WN * kTileKBytes);

  auto read_frags = [&](int stage, int t, v4i(&fa)[MT_M], v4i(&fb)[MT_N]) {
    const uint8_t *base = smem + stage * Cfg::STAGE_BYTES + foff[t];
#pragma unroll
    for (int i = 0; i < MT_M; ++i) fa[i] = *(const v4i *)(base + a_fbase + i * 32 * kTileKBytes);
#pragma unroll
    for (int j = 0; j < MT_N; ++j) fb[j] = *(const v4i *)(base + b_fbase + j * 32 * kTileKBytes);
  };

  // ---------------- scales ----------------
  // Per 32-row tile and K tile a lane ends up with one VGPR whose byte t is its
  // scale for K step t (selected with op_sel): the scale of (row, group 2t + fg)
  // with groups numbered 0..7 inside the K tile.
  uint32_t a_soff[MT_M], a_ssel[MT_M], b_soff[MT_N], b_ssel[MT_N];
#pragma unroll
  for (int i = 0; i < MT_M; ++i)
    scale_lane_setup(p.a_scale_shuffled, min(m0 + wave_m * Cfg::WM + i * 32 + fr, p.m - 1), fg, p.ks, p.ksp,
                     a_soff[i], a_ssel[i]);
#pragma unroll
  for (int j = 0; j < MT_N; ++j)
    scale_lane_setup(p.b_scale_shuffled, min(n0 + wave_n * Cfg::WN + j * 32 + fr, p.n - 1), fg, p.ks, p.ksp,
                     b_soff[j], b_ssel[j]);
  const ScaleAddr a_sa = {p.a_scale_shuffled ? 256 : 8, p.a_scale_shuffled ? 128 : 4};
  const ScaleAddr b_sa = {p.b_scale_shuffled ? 256 : 8, p.b_scale_shuffled ? 128 : 4};

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
        const bool shuffled = is_a ? p.a_scale_shuffled : p.b_scale_shuffled;
        const uint8_t *base = is_a ? p.a_scale : bs_ptr;
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
    const uint8_t *ab = p.a_scale + (int64_t)kt * a_sa.kt_stride;
    const uint8_t *bb = bs_ptr + (int64_t)kt * b_sa.kt_stride;
#pragma unroll
    for (int i = 0; i < MT_M; ++i) {
      raw_a[i][0] = *(const uint32_t *)(ab + a_soff[i]);
      raw_a[i][1] = *(const uint32_t *)(ab + a_sa.delta + a_soff[i]);
    }
#pragma unroll
    for (int j = 0; j < MT_N; ++j) {
      raw_b[j][0] = *(const uint32_t *)(bb + b_soff[j]);
      raw_b[j][1] = *(const uint32_t *)(bb + b_sa.delta + b_soff[j]);
    }
  };
  auto canon_scales = [&]() {
    const bool a_bytes = GENERIC_K && (p.ks & 7) != 0 && !p.a_scale_shuffled;
    const bool b_bytes = GENERIC_K && (p.ks & 7) != 0 && !p.b_scale_shuffled;
#pragma unroll
    for (int i = 0; i < MT_M; ++i)
      sc_a[i] = a_bytes ? raw_a[i][0] : perm_bytes(raw_a[i][1], raw_a[i][0], a_ssel[i]);
#pragma unroll
    for (int j = 0; j < MT_N; ++j)
      sc_b[j] = b_bytes ? raw_b[j][0] : perm_bytes(raw_b[j][1], raw_b[j][0], b_ssel[j]);
  };

  // ---------------- accumulators ----------------
  v16f acc[MT_M][MT_N];
#pragma unroll
  for (int i = 0; i < MT_M; ++i)
#pragma unroll
    for (int j = 0; j < MT_N; ++j)
#pragma unroll
      for (int g = 0; g < 16; ++g) acc[i][j][g] = 0.f;

  auto mfma_block = [&](const v4i(&fa)[MT_M], const v4i(&fb)[MT_N], auto t_tag) {
    constexpr int T = decltype(t_tag)::value;
#pragma unroll
    for (int i = 0; i < MT_M; ++i) {
      const v8i va = {fa[i].x, fa[i].y, fa[i].z, fa[i].w, 0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < MT_N; ++j) {
        const v8i vb = {fb[j].x, fb[j].y, fb[j].z, fb[j].w, 0, 0, 0, 0};
        // first port = B rows (N index), second port = A rows (M index)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vb, va, acc[i][j], 4, 4, T,
                                                                     (int)sc_b[j], T, (int)sc_a[i]);
      }
    }
  };
  typedef std::integral_constant<int, 0> T0;
  typedef std::integral_constant<int, 1> T1;
  typedef std::integral_constant<int, 2> T2;
  typedef std::integral_constant<int, 3> T3;

  // ---------------- main loop ----------------
  // Two LDS stages; the DMA of K tile it+2 is issued as soon as every wave has
  // finished reading tile it (3/4 through iteration it) and is waited for at
  // the same point of iteration it+1.  Fragments are double-buffered in
  // registers across the four 64-wide K steps of a tile.
  v4i fa0[MT_M], fb0[MT_N], fa1[MT_M], fb1[MT_N];

  issue_g2l(kt_begin, 0);
  load_scales(kt_begin);
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (nkt > 1) issue_g2l(kt_begin + 1, 1);
  canon_scales();
  if (nkt > 1) load_scales(kt_begin + 1);
  read_frags(0, 0, fa0, fb0);
  __builtin_amdgcn_sched_barrier(0);

  // One K tile.  The sched_barriers pin the phase order (the scheduler may
  // interleave inside a phase, i.e. the LDS reads of step t+1 with the MFMAs of
  // step t, but not merge phases, which would need every step's fragments
  // live at once).  HAS1: tile it+1 exists; HAS2: tile it+2 exists.
  // Issue order inside a phase: the LDS reads of the next K step go out first,
  // two behind each of the first MFMAs, so their latency is covered by the
  // remaining MFMAs of the phase.  Masks: 0x008 MFMA, 0x100 LDS read, 0x020 VMEM read.
  auto order_reads_then_mfma = [&]() {
#pragma unroll
    for (int r = 0; r < (MT_M + MT_N) / 2; ++r) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, MT_M * MT_N - (MT_M + MT_N) / 2, 0);
  };
  auto k_tile = [&](int it, auto has1_tag, auto has2_tag) {
    constexpr bool HAS1 = decltype(has1_tag)::value, HAS2 = decltype(has2_tag)::value;
    const int cur = it & 1;
    read_frags(cur, 1, fa1, fb1);
    mfma_block(fa0, fb0, T0{});
    order_reads_then_mfma();
    __builtin_amdgcn_sched_barrier(0);
    read_frags(cur, 2, fa0, fb0);
    mfma_block(fa1, fb1, T1{});
    order_reads_then_mfma();
    __builtin_amdgcn_sched_barrier(0);
    read_frags(cur, 3, fa1, fb1);
    mfma_block(fa0, fb0, T2{});
    order_reads_then_mfma();
    __builtin_amdgcn_sched_barrier(0);
    // Own DMA of tile it+1 and all fragment reads of stage `cur` are complete
    // before the barrier; after it every wave's are.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    if (HAS2) issue_g2l(kt_begin + it + 2, cur);
    if (HAS1) read_frags(cur ^ 1, 0, fa0, fb0);
    mfma_block(fa1, fb1, T3{});
    if (HAS2) {
      // DMA first (longest latency), LDS reads next, all within the first MFMAs
      constexpr int G = A_LD + B_LD, R = MT_M + MT_N, Q = MT_M * MT_N;
      constexpr int SLOTS = Q / 2;
#pragma unroll
      for (int r = 0; r < SLOTS; ++r) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, (G + SLOTS - 1) / SLOTS, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, (R + SLOTS - 1) / SLOTS, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, Q - SLOTS, 0);
    } else if (HAS1) {
      order_reads_then_mfma();
    }
    __builtin_amdgcn_sched_barrier(0);
    if (HAS1) canon_scales();
    if (HAS2) load_scales(kt_begin + it + 2);
    __builtin_amdgcn_sched_barrier(0);
  };
  int it = 0;
  for (; it < nkt - 2; ++it) k_tile(it, std::true_type{}, std::true_type{});
  if (it < nkt - 1) {
    k_tile(it, std::true_type{}, std::false_type{});
    ++it;
  }
  k_tile(it, std::false_type{}, std::false_type{});

  // ---------------- epilogue ----------------
  // acc[i][j][4q + e]: M row = lane%32, N column = 8q + 4*(lane/32) + e.
  const int64_t ldc = p.n;
  const bool vec_ok = (p.n & 3) == 0;
#pragma unroll
  for (int i = 0; i < MT_M; ++i) {
    const int m = m0 + wave_m * Cfg::WM + i * 32 + fr;
    if (m >= row_end) continue;
#pragma unroll
    for (int j = 0; j < MT_N; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wave_n * Cfg::WN + j * 32 + q * 8 + fg * 4;
        if (n >= p.n) continue;
        const v4f v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
        const int64_t idx = (int64_t)m * ldc + n;
        if (p.partial != nullptr) {
          float *dst = p.partial + (int64_t)split * p.m * ldc + idx;
          if (vec_ok) {
            *(v4f *)dst = v;
          } else {
            for (int r = 0; r < 4 && n + r < p.n; ++r) dst[r] = v[r];
          }
        } else if (p.out_bf16) {
          __bf16 *dst = (__bf16 *)p.c + idx;
          if (vec_ok) {
            typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
            const bf4 h = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
            *(bf4 *)dst = h;
          } else {
            for (int r = 0; r < 4 && n + r < p.n; ++r) dst[r] = (__bf16)v[r];
          }
        } else {
          float *dst = (float *)p.c + idx;
          if (vec_ok) {
            *(v4f *)dst = v;
          } else {
            for (int r = 0; r < 4 && n + r < p.n; ++r) dst[r] = v[r];
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
typedef TileCfg<256, 256, 2, 2> Cfg256x256w4;
typedef TileCfg<256, 256, 4, 2> Cfg256x256w8;
typedef TileCfg<128, 128, 2, 2> Cfg128x128w4;
typedef TileCfg<256, 128, 2, 2> Cfg256x128w4;
typedef TileCfg<128, 256, 2, 2> Cfg128x256w4;

void tile_variant_shape(int variant, int *bm, int *bn) {
  switch (variant) {
    case WAVE_MXFP4_VARIANT_T256x256_W2x2:
    case WAVE_MXFP4_VARIANT_T256x256_W4x2: *bm = 256; *bn = 256; break;
    case WAVE_MXFP4_VARIANT_T128x128_W2x2: *bm = 128; *bn = 128; break;
    case WAVE_MXFP4_VARIANT_T256x128_W2x2: *bm = 256; *bn = 128; break;
    case WAVE_MXFP4_VARIANT_T128x256_W2x2: *bm = 128; *bn = 256; break;
    default: *bm = 0; *bn = 0; break;
  }
}

template <class Cfg, bool GENERIC_K>
static hipError_t launch_cfg(const GemmParams &p, hipStream_t stream) {
  static bool attr_done = false;  // benign race: the attribute is idempotent
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void *)tile_gemm_kernel<Cfg, GENERIC_K>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_done = true;
  }
  const int total = p.tiles_m * p.tiles_n;
  const int per_xcd = (total + kNumXcd - 1) / kNumXcd;
  dim3 grid(per_xcd * kNumXcd, p.splits, 1);
  tile_gemm_kernel<Cfg, GENERIC_K><<<grid, dim3(Cfg::NT), Cfg::LDS_BYTES, stream>>>(p);
  return hipGetLastError();
}

// K % 256 != 0 (partial last K tile, scale rows that are not 8-byte multiples)
// is served by one extra instantiation of the 128x128 kernel; the caller maps
// every tile variant onto it for such K (see tile_variant_shape_for_k).
hipError_t launch_tile_gemm(const GemmParams &p, int variant, hipStream_t stream) {
  if ((p.k & (kTileK - 1)) != 0) return launch_cfg<Cfg128x128w4, true>(p, stream);
  switch (variant) {
    case WAVE_MXFP4_VARIANT_T256x256_W2x2: return launch_cfg<Cfg256x256w4, false>(p, stream);
    case WAVE_MXFP4_VARIANT_T256x256_W4x2: return launch_cfg<Cfg256x256w8, false>(p, stream);
    case WAVE_MXFP4_VARIANT_T128x128_W2x2: return launch_cfg<Cfg128x128w4, false>(p, stream);
    case WAVE_MXFP4_VARIANT_T256x128_W2x2: return launch_cfg<Cfg256x128w4, false>(p, stream);
    case WAVE_MXFP4_VARIANT_T128x256_W2x2: return launch_cfg<Cfg128x256w4, false>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace wave_mxfp4

// Mid-M MXFP4 GEMM for gfx950 (MI355X): 16 < M <= 256 against a wide B that comes from HBM.
//
// Up to M of about 200 the operation is still bound by reading B once (2*M*N*K flops against N*K/2 bytes), but M
// is too large for the streaming kernel's resident A (64 registers per 16 rows) and too small for the tile
// kernels, whose ring gives B two K tiles of prefetch next to A's: one tile per CU then waits for memory latency
// (128 x 28672 x 8192 ran at 2.9 TB/s there).  What this regime wants is all of LDS for B and a shallow, cheap
// path for A, which comes from L2.  Vector memory operations of a wave retire in issue order, so a wave that
// waits for a recent A tile also waits for every older B request: the two streams need different waves.
//
//   * One workgroup per strip of 4 * WV columns of C: four compute waves, 2 x 2 on the strip (each every second
//     32-row block and two of the strip's four groups of WV <= 32 columns; v_mfma_scale_f32_32x32x64_f8f6f4,
//     BM / 32 accumulator tiles, one A fragment per two MFMAs; side by side on one row block at BM = 32) and a
//     fifth, the producer wave, which does nothing but request A.  WV is chosen per problem so that the strips come out as a whole number of rounds over the CUs
//     (N = 28672 on 256 CUs: 28 columns per group, 256 workgroups).  The rows of a group's MFMA operand past WV
//     are zero-filled by the buffer descriptor (no memory request) and their columns are not stored.
//   * B goes into a ring of DB K tiles (four groups of 32 rows x 128 bytes each).  Compute wave w fetches group
//     w (4 DMA instructions of 8 rows x 128 bytes per K tile, whole cache lines, non-temporal) and waits for its
//     own requests only, with a counted vmcnt that leaves the younger DB - 2 K tiles in flight; the K tile's one
//     barrier then makes all four groups visible to all.  The groups' scales travel the same way: in MFMA32
//     order one DMA instruction per FOUR K tiles (the blocks of consecutive K tiles are contiguous) and a lane
//     reads its dword; row-major scales as 64 bytes of each of the 32 rows (8 K tiles per image, the 16-byte
//     pieces swizzled for conflict-free reads) from which a lane reads its row's piece of two K tiles and picks
//     the four bytes of its K tile with one v_perm, so neither order needs a pass of its own.
//   * The producer wave fetches A (BM rows x 128 bytes per K tile) and its scales into a ring of DA K tiles,
//     DA - 1 ahead, waits for its own requests, and meets the compute waves at the barrier: behind it A(j) is
//     visible to all and the slots of A(j - 1) and B(j - 1) are free.
//   * C leaves through the (by then idle) B ring, 4 KB per wave, 64 or 128 bytes per row and store.
//   * Workgroups start at different K tiles and walk around the end of K, so that the chip's requests of a
//     moment spread over the memory channels instead of all naming the same 128 bytes of every 4 KB row.
//   * A grouped (mixture of experts) problem of few rows per expert runs the same body with one workgroup per
//     (expert, strip); a wave skips the row blocks past its group's rows.
//
// Taken for K % 256 == 0 (at least 4 K tiles), N % 4 == 0, each scale tensor row-major, in MFMA32 order or in
// e8m0_shuffle order, the reference's format for preshuffled scales (all read as they are; B scales in a blocked
// order fix WV at 32, the row block of those layouts; a grouped problem takes A's row-major only), B row-major or
// preshuffled.  The reference runs these shapes
// through its generic tile kernel (tests/kernel/wave_gemm_mxfp_test.py:291-339); the result contract is the same.
#include <type_traits>

#include "mxfp4_tile_common.h"

namespace wave_mxfp4 {

namespace {

constexpr int kMidBN = 128, kMidCW = 4, kMidNT = (kMidCW + 1) * 64;
constexpr int kMidOnce = 2;  // the "nt" bit: B is read exactly once

// B_RM: B's scales are row-major: a group's image is then two buffers of 32 rows x 64 bytes (8 K tiles) instead
// of four buffers of 1 KB (4 K tiles).
// TWO_PER_CU (BM = 32 only): rings of three K tiles each, 78 KB of LDS, so that two workgroups share a CU and the
// one's prologue and C write run under the other's stream.  For problems of more workgroups than CUs (measured, 8
// experts x 14336 x 4096 at one row per expert: 47.0 -> 40.2 us, 6.2 TB/s; 64 experts x 2048 x 7168: 80.8 -> 74.1 us,
// 6.75 TB/s); with one workgroup per CU or fewer the deep rings are the better use of the LDS.
// A_OFF: A's scales are in MFMA32 order and the block of rows may start inside one of their 32-row blocks (a group
// of a grouped problem starts at any row): the images hold one block more.
template <int BM_, bool B_RM_, bool TWO_PER_CU_ = false, bool A_OFF_ = false>
struct MidCfg {
  static constexpr int BM = BM_, MT_M = BM / 32;
  static constexpr bool B_RM = B_RM_, TWO_PER_CU = TWO_PER_CU_, A_OFF = A_OFF_;
  static_assert(!TWO_PER_CU || BM == 32, "only the 32-row block leaves room for two workgroups");
  // The four compute waves sit WM x (4 / WM) on the strip: two row halves times two pairs of column groups from
  // BM = 64 on (one A fragment per two MFMAs), side by side on one row block at BM = 32.
  static constexpr int WM = BM >= 64 ? 2 : 1;
  static constexpr int A_SLOT = BM * kTileKBytes;
  // Ring depths, measured at N = 28672, K = 8192 (us at M = 64 / 128 / 192): A, which every workgroup re-reads
  // from L2 at the same moment as all the others, needs the deeper ring.  With no B traffic at all the kernel
  // took 17 / 22 us at two K tiles of A ahead: its latency, not B's, set the pace.
  //   (DA, DB) = (3, 7) / (3, 5) / (2, 5): 29.9 / 33.1 / 43.5     (6, 5) / (5, 3) / (3, 3): 27.9 / 31.4 / 39.0
  // Deeper still for A at the small blocks, re-measured later on the same shape: 32 rows (6, 7) -> (10, 6) 22.9 ->
  // 22.7 us, 64 rows (6, 5) -> (8, 4) 24.4 -> 24.3 (23.75 -> 23.4 with MFMA32 scales); at 128 rows (6, 2) lost
  // against (5, 3), 33.0 against 28.9 us.  A producer with more than 63 requests in flight is held at the counter's
  // limit by the hardware, and its wait is clamped there (it then waits for a few requests more than it must).
  // The 256-row block, whose K tile of A is 32 KB, takes (3, 2): a third K tile of A is worth more than B's third
  // and fourth (M = 256 / 224 / 200 at N = 28672, K = 8192 with (2, 4): 45.0 / 43.2 / 42.7 us, with (3, 2): 43.6 /
  // 41.1 / 39.9); at 192 rows (4, 2) against (3, 3) is a draw (36.4 / 35.6 against 37.7 / 35.0 us with row-major /
  // MFMA32 scales) and (3, 3) stays.
  static constexpr int DA = TWO_PER_CU ? 3 : BM <= 32 ? 10 : BM <= 64 ? 8 : BM <= 128 ? 5 : 3;  // K tiles of A in LDS
  static constexpr int DB = TWO_PER_CU ? 3 : BM <= 32 ? 6 : BM <= 64 ? 4 : BM <= 192 ? 3 : 2;   // K tiles of B in the ring
  static constexpr int LB = DB - 1;                                      // B is requested LB K tiles ahead
  static constexpr int AS_SLOT = (MT_M + (A_OFF ? 1 : 0)) * 1024;        // A scales of 4 K tiles (1 KB per 32 rows)
  // Scale groups of A in LDS: the one being read, (j / 4), up to the one requested with A(j + DA - 1); a group's
  // slot may be overwritten only when the group before it in that slot is no longer read: more than
  // ceil((DA - 1) / 4) slots (a power of two, for the slot index).
  static constexpr int AS_SLOTS = (DA - 1 + 3) / 4 + 1 <= 2 ? 2 : 4;
  static constexpr int A_RING = DA * A_SLOT, AS_RING = AS_SLOTS * AS_SLOT;
  static constexpr int B_RING = DB * kMidBN * kTileKBytes;               // B ring (16 KB per K tile: four 32-row groups)
  static constexpr int BS_WAVE = 4 * 1024;                               // one group's scale images
  static constexpr int LDS = A_RING + AS_RING + B_RING + kMidCW * BS_WAVE;
  static constexpr int A_LD = BM / 8;                                    // A DMA instructions per K tile (producer)
  static_assert(LDS <= (TWO_PER_CU ? 80 : 160) * 1024, "LDS");
  static_assert(MT_M % WM == 0 && B_RING >= kMidCW * 32 * 32 * 4, "whole row blocks per wave; the waves' C staging fits the ring");
  static_assert(4 * (LB - 1) + 2 <= 63, "vmcnt range");
};

// A_RM / B_RM: the operand's scales are row-major (else MFMA32 order, or with A_SH / B_SH e8m0_shuffle order: the
// same 256-byte blocks per 32 rows and K tile, fetched the same way; only the lane's read differs).  Template
// parameters, not run-time flags:
// a branch on the layout inside the K loop makes the compiler wait for every outstanding request at the join.
// One strip of one block of `m_rows` <= BM rows: A [m_rows, kp] at `a_base` with its scales at `as_base`, B [N, kp]
// at `b_base` (one expert's, for a grouped problem) with its scales at `bs_base`, C rows at `c_base`.
// GATED: the first GEMM of a gated MLP with the step behind it in its C write, as in the persistent kernel
// (mxfp4_gemm_persist.hip): B holds gate and up rows interleaved in blocks of 32, so the two column groups of a wave
// are gate and up of the same 32 activation columns, element for element in the same lane; written are the MXFP4
// codes of silu(gate) * up ([rows, N / 4] bytes at `c_base`) and one e8m0 scale per row and 32 columns in MFMA32
// order at p.epi_scale (row `m_abs0` + the block's row).  The arithmetic of the unfused pair of kernels, bit for bit.
template <class Cfg, bool A_RM, bool B_SH, bool A_SH, bool GATED = false>
__device__ __forceinline__ void mid_body(const GemmParams &p, const int wv, const uint8_t *a_base, const uint8_t *as_base,
                                         const uint8_t *b_base, const uint8_t *bs_base, uint8_t *c_base, const int m_rows,
                                         const int a_row32 = 0, const int m_abs0 = 0) {
  static_assert(!GATED || (!Cfg::B_RM && !B_SH), "gated epilogue: B scales in MFMA32 order (column groups of 32)");
  constexpr bool B_RM = Cfg::B_RM;
  constexpr int MT_M = Cfg::MT_M, DA = Cfg::DA, DB = Cfg::DB, LB = Cfg::LB;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  uint8_t *const a_ring = smem;
  uint8_t *const as_ring = smem + Cfg::A_RING;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kp = p.kp, nkt = p.k_tiles;
  const int n0 = blockIdx.x * (kMidCW * wv);
  const int k_tiles_blocks = nkt * 256;   // bytes of one 32-row block row of MFMA32 scales
  // Where this workgroup starts in K.  Workgroups that all walk K from tile 0 ask, at any moment, for the same
  // 128 bytes of every row of A and of B: a few L2 and memory channels take all requests of the chip (a bare
  // stream of B in this shape: 22.3 us; the same requests with the start rotated per workgroup: 18.0 us).  With
  // whole groups of 8 K tiles, the workgroups of an XCD (ids x, x + 8, ..) therefore start one K tile apart and
  // walk around the end of K; the sums are the same terms in another order.  The loops count a virtual K tile v
  // from v0 = start % 8, so that v and the K tile it stands for agree mod 8 and the scale groups (4 and 8 K
  // tiles) keep their places in the images.
  const bool rotate = (nkt & 7) == 0;
  const int k_start = rotate ? (int)(((blockIdx.y * gridDim.x + blockIdx.x) >> 3) % (uint32_t)nkt) : 0;
  const int v0 = k_start & 7, vend = v0 + nkt, k_base = k_start - v0;
  const int g_end = (vend + 3) >> 2, h_end = (vend + 7) >> 3;  // ends of the virtual groups of 4 and of 8
  auto tile_of = [&](int v) { const int t = v + k_base; return t >= nkt ? t - nkt : t; };
  auto group4_of = [&](int g) { const int t = g + (k_base >> 2); return rotate && t >= (nkt >> 2) ? t - (nkt >> 2) : t; };
  auto group8_of = [&](int h) { const int t = h + (k_base >> 3); return rotate && t >= (nkt >> 3) ? t - (nkt >> 3) : t; };
  constexpr bool a_rowmajor = A_RM, b_rowmajor = B_RM;

  if (wave == kMidCW) {
    // ================= the producer wave: A and its scales =================
    const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc_n(a_base, (int)min((int64_t)m_rows * kp, (int64_t)0x7FFFFFFF));
    // (blocked: `as_base` is the 32-row block that holds the first row, row a_row32 of it)
    const int64_t as_bytes = a_rowmajor ? (int64_t)m_rows * p.ks : (int64_t)((a_row32 + m_rows + 31) >> 5) * k_tiles_blocks;
    const __amdgpu_buffer_rsrc_t as_rsrc = make_rsrc_n(as_base, (int)min(as_bytes, (int64_t)0x7FFFFFFF));
    const int row0 = lane >> 3;  // instruction d fills rows 8d .. 8d + 7
    // chunk position lane % 8 of row r holds chunk (lane % 8) ^ ((r / 2) % 8); 8d is a multiple of 8, so the
    // swizzle depends on the lane alone when d is even, and flips bit 2 of it when d is odd
    const int goff_even = row0 * kp + (((lane & 7) ^ ((row0 >> 1) & 7)) << 4);
    const int goff_odd = row0 * kp + (((lane & 7) ^ (((row0 + 8) >> 1) & 7)) << 4);
    auto issue_a = [&](int v, int slot) {
      // past the last K tile: the same number of requests, from beyond the end of A (zeros into a slot nobody reads)
      const int soff = v < vend ? tile_of(v) * kTileKBytes : (int)0x80000000;
#pragma unroll
      for (int d = 0; d < Cfg::A_LD; ++d)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, WAVE_LDS_PTR(a_ring + slot * Cfg::A_SLOT + d * 1024), 16,
                                                 (d & 1) ? goff_odd : goff_even, soff + d * 8 * kp, 0, 0);
    };
    // scales of K tiles 4g .. 4g + 3, 1 KB per 32 rows, MT_M instructions.  MFMA32 order: the four 256-byte blocks
    // are contiguous (lane * 16).  Row-major: 32 bytes of each row; lane l fetches the half l / 32 of row l % 32
    // and the image is half-major (half * 512 + row * 16).
    const int as_goff = a_rowmajor ? (lane & 31) * p.ks + (lane >> 5) * 16 : lane * 16;
    const int as_gstep = a_rowmajor ? 32 : 1024, as_istep = a_rowmajor ? 32 * p.ks : k_tiles_blocks;
    auto issue_as = [&](int g) {
      const int soff = g < g_end ? group4_of(g) * as_gstep : (int)0x80000000;
#pragma unroll
      for (int i = 0; i < MT_M + (Cfg::A_OFF ? 1 : 0); ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(as_rsrc, WAVE_LDS_PTR(as_ring + (g & (Cfg::AS_SLOTS - 1)) * Cfg::AS_SLOT + i * 1024), 16,
                                                 as_goff, soff + i * as_istep, 0, 0);
    };
    // (a group's last K tiles may lie past K: those bytes belong to the next block or row, or lie past the
    // buffer; nobody reads them)
    // prologue: A(v0 .. v0 + DA - 2), with the scale groups they belong to in front
    for (int g = v0 >> 2; g <= (v0 + DA - 2) >> 2; ++g) issue_as(g);
#pragma unroll
    for (int j = 0; j < DA - 1; ++j) issue_a(v0 + j, j);
    int slot_next = DA - 1;  // slot of the K tile requested next
    for (int j = v0; j < vend; ++j) {
      // A(j) has landed: younger than it are A(j + 1 .. j + DA - 2) and at most one scale group
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0((DA - 2) * Cfg::A_LD < 63 ? (DA - 2) * Cfg::A_LD : 63));
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();  // A(j) visible to the compute waves; they are done with A(j - 1)
      asm volatile("" ::: "memory");
      const int jn = j + DA - 1;
      if ((jn & 3) == 0) issue_as(jn >> 2);  // (its slot's previous group is no longer read: AS_SLOTS)
      issue_a(jn, slot_next);
      slot_next = slot_next + 1 == DA ? 0 : slot_next + 1;
    }
    __builtin_amdgcn_s_barrier();  // (the compute waves' barrier in front of their C staging)
    if constexpr (GATED && Cfg::WM == 1) __builtin_amdgcn_s_barrier();  // (... and the one of their gate / up exchange)
    __builtin_amdgcn_s_waitcnt(0);
    return;
  }

  // ================= a compute wave =================
  // From BM = 64 on the four compute waves sit 2 x 2 on the strip: wave (wm, wn) multiplies every second row block
  // from block wm on and the strip's 32-row groups 2 wn and 2 wn + 1 of B (one A fragment per two MFMAs instead of
  // one per MFMA).  At BM = 32 they sit side by side, wave w on group w.  Either way each wave requests, and
  // waits for, the group `wave` of B and of its scales; the K tile's barrier makes all four groups visible to all.
  constexpr int WM = Cfg::WM, NJ = WM == 2 ? 2 : 1, MI = MT_M / WM;  // row blocks and column groups per wave
  const int wm = WM == 2 ? wave >> 1 : 0, wn = WM == 2 ? wave & 1 : wave;
  uint8_t *const b_ring = smem + Cfg::A_RING + Cfg::AS_RING;  // DB slots of 4 groups x 32 rows x 128 bytes
  uint8_t *const bs_all = b_ring + Cfg::B_RING;               // the four groups' scale images
  uint8_t *const bs_ring = bs_all + wave * Cfg::BS_WAVE;      // ... the one this wave fills
  const int nw0 = n0 + wave * wv;  // the wave's first column of C = first row of B
  const int cols = max(0, min(wv, p.n - nw0));  // columns it owns
  // B: the descriptor starts at the wave's first row (row-major) or at the 16-row block that holds it
  // (preshuffled) and ends with B; rows past N read zeros, like the operand rows past the wave's own columns
  const int b_blk = p.b_preshuffled ? (nw0 & ~15) : nw0, b_sub = nw0 - b_blk;
  const int64_t b_bytes = (int64_t)p.n * kp - (int64_t)b_blk * kp;
  const __amdgpu_buffer_rsrc_t b_rsrc =
      make_rsrc_n(b_base + (int64_t)b_blk * kp, (int)min(max(b_bytes, (int64_t)0), (int64_t)0x7FFFFFFF));
  // B scales: MFMA32 order from the wave's 32-row block on (there WV is 32), row-major from its first row on
  const int64_t bs_skip = b_rowmajor ? (int64_t)nw0 * p.ks : (int64_t)(nw0 >> 5) * k_tiles_blocks;
  const int64_t bs_bytes = (b_rowmajor ? (int64_t)p.n * p.ks : (int64_t)((p.n + 31) >> 5) * k_tiles_blocks) - bs_skip;
  const __amdgpu_buffer_rsrc_t bs_rsrc =
      make_rsrc_n(bs_base + bs_skip, (int)min(max(bs_bytes, (int64_t)0), (int64_t)0x7FFFFFFF));
  // B DMA: instruction d fills rows 8d .. 8d + 7 of the wave's 32 (LDS: row * 128, swizzled chunks)
  const int ld_row = lane >> 3;
  int b_goff[4];
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int r = d * 8 + ld_row, chunk = (lane & 7) ^ ((r >> 1) & 7), rb = r + b_sub;
    const int off = p.b_preshuffled ? (rb >> 4) * 16 * kp + (rb & 15) * 16 + (chunk >> 1) * 512 + (chunk & 1) * 256
                                    : r * kp + chunk * 16;
    b_goff[d] = r < cols ? off : (int)0x80000000;  // past the wave's columns: out of range, zeros, no request
  }
  const int b_kt_stride = p.b_preshuffled ? 2048 : kTileKBytes;
  auto issue_b = [&](int v, int slot) {
    const int soff = v < vend ? tile_of(v) * b_kt_stride : (int)0x80000000;
#pragma unroll
    for (int d = 0; d < 4; ++d)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, WAVE_LDS_PTR(b_ring + slot * 16384 + wave * 4096 + d * 1024), 16,
                                               b_goff[d], soff, 0, kMidOnce);
  };
  // MFMA32 order: the four 256-byte blocks of K tiles 4g .. 4g + 3 are contiguous, one instruction per group.
  auto issue_bs = [&](int g) {
    const int soff = g < g_end ? group4_of(g) * 1024 : (int)0x80000000;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(bs_rsrc, WAVE_LDS_PTR(bs_ring + (g & 3) * 1024), 16, lane * 16, soff, 0, 0);
  };
  // Row-major: 64 bytes of each of the group's rows (8 K tiles), 16 rows per instruction, two instructions per
  // image, the 16-byte pieces swizzled so that the lanes' reads of one piece per row are conflict-free (piece c
  // of row r at position c ^ (r / 4) % 4 of the row's 64 bytes).  Image h holds K tiles 8 h .. 8 h + 7.
  // (Fetched as 32 bytes of each of 32 rows per 4 K tiles, every instruction touched 32 cache lines and every
  // line was requested four times.)
  auto issue_bs8 = [&](int h) {
    const int soff = h < h_end ? group8_of(h) * 64 : (int)0x80000000;
#pragma unroll
    for (int dd = 0; dd < 2; ++dd) {
      const int r = dd * 16 + (lane >> 2);
      const int goff = r * p.ks + (((lane & 3) ^ ((r >> 2) & 3)) << 4);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(bs_rsrc, WAVE_LDS_PTR(bs_ring + (h & 1) * 2048 + dd * 1024), 16, goff, soff, 0,
                                               0);
    }
  };

  const int fr = lane & 31, fg = lane >> 5;
  uint32_t foff[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) foff[t] = (uint32_t)(fr * kTileKBytes + (((t * 2 + fg) ^ ((fr >> 1) & 7)) << 4));
  // A lane's scale dword of a K tile holds the bytes of its K steps 0 .. 3: groups fg, 2 + fg, 4 + fg, 6 + fg of
  // row fr.  MFMA32 order stores exactly that dword.  From a row-major image the lane reads the row's 16-byte
  // piece (K tiles j & ~1 and j | 1; one ds_read_b128 of 32 contiguous pieces - 8-byte reads at a 16-byte pitch
  // are bank conflicts, which made the scale reads 80 % of the kernel's LDS time on top of the fragment reads),
  // takes the half of its K tile and picks its four bytes with one v_perm.
  const uint32_t pick = fg ? 0x07050301u : 0x06040200u;
  auto pick_scales = [&](const v4i q, int j) -> uint32_t {
    const bool odd = (j & 1) != 0;
    return __builtin_amdgcn_perm((uint32_t)(odd ? q.w : q.y), (uint32_t)(odd ? q.z : q.x), pick);
  };
  // A lane's dword of a K tile's 256-byte block in e8m0_shuffle order
  // (wave_lang/kernel/wave/utils/mxfp_utils.py:113-128): group k of row r sits at byte
  // (k % 4) * 64 + (r % 16) * 4 + (k % 8) / 4 * 2 + r / 16 of the block.  The lane's K steps s = 0 .. 3 want groups
  // 2 s + fg: steps 0 and 2 are bytes r / 16 and 2 + r / 16 of the dword at fg * 64 + (r % 16) * 4, steps 1 and 3
  // the same bytes of the dword 128 bytes further on.
  auto shuffled_scales = [&](const uint8_t *blk) -> uint32_t {
    const uint32_t d0 = *(const uint32_t *)(blk + fg * 64 + (fr & 15) * 4);
    const uint32_t d1 = *(const uint32_t *)(blk + 128 + fg * 64 + (fr & 15) * 4);
    return __builtin_amdgcn_perm(d1, d0, 0x06020400u + (uint32_t)(fr >> 4) * 0x01010101u);
  };
  // MFMA32 order, a block of rows that starts at row a_row32 of a 32-row scale block: the lane's row fr of row block
  // i is row (a_row32 + fr) % 32 of image i + (a_row32 + fr) / 32
  const int a_lane_off = Cfg::A_OFF ? ((a_row32 + fr) >> 5) * 1024 + ((fg << 5) | ((a_row32 + fr) & 31)) * 4 : lane * 4;
  auto lane_scales = [&](const uint8_t *img, auto rm_tag, int j) -> uint32_t {
    if constexpr (decltype(rm_tag)::value) {
      return pick_scales(*(const v4i *)(img + ((j & 2) << 8) + fr * 16), j);
    } else if constexpr (A_SH) {
      return shuffled_scales(img + (j & 3) * 256);
    } else {
      return *(const uint32_t *)(img + (j & 3) * 256 + a_lane_off);
    }
  };
  // B, row-major: the piece (j / 2) % 4 of row fr in the swizzled 32 x 64-byte image of the K tile's group of 8
  auto lane_scales_b = [&](int g, int j) -> uint32_t {  // g: the 32-row group of the strip
    const uint8_t *img = bs_all + g * Cfg::BS_WAVE;
    if constexpr (B_RM) {
      const int c = (j >> 1) & 3;
      return pick_scales(*(const v4i *)(img + ((j >> 3) & 1) * 2048 + fr * 64 + ((c ^ ((fr >> 2) & 3)) << 4)), j);
    } else {
      const uint8_t *blk = img + ((j >> 2) & 3) * 1024 + (j & 3) * 256;  // the K tile's block
      if constexpr (B_SH) {
        static_assert(!Cfg::B_RM, "blocked layouts");
        return shuffled_scales(blk);
      } else {
        return *(const uint32_t *)(blk + lane * 4);
      }
    }
  };

  v16f acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int jn = 0; jn < NJ; ++jn)
#pragma unroll
      for (int g = 0; g < 16; ++g) acc[i][jn][g] = 0.f;

  // prologue: B(v0 .. v0 + LB - 1) with the scale groups they belong to in front (row-major: the second image
  // too when the walk starts inside the first, because the K loop requests an image at the start of the one before)
  if constexpr (B_RM) {
    issue_bs8(0);
    if (v0 != 0) issue_bs8(1);
  }
#pragma unroll
  for (int j = 0; j < LB; ++j) {
    if (!B_RM && (j == 0 || ((v0 + j) & 3) == 0)) issue_bs((v0 + j) >> 2);
    issue_b(v0 + j, j);
  }
  int slot = 0, slot_next = LB;  // slots of B(j) and of the K tile requested next
  int a_slot = 0;
  typedef std::integral_constant<int, 0> T0;
  typedef std::integral_constant<int, 1> T1;
  typedef std::integral_constant<int, 2> T2;
  typedef std::integral_constant<int, 3> T3;
  // Row block i of this wave is block WM i + wm of the tile, so that a block of fewer rows than BM (a small group
  // of a grouped problem) leaves both halves of the workgroup the same share; the blocks past the rows take no
  // fragment reads and no MFMAs: the K loop exists once per count of live blocks, with no branch inside it.
  const int live = min(max((m_rows - 32 * wm + 32 * WM - 1) / (32 * WM), 0), MI);
  auto k_loop = [&](auto live_tag) {
  constexpr int LIVE = decltype(live_tag)::value;
  for (int j = v0; j < vend; ++j) {
    // B(j) and its scales have landed: younger are B(j + 1 .. j + LB - 1), 4 requests each (and up to two scale
    // groups, which the count leaves out: it then waits for that much more than it must)
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(4 * (LB - 1)));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();  // A(j) is in LDS
    asm volatile("" ::: "memory");
    // the slot of B(j - 1) is free (its fragments were consumed before the wait above): request B(j + LB)
    const int jn = j + LB;
    if constexpr (B_RM) {
      // the image of the next 8 K tiles: its buffer held the previous image, last read in K tile j - 1, and the
      // requests are older than those K tiles' B
      if ((j & 7) == 0) issue_bs8((j >> 3) + 1);
    } else {
      if ((jn & 3) == 0) issue_bs(jn >> 2);
    }
    issue_b(jn, slot_next);
    slot_next = slot_next + 1 == DB ? 0 : slot_next + 1;

    const uint8_t *a_t = a_ring + a_slot * Cfg::A_SLOT + wm * 32 * kTileKBytes;
    const uint8_t *b_t = b_ring + slot * 16384 + wn * NJ * 4096;
    uint32_t sa[MI], sb[NJ];
#pragma unroll
    for (int i = 0; i < LIVE; ++i)
      sa[i] = lane_scales(as_ring + ((j >> 2) & (Cfg::AS_SLOTS - 1)) * Cfg::AS_SLOT + (WM * i + wm) * 1024, std::integral_constant<bool, A_RM>{}, j);
#pragma unroll
    for (int jn = 0; jn < NJ; ++jn) sb[jn] = lane_scales_b(wn * NJ + jn, j);
    auto step = [&](auto t_tag) {
      constexpr int T = decltype(t_tag)::value;
      v8i vb[NJ];
#pragma unroll
      for (int jn = 0; jn < NJ; ++jn) {
        const v4i fb = *(const v4i *)(b_t + jn * 4096 + foff[T]);
        vb[jn] = v8i{fb.x, fb.y, fb.z, fb.w, 0, 0, 0, 0};
      }
#pragma unroll
      for (int i = 0; i < LIVE; ++i) {
        const v4i fa = *(const v4i *)(a_t + i * WM * 32 * kTileKBytes + foff[T]);
        const v8i va = {fa.x, fa.y, fa.z, fa.w, 0, 0, 0, 0};
#pragma unroll
        for (int jn = 0; jn < NJ; ++jn)
          acc[i][jn] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vb[jn], va, acc[i][jn], 4, 4, T, (int)sb[jn], T,
                                                                       (int)sa[i]);
      }
    };
    step(T0{});
    step(T1{});
    step(T2{});
    step(T3{});
    slot = slot + 1 == DB ? 0 : slot + 1;
    a_slot = a_slot + 1 == DA ? 0 : a_slot + 1;
  }
  };
  auto with_live = [&](auto self, auto tag) -> void {
    constexpr int L = decltype(tag)::value;
    if constexpr (L == 0) {
      k_loop(tag);
    } else {
      if (live >= L)
        k_loop(tag);
      else
        self(self, std::integral_constant<int, L - 1>{});
    }
  };
  with_live(with_live, std::integral_constant<int, MI>{});
  // the trailing (empty) requests must have landed, and every wave must be done reading the last K tile, before
  // the ring becomes the C staging area
  __builtin_amdgcn_s_waitcnt(0);
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");

  if constexpr (GATED) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const int qrow = p.n >> 2;    // bytes of a row of codes
    const int act_ks = p.n >> 6;  // scale groups of a row of the activation
    const int s_kt = (act_ks + 7) >> 3;
    const __amdgpu_buffer_rsrc_t q_rsrc = make_rsrc_n(c_base, (int)min((int64_t)m_rows * qrow, (int64_t)0x7FFFFFFF));
    const __amdgpu_buffer_rsrc_t s_rsrc = make_rsrc_n(p.epi_scale, rsrc_bytes((int64_t)((p.m + 31) >> 5) * s_kt * 256));
    // the wave's 16 values of a row as 8 bf16 pairs: what the unfused GEMM would have stored
    auto pack_bf16 = [](const v16f &a, uint32_t (&out)[8]) {
#pragma unroll
      for (int w = 0; w < 8; ++w) {
        const bf16x2 h = {(__bf16)a[2 * w], (__bf16)a[2 * w + 1]};
        out[w] = __builtin_bit_cast(uint32_t, h);
      }
    };
    // silu(gate) * up of one row block and activation scale group `g`, quantised: the activation kernel's arithmetic
    auto emit = [&](int r_tile, int g, const uint32_t (&gb)[8], const uint32_t (&ub)[8]) {
      uint32_t h[8];
      uint32_t lo = 0, hi = 0;
#pragma unroll
      for (int w = 0; w < 8; ++w) {
        const float g0 = __builtin_bit_cast(float, gb[w] << 16), g1 = __builtin_bit_cast(float, gb[w] & 0xFFFF0000u);
        const float u0 = __builtin_bit_cast(float, ub[w] << 16), u1 = __builtin_bit_cast(float, ub[w] & 0xFFFF0000u);
        const float r0 = g0 * u0 * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g0 * -1.44269504088896340736f));
        const float r1 = g1 * u1 * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g1 * -1.44269504088896340736f));
        const bf16x2 o = {(__bf16)r0, (__bf16)r1};
        h[w] = __builtin_bit_cast(uint32_t, o);
        lo = max(lo, h[w] & 0x7FFFu);
        hi = max(hi, (h[w] >> 16) & 0x7FFFu);
      }
      // the group's largest magnitude: this lane's 16 columns and the other lane's
      const uint32_t mine = max(lo, hi);
      const auto both = __builtin_amdgcn_permlane32_swap(mine, mine, false, false);
      const uint32_t amax = max(both[0], both[1]) << 16;
      const uint32_t e = (amax + 0x200000u) >> 23;
      const uint32_t sb = e >= 255u ? 254u : (e > 2u ? e - 2u : 0u);
      const float sf = __builtin_bit_cast(float, sb ? sb << 23 : 0x00400000u);
      uint32_t c0 = 0, c1 = 0;
      c0 = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(c0, __builtin_bit_cast(bf16x2, h[0]), sf, 0);
      c0 = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(c0, __builtin_bit_cast(bf16x2, h[1]), sf, 1);
      c0 = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(c0, __builtin_bit_cast(bf16x2, h[2]), sf, 2);
      c0 = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(c0, __builtin_bit_cast(bf16x2, h[3]), sf, 3);
      c1 = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(c1, __builtin_bit_cast(bf16x2, h[4]), sf, 0);
      c1 = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(c1, __builtin_bit_cast(bf16x2, h[5]), sf, 1);
      c1 = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(c1, __builtin_bit_cast(bf16x2, h[6]), sf, 2);
      c1 = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(c1, __builtin_bit_cast(bf16x2, h[7]), sf, 3);
      // lanes 0..31 get the upper lanes' dword 0, lanes 32..63 the lower lanes' dword 1: each lane then holds
      // 8 consecutive bytes of its row's 16 (the lower lanes bytes 0..7, the upper lanes bytes 8..15)
      const auto sw = __builtin_amdgcn_permlane32_swap(c0, c1, false, false);
      v2i out;
      out.x = (int)__builtin_amdgcn_perm(sw[1], sw[0], 0x05040100u);
      out.y = (int)__builtin_amdgcn_perm(sw[1], sw[0], 0x07060302u);
      // (rows past the block's own lie past the end of the descriptor: dropped)
      __builtin_amdgcn_raw_buffer_store_b64(out, q_rsrc, r_tile * qrow + g * 16 + fg * 8, 0, 0);
      const int r_abs = m_abs0 + r_tile;
      const int s_off = ((r_abs >> 5) * s_kt + (g >> 3)) * 256 + (((g & 1) << 5) | (r_abs & 31)) * 4 + ((g & 7) >> 1);
      __builtin_amdgcn_raw_buffer_store_b8((uint8_t)sb, s_rsrc, fg == 0 && r_tile < m_rows ? s_off : (int)0x80000000, 0, 0);
    };
    if constexpr (WM == 2) {
      // the wave's column groups 2 wn and 2 wn + 1 are gate and up of the activation's group (n0 / 64) + wn
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        if (i >= live) break;
        uint32_t gb[8], ub[8];
        pack_bf16(acc[i][0], gb);
        pack_bf16(acc[i][1], ub);
        emit((WM * i + wm) * 32 + fr, (n0 >> 6) + wn, gb, ub);
      }
    } else {
      // one row block, the waves side by side: wave 2q holds the gate, wave 2q + 1 the up values of the
      // activation's group (n0 / 64) + q, element for element in the same lane and register.  The up waves hand
      // theirs over through the ring (free since the barrier above): 8 dwords per lane, lane-contiguous.
      uint8_t *xch = b_ring + (wave >> 1) * 2048 + lane * 4;
      uint32_t gb[8], ub[8];
      pack_bf16(acc[0][0], gb);
      if (wave & 1) {
#pragma unroll
        for (int w = 0; w < 8; ++w) *(uint32_t *)(xch + w * 256) = gb[w];
      }
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(63));
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      if (!(wave & 1)) {
#pragma unroll
        for (int w = 0; w < 8; ++w) ub[w] = *(const uint32_t *)(xch + w * 256);
        emit(fr, (n0 >> 6) + (wave >> 1), gb, ub);
      }
    }
    return;
  }
  // ---------------- C: accumulators -> the wave's ring -> global ----------------
  // acc[i][jn][4q + e] is row lane % 32, column 8q + 4 * (lane / 32) + e of the 32 x 32 tile (row block
  // WM i + wm, group NJ wn + jn).  A tile is staged as 32 rows of eight 4-column pieces and stored 8 rows per
  // instruction, a lane one piece (8 bytes of bf16, 16 of f32), the pieces past the group's columns left out.
  uint8_t *stage = b_ring + wave * 4096;
  const bool out_bf16 = p.out_bf16 != 0;
  const int elt = out_bf16 ? 2 : 4;
  const __amdgpu_buffer_rsrc_t c_rsrc =
      make_rsrc_n(c_base, (int)min((int64_t)m_rows * p.n * elt, (int64_t)0x7FFFFFFF));
  const int lr = lane >> 3, lc = lane & 7;
#pragma unroll
  for (int jn = 0; jn < NJ; ++jn) {
    const int gc0 = n0 + (wn * NJ + jn) * wv;                // the group's first column of C
    const bool mine = lc * 4 < min(wv, p.n - gc0);          // (negative past N: nothing stored)
    if (out_bf16) {
      typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        if (i >= live) break;
        const v16f &a = acc[i][jn];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const bf4 h = {(__bf16)a[4 * q], (__bf16)a[4 * q + 1], (__bf16)a[4 * q + 2], (__bf16)a[4 * q + 3]};
          *(bf4 *)(stage + fr * 64 + (((q * 2 + fg) ^ ((fr >> 2) & 7)) << 3)) = h;
        }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int r0 = 0; r0 < 32; r0 += 8) {
          const int r = r0 + lr, row = (WM * i + wm) * 32 + r;
          const v2i v = *(const v2i *)(stage + r * 64 + ((lc ^ ((r >> 2) & 7)) << 3));
          // rows past M lie past the end of C: dropped by the descriptor
          if (mine) __builtin_amdgcn_raw_buffer_store_b64(v, c_rsrc, (int)(((int64_t)row * p.n + gc0 + lc * 4) * 2), 0, 0);
        }
        asm volatile("" ::: "memory");
      }
    } else {
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        if (i >= live) break;
        const v16f &a = acc[i][jn];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const v4f v = {a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]};
          const int chunk = q * 2 + fg;
          *(v4f *)(stage + fr * 128 + ((chunk ^ (fr & 7)) << 4)) = v;
        }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int r0 = 0; r0 < 32; r0 += 8) {
          const int r = r0 + lr, row = (WM * i + wm) * 32 + r;
          const v4f v = *(const v4f *)(stage + r * 128 + ((lc ^ (r & 7)) << 4));
          if (mine)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, v), c_rsrc,
                                                   (int)(((int64_t)row * p.n + gc0 + lc * 4) * 4), 0, 0);
        }
        asm volatile("" ::: "memory");
      }
    }
  }
}

// GROUPED: blockIdx.y is the expert; its rows offsets[e] .. offsets[e + 1] (clamped to [0, M], not validated) are
// taken BM at a time - a group of more rows than BM streams its expert's B once per block of rows, which is what
// the table-driven persistent kernel is for; this one is for the few rows per expert of a small batch.
template <class Cfg, bool A_RM, bool GROUPED, bool B_SH, bool A_SH, bool GATED = false>
__global__ void __launch_bounds__(kMidNT, 1) mid_gemm_kernel(const GemmParams p, const int wv) {
  static_assert(!(A_RM && A_SH), "one layout");
  if constexpr (!GROUPED) {
    mid_body<Cfg, A_RM, B_SH, A_SH, GATED>(p, wv, p.a, p.a_scale, p.b, p.b_scale, (uint8_t *)p.c, p.m);
  } else {
    static_assert(A_RM || (Cfg::A_OFF && !A_SH), "a group may start at any row: A's scales row-major, or MFMA32 with room for the block it starts in");
    const int e = blockIdx.y;
    const int lo = __builtin_amdgcn_readfirstlane(min(max(p.offsets[e], 0), p.m));
    const int hi = __builtin_amdgcn_readfirstlane(min(max(p.offsets[e + 1], lo), p.m));
    const uint8_t *b = p.b + (int64_t)e * p.b_group_stride, *bs = p.b_scale + (int64_t)e * p.b_scale_group_stride;
    const int64_t c_row = GATED ? p.n >> 2 : (int64_t)p.n * (p.out_bf16 ? 2 : 4);  // bytes of a row of what is written
    for (int m0 = lo; m0 < hi; m0 += Cfg::BM) {
      const uint8_t *as = A_RM ? p.a_scale + (int64_t)m0 * p.ks : p.a_scale + (int64_t)(m0 >> 5) * p.k_tiles * 256;
      mid_body<Cfg, A_RM, B_SH, A_SH, GATED>(p, wv, p.a + (int64_t)m0 * p.kp, as, b, bs,
                          (uint8_t *)p.c + (int64_t)m0 * c_row, min(Cfg::BM, hi - m0), A_RM ? 0 : m0 & 31, m0);
      // every wave is done with the rings (the C staging's reads included) before the next block's requests
      __builtin_amdgcn_s_waitcnt(0);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
    }
  }
}

template <class Cfg, bool A_RM, bool GROUPED, bool B_SH, bool A_SH = false, bool GATED = false>
hipError_t launch_mid_kernel(const GemmParams &p, int wv, hipStream_t stream) {
  static LdsAttrOnce once;
  hipError_t e = allow_dynamic_lds(once, (const void *)mid_gemm_kernel<Cfg, A_RM, GROUPED, B_SH, A_SH, GATED>, Cfg::LDS);
  if (e != hipSuccess) return e;
  const int bn = kMidCW * wv;
  const dim3 grid((p.n + bn - 1) / bn, GROUPED ? p.num_groups : 1, 1);
  mid_gemm_kernel<Cfg, A_RM, GROUPED, B_SH, A_SH, GATED><<<grid, dim3(kMidNT), Cfg::LDS, stream>>>(p, wv);
  return hipGetLastError();
}

template <class Cfg, bool A_RM, bool GROUPED>
hipError_t launch_mid_layouts(const GemmParams &p, int wv, hipStream_t stream) {
  const bool b_sh = p.b_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE;
  if constexpr (!A_RM && !GROUPED) {
    if (p.a_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE) {
      if constexpr (!Cfg::B_RM) {
        if (b_sh) return launch_mid_kernel<Cfg, false, false, true, true>(p, wv, stream);
      }
      return launch_mid_kernel<Cfg, false, false, false, true>(p, wv, stream);
    }
  }
  if constexpr (!Cfg::B_RM) {
    if (b_sh) return launch_mid_kernel<Cfg, A_RM, GROUPED, true>(p, wv, stream);
  }
  return launch_mid_kernel<Cfg, A_RM, GROUPED, false>(p, wv, stream);
}

template <int BM, bool TWO = false>
hipError_t launch_mid_cfg(const GemmParams &p, int wv, hipStream_t stream) {
  const bool a_rm = p.a_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR, b_rm = p.b_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR;
  if (p.num_groups != 0) {  // (A's scales row-major or MFMA32: checked by mid_grouped_applies)
    if constexpr (BM <= 192) {
      if (!a_rm)
        return b_rm ? launch_mid_layouts<MidCfg<BM, true, TWO, true>, false, true>(p, wv, stream)
                    : launch_mid_layouts<MidCfg<BM, false, TWO, true>, false, true>(p, wv, stream);
    }
    return b_rm ? launch_mid_layouts<MidCfg<BM, true, TWO>, true, true>(p, wv, stream)
                : launch_mid_layouts<MidCfg<BM, false, TWO>, true, true>(p, wv, stream);
  }
  if (a_rm)
    return b_rm ? launch_mid_layouts<MidCfg<BM, true, TWO>, true, false>(p, wv, stream)
                : launch_mid_layouts<MidCfg<BM, false, TWO>, true, false>(p, wv, stream);
  return b_rm ? launch_mid_layouts<MidCfg<BM, true, TWO>, false, false>(p, wv, stream)
              : launch_mid_layouts<MidCfg<BM, false, TWO>, false, false>(p, wv, stream);
}

// Columns per compute wave: the narrowest strips (a multiple of 4 columns, 16 to 32) that still fit the number of
// rounds which strips of 128 columns would take on this many CUs.  B scales in MFMA32 order come in blocks of 32
// rows, so there a wave's strip is a block.  From 97 rows on a workgroup's time is mostly its copy of A (every
// workgroup reads all of it), so fewer, wider strips win even where they leave CUs idle (128 x 28672 x 8192 with
// row-major scales: 31.4 -> 29.8 us, 192 rows 39.9 -> 38.3 us; at 96 rows the narrow strips are still as good).
int mid_wave_cols(const GemmParams &p, int num_cus) {
  if (p.b_scale_layout != WAVE_MXFP4_SCALE_ROW_MAJOR || num_cus <= 0) return 32;
  if (p.num_groups == 0 && p.m > 96) return 32;
  const int64_t experts = p.num_groups != 0 ? p.num_groups : 1;
  const int64_t strips = (p.n + kMidBN - 1) / kMidBN * experts;
  const int64_t wgs = (strips + num_cus - 1) / num_cus * num_cus;   // whole rounds of the CUs
  const int64_t per_expert = wgs / experts > 0 ? wgs / experts : 1;  // strips of one expert
  int64_t wv = (p.n + 4 * per_expert - 1) / (4 * per_expert);
  wv = (wv + 3) / 4 * 4;
  return (int)(wv < 16 ? 16 : wv > 32 ? 32 : wv);
}

}  // namespace

int mid_max_m() { return 256; }

// Whether the mid-M kernel serves this problem.
bool mid_gemm_applies(const GemmParams &p) {
  if (p.num_groups != 0 || p.splits != 1 || p.partial != nullptr || p.m < 1 || p.m > mid_max_m()) return false;
  // (row-major, MFMA32, or e8m0_shuffle order, the reference's format for preshuffled scales)
  const auto layout_ok = [](int l) {
    return l == WAVE_MXFP4_SCALE_ROW_MAJOR || l == WAVE_MXFP4_SCALE_MFMA32 || l == WAVE_MXFP4_SCALE_E8M0_SHUFFLE;
  };
  if (!layout_ok(p.a_scale_layout) || !layout_ok(p.b_scale_layout)) return false;
  // A partial last K tile: both scale tensors in MFMA32 order.  Their padding groups hold 0 (2^-127 each), so the
  // products of whatever the last K tile's requests bring in from past the end of K - the start of the next row, or
  // the zeros the buffer descriptor returns past the last one - vanish in the f32 accumulators; the kernel walks
  // ceil(K / 256) K tiles and knows nothing of it.
  if ((p.k & (kTileK - 1)) != 0 &&
      (p.a_scale_layout != WAVE_MXFP4_SCALE_MFMA32 || p.b_scale_layout != WAVE_MXFP4_SCALE_MFMA32))
    return false;
  if ((p.k & 31) != 0 || p.k_tiles < 4 || (p.n & 3) != 0) return false;
  // 32-bit offsets: inside A, inside a wave's 48 rows of B, inside C, inside the scales of A and of a wave's rows
  if ((int64_t)p.m * p.kp >= ((int64_t)1 << 31) || (int64_t)48 * p.kp >= ((int64_t)1 << 31) ||
      (int64_t)p.m * p.n * 4 >= ((int64_t)1 << 31) || (int64_t)8 * p.k_tiles * 256 >= ((int64_t)1 << 31))
    return false;
  return true;
}

// Whether the mid-M kernel serves this grouped problem: row-major A scales (a group starts at any row), each
// expert's B scales row-major or MFMA32, whole K tiles.  Any group sizes are computed correctly; it pays for few rows
// per expert.
bool mid_grouped_applies(const GemmParams &p) {
  if (p.num_groups <= 0 || p.num_groups > 65535 || p.offsets == nullptr || p.splits != 1 || p.partial != nullptr) return false;
  if (p.a_scale_layout != WAVE_MXFP4_SCALE_ROW_MAJOR && p.a_scale_layout != WAVE_MXFP4_SCALE_MFMA32) return false;
  if (p.b_scale_layout != WAVE_MXFP4_SCALE_ROW_MAJOR && p.b_scale_layout != WAVE_MXFP4_SCALE_MFMA32 &&
      p.b_scale_layout != WAVE_MXFP4_SCALE_E8M0_SHUFFLE)
    return false;
  // (a partial last K tile: both scale tensors in MFMA32 order, as for the dense problem)
  if ((p.k & (kTileK - 1)) != 0 &&
      (p.a_scale_layout != WAVE_MXFP4_SCALE_MFMA32 || p.b_scale_layout != WAVE_MXFP4_SCALE_MFMA32))
    return false;
  if ((p.k & 31) != 0 || p.k_tiles < 4 || (p.n & 3) != 0) return false;
  if ((int64_t)256 * p.kp >= ((int64_t)1 << 31) || (int64_t)48 * p.kp >= ((int64_t)1 << 31) ||
      (int64_t)256 * p.n * 4 >= ((int64_t)1 << 31) || (int64_t)8 * p.k_tiles * 256 >= ((int64_t)1 << 31))
    return false;
  return true;
}

// `bm`: rows per block of a group (dense: M; grouped: the library's guess from the average group, a group of more
// rows takes several blocks).
hipError_t launch_mid_gemm(const GemmParams &p, int num_cus, hipStream_t stream, int bm) {
  if (bm <= 0) bm = p.m;
  // (a group's block with A scales in MFMA32 order holds one scale block more: no room for it beside 256 rows)
  if (p.num_groups != 0 && p.a_scale_layout != WAVE_MXFP4_SCALE_ROW_MAJOR && bm > 192) bm = 192;
  // more strips than CUs at the 32-row block: two workgroups per CU
  const int64_t strips = (int64_t)((p.n + kMidBN - 1) / kMidBN) * (p.num_groups != 0 ? p.num_groups : 1);
  const bool two = bm <= 32 && strips > num_cus;
  const int wv = mid_wave_cols(p, two ? 2 * num_cus : num_cus);
  if (two) return launch_mid_cfg<32, true>(p, wv, stream);
  if (bm <= 32) return launch_mid_cfg<32>(p, wv, stream);
  if (bm <= 64) return launch_mid_cfg<64>(p, wv, stream);
  if (bm <= 128) return launch_mid_cfg<128>(p, wv, stream);
  if (bm <= 192) return launch_mid_cfg<192>(p, wv, stream);
  return launch_mid_cfg<256>(p, wv, stream);
}

// The gated, quantising form (grouped): blocks of 32 (the up waves hand their values to the gate waves through LDS),
// 64, 128 or 192 rows (a wave holds both column groups of a pair), the experts' B scales in MFMA32 order, whole
// 128-column strips of gate / up pairs.
bool mid_gated_applies(const GemmParams &p) {
  return mid_grouped_applies(p) && p.epi_scale != nullptr && p.epi_scale_layout == WAVE_MXFP4_SCALE_MFMA32 &&
         p.b_scale_layout == WAVE_MXFP4_SCALE_MFMA32 && !p.b_preshuffled && p.out_bf16 && (p.n & 127) == 0 &&
         (int64_t)p.m * (p.n >> 2) < ((int64_t)1 << 31);
}

template <int BM, bool TWO = false>
static hipError_t launch_mid_gated_bm(const GemmParams &p, hipStream_t stream) {
  if (p.a_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR)
    return launch_mid_kernel<MidCfg<BM, false, TWO, false>, true, true, false, false, true>(p, 32, stream);
  return launch_mid_kernel<MidCfg<BM, false, TWO, true>, false, true, false, false, true>(p, 32, stream);
}

hipError_t launch_mid_gated(const GemmParams &p, int num_cus, hipStream_t stream, int bm) {
  // (the 32-row block: two workgroups per CU when there are more strips than CUs, as in launch_mid_gemm)
  if (bm <= 32)
    return (int64_t)(p.n / kMidBN) * p.num_groups > num_cus ? launch_mid_gated_bm<32, true>(p, stream)
                                                           : launch_mid_gated_bm<32>(p, stream);
  if (bm <= 64) return launch_mid_gated_bm<64>(p, stream);
  if (bm <= 128) return launch_mid_gated_bm<128>(p, stream);
  return launch_mid_gated_bm<192>(p, stream);
}

}  // namespace wave_mxfp4

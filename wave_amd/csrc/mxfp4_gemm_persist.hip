// Persistent tiled MXFP4 GEMM for gfx950 (MI355X): the large-shape fast path.
//
// Same tile machinery as the one-tile-per-workgroup kernel (256x256x256 tile,
// v_mfma_scale_f32_32x32x64_f8f6f4, five-slot LDS ring filled by 16-byte DMA,
// scales in the MFMA-native order), but one workgroup per CU walks a sequence
// of output tiles, and the operand stream does not stop at a tile boundary:
// while the last two K tiles of a tile are multiplied, the first two K tiles
// of the NEXT tile are already being fetched, so a new tile starts without the
// 3-4 us it otherwise takes to launch a workgroup and fill the ring.  The C
// tile is written from a single free ring slot (32 KB for the workgroup,
// passes of 32 rows through LDS so that every store instruction writes whole
// lines), and those stores are left in flight under the MFMAs of the next
// tile.  Vector memory operations retire in issue order (loads and stores
// share vmcnt), so the first wait of the new tile allows for the stores
// behind the loads it needs; from the second K tile on the stores must have
// drained, which by then they have had a whole K tile of time to do.
//
// Taken for N % 256 == 0, K >= 768 (K % 256 != 0 with a partial last K tile from
// K = 1024 on; any M: the last tile row reads
// and writes through descriptors that end with the tensors), MFMA-native
// scales for both operands, no split; grouped (MoE) problems by way of a table
// of M tiles.  Everything else runs the
// one-tile-per-workgroup kernel.  The reference writes one tile per workgroup
// (wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:38-145); the result
// contract is the same.
#include <type_traits>

#include "mxfp4_group_table.h"
#include "mxfp4_tile_common.h"

namespace wave_mxfp4 {

// Into how many parts along K the tiles of a sparsely filled last round are cut (1 = left whole): `rest` tile ids
// in that round on `grid` workgroups, tiles of `k_tiles` K tiles.  Cost of the last round in us: a tile's K tiles
// at the measured 1.85 us each, divided among the parts, plus writing and re-reading the f32 parts (about 4 TB/s)
// and the launch of the kernel that sums them.  Host code for dense problems; a grouped problem's tile count is
// only known on the device, where the GEMM and the summing kernel both evaluate this.
__host__ __device__ inline int tail_parts_rule(int rest, int grid, int k_tiles) {
  if (rest <= 0 || rest * 2 > grid) return 1;
  // (whole nanoseconds: the GEMM and the summing kernel must come to the same answer, which floating point
  // contracted differently in two places would not promise)
  const int tile_ns = 1850 * k_tiles;
  int parts = 1, best = tile_ns;
  for (int c = 2; c <= 8 && c * rest <= grid && k_tiles / c >= 4; ++c) {
    const int ns = tile_ns / c + 2 * rest * c * (256 * 256 * 4 / 4000) + 6000;
    if (ns * 10 < best * 9) best = ns, parts = c;
  }
  return parts;
}

// Tile id -> (M tile, N tile) of a grouped problem: the same XCD regrouping as map_tile, but the bands the sequence
// walks column by column are the table's (at most 8 tiles of one expert), not fixed runs of 8 tile rows.
// (the full tiles first, then the table's short tiles: grouped_tile_of_id)
__device__ __forceinline__ bool map_grouped_tile(const int32_t *table, int tiles, int full, int tiles_n, int id, int &tm, int &tn) {
  return grouped_tile_of_id(tiles, full, tiles_n, id,
                            [table](int t) { return __builtin_amdgcn_readfirstlane(table[4 * (1 + t) + 3]); }, tm, tn);
}

enum KtKind {
  kSteadyTail = 4,  // kSteady whose K tile j+2 is a partial last K tile (TAIL kernels: j = nkt - 3)
  kSteady = 0,  // K tiles j+1, j+2 belong to this output tile
  kFirst = 1,   // first K tile of an output tile (B(1) was fetched whole ahead of it)
  kBound1 = 2,  // K tile j+2 is K tile 0 of the next output tile
  kBound2 = 3   // K tiles j+1, j+2 are K tiles 0, 1 of the next output tile
};

// OUT_BF16 is a template parameter so that the C stores are straight-line code:
// behind a run-time branch the compiler's wait insertion has to assume the
// store-free path and waits for the stores long before it must.
// GROUPED: the M tiles come from a table (first row, rows, expert) built on the
// device from the group offsets; a tile's rows past its group are computed and
// dropped like rows past M.  A tile starts at any row, so a lane finds its row's
// scales in block (first % 32 + row in tile) / 32 from the tile's first block, at
// lane (first % 32 + row) % 32 of it: one dword per lane as before, from two
// neighbouring blocks per wave instruction instead of one.
// TAIL: K % 256 != 0.  The lanes whose 16-byte chunk lies past the end of K fetch
// the last K tile from beyond the buffer descriptor (zeros land in LDS): their
// offset gets its top bit flipped just before that tile's DMA is issued and
// flipped back after it, at fixed places of two peeled K tiles, so the steady
// loop and the instruction counts the waits rely on are untouched.
// SPLIT: the tiles of the last round, which only part of the workgroups would
// get one of, are cut along K into p.tail_parts parts instead, one part per
// workgroup (its last item); the parts go to p.tail_partial as f32 tiles and a
// small kernel adds them up.  A 288-tile problem on 256 CUs then takes 1 + 1/8
// tile times instead of 2.  For a grouped problem the number of parts is worked
// out on the device (tail_parts_rule on the table's tile count), by this kernel
// and by the one that sums, and may come out as 1: then the tiles stay whole.
// FMT_A / FMT_B: element format codes of the scaled MFMA, 4 = e2m1 (MXFP4); 0 = e4m3, 1 = e5m2 (MXFP8, both
// operands 8-bit: a 128-byte K tile is then 128 elements = two 64-deep K steps of 32 bytes per lane, the MFMA
// takes 64 cycles instead of 32, and one MFMA32 scale block serves two K tiles; dense, whole K tiles, no cut).
// SHUF: both scale tensors in e8m0_shuffle order (the reference's preshuffled format,
// wave_lang/kernel/wave/utils/mxfp_utils.py:113-128), read in place.  It keeps the same 256-byte blocks per 32 rows
// and K tile in the same order as MFMA32; inside a block the four bytes of a lane (row r, K half h: groups 2t + h of
// the K steps t = 0..3) sit in two dwords, (16h + r % 16) for t = 0, 2 and 32 further on for t = 1, 3, at bytes
// (r % 32) / 16 and 2 + (r % 32) / 16: two loads and one v_perm where MFMA32 takes one load and a move.
// GATED: the step behind the first GEMM of a gated MLP, fused into the C write.  B holds the gate and up projections
// interleaved in blocks of 32 rows (rows 64 b .. 64 b + 31: gate rows 32 b .., rows 64 b + 32 .. 64 b + 63: up rows
// 32 b ..), so that a wave's accumulator tiles (i, 2 jp) and (i, 2 jp + 1) hold gate and up of the same 32 rows x 32
// columns of the activation, element for element in the same lane.  The kernel writes, instead of C [M, N], the
// MXFP4 quantisation of silu(gate) * up [M, N / 2]: packed e2m1 to p.c ([M, N / 4] bytes) and one e8m0 scale per
// row and 32 columns to p.epi_scale (MFMA32 order, what the next GEMM reads).  Arithmetic as in the unfused pair of kernels, bit for
// bit: gate and up rounded to bf16 (the GEMM's output there), silu(g) * u in f32 with the hardware exp2 and
// reciprocal, rounded to bf16, then the quantiser's scale rule and conversion (mxfp4_quant.hip).  A row's 32
// columns sit in two lanes (l and l + 32), which exchange their maxima and halves of their codes with
// v_permlane32_swap.
template <class Cfg, bool OUT_BF16, bool GROUPED, bool TAIL, bool SPLIT, int FMT_A = 4, int FMT_B = 4, bool SHUF = false,
          bool GATED = false>
__device__ __forceinline__ void persist_body(const GemmParams &p) {
  constexpr bool FP8 = FMT_A != 4 || FMT_B != 4;
  static_assert(!GATED || (!FP8 && !TAIL && !SPLIT && OUT_BF16 && Cfg::NWAVES == 8 && Cfg::BN == 256),
                "gated epilogue: whole K tiles, no cut, the 8-wave 256x256 tiles");
  static_assert(!SHUF || (!FP8 && !GROUPED && !TAIL), "scales in e8m0_shuffle order: dense MXFP4 problems with whole K tiles");
  constexpr bool B4 = FP8 && FMT_B == 4;  // 8-bit A against 4-bit B [N, K/2]: the lower half of B's LDS rows
  constexpr bool A4 = FP8 && FMT_A == 4;  // 4-bit A [M, K/2] against 8-bit B, the same way round
  static_assert(!FP8 || (!GROUPED && !TAIL && !SPLIT), "MXFP8: dense problems with whole K tiles");
  constexpr int BM = Cfg::BM, BN = Cfg::BN, MT_M = Cfg::MT_M, MT_N = Cfg::MT_N;
  constexpr int NWAVES = Cfg::NWAVES, A_LD = Cfg::A_LD, B_LD = Cfg::B_LD;
  constexpr int SLOT = Cfg::SLOT_BYTES, RING = Cfg::RING_SLOTS;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wave_m = wave / Cfg::WAVES_N, wave_n = wave % Cfg::WAVES_N;
  const int kp = p.kp, nkt = p.k_tiles;
  // SHORTS: a grouped problem's short tiles (a group's last M tile of at most 64 rows, listed behind the full ones
  // in the table) run after all full tiles, with the eight waves side by side on the tile's 64 rows (each 64 x 32:
  // two MFMAs per K step instead of eight).  The operand streams, their waits and the barrier are the full
  // tile's, request for request, so full and short tiles follow each other in any order.
  constexpr bool SHORTS = GROUPED && !SPLIT && !FP8 && !GATED && Cfg::NWAVES == 8 && Cfg::BN == 256 && Cfg::WAVES_M == 4;
  const int tiles_m = GROUPED ? __builtin_amdgcn_readfirstlane(p.tile_table[0]) : p.tiles_m;
  const int tiles_full = GROUPED ? __builtin_amdgcn_readfirstlane(p.tile_table[1]) : tiles_m;
  const int total = tiles_m * p.tiles_n;
  // ids of the tile walk (the padding ids of the XCD regrouping included)
  const int padded = GROUPED ? grouped_walk_ids(tiles_m, tiles_full, p.tiles_n) : (total + kNumXcd - 1) / kNumXcd * kNumXcd;
  const int k_tiles_blocks = (p.ksp >> 3) * 256;  // bytes of one 32-row scale tile row

  // ---------------- the tile sequence of this workgroup ----------------
  // Workgroup w takes ids w, w + grid, w + 2*grid, ...: the grid is a multiple
  // of the XCD count, so all of them map to the same XCD's run of tiles.
  // a_lim / as_lim: bytes of A and of its scale blocks from the tile's first row to the end of the tensor
  // (M need not be a multiple of the tile: rows past it read zeros and are never stored)
  const uint8_t *a_base[2], *b_base[2], *as_base[2], *bs_base[2];
  // c_rows: rows of the tile that are stored
  // nkt_of / part_of / tail_on: K tiles of the item, its slot in tail_partial (-1: a whole tile), and whether
  // its K range ends with the (partial) last K tile of the problem
  int m0[2], n0[2], a_lim[2], as_lim[2], b_lim[2], bs_lim[2], c_rows[2], nkt_of[2], part_of[2];
  int a_row32[2] = {0, 0};  // grouped: the tile's first row inside its 32-row scale block
  bool tail_on[2];
  bool is_short[2] = {false, false};
  const int m_blocks = (p.m + 31) >> 5;
  const int b_kt_stride = p.b_preshuffled ? 2048 : B4 ? kTileKBytes / 2 : kTileKBytes;
  auto map_grouped = [&](int id, int &tm, int &tn) -> bool {
    return map_grouped_tile(p.tile_table, tiles_m, tiles_full, p.tiles_n, id, tm, tn);
  };
  // (grouped: the tile count, and with it whether the last round is cut, is only known here)
  const int tail_parts = !SPLIT ? 1
                         : GROUPED ? tail_parts_rule(padded - total / (int)gridDim.x * (int)gridDim.x, (int)gridDim.x, nkt)
                                   : p.tail_parts;
  auto set_tile = [&](int which, int pid) -> bool {
    int tm, tn, kt_lo = 0;
    nkt_of[which] = nkt;
    part_of[which] = -1;
    if (SPLIT && tail_parts > 1 && pid >= total / (int)gridDim.x * (int)gridDim.x) {
      // the last round: workgroup w takes part w % parts of tile (whole rounds) + w / parts
      const int whole = total / (int)gridDim.x * (int)gridDim.x, w = pid - whole;
      if (w >= (int)gridDim.x) return false;
      const int r = w / tail_parts, i = w - r * tail_parts;
      if (whole + r >= padded) return false;  // (ids up to `padded`: map_tile skips the padding ids among them)
      pid = whole + r;
      const int base = nkt / tail_parts, rem = nkt - base * tail_parts;
      nkt_of[which] = base + (i < rem ? 1 : 0);
      kt_lo = i * base + min(i, rem);
      part_of[which] = r * tail_parts + i;
      if (!(GROUPED ? map_grouped(pid, tm, tn) : map_tile(pid, tiles_m, p.tiles_n, tm, tn))) return false;
    } else if (pid >= padded || !(GROUPED ? map_grouped(pid, tm, tn) : map_tile(pid, tiles_m, p.tiles_n, tm, tn))) {
      return false;
    }
    tail_on[which] = TAIL && kt_lo + nkt_of[which] == nkt;
    n0[which] = tn * BN;
    if (GROUPED) {
      const int32_t *ent = p.tile_table + 4 * (1 + tm);
      const int first = __builtin_amdgcn_readfirstlane(ent[0]), rows = __builtin_amdgcn_readfirstlane(ent[1]);
      const int expert = __builtin_amdgcn_readfirstlane(ent[2]);
      m0[which] = first;
      c_rows[which] = rows;
      b_base[which] = p.b + (int64_t)expert * p.b_group_stride + (int64_t)n0[which] * kp;
      bs_base[which] = p.b_scale + (int64_t)expert * p.b_scale_group_stride + (int64_t)(n0[which] >> 5) * k_tiles_blocks;
      a_row32[which] = first & 31;
      is_short[which] = SHORTS && tm >= tiles_full;
      as_base[which] = p.a_scale + (int64_t)(first >> 5) * k_tiles_blocks;
      as_lim[which] = (int)min((int64_t)(m_blocks - (first >> 5)) * k_tiles_blocks, (int64_t)0x7FFFFFFF);
    } else {
      m0[which] = tm * BM;
      c_rows[which] = p.m - m0[which];
      b_base[which] = p.b + (int64_t)n0[which] * (B4 ? kp >> 1 : kp);
      bs_base[which] = p.b_scale + (int64_t)(n0[which] >> 5) * k_tiles_blocks;
      as_base[which] = p.a_scale + (int64_t)(m0[which] >> 5) * k_tiles_blocks;
      as_lim[which] = (int)min((int64_t)(m_blocks - (m0[which] >> 5)) * k_tiles_blocks, (int64_t)0x7FFFFFFF);
    }
    // B and its scales end with the tensor (grouped: with the expert's)
    b_lim[which] = rsrc_bytes(((int64_t)p.n - n0[which]) * (B4 ? kp >> 1 : kp));
    bs_lim[which] = rsrc_bytes((int64_t)(((p.n + 31) >> 5) - (n0[which] >> 5)) * k_tiles_blocks);
    a_base[which] = p.a + (int64_t)m0[which] * (A4 ? kp >> 1 : kp);
    // (grouped: A ends with the tile's own rows.  The rows of the next group would do as padding, their results
    // are dropped, but zeros cost the matrix pipes far less power than data does, and power is what bounds the
    // kernel.)
    a_lim[which] = (int)min((int64_t)max(GROUPED ? c_rows[which] : p.m - m0[which], 0) * (A4 ? kp >> 1 : kp), (int64_t)0x7FFFFFFF);
    if (SPLIT) {  // the item's K range starts at K tile kt_lo: move the bases there
      a_base[which] += kt_lo * kTileKBytes;
      a_lim[which] = max(a_lim[which] - kt_lo * kTileKBytes, 0);
      b_base[which] += (int64_t)kt_lo * b_kt_stride;
      as_base[which] += kt_lo * 256;
      as_lim[which] = max(as_lim[which] - kt_lo * 256, 0);
      bs_base[which] += kt_lo * 256;
      b_lim[which] = max(b_lim[which] - kt_lo * b_kt_stride, 0);
      bs_lim[which] = max(bs_lim[which] - kt_lo * 256, 0);
    }
    return true;
  };
  // Item `step` of this workgroup's walk is tile id blockIdx.x + step * gridDim.x: all its full tiles, then its short
  // ones.  (Measured at 8 experts x 14336 x 4096, 8192 rows in multinomial groups, 1792 full and 224 short tiles:
  // short tiles placed between the full ones instead - at a position that differs from workgroup to workgroup, or
  // from XCD to XCD - so that their requests for B meet less competition, took 11-12 us longer: the workgroups of
  // an XCD then no longer run the tiles of a band together, and what they share of A and B is fetched again.)
  const int grid = (int)gridDim.x;
  const int walk_items = (int)blockIdx.x < padded ? (padded - (int)blockIdx.x + grid - 1) / grid : 0;
  auto id_of = [&](int step) -> int { return (int)blockIdx.x + step * grid; };
  // (padding ids of the XCD regrouping map to no tile: the walk steps over them)
  int step = 0;
  if constexpr (SHORTS) {
    while (step < walk_items && !set_tile(0, id_of(step))) ++step;
    if (step >= walk_items) return;
  } else {
    if (!set_tile(0, id_of(0))) return;
  }

  // ---------------- global -> LDS addressing (see the one-tile kernel) ----------------
  const int ld_row0 = wave * 8 + (lane >> 3);
  const int ld_chunk = (lane & 7) ^ ((ld_row0 >> 1) & 7);
  // DMA instruction d of a wave fills rows 8*NWAVES*d further down: one per-lane
  // offset per operand, the rest is scalar (registers are what this kernel is short of).
  const int kpb = B4 ? kp >> 1 : kp;  // bytes of a row of B
  const int kpa = A4 ? kp >> 1 : kp;  // bytes of a row of A
  int a_goff = ld_row0 * kpa + ld_chunk * 16;
  if (A4 && ld_chunk >= 4) a_goff = (int)0x80000000;  // the upper half of the LDS row: no request, zeros
  int b_goff = p.b_preshuffled ? (ld_row0 >> 4) * 16 * kp + (ld_row0 & 15) * 16 + (ld_chunk >> 1) * 512 +
                                           (ld_chunk & 1) * 256
                                     : ld_row0 * kpb + ld_chunk * 16;
  if (B4 && ld_chunk >= 4) b_goff = (int)0x80000000;  // the upper half of the LDS row: no request, zeros
  const int ld_step = NWAVES * 8 * kpa;  // bytes between consecutive d, either layout (8*NWAVES is a multiple of 16)
  const int ld_step_b = NWAVES * 8 * kpb;
  const bool tail_lane = TAIL && ld_chunk >= ((p.k & (kTileK - 1)) >> 5);
  auto flip_tail = [&](int &goff) { goff ^= tail_lane && (!SPLIT || tail_on[0]) ? (int)0x80000000 : 0; };

  // DMA instructions [d0, d1) of operand `op` (0 = A, 1 = B), K tile `kt` of
  // output tile `which` (0 = current, 1 = next), into ring slot `slot`.
  auto issue_g2l = [&](int which, int op, int kt, int slot, int d0, int d1) {
    uint8_t *dst_tile = smem + slot * SLOT;
    const __amdgpu_buffer_rsrc_t rsrc =
        op == 0 ? make_rsrc_n(a_base[which], a_lim[which]) : make_rsrc_n(b_base[which], b_lim[which]);
    const int soff = op == 0 ? kt * (A4 ? kTileKBytes / 2 : kTileKBytes) : kt * b_kt_stride;
#pragma unroll
    for (int d = d0; d < d1; ++d) {
      uint8_t *dst = dst_tile + (d * NWAVES + wave) * 1024;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, WAVE_LDS_PTR(dst), 16, op == 0 ? a_goff : b_goff,
                                               soff + d * (op == 0 ? ld_step : ld_step_b), 0, 0);
    }
  };

  // ---------------- fragments ----------------
  const int fr = lane & 31, fg = lane >> 5;
  // (MXFP8: K step s takes 32 bytes per lane in two halves, chunks 4s + fg and 4s + 2 + fg; foff[2s + h] is half h)
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
  uint32_t foff_b4[2];  // a 4-bit operand against an 8-bit one: its K step s is the chunk 2s + fg of the row's lower half
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

  // short tile: the wave's operands are rows 0..63 of A (two fragments) and its own 32 rows of B (one)
  auto read_frags_short = [&](int slot_a, int slot_b, int t, Frag(&fa)[MT_M], FragB(&fb)[MT_N]) {
    if constexpr (SHORTS) {
      const uint8_t *ba = smem + slot_a * SLOT + foff[t];
      const uint8_t *bb = smem + slot_b * SLOT + wave * 32 * kTileKBytes + foff[t];
      fa[0] = *(const v4i *)ba;
      fa[1] = *(const v4i *)(ba + 32 * kTileKBytes);
      fb[0] = *(const v4i *)bb;
    }
  };

  // The first fragments of the NEXT output tile, full or short (one sequence of six reads with that tile's bases,
  // not a branch between two sequences: the fragment registers of two paths would have to meet in one place, and
  // the register allocation of the whole loop fell apart over that.  A short tile has one fragment of B: its
  // three surplus reads repeat it.)
  auto read_frags_next_tile = [&](int slot_a, int slot_b, Frag(&fa)[MT_M], FragB(&fb)[MT_N]) {
    if constexpr (SHORTS) {
      const bool ns = is_short[1];
      const uint8_t *ba = smem + slot_a * SLOT + (ns ? 0u : a_fbase) + foff[0];
      const uint8_t *bb = smem + slot_b * SLOT + (ns ? (uint32_t)(wave * 32 * kTileKBytes) : b_fbase) + foff[0];
      const int b_step = ns ? 0 : 32 * kTileKBytes;
#pragma unroll
      for (int i = 0; i < MT_M; ++i) fa[i] = *(const v4i *)(ba + i * 32 * kTileKBytes);
#pragma unroll
      for (int jj = 0; jj < MT_N; ++jj) fb[jj] = *(const v4i *)(bb + jj * b_step);
    }
  };

  // ---------------- scales (MFMA-native order: one dword per lane, 32 rows and K tile) ----------------
  const int a_srow = ((wave_m * Cfg::WM) >> 5) * k_tiles_blocks, b_srow = ((wave_n * Cfg::WN) >> 5) * k_tiles_blocks;
  const int s_lane = SHUF ? ((lane >> 5) * 16 + (lane & 15)) * 4 : lane * 4;
  const uint32_t s_sel = (lane & 16) ? 0x07030501u : 0x06020400u;  // SHUF: the lane's bytes of its two dwords
  uint32_t raw_a[MT_M], raw_b[MT_N], sc_a[MT_M], sc_b[MT_N];
  uint32_t raw_a2[SHUF ? MT_M : 1], raw_b2[SHUF ? MT_N : 1];  // SHUF: the dwords of the odd K steps
  auto sblk = [](int kt) { return FP8 ? kt >> 1 : kt; };  // MXFP8: one MFMA32 block serves two K tiles
  auto load_scales = [&](int which, int kt) {
    const __amdgpu_buffer_rsrc_t ra = make_rsrc_n(as_base[which], as_lim[which]), rb = make_rsrc_n(bs_base[which], bs_lim[which]);
    int a_lane = s_lane;
    if constexpr (GROUPED) {
      const int t = a_row32[which] + (lane & 31);
      a_lane = ((t & 31) + (lane & 32)) * 4 + (t >> 5) * k_tiles_blocks;
    }
    // (a short tile: the blocks of rows 0..63 and of the wave's 32 columns; the three further B requests stay, for
    // the count of requests in flight, and read blocks that are not used)
    const int a_sr = SHORTS && is_short[which] ? 0 : a_srow;
    const int b_sr = SHORTS && is_short[which] ? wave * k_tiles_blocks : b_srow;
#pragma unroll
    for (int i = 0; i < MT_M; ++i) {
      raw_a[i] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(ra, a_lane, a_sr + i * k_tiles_blocks + sblk(kt) * 256, 0);
      if constexpr (SHUF)
        raw_a2[i] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(ra, a_lane, a_sr + i * k_tiles_blocks + sblk(kt) * 256 + 128, 0);
    }
#pragma unroll
    for (int j = 0; j < MT_N; ++j) {
      raw_b[j] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rb, s_lane, b_sr + j * k_tiles_blocks + sblk(kt) * 256, 0);
      if constexpr (SHUF)
        raw_b2[j] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rb, s_lane, b_sr + j * k_tiles_blocks + sblk(kt) * 256 + 128, 0);
    }
  };
  // Real register moves, pinned here (a compiler copy would be folded into the
  // loop's phi and wait for the next scale load at the top of every iteration).
  // (MXFP8, `kt` = the K tile the scales are for: its two K steps' bytes are bytes 0, 1 of the block's dword for
  // the even K tile of a pair and bytes 2, 3 for the odd one)
  auto canon_scales = [&](int kt) {
    if constexpr (FP8) {
      const int shift = (kt & 1) * 16;
#pragma unroll
      for (int i = 0; i < MT_M; ++i) asm volatile("v_lshrrev_b32 %0, %1, %2" : "=v"(sc_a[i]) : "s"(shift), "v"(raw_a[i]));
#pragma unroll
      for (int j = 0; j < MT_N; ++j) asm volatile("v_lshrrev_b32 %0, %1, %2" : "=v"(sc_b[j]) : "s"(shift), "v"(raw_b[j]));
    } else if constexpr (SHUF) {
#pragma unroll
      for (int i = 0; i < MT_M; ++i)
        asm volatile("v_perm_b32 %0, %1, %2, %3" : "=v"(sc_a[i]) : "v"(raw_a2[i]), "v"(raw_a[i]), "v"(s_sel));
#pragma unroll
      for (int j = 0; j < MT_N; ++j)
        asm volatile("v_perm_b32 %0, %1, %2, %3" : "=v"(sc_b[j]) : "v"(raw_b2[j]), "v"(raw_b[j]), "v"(s_sel));
    } else {
#pragma unroll
      for (int i = 0; i < MT_M; ++i) asm volatile("v_mov_b32 %0, %1" : "=v"(sc_a[i]) : "v"(raw_a[i]));
#pragma unroll
      for (int j = 0; j < MT_N; ++j) asm volatile("v_mov_b32 %0, %1" : "=v"(sc_b[j]) : "v"(raw_b[j]));
    }
  };

  // ---------------- accumulators and MFMA ----------------
  v16f acc[MT_M][MT_N];  // started from 0 by the first K step of every tile

  // ZERO: start the tile's sums from 0 (the first K step of a new output tile).
  auto mfma_block = [&](const Frag(&fa)[MT_M], const FragB(&fb)[MT_N], auto t_tag, auto zero_tag) {
    constexpr int T = decltype(t_tag)::value;
    constexpr bool ZERO = decltype(zero_tag)::value;
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
        v16f c = acc[i][j];
        if (ZERO) {
#pragma unroll
          for (int g = 0; g < 16; ++g) c[g] = 0.f;
        }
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vb, va, c, FMT_B, FMT_A, T, (int)sc_b[j], T, (int)sc_a[i]);
      }
    }
  };
  // short tile: 64 rows x the wave's 32 columns, accumulated in acc[0][0] and acc[1][0]
  auto mfma_short = [&](const Frag(&fa)[MT_M], const FragB(&fb)[MT_N], auto t_tag, auto zero_tag) {
    if constexpr (SHORTS) {
      constexpr int T = decltype(t_tag)::value;
      constexpr bool ZERO = decltype(zero_tag)::value;
      const v8i vb = v8i{fb[0].x, fb[0].y, fb[0].z, fb[0].w, 0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const v8i va = v8i{fa[i].x, fa[i].y, fa[i].z, fa[i].w, 0, 0, 0, 0};
        v16f c = acc[i][0];
        if (ZERO) {
#pragma unroll
          for (int g = 0; g < 16; ++g) c[g] = 0.f;
        }
        acc[i][0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vb, va, c, 4, 4, T, (int)sc_b[0], T, (int)sc_a[i]);
      }
    }
  };
  typedef std::integral_constant<int, 0> T0;
  typedef std::integral_constant<int, 1> T1;
  typedef std::integral_constant<int, 2> T2;
  typedef std::integral_constant<int, 3> T3;

  constexpr int HALF_LD = (A_LD > B_LD ? A_LD : B_LD) / 2;
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

  // C store instructions per wave and tile (1 KB each)
  constexpr int NS_BF16 = Cfg::WM * Cfg::WN * 2 / 1024, NS_F32 = Cfg::WM * Cfg::WN * 4 / 1024;
  constexpr int NS_GATED = MT_M * (MT_N / 2) * 2;  // per accumulator pair: one store of codes, one of scale bytes
  constexpr int kWaitFirstBf16 = GATED ? NS_GATED + A_LD : NS_BF16 + A_LD > 63 ? 63 : NS_BF16 + A_LD;
  constexpr int kWaitFirstF32 = NS_F32 + A_LD > 63 ? 63 : NS_F32 + A_LD;

  // ---------------- one K tile (phases as in the one-tile kernel) ----------------
  //   P0: second half of B(j+1)      P1, P2: A(j+2)      P3: barrier, first half of B(j+2)
  // with (j+1), (j+2) running on into the next output tile at a boundary.
  Frag fa0[MT_M], fa1[MT_M];
  FragB fb0[MT_N], fb1[MT_N];
  // MXFP8: one MFMA, two fragment halves each for its operands, and a DMA instruction while there are any
  auto order_phase8 = [&]() {
#pragma unroll
    for (int g = 0; g < MT_M * MT_N; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
  };
  // PENDING: the C stores of the previous output tile are in the queue (every tile but the first).
  // SHORT: the current output tile is a short tile (its MFMAs and fragment reads; everything else is the same)
  auto order_phase_short = [&]() {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
  };
  auto k_tile = [&](int j, int sa, int sb, auto kind_tag, auto pending_tag, auto short_tag) {
    constexpr int KIND = decltype(kind_tag)::value;
    constexpr bool PENDING = decltype(pending_tag)::value;
    constexpr bool SHORT = decltype(short_tag)::value;
    static_assert(!SHORT || SHORTS, "short tiles: the grouped 8-wave kernel");
    auto rd = [&](int slot_a, int slot_b, int t, Frag(&fa)[MT_M], FragB(&fb)[MT_N]) {
      if constexpr (SHORT) read_frags_short(slot_a, slot_b, t, fa, fb);
      else read_frags(slot_a, slot_b, t, fa, fb);
    };
    auto mm = [&](const Frag(&fa)[MT_M], const FragB(&fb)[MT_N], auto t_tag, auto zero_tag) {
      if constexpr (SHORT) mfma_short(fa, fb, t_tag, zero_tag);
      else mfma_block(fa, fb, t_tag, zero_tag);
    };
    auto order = [&]() {
      if constexpr (SHORT) order_phase_short();
      else order_phase();
    };
    static_assert(TAIL || KIND != kSteadyTail, "kSteadyTail belongs to the TAIL kernels");
    constexpr int W1 = KIND == kBound2 ? 1 : 0;                      // output tile of K tile j+1
    constexpr int W2 = (KIND == kBound1 || KIND == kBound2) ? 1 : 0;  // ... of K tile j+2
    const int kt1 = KIND == kBound2 ? 0 : j + 1;
    const int kt2 = KIND == kBound1 ? 0 : KIND == kBound2 ? 1 : j + 2;
    typedef std::integral_constant<bool, KIND == kFirst> Zero;
    typedef std::false_type Keep;
    const int sa1 = sa + 2 >= RING ? sa + 2 - RING : sa + 2;
    const int sb1 = sa + 3 >= RING ? sa + 3 - RING : sa + 3;
    const int sa2 = sa + 4 >= RING ? sa + 4 - RING : sa + 4;
    if constexpr (FP8) {
      // two K steps of 64-cycle MFMAs, two phases: A(j+2) in the first, the barrier, all of B(j+2) in the second,
      // so that every request has a whole K tile to land in (with B's second half requested in the first phase,
      // as the four-phase MXFP4 sequence does, it had half a K tile, and the waves waited for it)
      read_frags(sa, sb, 1, fa1, fb1);
      mfma_block(fa0, fb0, T0{}, Zero{});
      issue_g2l(W2, 0, kt2, sa2, 0, A_LD);
      order_phase8();
      __builtin_amdgcn_sched_barrier(0);
      if (KIND == kFirst && PENDING) {
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(OUT_BF16 ? kWaitFirstBf16 : kWaitFirstF32));
      } else {
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(A_LD));
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      issue_g2l(W2, 1, kt2, sa, 0, B_LD);  // (ahead of the phase's MFMAs: spread between them it cost 10 %)
      __builtin_amdgcn_sched_barrier(0);
      read_frags(sa1, sb1, 0, fa0, fb0);
      mfma_block(fa1, fb1, T1{}, Keep{});
      order_phase8();
      __builtin_amdgcn_sched_barrier(0);
      canon_scales(kt1);
      load_scales(W2, kt2);
      __builtin_amdgcn_sched_barrier(0);
      return;
    }
    rd(sa, sb, 1, fa1, fb1);
    mm(fa0, fb0, T0{}, Zero{});
    if (KIND != kFirst) issue_g2l(W1, 1, kt1, sb1, B_LD / 2, B_LD);
    if (TAIL && KIND == kBound1) flip_tail(b_goff);  // the second half of B of the partial K tile is out: back
    if (TAIL && KIND == kSteadyTail) flip_tail(a_goff);
    order();
    __builtin_amdgcn_sched_barrier(0);
    rd(sa, sb, 2, fa0, fb0);
    mm(fa1, fb1, T1{}, Keep{});
    issue_g2l(W2, 0, kt2, sa2, 0, A_LD / 2);
    order();
    __builtin_amdgcn_sched_barrier(0);
    rd(sa, sb, 3, fa1, fb1);
    mm(fa0, fb0, T2{}, Keep{});
    issue_g2l(W2, 0, kt2, sa2, A_LD / 2, A_LD);
    if (TAIL && KIND == kSteadyTail) flip_tail(a_goff), flip_tail(b_goff);  // A back; B until kBound1's first phase
    order();
    __builtin_amdgcn_sched_barrier(0);
    // Everything this wave issued up to B(j+1) has landed.  Younger than that:
    // the A_LD instructions of A(j+2) and, in the first K tile after a
    // boundary, the C stores of the previous output tile.
    if (KIND == kFirst && PENDING) {
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(OUT_BF16 ? kWaitFirstBf16 : kWaitFirstF32));
    } else {
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(A_LD));
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    // the first fragments of the next K tile; at the end of an output tile they are the next tile's, in ITS shape
    if constexpr (SHORTS && KIND == kBound2) {
      read_frags_next_tile(sa1, sb1, fa0, fb0);
    } else {
      rd(sa1, sb1, 0, fa0, fb0);
    }
    mm(fa1, fb1, T3{}, Keep{});
    issue_g2l(W2, 1, kt2, sa, 0, B_LD / 2);
    order();
    __builtin_amdgcn_sched_barrier(0);
    canon_scales(kt1);
    load_scales(W2, kt2);
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---------------- C tile: accumulators -> one ring slot -> global ----------------
  // acc[i][jn][4q + e] is row lane%32, column 8q + 4*(lane/32) + e of the 32x32
  // tile (i, jn).  Each wave owns 1/NWAVES of the slot: 32 rows whose 16-byte
  // chunk c sits at position c ^ (row % chunks per row) (conflict-free 16-byte
  // reads, two-way on the 8-byte writes), written pass by pass and read back as
  // whole rows, 16 bytes per lane.
  // `cbase`: the tile's first row; `f32_tag`: store f32 whatever the kernel's output type (the parts of SPLIT)
  auto store_tile = [&](int slot, uint8_t *cbase, int ldc, int tn0, int rows, auto f32_tag) {
    constexpr bool out_bf16 = OUT_BF16 && !decltype(f32_tag)::value;
    constexpr int SW = SLOT / NWAVES;  // staging bytes of a wave
    constexpr int RP = SW / 32;        // row pitch
    constexpr int NCH = RP / 16;       // chunks per row
    constexpr int LPR = NCH, RPI = 64 / LPR;
    uint8_t *stage = smem + slot * SLOT + wave * SW;
    const int wn0 = tn0 + wave_n * Cfg::WN;
    // Staging addresses are recomputed from the lane id at every tile: hoisted
    // out of the tile loop they would sit in registers through the main loop,
    // which has none to spare (a spill there costs a wait for the whole queue).
    int lane_v = lane;
    asm volatile("" : "+v"(lane_v));
    const int fr = lane_v & 31, fg = lane_v >> 5;
    const int lr = lane_v / LPR, lc = lane_v % LPR;
    // C goes out through a descriptor that ends with the tile's last valid row: rows past M (or past the
    // tile's group) are dropped
    constexpr int ELT = out_bf16 ? 2 : 4;
    // Grouped: non-temporal stores (the nt bit).  Every expert's B streams from HBM once, and a round's C tiles,
    // as many bytes as the XCD's L2 holds, written back lazily from there, got in the way of it: 8 experts x 1024
    // rows x 14336 x 4096 236 -> 221 us, multinomial groups 258 -> 244 us.  A dense problem, whose B the XCDs
    // share through the Infinity Cache, loses 1-2 % with them (8192^3: 237 -> 241 us) and keeps the default.
    // MXFP8 (twice the operand bytes, f32 C: more than the Infinity Cache holds at 8192^3) gains 2 %.
    constexpr int kStorePolicy = (GROUPED || FP8) ? 2 : 0;
    const __amdgpu_buffer_rsrc_t c_rsrc = make_rsrc_n(cbase, (int)min((int64_t)rows * ldc * ELT, (int64_t)0x7FFFFFFF));
    const int wr0 = wave_m * Cfg::WM;  // the wave's first row inside the tile
    if (out_bf16) {
      constexpr int CP = RP / 2, JP = CP / 32;  // columns, 32-column tiles per pass
      constexpr int REM = MT_N % JP;            // 32-column tiles left for a narrower last pass
      static_assert(REM == 0 || (JP == 2 && REM == 1), "odd wave tiles: 8-wave configurations only");
      typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int i = 0; i < MT_M; ++i) {
#pragma unroll
        for (int jg = 0; jg < MT_N / JP; ++jg) {
#pragma unroll
          for (int jj = 0; jj < JP; ++jj) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const v16f &a = acc[i][jg * JP + jj];
              const bf4 h = {(__bf16)a[4 * q], (__bf16)a[4 * q + 1], (__bf16)a[4 * q + 2], (__bf16)a[4 * q + 3]};
              const int chunk = jj * 4 + q;
              *(bf4 *)(stage + fr * RP + ((chunk ^ (fr & (NCH - 1))) << 4) + fg * 8) = h;
            }
          }
          asm volatile("" ::: "memory");
#pragma unroll
          for (int r0 = 0; r0 < 32; r0 += RPI) {
            const int r = r0 + lr;
            const v4i v = *(const v4i *)(stage + r * RP + ((lc ^ (r & (NCH - 1))) << 4));
            __builtin_amdgcn_raw_buffer_store_b128(v, c_rsrc, ((wr0 + i * 32 + r) * ldc + wn0 + jg * CP + lc * 8) * 2,
                                                       0, kStorePolicy);
          }
          asm volatile("" ::: "memory");
        }
        if constexpr (REM != 0) {
          // the last 32 columns: rows of 64 bytes, four lanes a row, 16 rows per store instruction
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const v16f &a = acc[i][MT_N - 1];
            const bf4 h = {(__bf16)a[4 * q], (__bf16)a[4 * q + 1], (__bf16)a[4 * q + 2], (__bf16)a[4 * q + 3]};
            *(bf4 *)(stage + fr * RP + ((q ^ (fr & (NCH - 1))) << 4) + fg * 8) = h;
          }
          asm volatile("" ::: "memory");
          const int lr4 = lane_v >> 2, lc4 = lane_v & 3;
#pragma unroll
          for (int r0 = 0; r0 < 32; r0 += 16) {
            const int r = r0 + lr4;
            const v4i v = *(const v4i *)(stage + r * RP + ((lc4 ^ (r & (NCH - 1))) << 4));
            __builtin_amdgcn_raw_buffer_store_b128(v, c_rsrc, ((wr0 + i * 32 + r) * ldc + wn0 + (MT_N - 1) * 32 + lc4 * 8) * 2,
                                                       0, kStorePolicy);
          }
          asm volatile("" ::: "memory");
        }
      }
    } else {
      constexpr int CP = RP / 4, JP = CP / 32;
#pragma unroll
      for (int i = 0; i < MT_M; ++i) {
#pragma unroll
        for (int jg = 0; jg < MT_N / JP; ++jg) {
#pragma unroll
          for (int jj = 0; jj < JP; ++jj) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const v16f &a = acc[i][jg * JP + jj];
              const v4f v = {a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]};
              const int chunk = jj * 8 + q * 2 + fg;
              *(v4f *)(stage + fr * RP + ((chunk ^ (fr & (NCH - 1))) << 4)) = v;
            }
          }
          asm volatile("" ::: "memory");
#pragma unroll
          for (int r0 = 0; r0 < 32; r0 += RPI) {
            const int r = r0 + lr;
            const v4f v = *(const v4f *)(stage + r * RP + ((lc ^ (r & (NCH - 1))) << 4));
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, v), c_rsrc,
                                                       ((wr0 + i * 32 + r) * ldc + wn0 + jg * CP + lc * 4) * 4, 0, kStorePolicy);
          }
          asm volatile("" ::: "memory");
        }
      }
    }
  };

  // The gated, quantised C (GATED): see the head of this function.
  auto store_gated = [&](int tile_m0, int tn0, int rows) {
    if constexpr (GATED) {
      typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
      int lane_v = lane;
      asm volatile("" : "+v"(lane_v));
      const int fr = lane_v & 31, fg = lane_v >> 5;
      const int qrow = p.n >> 2;                       // bytes of a row of codes
      const int act_ks = p.n >> 6;                     // scale groups of a row
      const __amdgpu_buffer_rsrc_t q_rsrc =
          make_rsrc_n((uint8_t *)p.c + (int64_t)tile_m0 * qrow, (int)min((int64_t)rows * qrow, (int64_t)0x7FFFFFFF));
      const int s_kt = (act_ks + 7) >> 3;               // K tiles of the activation (MFMA32 blocks per 32 rows)
      const __amdgpu_buffer_rsrc_t s_rsrc = make_rsrc_n(p.epi_scale, rsrc_bytes((int64_t)((p.m + 31) >> 5) * s_kt * 256));
      // (the accumulators are complete here: without this the last K tile's MFMAs are moved down between the
      // conversions below, with their operand fragments parked in scratch memory)
#pragma unroll
      for (int i = 0; i < MT_M; ++i)
#pragma unroll
        for (int j = 0; j < MT_N; ++j) asm volatile("" : "+v"(acc[i][j]));
#pragma unroll
      for (int i = 0; i < MT_M; ++i) {
        const int r_tile = wave_m * Cfg::WM + i * 32 + fr;   // row inside the tile
#pragma unroll
        for (int jp = 0; jp < MT_N / 2; ++jp) {
          const v16f &ga = acc[i][2 * jp], &ua = acc[i][2 * jp + 1];
          uint32_t h[8];
          uint32_t lo = 0, hi = 0;
#pragma unroll
          for (int w = 0; w < 8; ++w) {
            // the GEMM's bf16 output of the unfused pipeline, then its activation kernel's arithmetic
            const bf16x2 g2 = {(__bf16)ga[2 * w], (__bf16)ga[2 * w + 1]}, u2 = {(__bf16)ua[2 * w], (__bf16)ua[2 * w + 1]};
            const uint32_t gb = __builtin_bit_cast(uint32_t, g2), ub = __builtin_bit_cast(uint32_t, u2);
            const float g0 = __builtin_bit_cast(float, gb << 16), g1 = __builtin_bit_cast(float, gb & 0xFFFF0000u);
            const float u0 = __builtin_bit_cast(float, ub << 16), u1 = __builtin_bit_cast(float, ub & 0xFFFF0000u);
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
          // codes: dword 0 = columns 8q + 4 fg + 0..3 of q = 0, 1, dword 1 = of q = 2, 3 (two bytes each)
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
          const int g = (tn0 >> 6) + wave_n * (MT_N / 2) + jp;  // the activation's scale group
          __builtin_amdgcn_raw_buffer_store_b64(out, q_rsrc, r_tile * qrow + g * 16 + fg * 8, 0, 0);
          // one scale byte per row, from the lower lanes; rows past the tile's own are some other tile's
          const int r_abs = tile_m0 + r_tile;
          const int s_off = ((r_abs >> 5) * s_kt + (g >> 3)) * 256 + (((g & 1) << 5) | (r_abs & 31)) * 4 + ((g & 7) >> 1);
          __builtin_amdgcn_raw_buffer_store_b8((uint8_t)sb, s_rsrc, fg == 0 && r_tile < rows ? s_off : (int)0x80000000, 0, 0);
          __builtin_amdgcn_sched_barrier(0);  // one pair of accumulator tiles at a time through the vector registers
        }
      }
      asm volatile("" ::: "memory");
    }
  };

  // A short tile's C: acc[i][0][4q + e] is row 32 i + lane % 32, column 32 wave + 8q + 4 (lane / 32) + e of the tile;
  // eight stores of 8 or 16 bytes per lane, then as many more beyond the descriptor (dropped, but counted) as
  // bring the number of store instructions to a full tile's, which the first wait of the next tile counts on.
  auto store_short = [&](uint8_t *cbase, int ldc, int tn0, int rows) {
    if constexpr (SHORTS) {
      constexpr int ELT = OUT_BF16 ? 2 : 4;
      const __amdgpu_buffer_rsrc_t c_rsrc = make_rsrc_n(cbase, (int)min((int64_t)rows * ldc * ELT, (int64_t)0x7FFFFFFF));
      int lane_v = lane;
      asm volatile("" : "+v"(lane_v));
      const int fr = lane_v & 31, fg = lane_v >> 5;
      const int col0 = tn0 + wave * 32 + fg * 4;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const v16f &a = acc[i][0];
          const int off = ((i * 32 + fr) * ldc + col0 + q * 8) * ELT;
          if constexpr (OUT_BF16) {
            typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
            const bf4 h = {(__bf16)a[4 * q], (__bf16)a[4 * q + 1], (__bf16)a[4 * q + 2], (__bf16)a[4 * q + 3]};
            __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2i, h), c_rsrc, off, 0, 2);
          } else {
            const v4f v = {a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]};
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, v), c_rsrc, off, 0, 2);
          }
        }
      }
      // (each to an address of its own, far beyond the descriptor and not next to another: the compiler deletes a
      // store that a later one overwrites, and joins neighbours into one instruction)
#pragma unroll
      for (int d = 8; d < (OUT_BF16 ? NS_BF16 : NS_F32); ++d)
        __builtin_amdgcn_raw_buffer_store_b32(0, c_rsrc, 0x40000000 + 64 * d, 0, 0);
      asm volatile("" ::: "memory");
    }
  };

  // ---------------- prologue of the first tile ----------------
  issue_g2l(0, 0, 0, 0, 0, A_LD);
  issue_g2l(0, 1, 0, 1, 0, B_LD);
  load_scales(0, 0);
  issue_g2l(0, 0, 1, 2, 0, A_LD);
  issue_g2l(0, 1, 1, 3, 0, B_LD);
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(A_LD + B_LD));
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  canon_scales(0);
  load_scales(0, 1);
  bool short_first = false;
  if constexpr (SHORTS) short_first = is_short[0];
  if (short_first) read_frags_short(0, 1, 0, fa0, fb0);
  else read_frags(0, 1, 0, fa0, fb0);
  __builtin_amdgcn_sched_barrier(0);

  // ---------------- the tiles ----------------
  // After the last tile the stream simply runs on into a repeat of that tile's
  // first two K tiles (valid memory, never multiplied): one code path, no drain.
  // The first tile is peeled off the loop: with it inside, the compiler's own
  // waits (for the scale registers) would have to assume its store-free queue
  // for every tile.
  int sa = 0, part_stage = -1;
  auto next_slot = [&](int s) { return s + 2 >= RING ? s + 2 - RING : s + 2; };
  auto b_slot = [&](int s) { return s + 1 >= RING ? 0 : s + 1; };
  // Returns 0: that was the workgroup's last tile; 1: a full tile follows; 2: a short tile follows.
  auto run_tile = [&](auto pending_tag, auto short_tag) -> int {
    constexpr bool SHORT = decltype(short_tag)::value;
    int nstep = step + 1;
    bool has_next = set_tile(1, id_of(nstep));
    if constexpr (SHORTS) {
      while (!has_next && nstep + 1 < walk_items) has_next = set_tile(1, id_of(++nstep));
    }
    if (!has_next) {
      m0[1] = m0[0], n0[1] = n0[0], a_lim[1] = a_lim[0], as_lim[1] = as_lim[0], c_rows[1] = c_rows[0];
      b_lim[1] = b_lim[0], bs_lim[1] = bs_lim[0];
      nkt_of[1] = nkt_of[0], part_of[1] = part_of[0], tail_on[1] = tail_on[0], a_row32[1] = a_row32[0];
      a_base[1] = a_base[0], b_base[1] = b_base[0], as_base[1] = as_base[0], bs_base[1] = bs_base[0];
      is_short[1] = is_short[0];
    }
    const int nk = SPLIT ? nkt_of[0] : nkt;  // K tiles of this item
    k_tile(0, sa, b_slot(sa), std::integral_constant<int, kFirst>{}, pending_tag, short_tag);
    sa = next_slot(sa);
    for (int j = 1; j < nk - (TAIL ? 3 : 2); ++j) {
      k_tile(j, sa, b_slot(sa), std::integral_constant<int, kSteady>{}, pending_tag, short_tag);
      sa = next_slot(sa);
    }
    if constexpr (TAIL) {  // nk >= 4
      k_tile(nk - 3, sa, b_slot(sa), std::integral_constant<int, kSteadyTail>{}, pending_tag, short_tag);
      sa = next_slot(sa);
    }
    k_tile(nk - 2, sa, b_slot(sa), std::integral_constant<int, kBound1>{}, pending_tag, short_tag);
    sa = next_slot(sa);
    const int stage_slot = b_slot(sa);
    k_tile(nk - 1, sa, stage_slot, std::integral_constant<int, kBound2>{}, pending_tag, short_tag);
    // second half of B(1) of the next tile, ahead of the C stores (its first
    // half went into slot `sa` in the last phase above)
    if constexpr (!FP8) issue_g2l(1, 1, 1, sa, B_LD / 2, B_LD);
    sa = next_slot(sa);
    __builtin_amdgcn_sched_barrier(0);
    if (SPLIT && part_of[0] >= 0) {  // a part of a tile of the last round: always the workgroup's last item,
      part_stage = stage_slot;       // stored after the loop (a second store path in here costs the loop registers)
      return 0;
    }
    if constexpr (GATED)
      store_gated(m0[0], n0[0], c_rows[0]);
    else if constexpr (SHORT)
      store_short((uint8_t *)p.c + (int64_t)m0[0] * p.n * (OUT_BF16 ? 2 : 4), p.n, n0[0], c_rows[0]);
    else
      store_tile(stage_slot, (uint8_t *)p.c + (int64_t)m0[0] * p.n * (OUT_BF16 ? 2 : 4), p.n, n0[0], c_rows[0],
                 std::false_type{});
    if (!has_next) return 0;
    // the staging slot is the next target of the A stream: all waves must be done reading it
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(63));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    step = nstep;
    m0[0] = m0[1], n0[0] = n0[1], a_lim[0] = a_lim[1], as_lim[0] = as_lim[1], c_rows[0] = c_rows[1];
    b_lim[0] = b_lim[1], bs_lim[0] = bs_lim[1];
    nkt_of[0] = nkt_of[1], part_of[0] = part_of[1], tail_on[0] = tail_on[1], a_row32[0] = a_row32[1];
    a_base[0] = a_base[1], b_base[0] = b_base[1], as_base[0] = as_base[1], bs_base[0] = bs_base[1];
    is_short[0] = is_short[1];
    return SHORTS && is_short[0] ? 2 : 1;
  };
  int more = 2;
  if (!short_first) more = run_tile(std::false_type{}, std::false_type{});
  if constexpr (SHORTS) {
    if (short_first) {
      // no tile before this one: as many dropped stores as a tile's, so that the first wait of the first short
      // tile finds the queue it counts on (one instantiation then serves every short tile)
      const __amdgpu_buffer_rsrc_t none = make_rsrc_n(p.c, 0);
#pragma unroll
      for (int d = 0; d < (OUT_BF16 ? NS_BF16 : NS_F32); ++d) __builtin_amdgcn_raw_buffer_store_b32(0, none, 64 * d, 0, 0);
      asm volatile("" ::: "memory");
    }
    while (more != 0) more = more == 2 ? run_tile(std::true_type{}, std::true_type{}) : run_tile(std::true_type{}, std::false_type{});
  } else {
    while (more == 1) more = run_tile(std::true_type{}, std::false_type{});
  }
  if (SPLIT && part_stage >= 0)
    store_tile(part_stage, (uint8_t *)(p.tail_partial + (int64_t)part_of[0] * BM * BN), BN, 0, BM, std::true_type{});
  __builtin_amdgcn_s_waitcnt(0);  // the trailing DMA must not outlive the workgroup's LDS
}

template <class Cfg, bool OUT_BF16, bool GROUPED, bool TAIL, bool SPLIT, bool SHUF = false>
__global__ void __launch_bounds__(Cfg::NT, 1) persist_gemm_kernel(const GemmParams p) {
  persist_body<Cfg, OUT_BF16, GROUPED, TAIL, SPLIT, 4, 4, SHUF>(p);
}

template <class Cfg, bool GROUPED>
__global__ void __launch_bounds__(Cfg::NT, 1) persist_gemm_gated_kernel(const GemmParams p) {
  persist_body<Cfg, true, GROUPED, false, false, 4, 4, false, true>(p);
}

template <class Cfg, bool OUT_BF16, int FMT_A, int FMT_B>
__global__ void __launch_bounds__(Cfg::NT, 1) persist_gemm_fp8_kernel(const GemmParams p) {
  persist_body<Cfg, OUT_BF16, false, false, false, FMT_A, FMT_B>(p);
}

// Adds up the parts of the tiles of the last round (SPLIT) and writes them to C: one workgroup per 8 rows of a
// tile, a thread per 4 columns and row (two of them: with 32 rows per workgroup the loads of a thread's eight
// turns came one after the other, 11.5 us for 64 tiles of 3 parts).  Grouped: launched for the most tile ids a cut round can have; how many
// there are, and whether the round was cut at all, follows from the table's tile count as in the GEMM.
constexpr int kSumRows = 8;
template <class Cfg, bool GROUPED>
__global__ void __launch_bounds__(256) persist_tail_sum_kernel(const GemmParams p, int grid_main) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN;
  const int tiles_m = GROUPED ? p.tile_table[0] : p.tiles_m;
  const int total = tiles_m * p.tiles_n, whole = total / grid_main * grid_main;
  const int padded = (total + kNumXcd - 1) / kNumXcd * kNumXcd;
  const int parts = GROUPED ? tail_parts_rule(padded - whole, grid_main, p.k_tiles) : p.tail_parts;
  const int r = blockIdx.x / (BM / kSumRows), band = blockIdx.x % (BM / kSumRows);
  if (GROUPED && (parts <= 1 || whole + r >= padded)) return;
  int tm, tn;
  if (!(GROUPED ? map_grouped_tile(p.tile_table, tiles_m, p.tile_table[1], p.tiles_n, whole + r, tm, tn)
                : map_tile(whole + r, p.tiles_m, p.tiles_n, tm, tn)))
    return;  // a padding id
  int m_first = tm * BM, m_end = p.m;
  if (GROUPED) {  // the tile's rows: its group's, from the table
    m_first = p.tile_table[4 * (1 + tm)];
    m_end = m_first + p.tile_table[4 * (1 + tm) + 1];
  }
  const float *part = p.tail_partial + (int64_t)r * parts * BM * BN;
  for (int e = threadIdx.x; e < kSumRows * BN / 4; e += 256) {
    const int row = band * kSumRows + e / (BN / 4), col = (e % (BN / 4)) * 4;
    const int m = m_first + row, n = tn * BN + col;
    if (m >= m_end) continue;
    v4f sum = *(const v4f *)(part + (int64_t)row * BN + col);
    for (int i = 1; i < parts; ++i) sum += *(const v4f *)(part + ((int64_t)i * BM + row) * BN + col);
    if (p.out_bf16) {
      typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
      *(bf4 *)((__bf16 *)p.c + (int64_t)m * p.n + n) = bf4{(__bf16)sum.x, (__bf16)sum.y, (__bf16)sum.z, (__bf16)sum.w};
    } else {
      *(v4f *)((float *)p.c + (int64_t)m * p.n + n) = sum;
    }
  }
}

template <class Cfg, bool OUT_BF16, bool GROUPED, bool TAIL, bool SPLIT, bool SHUF = false>
static hipError_t launch_persist_out(const GemmParams &p, int grid_x, hipStream_t stream) {
  static LdsAttrOnce once;
  hipError_t e = allow_dynamic_lds(once, (const void *)persist_gemm_kernel<Cfg, OUT_BF16, GROUPED, TAIL, SPLIT, SHUF>,
                                   Cfg::LDS_BYTES);
  if (e != hipSuccess) return e;
  persist_gemm_kernel<Cfg, OUT_BF16, GROUPED, TAIL, SPLIT, SHUF>
      <<<dim3(grid_x, 1, 1), dim3(Cfg::NT), Cfg::LDS_BYTES, stream>>>(p);
  e = hipGetLastError();
  if (SPLIT && e == hipSuccess) {
    const int total = p.tiles_m * p.tiles_n;
    // tile ids of the last round (grouped: the most a round that is cut can have, the kernel knows how many there are)
    const int ids = GROUPED ? grid_x / 2 : (total + kNumXcd - 1) / kNumXcd * kNumXcd - total / grid_x * grid_x;
    persist_tail_sum_kernel<Cfg, GROUPED><<<dim3(ids * (Cfg::BM / kSumRows)), 256, 0, stream>>>(p, grid_x);
    e = hipGetLastError();
  }
  return e;
}

template <class Cfg, bool OUT_BF16>
static hipError_t launch_persist_dense(const GemmParams &p, int grid_x, hipStream_t stream) {
  const bool tail = (p.k & (kTileK - 1)) != 0;
  if constexpr (Cfg::NWAVES == 8) {
    // (both tensors, whole K tiles: persist_gemm_applies; a call without scratch, so no cut of the last round)
    if (p.a_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE)
      return launch_persist_out<Cfg, OUT_BF16, false, false, false, true>(p, grid_x, stream);
  }
  if constexpr (Cfg::NWAVES == 8 && Cfg::BN == 256) {  // (the 4-wave kernel has no registers to spare for the split bookkeeping)
    if (p.tail_parts > 1)
      return tail ? launch_persist_out<Cfg, OUT_BF16, false, true, true>(p, grid_x, stream)
                  : launch_persist_out<Cfg, OUT_BF16, false, false, true>(p, grid_x, stream);
  }
  return tail ? launch_persist_out<Cfg, OUT_BF16, false, true, false>(p, grid_x, stream)
              : launch_persist_out<Cfg, OUT_BF16, false, false, false>(p, grid_x, stream);
}

template <class Cfg>
static hipError_t launch_persist_cfg(const GemmParams &p, int grid_x, hipStream_t stream) {
  if (p.tile_table != nullptr) {
    if constexpr (Cfg::NWAVES == 8 && Cfg::BN == 256) {
      if (p.tail_partial != nullptr)  // few rounds: a sparsely filled last one is cut along K (decided on the device)
        return p.out_bf16 ? launch_persist_out<Cfg, true, true, false, true>(p, grid_x, stream)
                          : launch_persist_out<Cfg, false, true, false, true>(p, grid_x, stream);
    }
    return p.out_bf16 ? launch_persist_out<Cfg, true, true, false, false>(p, grid_x, stream)
                      : launch_persist_out<Cfg, false, true, false, false>(p, grid_x, stream);
  }
  return p.out_bf16 ? launch_persist_dense<Cfg, true>(p, grid_x, stream) : launch_persist_dense<Cfg, false>(p, grid_x, stream);
}

// How many parts the tiles of the last round should be cut into along K (1 = leave them whole), and the bytes
// of f32 scratch that takes.  Only when less than half of the workgroups would get a tile in that round,
// every part keeps at least four K tiles and the estimate says it pays.
int persist_tail_parts(const GemmParams &p, int variant, int num_cus, size_t *partial_bytes) {
  *partial_bytes = 0;
  if (variant != WAVE_MXFP4_VARIANT_T256x256_W4x2 || p.num_groups != 0 || !persist_gemm_applies(p, variant, num_cus))
    return 1;
  const int grid = num_cus / kNumXcd * kNumXcd;
  const int64_t total = (int64_t)p.tiles_m * p.tiles_n;
  if (total % grid == 0) return 1;
  // tile ids of the last round, the XCD padding ids among them included (they get a slot and stay unused)
  const int rest = (int)((total + kNumXcd - 1) / kNumXcd * kNumXcd - total / grid * grid);
  if (rest * 2 > grid) return 1;
  const int parts = tail_parts_rule(rest, grid, p.k_tiles);
  if (parts > 1) *partial_bytes = (size_t)rest * parts * 256 * 256 * sizeof(float);
  return parts;
}

// Whether 256x192 tiles serve a dense problem better than 256x256 tiles.  The kernels are bound by power, not by
// issue slots, so a partly filled last round costs less than a full one: measured on both tile shapes over the
// reference's shape list (K = 16000), a last round that gives a fraction f of the workgroups a tile takes
// 0.4 + 0.6 f of a full round's time (about 1 / parts + 0.2, at least 0.4, when its tiles are cut along K into
// `parts256` parts instead), and a round of 256x192 tiles 0.785 of a round of 256x256 tiles.  With fewer than 8 tile rows the wider tiles kept
// their lead (1024 x 24576: the XCDs' bands of the tile walk are 8 tile rows high).
bool persist_prefers_192(const GemmParams &p, int num_cus, int parts256) {
  if (p.num_groups != 0 || p.n % 192 != 0 || p.splits != 1) return false;
  const int grid = num_cus / kNumXcd * kNumXcd;
  if (grid < kNumXcd) return false;
  const int64_t tm = (p.m + 255) / 256, t256 = tm * ((p.n + 255) / 256), t192 = tm * (p.n / 192);
  if (t192 <= grid || tm < 8) return false;
  const auto rounds = [grid](int64_t tiles, int parts) {
    const double f = (double)(tiles % grid) / grid;
    const double cut = 1.0 / parts + 0.2;
    return (double)(tiles / grid) + (f == 0.0 ? 0.0 : parts > 1 ? (cut > 0.4 ? cut : 0.4) : 0.4 + 0.6 * f);
  };
  return 0.785 * rounds(t192, 1) < 0.95 * rounds(t256, parts256);
}

// The same question where N is a multiple of 192 but not of 256: the 256x256 tiles then run one per workgroup, in
// whole rounds over the CUs, and the persistent kernel on 256x192 tiles is the alternative from more tiles than
// workgroups on, at any number of tile rows (896 x 19584 x 3584: 308 tiles in two rounds 63.3 us, 408 narrower tiles
// 51.7; 1183 x 19584: 66.8 -> 55.4; 640 x 19584, 231 tiles in one round, stays: 38.1 against 45.4; 1536 x 19584,
// 462 against 612 tiles, stays: 70.7 against 76.4).
bool persist_192_over_tile_kernel(const GemmParams &p, int num_cus) {
  if (p.num_groups != 0 || p.n % 192 != 0 || p.n % 256 == 0 || p.splits != 1) return false;
  const int grid = num_cus / kNumXcd * kNumXcd;
  if (grid < kNumXcd) return false;
  const int64_t tm = (p.m + 255) / 256, t256 = tm * ((p.n + 255) / 256), t192 = tm * (p.n / 192);
  if (t192 <= grid) return false;
  const double f = (double)(t192 % grid) / grid;
  const double r192 = (double)(t192 / grid) + (f == 0.0 ? 0.0 : 0.4 + 0.6 * f);
  return 0.785 * r192 < (double)((t256 + num_cus - 1) / num_cus);
}

// Whether the persistent kernel serves this problem with `num_cus` CUs.
bool persist_gemm_applies(const GemmParams &p, int variant, int num_cus) {
  if (variant != WAVE_MXFP4_VARIANT_T256x256_W2x2 && variant != WAVE_MXFP4_VARIANT_T256x256_W4x2 &&
      variant != WAVE_MXFP4_VARIANT_T256x192_W4x2)
    return false;
  const int bn = variant == WAVE_MXFP4_VARIANT_T256x192_W4x2 ? 192 : 256;
  // (a grouped problem comes with its M tile table, or not at all)
  if ((p.num_groups != 0) != (p.tile_table != nullptr) || p.splits != 1 || p.partial != nullptr) return false;
  // both scale tensors in MFMA32 order; or, 8-wave kernels on dense problems with whole K tiles, both in
  // e8m0_shuffle order
  const bool shuffled = p.a_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE && p.b_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE &&
                        variant != WAVE_MXFP4_VARIANT_T256x256_W2x2 && p.num_groups == 0 && (p.k & (kTileK - 1)) == 0;
  if (!shuffled && (p.a_scale_layout != WAVE_MXFP4_SCALE_MFMA32 || p.b_scale_layout != WAVE_MXFP4_SCALE_MFMA32)) return false;
  if (p.n % bn != 0 || p.tiles_n != p.n / bn || p.k_tiles < 3) return false;  // any M
  // a partial last K tile: dense problems with at least four K tiles
  if ((p.k & (kTileK - 1)) != 0 && (p.num_groups != 0 || p.k_tiles < 4)) return false;
  if (p.out_bf16 ? (p.n & 7) != 0 : (p.n & 3) != 0) return false;
  // 32-bit offsets inside one operand tile, and more tiles than workgroups
  if ((int64_t)256 * p.kp >= ((int64_t)1 << 31) || (int64_t)256 * p.n * 4 >= ((int64_t)1 << 31)) return false;
  const int grid = num_cus / kNumXcd * kNumXcd;
  // (grouped: tiles_m is an upper bound, the rows give the estimate)
  const int64_t tiles_m = p.num_groups != 0 ? p.m / 256 : p.tiles_m;
  return grid >= kNumXcd && tiles_m * p.tiles_n > grid;
}

// MXFP8 (`p` in byte geometry: kp = K bytes per row, k_tiles = K / 128): the 8-wave 256x256 configuration, dense.
bool persist_gemm_fp8_applies(const GemmParams &p, int num_cus) {
  if (p.num_groups != 0 || p.tile_table != nullptr || p.splits != 1 || p.partial != nullptr || p.b_preshuffled) return false;
  if (p.a_scale_layout != WAVE_MXFP4_SCALE_MFMA32 || p.b_scale_layout != WAVE_MXFP4_SCALE_MFMA32) return false;
  if ((p.n & 255) != 0 || p.tiles_n != p.n / 256 || (p.k & 255) != 0 || p.k_tiles < 4) return false;
  if ((int64_t)256 * p.kp >= ((int64_t)1 << 31) || (int64_t)256 * p.n * 4 >= ((int64_t)1 << 31)) return false;
  const int grid = num_cus / kNumXcd * kNumXcd;
  return grid >= kNumXcd && (int64_t)p.tiles_m * p.tiles_n > grid;
}

template <class Cfg, bool OUT_BF16, int FMT_A, int FMT_B>
static hipError_t launch_persist_fp8_out(const GemmParams &p, int grid_x, hipStream_t stream) {
  static LdsAttrOnce once;
  hipError_t e = allow_dynamic_lds(once, (const void *)persist_gemm_fp8_kernel<Cfg, OUT_BF16, FMT_A, FMT_B>, Cfg::LDS_BYTES);
  if (e != hipSuccess) return e;
  persist_gemm_fp8_kernel<Cfg, OUT_BF16, FMT_A, FMT_B><<<dim3(grid_x, 1, 1), dim3(Cfg::NT), Cfg::LDS_BYTES, stream>>>(p);
  return hipGetLastError();
}

template <int FMT_A, int FMT_B>
static hipError_t launch_persist_fp8_fmt(const GemmParams &p, int grid_x, hipStream_t stream) {
  typedef TileCfg<256, 256, 4, 2> Cfg;
  return p.out_bf16 ? launch_persist_fp8_out<Cfg, true, FMT_A, FMT_B>(p, grid_x, stream)
                    : launch_persist_fp8_out<Cfg, false, FMT_A, FMT_B>(p, grid_x, stream);
}

// a_fmt, b_fmt: 0 = e4m3, 1 = e5m2, 2 = e2m1 (packed, two per byte; one operand at most)
hipError_t launch_persist_gemm_fp8(const GemmParams &p, int num_cus, int a_fmt, int b_fmt, hipStream_t stream) {
  const int grid = num_cus / kNumXcd * kNumXcd;
  if (a_fmt == 2 && b_fmt == 2) return hipErrorInvalidValue;  // (both 4-bit: the MXFP4 entry point)
  if (a_fmt == 2) return b_fmt ? launch_persist_fp8_fmt<4, 1>(p, grid, stream) : launch_persist_fp8_fmt<4, 0>(p, grid, stream);
  const int a_e5m2 = a_fmt;
  if (b_fmt == 2) return a_e5m2 ? launch_persist_fp8_fmt<1, 4>(p, grid, stream) : launch_persist_fp8_fmt<0, 4>(p, grid, stream);
  if (a_e5m2) return b_fmt ? launch_persist_fp8_fmt<1, 1>(p, grid, stream) : launch_persist_fp8_fmt<1, 0>(p, grid, stream);
  return b_fmt ? launch_persist_fp8_fmt<0, 1>(p, grid, stream) : launch_persist_fp8_fmt<0, 0>(p, grid, stream);
}

// The gated, quantising kernel: the 8-wave 256x256 tiles, dense or grouped by table, whole K tiles, N = twice the
// activation's width in whole 256-column tiles, MFMA32 scales, more tiles than workgroups.
bool persist_gated_applies(const GemmParams &p, int num_cus) {
  if (!p.out_bf16 || p.epi_scale == nullptr || (p.k & (kTileK - 1)) != 0 || p.tail_partial != nullptr || p.tail_parts > 1)
    return false;
  if (p.epi_scale_layout != WAVE_MXFP4_SCALE_MFMA32) return false;
  if (p.a_scale_layout != WAVE_MXFP4_SCALE_MFMA32 || p.b_scale_layout != WAVE_MXFP4_SCALE_MFMA32) return false;
  if ((int64_t)p.m * (p.n >> 6) >= ((int64_t)1 << 31) || (int64_t)((p.m + 31) >> 5) * (((p.n >> 6) + 7) >> 3) * 256 >= ((int64_t)1 << 31))
    return false;
  return persist_gemm_applies(p, WAVE_MXFP4_VARIANT_T256x256_W4x2, num_cus);
}

hipError_t launch_persist_gated(const GemmParams &p, int num_cus, hipStream_t stream) {
  typedef TileCfg<256, 256, 4, 2> Cfg;
  const int grid = num_cus / kNumXcd * kNumXcd;
  static LdsAttrOnce once[2];
  const bool grouped = p.tile_table != nullptr;
  const void *fn = grouped ? (const void *)persist_gemm_gated_kernel<Cfg, true> : (const void *)persist_gemm_gated_kernel<Cfg, false>;
  const hipError_t e = allow_dynamic_lds(once[grouped ? 1 : 0], fn, Cfg::LDS_BYTES);
  if (e != hipSuccess) return e;
  if (grouped)
    persist_gemm_gated_kernel<Cfg, true><<<dim3(grid, 1, 1), dim3(Cfg::NT), Cfg::LDS_BYTES, stream>>>(p);
  else
    persist_gemm_gated_kernel<Cfg, false><<<dim3(grid, 1, 1), dim3(Cfg::NT), Cfg::LDS_BYTES, stream>>>(p);
  return hipGetLastError();
}

hipError_t launch_persist_gemm(const GemmParams &p, int variant, int num_cus, hipStream_t stream) {
  const int grid = num_cus / kNumXcd * kNumXcd;
  if (variant == WAVE_MXFP4_VARIANT_T256x256_W2x2) return launch_persist_cfg<TileCfg<256, 256, 2, 2>>(p, grid, stream);
  if (variant == WAVE_MXFP4_VARIANT_T256x192_W4x2) return launch_persist_cfg<TileCfg<256, 192, 4, 2>>(p, grid, stream);
  return launch_persist_cfg<TileCfg<256, 256, 4, 2>>(p, grid, stream);
}

}  // namespace wave_mxfp4

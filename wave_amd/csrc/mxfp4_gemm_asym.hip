// Asymmetric persistent MXFP4 GEMM for gfx950 (MI355X): A through LDS, preshuffled B straight
// from global memory into registers.
//
// The counterpart of the reference's best kernel family
// (wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:950-991 with the schedule of
// wave_lang/kernel/wave/schedules/gemm_mxfp4_double_buffer.py:1781-2222: "A (data + scale):
// global -> LDS -> VGPRs, B (data + scale): global -> VGPRs directly"), designed for what
// bounds the symmetric kernels on this chip: with both operands in LDS the 160 KB hold 2.5 K
// tiles, so a tile of B has to arrive within about three quarters of a K tile's time of its
// request, and the waves wait for it.  Here
//   * a workgroup is 4 waves side by side along N: each owns all 256 rows and 64 columns of the
//     256 x 256 output tile (8 x 2 MFMA tiles of 32 x 32, v_mfma_scale_f32_32x32x64_f8f6f4);
//   * A (and its scales) goes global -> LDS by DMA into a ring of FOUR K tiles, requested three
//     K tiles ahead of its use;
//   * B needs no LDS: in b_preshuffle order the 16 bytes a lane feeds to one MFMA are where one
//     coalesced 16-byte load per lane finds them (256 contiguous bytes per 16 lanes).  Every
//     B fragment register is reloaded right after the MFMAs that read it, with the data of two
//     K tiles later (1.75 K tiles of time for the load), 64 registers in all;
//   * so about 190 KB per CU are in flight instead of 96 KB, at one wave per SIMD;
//   * one workgroup per CU walks a sequence of output tiles and the operand streams run on
//     across tile boundaries (the requests for the next tile's first K tiles go out while the
//     last K tiles of this one are multiplied); C leaves through a per-wave staging area
//     outside the ring, whole 128-byte lines per store instruction.
// One barrier per K tile.  All waits are counted (s_waitcnt vmcnt(n)), never for an empty queue:
// vector memory operations retire in issue order, and every wave issues the same 19 of them per
// K tile in a fixed order.
//
// Taken for preshuffled B, N % 256 == 0, K % 512 == 0 (the B registers alternate between even and
// odd K tiles), K >= 1536, both scale tensors in MFMA32 order or both in e8m0_shuffle order (SHUF: the
// same 256-byte blocks, a lane's four bytes in two dwords 128 bytes apart, put together by a v_perm),
// dense, no split.  Any M.
#include <type_traits>

#include "mxfp4_tile_common.h"

namespace wave_mxfp4 {

namespace {

constexpr int kAsymBM = 256, kAsymBN = 256, kAsymWaves = 4, kAsymNT = kAsymWaves * 64;
constexpr int kARing = 4;                       // K tiles of A in LDS
constexpr int kASlot = kAsymBM * kTileKBytes;   // 32 KB
constexpr int kSSlot = kAsymWaves * 1024;       // A scales of one K tile: 2 KB used, 1 KB per wave written
constexpr int kStage = 4096;                    // C staging per wave
constexpr int kAsymLds = kARing * kASlot + kARing * kSSlot + kAsymWaves * kStage;  // 160 KB
constexpr int kALd = kAsymBM / 8 / kAsymWaves;  // A DMA instructions per wave and K tile (8)
// Vector memory operations per wave and K tile: A 8, A scales 1, B 8, B scales 2 (4 in e8m0_shuffle order).
constexpr int ops_per_k_tile(bool shuf) { return kALd + 1 + 8 + (shuf ? 4 : 2); }
// At the wait of K tile g (before its fourth K step) A and its scales of K tile g + 1 must have landed.  They
// were requested in K tile g - 2 (at the latest as the last operations of its fourth K step: the compiler may
// order the requests of one K step among themselves), followed by the 19 of K tile g - 1 and the 14 of the first
// three K steps of K tile g (16 with four B scale requests, which go out in the second K step).
constexpr int wait_steady(bool shuf) { return ops_per_k_tile(shuf) + (shuf ? 16 : 14); }
static_assert(kAsymLds <= 160 * 1024, "LDS");

template <bool OUT_BF16, bool SHUF>
__device__ __forceinline__ void asym_body(const GemmParams &p) {
  constexpr int BM = kAsymBM, BN = kAsymBN, NW = kAsymWaves;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  uint8_t *const s_ring = smem + kARing * kASlot;   // scale ring
  uint8_t *const c_stage = s_ring + kARing * kSSlot;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kp = p.kp, nkt = p.k_tiles;
  const int total = p.tiles_m * p.tiles_n;
  const int padded = (total + kNumXcd - 1) / kNumXcd * kNumXcd;
  const int k_tiles_blocks = nkt * 256;  // bytes of one 32-row block row of scales (MFMA32 order)
  const int m_blocks = (p.m + 31) >> 5;

  // ---------------- the output tiles of this workgroup: [0] = being multiplied, [1] = the one after ----------------
  const uint8_t *a_base[2], *b_base[2], *as_base[2], *bs_base[2];
  int m0[2], n0[2], a_lim[2], as_lim[2], b_lim[2], bs_lim[2];
  auto set_tile = [&](int which, int pid) -> bool {
    int tm, tn;
    if (pid >= padded || !map_tile(pid, p.tiles_m, p.tiles_n, tm, tn)) return false;
    m0[which] = tm * BM;
    n0[which] = tn * BN;
    a_base[which] = p.a + (int64_t)m0[which] * kp;
    a_lim[which] = (int)min((int64_t)max(p.m - m0[which], 0) * kp, (int64_t)0x7FFFFFFF);
    as_base[which] = p.a_scale + (int64_t)(m0[which] >> 5) * k_tiles_blocks;
    as_lim[which] = (int)min((int64_t)max(m_blocks - (m0[which] >> 5), 0) * k_tiles_blocks, (int64_t)0x7FFFFFFF);
    // 16-row blocks of preshuffled B are contiguous: the tile's columns start at byte n0 * kp
    b_base[which] = p.b + (int64_t)n0[which] * kp;
    b_lim[which] = (int)min((int64_t)(p.n - n0[which]) * kp, (int64_t)0x7FFFFFFF);
    bs_base[which] = p.b_scale + (int64_t)(n0[which] >> 5) * k_tiles_blocks;
    bs_lim[which] = (int)min((int64_t)((p.n - n0[which]) >> 5) * k_tiles_blocks, (int64_t)0x7FFFFFFF);
    return true;
  };
  auto copy_tile = [&](int dst, int src) {
    m0[dst] = m0[src], n0[dst] = n0[src], a_lim[dst] = a_lim[src], as_lim[dst] = as_lim[src];
    b_lim[dst] = b_lim[src], bs_lim[dst] = bs_lim[src];
    a_base[dst] = a_base[src], b_base[dst] = b_base[src], as_base[dst] = as_base[src], bs_base[dst] = bs_base[src];
  };
  int pid = blockIdx.x;
  if (!set_tile(0, pid)) return;
  if (!set_tile(1, pid + (int)gridDim.x)) copy_tile(1, 0);  // past the end the streams re-read this tile: valid memory

  // ---------------- per-lane offsets ----------------
  // A DMA (as in the symmetric kernels): instruction d of a wave fills LDS rows (d * 4 + wave) * 8 .. + 7; lane t
  // lands at row t / 8, chunk position t % 8, which must hold chunk (t % 8) ^ swz(row), swz(row) = (row / 2) % 8.
  const int ld_row0 = wave * 8 + (lane >> 3);
  const int a_goff = ld_row0 * kp + (((lane & 7) ^ ((ld_row0 >> 1) & 7)) << 4);
  const int a_step = NW * 8 * kp;  // bytes between consecutive d
  // A scale DMA: lanes 0..15 fetch block 2 * wave, lanes 16..31 block 2 * wave + 1 (16 bytes each) of the tile's
  // eight 256-byte blocks of a K tile; the other half of the wave points past the end of any buffer (zeros land
  // in the unused upper half of the wave's kilobyte).
  const int as_goff = lane < 32 ? (2 * wave + (lane >> 4)) * k_tiles_blocks + (lane & 15) * 16 : (int)0x80000000;
  // B fragment of the 32x32x64 MFMA straight from b_preshuffle order: lane = (row r = lane % 32, K half = lane / 32)
  const int fr = lane & 31, fg = lane >> 5;
  const int b_goff = wave * 64 * kp + (fr >> 4) * 16 * kp + fg * 256 + (fr & 15) * 16;
  // the lane's dword of a 256-byte scale block (SHUF: the first of its two, the other 128 bytes on)
  const int s_lane = SHUF ? ((lane >> 5) * 16 + (lane & 15)) * 4 : lane * 4;
  const uint32_t s_sel = (lane & 16) ? 0x07030501u : 0x06020400u;  // SHUF: the lane's bytes of the two dwords
  const int bs_goff = (2 * wave) * k_tiles_blocks + s_lane;
  // A fragment reads: row fr of a 32-row block, chunk 2t + fg at its swizzled position
  uint32_t foff[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) foff[t] = (uint32_t)(fr * kTileKBytes + (((t * 2 + fg) ^ ((fr >> 1) & 7)) << 4));

  // ---------------- request streams: K tile `kt` of output tile `which` ----------------
  auto issue_a = [&](int which, int kt, int slot, int d0, int d1) {
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc_n(a_base[which], a_lim[which]);
#pragma unroll
    for (int d = d0; d < d1; ++d)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, WAVE_LDS_PTR(smem + slot * kASlot + (d * NW + wave) * 1024), 16, a_goff,
                                               kt * kTileKBytes + d * a_step, 0, 0);
  };
  auto issue_as = [&](int which, int kt, int slot) {
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc_n(as_base[which], as_lim[which]);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, WAVE_LDS_PTR(s_ring + slot * kSSlot + wave * 1024), 16, as_goff, kt * 256,
                                             0, 0);
  };
  // the two B fragments (32-column halves jn = 0, 1 of the wave's 64 columns) of K step t
  auto load_b = [&](int which, int kt, int t, v4i (&dst)[2]) {
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc_n(b_base[which], b_lim[which]);
#pragma unroll
    for (int jn = 0; jn < 2; ++jn)
      dst[jn] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, b_goff, (kt * 4 + t) * 512 + jn * 32 * kp, 0);
  };
  auto load_bs = [&](int which, int kt, uint32_t (&dst)[2], uint32_t (&dst2)[2]) {
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc_n(bs_base[which], bs_lim[which]);
#pragma unroll
    for (int jn = 0; jn < 2; ++jn) {
      dst[jn] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, bs_goff, jn * k_tiles_blocks + kt * 256, 0);
      if constexpr (SHUF)
        dst2[jn] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, bs_goff, jn * k_tiles_blocks + kt * 256 + 128, 0);
    }
  };

  // ---------------- registers ----------------
  v16f acc[8][2];
  v4i bq[2][4][2];          // [parity of the K tile][K step][jn]
  uint32_t sb_cur[2][2], sb_in[2][2];  // B scales in use / arriving, per parity
  uint32_t sb_in2[2][2];               // SHUF: the second dword of the arriving ones
  uint32_t sa[2][8];        // A scales per parity
  v4i afr[2][8];            // A fragments, double buffered by K step

  auto read_a = [&](int slot, int t, v4i (&dst)[8]) {
    const uint8_t *base = smem + slot * kASlot + foff[t];
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[i] = *(const v4i *)(base + i * 32 * kTileKBytes);
  };
  auto read_sa = [&](int slot, uint32_t (&dst)[8]) {
    // block i of the tile's eight was fetched by wave i / 2 into the lower half of its kilobyte
    const uint8_t *base = s_ring + slot * kSSlot + s_lane;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t d0 = *(const uint32_t *)(base + (i >> 1) * 1024 + (i & 1) * 256);
      if constexpr (SHUF)
        dst[i] = __builtin_amdgcn_perm(*(const uint32_t *)(base + (i >> 1) * 1024 + (i & 1) * 256 + 128), d0, s_sel);
      else
        dst[i] = d0;
    }
  };
  auto mfma_step = [&](const v4i (&fa)[8], const v4i (&fb)[2], const uint32_t (&sca)[8], const uint32_t (&scb)[2], auto t_tag,
                       auto zero_tag) {
    constexpr int T = decltype(t_tag)::value;
    constexpr bool ZERO = decltype(zero_tag)::value;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const v8i va = {fa[i].x, fa[i].y, fa[i].z, fa[i].w, 0, 0, 0, 0};
#pragma unroll
      for (int jn = 0; jn < 2; ++jn) {
        const v8i vb = {fb[jn].x, fb[jn].y, fb[jn].z, fb[jn].w, 0, 0, 0, 0};
        v16f c = acc[i][jn];
        if (ZERO) {
#pragma unroll
          for (int g = 0; g < 16; ++g) c[g] = 0.f;
        }
        // operands swapped (B rows as the matrix A of the instruction): a lane's 4 accumulator registers of a
        // group are 4 consecutive N
        acc[i][jn] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vb, va, c, 4, 4, T, (int)scb[jn], T, (int)sca[i]);
      }
    }
  };
  // one K step's instruction mix: MFMAs with the LDS reads and the memory requests spread between them
  auto order_step = [&]() {
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
  };
  typedef std::integral_constant<int, 0> T0;
  typedef std::integral_constant<int, 1> T1;
  typedef std::integral_constant<int, 2> T2;
  typedef std::integral_constant<int, 3> T3;
  typedef std::false_type Keep;

  // ---------------- one K tile ----------------
  // j: K tile of the current output tile; sl: its ring slot; PAR: parity of j; ZERO: first K tile of an output
  // tile; WAITN: operations that may still be in flight at the wait.
  //   K step 0: A(j+3) d 0,1; B(j+1) K step 3   (the registers the previous K tile's last K step just read)
  //   K step 1: A(j+3) d 2,3; B(j+2) K step 0; B scales (j+2)
  //   K step 2: A(j+3) d 4,5; B(j+2) K step 1
  //   K step 3: wait, barrier; A(j+3) d 6,7; A scales (j+3); B(j+2) K step 2
  // INNER: every K tile requested from here (up to j + 3) still belongs to the current output tile, so the
  // descriptors are loop constants; otherwise they are picked per stream (a few dozen scalar selects per K tile,
  // which a wave that is alone on its SIMD cannot hide: only the last four K tiles of an output tile pay them).
  auto k_tile = [&](int j, int sl, auto par_tag, auto zero_tag, auto wait_tag, auto inner_tag) {
    constexpr int PAR = decltype(par_tag)::value;
    constexpr int WAITN = decltype(wait_tag)::value;
    constexpr bool INNER = decltype(inner_tag)::value;
    const int ja = j + 3, wa = !INNER && ja >= nkt ? 1 : 0, kta = ja - (wa ? nkt : 0);
    const int jb1 = j + 1, wb1 = !INNER && jb1 >= nkt ? 1 : 0, ktb1 = jb1 - (wb1 ? nkt : 0);
    const int jb2 = j + 2, wb2 = !INNER && jb2 >= nkt ? 1 : 0, ktb2 = jb2 - (wb2 ? nkt : 0);
    const int sl_a = (sl + 3) & 3, sl_n = (sl + 1) & 3;

    // this K tile's B scales were requested two K tiles ago into sb_in: real moves, pinned here (a compiler copy
    // would be folded into a phi of the loop and wait wherever that lands)
#pragma unroll
    for (int jn = 0; jn < 2; ++jn) {
      if constexpr (SHUF)
        asm volatile("v_perm_b32 %0, %1, %2, %3" : "=v"(sb_cur[PAR][jn]) : "v"(sb_in2[PAR][jn]), "v"(sb_in[PAR][jn]), "v"(s_sel));
      else
        asm volatile("v_mov_b32 %0, %1" : "=v"(sb_cur[PAR][jn]) : "v"(sb_in[PAR][jn]));
    }
    read_a(sl, 1, afr[1]);
    mfma_step(afr[0], bq[PAR][0], sa[PAR], sb_cur[PAR], T0{}, zero_tag);
    issue_a(wa, kta, sl_a, 0, 2);
    load_b(wb1, ktb1, 3, bq[PAR ^ 1][3]);
    order_step();
    __builtin_amdgcn_sched_barrier(0);

    read_a(sl, 2, afr[0]);
    mfma_step(afr[1], bq[PAR][1], sa[PAR], sb_cur[PAR], T1{}, Keep{});
    issue_a(wa, kta, sl_a, 2, 4);
    load_b(wb2, ktb2, 0, bq[PAR][0]);
    load_bs(wb2, ktb2, sb_in[PAR], sb_in2[PAR]);
    order_step();
    __builtin_amdgcn_sched_barrier(0);

    read_a(sl, 3, afr[1]);
    mfma_step(afr[0], bq[PAR][2], sa[PAR], sb_cur[PAR], T2{}, Keep{});
    issue_a(wa, kta, sl_a, 4, 6);
    load_b(wb2, ktb2, 1, bq[PAR][1]);
    order_step();
    __builtin_amdgcn_sched_barrier(0);

    // A(j+1) and its scales, requested two K tiles ago by all four waves, must be in LDS: each wave waits for
    // its own part, the barrier makes the parts visible to all.  It also tells that every wave has read the
    // last fragments of A(j-1)... (its slot is the target of the requests that follow).
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(WAITN));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    read_a(sl_n, 0, afr[0]);
    read_sa(sl_n, sa[PAR ^ 1]);
    mfma_step(afr[1], bq[PAR][3], sa[PAR], sb_cur[PAR], T3{}, Keep{});
    issue_a(wa, kta, sl_a, 6, 8);
    issue_as(wa, kta, sl_a);
    load_b(wb2, ktb2, 2, bq[PAR][2]);
    order_step();
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---------------- C tile: accumulators -> the wave's staging area -> global, whole lines per store ----------------
  // acc[i][jn][4q + e] is row lane % 32, column 8q + 4 * (lane / 32) + e of the 32 x 32 tile (i, jn).
  auto store_tile = [&]() {
    uint8_t *stage = c_stage + wave * kStage;
    int lane_v = lane;
    asm volatile("" : "+v"(lane_v));  // addresses recomputed here: they must not live through the main loop
    const int sfr = lane_v & 31, sfg = lane_v >> 5;
    const int lr = lane_v >> 3, lc = lane_v & 7;
    constexpr int ELT = OUT_BF16 ? 2 : 4;
    const int rows = p.m - m0[0];
    const __amdgpu_buffer_rsrc_t c_rsrc =
        make_rsrc_n((uint8_t *)p.c + (int64_t)m0[0] * p.n * ELT, (int)min((int64_t)rows * p.n * ELT, (int64_t)0x7FFFFFFF));
    const int wn0 = n0[0] + wave * 64;
    if (OUT_BF16) {
      typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int i = 0; i < 8; ++i) {  // 32 rows x 64 columns = 32 x 128 bytes
#pragma unroll
        for (int jn = 0; jn < 2; ++jn) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const v16f &a = acc[i][jn];
            const bf4 h = {(__bf16)a[4 * q], (__bf16)a[4 * q + 1], (__bf16)a[4 * q + 2], (__bf16)a[4 * q + 3]};
            const int chunk = jn * 4 + q;
            *(bf4 *)(stage + sfr * 128 + ((chunk ^ (sfr & 7)) << 4) + sfg * 8) = h;
          }
          __builtin_amdgcn_sched_barrier(0);  // 16 accumulator registers at a time through the vector registers
        }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int r0 = 0; r0 < 32; r0 += 8) {
          const int r = r0 + lr;
          const v4i v = *(const v4i *)(stage + r * 128 + ((lc ^ (r & 7)) << 4));
          __builtin_amdgcn_raw_buffer_store_b128(v, c_rsrc, ((i * 32 + r) * p.n + wn0 + lc * 8) * 2, 0, 0);
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);  // one row block at a time: the accumulators stay where they are until then
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
#pragma unroll
        for (int jn = 0; jn < 2; ++jn) {  // 32 rows x 32 columns = 32 x 128 bytes
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const v16f &a = acc[i][jn];
            const v4f v = {a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]};
            const int chunk = q * 2 + sfg;
            *(v4f *)(stage + sfr * 128 + ((chunk ^ (sfr & 7)) << 4)) = v;
          }
          asm volatile("" ::: "memory");
#pragma unroll
          for (int r0 = 0; r0 < 32; r0 += 8) {
            const int r = r0 + lr;
            const v4f v = *(const v4f *)(stage + r * 128 + ((lc ^ (r & 7)) << 4));
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, v), c_rsrc,
                                                   ((i * 32 + r) * p.n + wn0 + jn * 32 + lc * 4) * 4, 0, 0);
          }
          asm volatile("" ::: "memory");
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };
  constexpr int NS = OUT_BF16 ? 32 : 64;  // C store instructions per wave and tile

  // ---------------- prologue: the requests of the three K tiles "before" K tile 0, in the steady order ----------------
  issue_a(0, 0, 0, 0, kALd);
  issue_as(0, 0, 0);
  issue_a(0, 1, 1, 0, kALd);
  issue_as(0, 1, 1);
#pragma unroll
  for (int t = 0; t < 3; ++t) load_b(0, 0, t, bq[0][t]);
  load_bs(0, 0, sb_in[0], sb_in2[0]);
  issue_a(0, 2, 2, 0, 2);
  load_b(0, 0, 3, bq[0][3]);
  issue_a(0, 2, 2, 2, 4);
  load_b(0, 1, 0, bq[1][0]);
  load_bs(0, 1, sb_in[1], sb_in2[1]);
  issue_a(0, 2, 2, 4, 6);
  load_b(0, 1, 1, bq[1][1]);
  issue_a(0, 2, 2, 6, 8);
  issue_as(0, 2, 2);
  load_b(0, 1, 2, bq[1][2]);
  // everything but the last K tile's worth has landed (the one-time cost of filling the pipeline)
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(ops_per_k_tile(SHUF)));
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  read_a(0, 0, afr[0]);
  read_sa(0, sa[0]);
  __builtin_amdgcn_sched_barrier(0);

  // ---------------- the tiles ----------------
  typedef std::integral_constant<int, 0> Even;
  typedef std::integral_constant<int, 1> Odd;
  constexpr int kWaitSteady = wait_steady(SHUF);
  typedef std::integral_constant<int, kWaitSteady> WaitSteady;
  typedef std::integral_constant<int, (kWaitSteady + NS > 63 ? 63 : kWaitSteady + NS)> WaitAfterStore;
  int sl = 0;
  // PENDING: the C stores of the previous output tile are in the queue, between the requests the first wait counts
  auto run_tile = [&](auto pending_tag) -> bool {
    constexpr bool PENDING = decltype(pending_tag)::value;
    typedef typename std::conditional<PENDING, WaitAfterStore, WaitSteady>::type WaitFirst;
    typedef std::true_type Inner;
    typedef std::false_type Edge;
    k_tile(0, sl, Even{}, std::true_type{}, WaitFirst{}, Inner{});  // (nkt >= 6: K tiles 3 and 4 exist)
    k_tile(1, (sl + 1) & 3, Odd{}, Keep{}, WaitSteady{}, Inner{});
    sl = (sl + 2) & 3;
    int j = 2;
    for (; j + 4 < nkt; j += 2) {
      k_tile(j, sl, Even{}, Keep{}, WaitSteady{}, Inner{});
      k_tile(j + 1, (sl + 1) & 3, Odd{}, Keep{}, WaitSteady{}, Inner{});
      sl = (sl + 2) & 3;
    }
    for (; j < nkt; j += 2) {  // the last two pairs: their requests run on into the next output tile
      k_tile(j, sl, Even{}, Keep{}, WaitSteady{}, Edge{});
      k_tile(j + 1, (sl + 1) & 3, Odd{}, Keep{}, WaitSteady{}, Edge{});
      sl = (sl + 2) & 3;
    }
    __builtin_amdgcn_sched_barrier(0);
    store_tile();
    const int npid = pid + (int)gridDim.x;
    if (npid >= padded) return false;
    {
      int tm, tn;
      if (!map_tile(npid, p.tiles_m, p.tiles_n, tm, tn)) return false;
    }
    pid = npid;
    copy_tile(0, 1);
    if (!set_tile(1, pid + (int)gridDim.x)) copy_tile(1, 0);
    __builtin_amdgcn_sched_barrier(0);
    return true;
  };
  if (run_tile(std::false_type{})) {
    while (run_tile(std::true_type{})) {
    }
  }
  __builtin_amdgcn_s_waitcnt(0);  // the trailing requests must not outlive the workgroup's LDS and registers
}

template <bool OUT_BF16, bool SHUF = false>
__global__ void __launch_bounds__(kAsymNT, 1) asym_gemm_kernel(const GemmParams p) {
  asym_body<OUT_BF16, SHUF>(p);
}

template <bool OUT_BF16, bool SHUF>
hipError_t launch_asym_out(const GemmParams &p, int grid_x, hipStream_t stream) {
  static LdsAttrOnce once;
  hipError_t e = allow_dynamic_lds(once, (const void *)asym_gemm_kernel<OUT_BF16, SHUF>, kAsymLds);
  if (e != hipSuccess) return e;
  asym_gemm_kernel<OUT_BF16, SHUF><<<dim3(grid_x, 1, 1), dim3(kAsymNT), kAsymLds, stream>>>(p);
  return hipGetLastError();
}

}  // namespace

// Whether the asymmetric kernel serves this problem (`forced`: the caller named the variant, so a problem with
// fewer tiles than CUs is taken too).
bool asym_gemm_applies(const GemmParams &p, int num_cus, bool forced) {
  if (!p.b_preshuffled || p.num_groups != 0 || p.tile_table != nullptr || p.splits != 1 || p.partial != nullptr) return false;
  const bool shuffled = p.a_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE && p.b_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE;
  if (!shuffled && (p.a_scale_layout != WAVE_MXFP4_SCALE_MFMA32 || p.b_scale_layout != WAVE_MXFP4_SCALE_MFMA32)) return false;
  if ((p.n & 255) != 0 || (p.k & 511) != 0 || p.k_tiles < 6 || p.m < 1) return false;
  // 32-bit offsets inside one operand tile and one C tile
  if ((int64_t)256 * p.kp >= ((int64_t)1 << 31) || (int64_t)256 * p.n * 4 >= ((int64_t)1 << 31)) return false;
  if ((int64_t)8 * p.k_tiles * 256 >= ((int64_t)1 << 31)) return false;
  const int grid = num_cus / kNumXcd * kNumXcd;
  if (grid < kNumXcd) return false;
  const int64_t tiles = (int64_t)((p.m + 255) / 256) * (p.n / 256);
  return forced || tiles > grid;
}

hipError_t launch_asym_gemm(const GemmParams &p, int num_cus, hipStream_t stream) {
  const int grid = num_cus / kNumXcd * kNumXcd;
  if (p.a_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE)
    return p.out_bf16 ? launch_asym_out<true, true>(p, grid, stream) : launch_asym_out<false, true>(p, grid, stream);
  return p.out_bf16 ? launch_asym_out<true, false>(p, grid, stream) : launch_asym_out<false, false>(p, grid, stream);
}

}  // namespace wave_mxfp4

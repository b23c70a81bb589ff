// MXFP4 GEMM for 64 < M <= 256 against a wide, preshuffled B that comes from HBM (gfx950, MI355X):
// A through LDS, B straight from global memory into registers, one workgroup per strip of 128 columns.
//
// In this range the operation is still bound by reading B once, and what limits a CU is how long before its use
// it can ask for B: a request takes 2-3 us to come back under load, and with A and B both landing in LDS (the
// strip kernel for row-major B) the ring of B holds three K tiles at 128 rows.  Here, as in the reference's
// asymmetric kernels (wave_lang/kernel/wave/templates/tagged_mxfp4_gemm.py:950-991, schedule
// wave_lang/kernel/wave/schedules/gemm_mxfp4_double_buffer.py:1781-2222: "B (data + scale): global -> VGPRs
// directly"),
//   * a workgroup is 4 waves side by side along N: each owns all BM rows (128 or 256) and 32 columns of the
//     strip (BM / 32 MFMA tiles of 32 x 32, v_mfma_scale_f32_32x32x64_f8f6f4);
//   * A and its scales go global -> LDS by DMA into a ring that takes all of the LDS: 8 K tiles at BM = 128,
//     4 at BM = 256, requested 5 / 3 K tiles ahead;
//   * B needs no LDS: in b_preshuffle order the 16 bytes a lane feeds to one MFMA are one coalesced 16-byte load
//     (256 contiguous bytes per 16 lanes), non-temporal.  Four K tiles of B fragments live in registers; each
//     register is reloaded right after the MFMA that read it with the data of four K tiles later (a wave has at
//     most 63 memory operations in flight; eight K tiles of B were measured and are no faster);
//   * a workgroup starts at its own K tile and walks around the end of K: all workgroups asking for the same 128
//     bytes of every row at once would keep a few memory channels busy and the rest idle.  The sums of a strip
//     are the same terms in another order.
// One barrier per K tile.  The waits for A are counted (s_waitcnt vmcnt(n)): vector memory operations retire in
// issue order, and every wave issues the same operations per K tile in a fixed order.
//
// Taken for preshuffled B, both scale tensors in MFMA32 order, N % 32 == 0, K a multiple of 1024 (BM = 256) or
// 2048 (BM = 128): the K loop is unrolled over the ring.  Dense, no split.
#include <type_traits>

#include "mxfp4_tile_common.h"

namespace wave_mxfp4 {

namespace {

constexpr int kMidbWaves = 4, kMidbNT = kMidbWaves * 64, kMidbBN = 128;
constexpr int kMidbOnce = 2;   // the "nt" bit: B is read exactly once (M = 128: 31.4 -> 30.1 us on one box)
constexpr int kMidbBSets = 4;  // K tiles of B fragments in registers (8 of them: 31.6 us against 29.6)
constexpr int kMidbDead = (int)0x80000000;  // a scalar offset past the end of any descriptor: nothing is fetched

template <int BM_>
struct MidbCfg {
  static constexpr int BM = BM_, MT = BM / 32;
  static constexpr int SLOT = BM * kTileKBytes;        // 16 / 32 KB of A per K tile
  static constexpr int RING = BM == 256 ? 4 : 8;       // K tiles of A in LDS = K tiles of B in registers = unroll
  static constexpr int LA = BM == 256 ? 3 : 5;         // A is requested this many K tiles ahead (7 at BM = 128: the same)
  static constexpr int SSLOT = MT * 256;               // A scales of one K tile
  static constexpr int STAGE = 4096;                   // C staging per wave
  static constexpr int LDS = RING * SLOT + RING * SSLOT + kMidbWaves * STAGE;
  static constexpr int A_LD = BM / 8 / kMidbWaves;     // A DMA instructions per wave and K tile (4 / 8)
  static constexpr int AS_LD = MT / kMidbWaves;        // A scale DMA instructions per wave and K tile (1 / 2)
  static constexpr int OPS = A_LD + AS_LD + 4 + 1;     // vector memory operations per wave and K tile
  // At the wait of K tile j (before its fourth K step) A(j + 1) and its scales must have landed.  They were
  // requested in K tile j + 1 - LA, at the latest as the last operations of its fourth K step, followed by the
  // operations of LA - 2 whole K tiles and those of the first three K steps of K tile j.
  static constexpr int OPS_3 = (A_LD / 4 + 1) * 3;
  static constexpr int WAIT = (LA - 2) * OPS + OPS_3;
  static_assert(LDS <= 160 * 1024, "LDS");
  static_assert(WAIT <= 63, "vmcnt holds 6 bits");
};

template <class Cfg, bool OUT_BF16>
__device__ __forceinline__ void midb_body(const GemmParams &p) {
  constexpr int MT = Cfg::MT, NW = kMidbWaves, RING = Cfg::RING, LA = Cfg::LA;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  uint8_t *const s_ring = smem + RING * Cfg::SLOT;
  uint8_t *const c_stage = s_ring + RING * Cfg::SSLOT;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kp = p.kp, nkt = p.k_tiles;
  const int k_tiles_blocks = nkt * 256;  // bytes of one 32-row block row of scales (MFMA32 order)
  const int n0 = blockIdx.x * kMidbBN;
  // workgroups w, w + 8, ... share an XCD: consecutive ones of them start one K tile apart
  const int kt_start = (int)(blockIdx.x / kNumXcd) % nkt;
  auto wrap = [&](int kt) { return kt >= nkt ? kt - nkt : kt; };  // kt < 2 * nkt

  // descriptors end with their tensors
  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc_n(p.a, rsrc_bytes((int64_t)p.m * kp));
  const __amdgpu_buffer_rsrc_t as_rsrc = make_rsrc_n(p.a_scale, rsrc_bytes((int64_t)((p.m + 31) >> 5) * k_tiles_blocks));
  // 16-row blocks of preshuffled B are contiguous: the strip's columns start at byte n0 * kp
  const __amdgpu_buffer_rsrc_t b_rsrc = make_rsrc_n(p.b + (int64_t)n0 * kp, rsrc_bytes((int64_t)(p.n - n0) * kp));
  const __amdgpu_buffer_rsrc_t bs_rsrc = make_rsrc_n(p.b_scale + (int64_t)(n0 >> 5) * k_tiles_blocks,
                                                     rsrc_bytes((int64_t)((p.n - n0) >> 5) * k_tiles_blocks));

  // ---------------- per-lane offsets ----------------
  // A DMA: instruction d of a wave fills LDS rows (d * 4 + wave) * 8 .. + 7; lane t lands at row t / 8, chunk
  // position t % 8, which must hold chunk (t % 8) ^ swz(row), swz(row) = (row / 2) % 8.
  const int ld_row0 = wave * 8 + (lane >> 3);
  const int a_goff = ld_row0 * kp + (((lane & 7) ^ ((ld_row0 >> 1) & 7)) << 4);
  const int a_step = NW * 8 * kp;  // bytes between consecutive d
  // B fragment of the 32x32x64 MFMA straight from b_preshuffle order: lane = (row r = lane % 32, K half = lane / 32)
  const int fr = lane & 31, fg = lane >> 5;
  const int b_goff = wave * 32 * kp + (fr >> 4) * 16 * kp + fg * 256 + (fr & 15) * 16;
  const int s_goff = lane * 4;  // a lane's dword of a 256-byte scale block
  // A fragment reads: row fr of a 32-row block, chunk 2t + fg at its swizzled position
  uint32_t foff[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) foff[t] = (uint32_t)(fr * kTileKBytes + (((t * 2 + fg) ^ ((fr >> 1) & 7)) << 4));

  // ---------------- request streams ----------------
  // `dead`: 0, or kMidbDead for the requests that the last turn of the walk issues for K tiles past its end: the
  // scalar offset puts them past the end of the descriptor, they fetch nothing and land zeros that nobody reads.
  // quarter q of the A DMA instructions of K tile kt into ring slot `slot`
  auto issue_a = [&](int kt, int slot, int q, int dead) {
#pragma unroll
    for (int d = q * (Cfg::A_LD / 4); d < (q + 1) * (Cfg::A_LD / 4); ++d)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, WAVE_LDS_PTR(smem + slot * Cfg::SLOT + (d * NW + wave) * 1024), 16,
                                               a_goff, (kt * kTileKBytes + d * a_step) | dead, 0, 0);
  };
  // A scales: a wave instruction of 4 bytes per lane moves one 256-byte block (32 rows x one K tile)
  auto issue_as = [&](int kt, int slot, int dead) {
#pragma unroll
    for (int b = 0; b < Cfg::AS_LD; ++b) {
      const int rb = wave * Cfg::AS_LD + b;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(as_rsrc, WAVE_LDS_PTR(s_ring + slot * Cfg::SSLOT + rb * 256), 4, s_goff,
                                               (rb * k_tiles_blocks + kt * 256) | dead, 0, 0);
    }
  };
  auto load_b = [&](int kt, int t, v4i &dst, int dead) {
    dst = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, b_goff, ((kt * 4 + t) * 512) | dead, kMidbOnce);
  };
  auto load_bs = [&](int kt, uint32_t &dst, int dead) {
    dst = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(bs_rsrc, s_goff, (wave * k_tiles_blocks + kt * 256) | dead, 0);
  };

  // ---------------- registers ----------------
  v16f acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int g = 0; g < 16; ++g) acc[i][g] = 0.f;
  v4i bq[kMidbBSets][4];        // [K tile mod sets][K step]
  uint32_t sb_in[kMidbBSets];   // B scales arriving, per set
  uint32_t sb_cur;        // ... of the K tile being multiplied
  uint32_t sa[2][MT];     // A scales per parity of the K tile
  v4i afr[2][MT];         // A fragments, double buffered by K step

  auto read_a = [&](int slot, int t, v4i (&dst)[MT]) {
    const uint8_t *base = smem + slot * Cfg::SLOT + foff[t];
#pragma unroll
    for (int i = 0; i < MT; ++i) dst[i] = *(const v4i *)(base + i * 32 * kTileKBytes);
  };
  auto read_sa = [&](int slot, uint32_t (&dst)[MT]) {
    const uint8_t *base = s_ring + slot * Cfg::SSLOT + lane * 4;
#pragma unroll
    for (int i = 0; i < MT; ++i) dst[i] = *(const uint32_t *)(base + i * 256);
  };
  auto mfma_step = [&](const v4i (&fa)[MT], const v4i &fb, const uint32_t (&sca)[MT], uint32_t scb, auto t_tag) {
    constexpr int T = decltype(t_tag)::value;
    const v8i vb = {fb.x, fb.y, fb.z, fb.w, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const v8i va = {fa[i].x, fa[i].y, fa[i].z, fa[i].w, 0, 0, 0, 0};
      // operands swapped (B rows as the matrix A of the instruction): a lane's 4 accumulator registers of a
      // group are 4 consecutive N
      acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vb, va, acc[i], 4, 4, T, (int)scb, T, (int)sca[i]);
    }
  };
  // one K step's instruction mix: MFMAs with the LDS reads and the memory requests spread between them
  auto order_step = [&]() {
#pragma unroll
    for (int g = 0; g < MT; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
  };
  typedef std::integral_constant<int, 0> T0;
  typedef std::integral_constant<int, 1> T1;
  typedef std::integral_constant<int, 2> T2;
  typedef std::integral_constant<int, 3> T3;

  // ---------------- one K tile ----------------
  // U: position in the turn of the ring = the K tile's ring slot, U % 4 its B register set; ka / kb: the K tiles
  // that the A ring and the B registers are refilled with (LA and 4 positions further along the walk).
  //   K step t < 3: a quarter of A(ka); B(kb) K step t into the register this step just read
  //   K step 3:     wait, barrier; the last quarter of A(ka) and its scales; B(kb) K step 3 and its scales
  auto k_tile = [&](int ka, int kb, auto u_tag, int dead_a, int dead_b) {
    constexpr int U = decltype(u_tag)::value;
    constexpr int PAR = U & 1, SB = U % kMidbBSets;
    constexpr int SL_A = (U + LA) % RING, SL_N = (U + 1) % RING;
    // this K tile's B scales were requested four K tiles ago: a real move, pinned here (a compiler copy would be folded
    // into a phi of the loop and wait wherever that lands)
    asm volatile("v_mov_b32 %0, %1" : "=v"(sb_cur) : "v"(sb_in[SB]));
    read_a(U, 1, afr[1]);
    mfma_step(afr[0], bq[SB][0], sa[PAR], sb_cur, T0{});
    issue_a(ka, SL_A, 0, dead_a);
    load_b(kb, 0, bq[SB][0], dead_b);
    order_step();
    __builtin_amdgcn_sched_barrier(0);

    read_a(U, 2, afr[0]);
    mfma_step(afr[1], bq[SB][1], sa[PAR], sb_cur, T1{});
    issue_a(ka, SL_A, 1, dead_a);
    load_b(kb, 1, bq[SB][1], dead_b);
    order_step();
    __builtin_amdgcn_sched_barrier(0);

    read_a(U, 3, afr[1]);
    mfma_step(afr[0], bq[SB][2], sa[PAR], sb_cur, T2{});
    issue_a(ka, SL_A, 2, dead_a);
    load_b(kb, 2, bq[SB][2], dead_b);
    order_step();
    __builtin_amdgcn_sched_barrier(0);

    // A of the next K tile and its scales, requested by all four waves, must be in LDS: each wave waits for its
    // own part, the barrier makes the parts visible to all.  It also tells that every wave has read the last
    // fragments of this K tile; the slot of the K tile before it is the target of this K tile's requests.
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(Cfg::WAIT));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    read_a(SL_N, 0, afr[0]);
    read_sa(SL_N, sa[PAR ^ 1]);
    mfma_step(afr[1], bq[SB][3], sa[PAR], sb_cur, T3{});
    issue_a(ka, SL_A, 3, dead_a);
    issue_as(ka, SL_A, dead_a);
    load_b(kb, 3, bq[SB][3], dead_b);
    load_bs(kb, sb_in[SB], dead_b);
    order_step();
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---------------- prologue: A of the first LA K tiles, B of the first four ----------------
#pragma unroll
  for (int s = 0; s < LA; ++s) {
    const int kt = wrap(kt_start + s);
#pragma unroll
    for (int q = 0; q < 4; ++q) issue_a(kt, s, q, 0);
    issue_as(kt, s, 0);
  }
#pragma unroll
  for (int s = 0; s < kMidbBSets; ++s) {
    const int kt = wrap(kt_start + s);
#pragma unroll
    for (int t = 0; t < 4; ++t) load_b(kt, t, bq[s][t], 0);
    load_bs(kt, sb_in[s], 0);
  }
  // the one-time cost of filling the pipeline: everything lands
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  read_a(0, 0, afr[0]);
  read_sa(0, sa[0]);
  __builtin_amdgcn_sched_barrier(0);

  // ---------------- the K walk, unrolled over the ring ----------------
  // ka, kb: the K tiles LA and 4 positions ahead of the walk, wrapped around the end of K.  In the last turn position U still asks for A of position
  // U + LA and for B of position U + 4 (inside the walk while those are below RING): dead requests beyond.  (Run-
  // time flags of one loop: with the last turn peeled off as code of its own the compiler ran out of registers.)
  int ka = wrap(kt_start + LA), kb = wrap(kt_start + kMidbBSets);
  auto step = [&](auto u_tag, int dead_a, int dead_b) {
    k_tile(ka, kb, u_tag, dead_a, dead_b);
    ka = ka + 1 == nkt ? 0 : ka + 1;
    kb = kb + 1 == nkt ? 0 : kb + 1;
  };
  for (int j = 0; j < nkt; j += RING) {
    const int dead = j + RING >= nkt ? kMidbDead : 0;
#define MIDB_STEP(U) step(std::integral_constant<int, U>{}, U + LA < RING ? 0 : dead, U + kMidbBSets < RING ? 0 : dead)
    MIDB_STEP(0);
    MIDB_STEP(1);
    MIDB_STEP(2);
    MIDB_STEP(3);
    if constexpr (RING == 8) {
      MIDB_STEP(4);
      MIDB_STEP(5);
      MIDB_STEP(6);
      MIDB_STEP(7);
    }
#undef MIDB_STEP
  }
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(0);  // the trailing requests must not outlive the workgroup's LDS and registers

  // ---------------- C: accumulators -> the wave's staging area -> global ----------------
  // acc[i][4q + e] is row lane % 32, column 8q + 4 * (lane / 32) + e of the wave's 32 x 32 tile of row block i.
  const int wn0 = n0 + wave * 32;
  if (wn0 >= p.n) return;  // N % 32 == 0: a wave's columns are all inside N or all outside
  uint8_t *stage = c_stage + wave * Cfg::STAGE;
  constexpr int ELT = OUT_BF16 ? 2 : 4;
  // rows past M lie past the end of the descriptor and are dropped
  const __amdgpu_buffer_rsrc_t c_rsrc = make_rsrc_n(p.c, rsrc_bytes((int64_t)p.m * p.n * ELT));
  if (OUT_BF16) {
    typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
    const int lr = lane >> 2, lc = lane & 3;
#pragma unroll
    for (int i = 0; i < MT; ++i) {  // 32 rows x 32 columns = 32 x 64 bytes
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const v16f &a = acc[i];
        const bf4 h = {(__bf16)a[4 * q], (__bf16)a[4 * q + 1], (__bf16)a[4 * q + 2], (__bf16)a[4 * q + 3]};
        *(bf4 *)(stage + fr * 64 + ((q ^ ((fr >> 1) & 3)) << 4) + fg * 8) = h;
      }
      asm volatile("" ::: "memory");
#pragma unroll
      for (int r0 = 0; r0 < 32; r0 += 16) {
        const int r = r0 + lr;
        const v4i v = *(const v4i *)(stage + r * 64 + ((lc ^ ((r >> 1) & 3)) << 4));
        __builtin_amdgcn_raw_buffer_store_b128(v, c_rsrc, ((i * 32 + r) * p.n + wn0 + lc * 8) * 2, 0, 0);
      }
      asm volatile("" ::: "memory");
    }
  } else {
    const int lr = lane >> 3, lc = lane & 7;
#pragma unroll
    for (int i = 0; i < MT; ++i) {  // 32 rows x 32 columns = 32 x 128 bytes
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const v16f &a = acc[i];
        const v4f v = {a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]};
        const int chunk = q * 2 + fg;
        *(v4f *)(stage + fr * 128 + ((chunk ^ (fr & 7)) << 4)) = v;
      }
      asm volatile("" ::: "memory");
#pragma unroll
      for (int r0 = 0; r0 < 32; r0 += 8) {
        const int r = r0 + lr;
        const v4f v = *(const v4f *)(stage + r * 128 + ((lc ^ (r & 7)) << 4));
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, v), c_rsrc, ((i * 32 + r) * p.n + wn0 + lc * 4) * 4, 0,
                                               0);
      }
      asm volatile("" ::: "memory");
    }
  }
}

template <class Cfg, bool OUT_BF16>
__global__ void __launch_bounds__(kMidbNT, 1) midb_gemm_kernel(const GemmParams p) {
  midb_body<Cfg, OUT_BF16>(p);
}

template <class Cfg, bool OUT_BF16>
hipError_t launch_midb_out(const GemmParams &p, hipStream_t stream) {
  static LdsAttrOnce once;
  hipError_t e = allow_dynamic_lds(once, (const void *)midb_gemm_kernel<Cfg, OUT_BF16>, Cfg::LDS);
  if (e != hipSuccess) return e;
  const int strips = (p.n + kMidbBN - 1) / kMidbBN;
  midb_gemm_kernel<Cfg, OUT_BF16><<<dim3(strips, 1, 1), dim3(kMidbNT), Cfg::LDS, stream>>>(p);
  return hipGetLastError();
}

// rows of the block the kernel takes for `m` rows, 0 if none does
int midb_block_rows(const GemmParams &p) {
  if (p.m < 1 || p.m > 256) return 0;
  const int bm = p.m <= 128 ? 128 : 256;
  const int unroll = bm == 256 ? MidbCfg<256>::RING : MidbCfg<128>::RING;
  return p.k_tiles % unroll == 0 ? bm : (bm == 128 && p.k_tiles % MidbCfg<256>::RING == 0 ? 256 : 0);
}

}  // namespace

// Whether the kernel serves this problem: preshuffled B, dense, both scale tensors in MFMA32 order, whole K
// tiles in whole turns of the ring.
bool midb_gemm_applies(const GemmParams &p) {
  if (!p.b_preshuffled || p.num_groups != 0 || p.tile_table != nullptr || p.splits != 1 || p.partial != nullptr) return false;
  if (p.a_scale_layout != WAVE_MXFP4_SCALE_MFMA32 || p.b_scale_layout != WAVE_MXFP4_SCALE_MFMA32) return false;
  if ((p.n & 31) != 0 || (p.k & (kTileK - 1)) != 0 || p.k_tiles * 256 != p.k) return false;
  if (midb_block_rows(p) == 0) return false;
  // 32-bit offsets: a strip of B, all of A, all of C
  if ((int64_t)kMidbBN * p.kp >= ((int64_t)1 << 31) || (int64_t)256 * p.kp >= ((int64_t)1 << 31) ||
      (int64_t)256 * p.n * 4 >= ((int64_t)1 << 31) || (int64_t)8 * p.k_tiles * 256 >= ((int64_t)1 << 31))
    return false;
  return true;
}

hipError_t launch_midb_gemm(const GemmParams &p, hipStream_t stream) {
  if (midb_block_rows(p) == 128)
    return p.out_bf16 ? launch_midb_out<MidbCfg<128>, true>(p, stream) : launch_midb_out<MidbCfg<128>, false>(p, stream);
  return p.out_bf16 ? launch_midb_out<MidbCfg<256>, true>(p, stream) : launch_midb_out<MidbCfg<256>, false>(p, stream);
}

}  // namespace wave_mxfp4

// Asymmetric persistent MXFP8 GEMM for gfx950 (MI355X): A through LDS, B straight from global memory into
// registers, out of a preshuffled 8-bit layout of this library (wave_mxfp8_b_preshuffle).
//
// The 8-bit form of mxfp4_gemm_asym.hip (the reference's "A: global -> LDS -> VGPRs, B: global -> VGPRs directly"
// schedule, wave_lang/kernel/wave/schedules/gemm_mxfp4_double_buffer.py:1781-2222, applied to the operands of
// tests/kernel/wave_gemm_mxfp_test.py:416-501).  With both 8-bit operands in LDS the 160 KB hold 2.5 K tiles of 128
// elements; here LDS holds four K tiles of A and the registers two K tiles of B.
//   * A workgroup is 4 waves side by side along N: each owns all 256 rows and 64 columns of the 256 x 256 output
//     tile (8 x 2 MFMA tiles of 32 x 32, v_mfma_scale_f32_32x32x64_f8f6f4 with 8-bit operands: 32 bytes per lane
//     and operand, 64 cycles per instruction).
//   * A K tile is 128 elements = 128 bytes of a row = two K steps.  A K step's 16 MFMAs run as two phases of 8 (row
//     blocks 0..3, then 4..7), so that the A fragments are double buffered by half a K step: 64 registers, as
//     many as the 4-bit kernel needs for whole K steps.  Four phases per K tile, each with the request mix of one
//     K step of the 4-bit kernel: the counted waits are the same.
//   * B [N, K] in preshuffled order: blocks of 32 rows x 128 bytes (one K tile), 4 KB each, block (n / 32, kt) at
//     ((n / 32) * K / 128 + kt) * 4096; inside, the 16-byte pieces in the order [K step 0..1][half 0..1][lane 0..63],
//     lane = 32 * g + r holding row r's bytes 64 * step + 32 * half + 16 * g .. + 15 of the K tile: one coalesced
//     kilobyte per load instruction, and a wave walks its 32 rows' K tiles front to back.  (The instruction takes
//     a lane's 32 bytes of an 8-bit operand as two halves 32 bytes apart in K.)
//   * Scales: both tensors in MFMA32 order; one 256-byte block serves two K tiles (bytes 0, 1 of a lane's dword
//     for the even one, 2, 3 for the odd one, picked by the instruction's byte selector, a constant per phase).
//   * FMT_B = 4: 8-bit A against packed MXFP4 B [N, K/2] in the reference's b_preshuffle order
//     (wave_lang/kernel/wave/utils/mxfp_utils.py:98-110), read as the MXFP4 B-direct kernel reads it: a K step is
//     one 16-byte load per lane and column half, four B loads per K tile instead of eight.
// Taken for N % 256 == 0, K % 256 == 0, K >= 768, A 8-bit (e4m3 / e5m2), B 8-bit or e2m1, dense.  Any M.
#include <type_traits>

#include "mxfp4_tile_common.h"

namespace wave_mxfp4 {

namespace {

constexpr int kBM = 256, kBN = 256, kNW = 4, kNT = kNW * 64;
constexpr int kARing = 4;                 // K tiles of A in LDS
constexpr int kASlot = kBM * kTileKBytes;  // 32 KB
constexpr int kSSlot = kNW * 1024;         // A scales of one K tile: 2 KB used, 1 KB per wave written
constexpr int kStage = 4096;               // C staging per wave
constexpr int kLds = kARing * kASlot + kARing * kSSlot + kNW * kStage;  // 160 KB
constexpr int kALd = kBM / 8 / kNW;        // A DMA instructions per wave and K tile (8)
// Vector memory operations per wave and K tile: A 8, A scales 1, B 8 (two K steps x two column halves x two
// 16-byte halves; a 4-bit B: one 16-byte load each, 4), B scales 2.
constexpr int ops_per_k_tile(bool b4) { return kALd + 1 + (b4 ? 4 : 8) + 2; }
// At the wait of K tile g (before its fourth phase) A and its scales of K tile g + 1 must have landed.  They were
// requested in K tile g - 2 (at the latest as the last operations of its fourth phase), followed by the 19 (15) of
// K tile g - 1 and the 4 + 4 + 6 (3 + 3 + 5) of the first three phases of K tile g.
constexpr int wait_steady(bool b4) { return ops_per_k_tile(b4) + (b4 ? 11 : 14); }
static_assert(kLds <= 160 * 1024, "LDS");

template <bool OUT_BF16, int FMT_A, int FMT_B>
__device__ __forceinline__ void asym8_body(const GemmParams &p) {
  constexpr int BM = kBM, BN = kBN, NW = kNW;
  constexpr bool B4 = FMT_B == 4;
  static_assert(FMT_A == 0 || FMT_A == 1, "A is 8-bit");
  typedef typename std::conditional<B4, v4i, v8i>::type FragB;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  uint8_t *const s_ring = smem + kARing * kASlot;
  uint8_t *const c_stage = s_ring + kARing * kSSlot;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kp = p.kp, nkt = p.k_tiles;  // bytes of a row of A, K tiles of 128 elements
  const int kpb = B4 ? kp >> 1 : kp;     // bytes of a row of B
  const int total = p.tiles_m * p.tiles_n;
  const int padded = (total + kNumXcd - 1) / kNumXcd * kNumXcd;
  const int s_stride = (nkt >> 1) * 256;  // bytes of one 32-row block row of scales (MFMA32 order, K % 256 == 0)
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
    as_base[which] = p.a_scale + (int64_t)(m0[which] >> 5) * s_stride;
    as_lim[which] = (int)min((int64_t)max(m_blocks - (m0[which] >> 5), 0) * s_stride, (int64_t)0x7FFFFFFF);
    // the 32-row blocks of a column tile are contiguous: they start at byte n0 * kp
    b_base[which] = p.b + (int64_t)n0[which] * kpb;
    b_lim[which] = (int)min((int64_t)(p.n - n0[which]) * kpb, (int64_t)0x7FFFFFFF);
    bs_base[which] = p.b_scale + (int64_t)(n0[which] >> 5) * s_stride;
    bs_lim[which] = (int)min((int64_t)((p.n - n0[which]) >> 5) * s_stride, (int64_t)0x7FFFFFFF);
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
  // A DMA: instruction d of a wave fills LDS rows (d * 4 + wave) * 8 .. + 7; lane t lands at row t / 8, chunk
  // position t % 8, which must hold chunk (t % 8) ^ swz(row), swz(row) = (row / 2) % 8.
  const int ld_row0 = wave * 8 + (lane >> 3);
  const int a_goff = ld_row0 * kp + (((lane & 7) ^ ((ld_row0 >> 1) & 7)) << 4);
  const int a_step = NW * 8 * kp;  // bytes between consecutive d
  // A scale DMA: lanes 0..15 fetch block 2 * wave, lanes 16..31 block 2 * wave + 1 (16 bytes each) of the tile's
  // eight 256-byte blocks; the other half of the wave points past the end of any buffer.
  const int as_goff = lane < 32 ? (2 * wave + (lane >> 4)) * s_stride + (lane & 15) * 16 : (int)0x80000000;
  const int fr = lane & 31, fg = lane >> 5;
  // B: the lane's 16 bytes of a kilobyte; the wave's 64 columns are the 32-row blocks 2 * wave and 2 * wave + 1
  // (4-bit B in b_preshuffle order: 16-row blocks, a K step of a block 512 bytes, lane = (row fr, K half fg))
  const int b_goff = B4 ? wave * 64 * kpb + (fr >> 4) * 16 * kpb + fg * 256 + (fr & 15) * 16 : wave * 64 * kp + lane * 16;
  const int bs_goff = (2 * wave) * s_stride + lane * 4;
  // A fragment reads: row fr of a 32-row block; K step s takes the chunks 4 s + fg and 4 s + 2 + fg
  uint32_t foff[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
    foff[t] = (uint32_t)(fr * kTileKBytes + ((((t >> 1) * 4 + (t & 1) * 2 + fg) ^ ((fr >> 1) & 7)) << 4));

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
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, WAVE_LDS_PTR(s_ring + slot * kSSlot + wave * 1024), 16, as_goff,
                                             (kt >> 1) * 256, 0, 0);
  };
  // the B fragment of K step s for the 32-column half jn of the wave's 64 columns
  auto load_b = [&](int which, int kt, int s, int jn, FragB &dst) {
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc_n(b_base[which], b_lim[which]);
    if constexpr (B4) {
      dst = __builtin_amdgcn_raw_buffer_load_b128(rsrc, b_goff, jn * 32 * kpb + (kt * 2 + s) * 512, 0);
    } else {
      const int soff = jn * 32 * kp + kt * 4096 + s * 2048;
      const v4i lo = __builtin_amdgcn_raw_buffer_load_b128(rsrc, b_goff, soff, 0);
      const v4i hi = __builtin_amdgcn_raw_buffer_load_b128(rsrc, b_goff, soff + 1024, 0);
      dst = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
  };
  auto load_bs = [&](int which, int kt, uint32_t (&dst)[2]) {
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc_n(bs_base[which], bs_lim[which]);
#pragma unroll
    for (int jn = 0; jn < 2; ++jn)
      dst[jn] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, bs_goff, jn * s_stride + (kt >> 1) * 256, 0);
  };

  // ---------------- registers ----------------
  v16f acc[8][2];
  FragB bq[2][2][2];                   // [parity of the K tile][K step][jn]
  uint32_t sb_cur[2][2], sb_in[2][2];  // B scales in use / arriving, per parity
  uint32_t sa[2][8];                   // A scales per parity
  v8i afr[2][4];                       // A fragments of four row blocks, double buffered by phase

  // row blocks 4 hh .. 4 hh + 3 of K step s
  auto read_a = [&](int slot, int s, int hh, v8i (&dst)[4]) {
    const uint8_t *lo = smem + slot * kASlot + hh * 4 * 32 * kTileKBytes + foff[2 * s];
    const uint8_t *hi = smem + slot * kASlot + hh * 4 * 32 * kTileKBytes + foff[2 * s + 1];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const v4i l = *(const v4i *)(lo + i * 32 * kTileKBytes);
      const v4i h = *(const v4i *)(hi + i * 32 * kTileKBytes);
      dst[i] = v8i{l.x, l.y, l.z, l.w, h.x, h.y, h.z, h.w};
    }
  };
  auto read_sa = [&](int slot, uint32_t (&dst)[8]) {
    // block i of the tile's eight was fetched by wave i / 2 into the lower half of its kilobyte
    const uint8_t *base = s_ring + slot * kSSlot + lane * 4;
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[i] = *(const uint32_t *)(base + (i >> 1) * 1024 + (i & 1) * 256);
  };
  // T: the byte of the scale dwords (2 * parity of the K tile + K step); HH: which four row blocks
  auto mfma_phase = [&](const v8i (&fa)[4], const FragB (&fb)[2], const uint32_t (&sca)[8], const uint32_t (&scb)[2],
                        auto t_tag, auto hh_tag, auto zero_tag) {
    constexpr int T = decltype(t_tag)::value;
    constexpr int HH = decltype(hh_tag)::value;
    constexpr bool ZERO = decltype(zero_tag)::value;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int jn = 0; jn < 2; ++jn) {
        v16f c = acc[4 * HH + i][jn];
        if (ZERO) {
#pragma unroll
          for (int g = 0; g < 16; ++g) c[g] = 0.f;
        }
        // operands swapped (B rows as the matrix A of the instruction): a lane's 4 accumulator registers of a
        // group are 4 consecutive N
        v8i vb;
        if constexpr (B4) vb = v8i{fb[jn].x, fb[jn].y, fb[jn].z, fb[jn].w, 0, 0, 0, 0};
        else vb = fb[jn];
        acc[4 * HH + i][jn] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vb, fa[i], c, FMT_B, FMT_A, T, (int)scb[jn], T,
                                                                              (int)sca[4 * HH + i]);
      }
    }
  };
  // one phase's instruction mix: MFMAs with the LDS reads and the memory requests spread between them
  auto order_phase = [&]() {
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
  };
  typedef std::integral_constant<int, 0> I0;
  typedef std::integral_constant<int, 1> I1;
  typedef std::false_type Keep;

  // ---------------- one K tile ----------------
  // j: K tile of the current output tile; sl: its ring slot; PAR: parity of j; ZERO: first K tile of an output
  // tile; WAITN: operations that may still be in flight at the wait.
  //   phase 0 (K step 0, row blocks 0..3): A(j+3) d 0,1; B(j+1) K step 1, columns 0..31
  //   phase 1 (K step 0, row blocks 4..7): A(j+3) d 2,3; B(j+1) K step 1, columns 32..63
  //   phase 2 (K step 1, row blocks 0..3): A(j+3) d 4,5; B(j+2) K step 0, columns 0..31; B scales (j+2)
  //   phase 3 (K step 1, row blocks 4..7): wait, barrier; A(j+3) d 6,7; A scales (j+3); B(j+2) K step 0, columns 32..63
  // (every B register is requested anew right after the phases that read it)
  // INNER: every K tile requested from here (up to j + 3) still belongs to the current output tile.
  auto k_tile = [&](int j, int sl, auto par_tag, auto zero_tag, auto wait_tag, auto inner_tag) {
    constexpr int PAR = decltype(par_tag)::value;
    constexpr int WAITN = decltype(wait_tag)::value;
    constexpr bool INNER = decltype(inner_tag)::value;
    typedef std::integral_constant<int, 2 * PAR> S0;
    typedef std::integral_constant<int, 2 * PAR + 1> S1;
    const int ja = j + 3, wa = !INNER && ja >= nkt ? 1 : 0, kta = ja - (wa ? nkt : 0);
    const int jb1 = j + 1, wb1 = !INNER && jb1 >= nkt ? 1 : 0, ktb1 = jb1 - (wb1 ? nkt : 0);
    const int jb2 = j + 2, wb2 = !INNER && jb2 >= nkt ? 1 : 0, ktb2 = jb2 - (wb2 ? nkt : 0);
    const int sl_a = (sl + 3) & 3, sl_n = (sl + 1) & 3;

    // this K tile's B scales were requested two K tiles ago into sb_in: real moves, pinned here
#pragma unroll
    for (int jn = 0; jn < 2; ++jn) asm volatile("v_mov_b32 %0, %1" : "=v"(sb_cur[PAR][jn]) : "v"(sb_in[PAR][jn]));

    read_a(sl, 0, 1, afr[1]);
    mfma_phase(afr[0], bq[PAR][0], sa[PAR], sb_cur[PAR], S0{}, I0{}, zero_tag);
    issue_a(wa, kta, sl_a, 0, 2);
    load_b(wb1, ktb1, 1, 0, bq[PAR ^ 1][1][0]);
    order_phase();
    __builtin_amdgcn_sched_barrier(0);

    read_a(sl, 1, 0, afr[0]);
    mfma_phase(afr[1], bq[PAR][0], sa[PAR], sb_cur[PAR], S0{}, I1{}, zero_tag);
    issue_a(wa, kta, sl_a, 2, 4);
    load_b(wb1, ktb1, 1, 1, bq[PAR ^ 1][1][1]);
    order_phase();
    __builtin_amdgcn_sched_barrier(0);

    read_a(sl, 1, 1, afr[1]);
    mfma_phase(afr[0], bq[PAR][1], sa[PAR], sb_cur[PAR], S1{}, I0{}, Keep{});
    issue_a(wa, kta, sl_a, 4, 6);
    load_b(wb2, ktb2, 0, 0, bq[PAR][0][0]);
    load_bs(wb2, ktb2, sb_in[PAR]);
    order_phase();
    __builtin_amdgcn_sched_barrier(0);

    // A(j+1) and its scales, requested two K tiles ago by all four waves, must be in LDS: each wave waits for
    // its own part, the barrier makes the parts visible to all.  It also tells that every wave has read the
    // last fragments of A(j-1)... (its slot is the target of the requests that follow).
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(WAITN));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    read_a(sl_n, 0, 0, afr[0]);
    read_sa(sl_n, sa[PAR ^ 1]);
    mfma_phase(afr[1], bq[PAR][1], sa[PAR], sb_cur[PAR], S1{}, I1{}, Keep{});
    issue_a(wa, kta, sl_a, 6, 8);
    issue_as(wa, kta, sl_a);
    load_b(wb2, ktb2, 0, 1, bq[PAR][0][1]);
    order_phase();
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
            // (f32 C of a large problem is more than the memory-side cache holds: stored past it)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, v), c_rsrc,
                                                   ((i * 32 + r) * p.n + wn0 + jn * 32 + lc * 4) * 4, 0, 2);
          }
          asm volatile("" ::: "memory");
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };
  constexpr int NS = OUT_BF16 ? 32 : 64;  // C store instructions per wave and tile

  // ---------------- prologue: what the K tiles "before" K tile 0 would have requested, the last in the steady order ----------------
  issue_a(0, 0, 0, 0, kALd);
  issue_as(0, 0, 0);
  issue_a(0, 1, 1, 0, kALd);
  issue_as(0, 1, 1);
  load_b(0, 0, 0, 0, bq[0][0][0]);
  load_b(0, 0, 0, 1, bq[0][0][1]);
  load_bs(0, 0, sb_in[0]);
  issue_a(0, 2, 2, 0, 2);
  load_b(0, 0, 1, 0, bq[0][1][0]);
  issue_a(0, 2, 2, 2, 4);
  load_b(0, 0, 1, 1, bq[0][1][1]);
  issue_a(0, 2, 2, 4, 6);
  load_b(0, 1, 0, 0, bq[1][0][0]);
  load_bs(0, 1, sb_in[1]);
  issue_a(0, 2, 2, 6, 8);
  issue_as(0, 2, 2);
  load_b(0, 1, 0, 1, bq[1][0][1]);
  // everything but the last K tile's worth has landed (the one-time cost of filling the pipeline)
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(ops_per_k_tile(B4)));
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  read_a(0, 0, 0, afr[0]);
  read_sa(0, sa[0]);
  __builtin_amdgcn_sched_barrier(0);

  // ---------------- the tiles ----------------
  typedef std::integral_constant<int, 0> Even;
  typedef std::integral_constant<int, 1> Odd;
  constexpr int kWaitSteady = wait_steady(B4);
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

template <bool OUT_BF16, int FMT_A, int FMT_B>
__global__ void __launch_bounds__(kNT, 1) asym8_gemm_kernel(const GemmParams p) {
  asym8_body<OUT_BF16, FMT_A, FMT_B>(p);
}

template <bool OUT_BF16, int FMT_A, int FMT_B>
hipError_t launch_out(const GemmParams &p, int grid_x, hipStream_t stream) {
  static LdsAttrOnce once;
  hipError_t e = allow_dynamic_lds(once, (const void *)asym8_gemm_kernel<OUT_BF16, FMT_A, FMT_B>, kLds);
  if (e != hipSuccess) return e;
  asym8_gemm_kernel<OUT_BF16, FMT_A, FMT_B><<<dim3(grid_x, 1, 1), dim3(kNT), kLds, stream>>>(p);
  return hipGetLastError();
}

template <int FMT_A, int FMT_B>
hipError_t launch_fmt(const GemmParams &p, int grid_x, hipStream_t stream) {
  return p.out_bf16 ? launch_out<true, FMT_A, FMT_B>(p, grid_x, stream) : launch_out<false, FMT_A, FMT_B>(p, grid_x, stream);
}

}  // namespace

// Whether the kernel serves this problem (`p` in the geometry of an 8-bit A: kp = K bytes of a row, k_tiles = K / 128;
// B in the preshuffled 8-bit order, or packed MXFP4 in b_preshuffle order; both scale tensors in MFMA32 order).
bool asym8_gemm_applies(const GemmParams &p, int num_cus) {
  if (p.num_groups != 0 || p.tile_table != nullptr || p.splits != 1 || p.partial != nullptr) return false;
  if (p.a_scale_layout != WAVE_MXFP4_SCALE_MFMA32 || p.b_scale_layout != WAVE_MXFP4_SCALE_MFMA32) return false;
  if ((p.n & 255) != 0 || (p.k & 255) != 0 || p.k_tiles < 6 || (p.k_tiles & 1) != 0 || p.m < 1 || p.kp != p.k) return false;
  // 32-bit offsets inside one operand tile and one C tile
  if ((int64_t)256 * p.kp >= ((int64_t)1 << 31) || (int64_t)256 * p.n * 4 >= ((int64_t)1 << 31)) return false;
  if ((int64_t)8 * p.k_tiles * 128 >= ((int64_t)1 << 31)) return false;
  return num_cus / kNumXcd * kNumXcd >= kNumXcd;
}

// a_fmt: 0 = e4m3, 1 = e5m2; b_fmt: the same, or 2 = e2m1
hipError_t launch_asym8_gemm(const GemmParams &p, int num_cus, int a_fmt, int b_fmt, hipStream_t stream) {
  const int grid = num_cus / kNumXcd * kNumXcd;
  if (a_fmt == 0)
    return b_fmt == 0 ? launch_fmt<0, 0>(p, grid, stream) : b_fmt == 1 ? launch_fmt<0, 1>(p, grid, stream)
           : b_fmt == 2 ? launch_fmt<0, 4>(p, grid, stream) : hipErrorInvalidValue;
  if (a_fmt == 1)
    return b_fmt == 0 ? launch_fmt<1, 0>(p, grid, stream) : b_fmt == 1 ? launch_fmt<1, 1>(p, grid, stream)
           : b_fmt == 2 ? launch_fmt<1, 4>(p, grid, stream) : hipErrorInvalidValue;
  return hipErrorInvalidValue;
}

}  // namespace wave_mxfp4

// Streaming skinny-M (decode shape) MXFP4 GEMM for gfx950: M <= 64, N large.
//
// The operation is bound by reading B once from HBM (2*M*N*K flops against
// N*K/2 bytes), so the kernel is organised around the memory system:
//
// * B goes global -> LDS with 16-byte-per-lane DMA (buffer_load ... lds), one
//   instruction = 1 KB contiguous of one B row = 8 whole cache lines.  (Loading
//   MFMA fragments straight from global touches 16 half lines per instruction
//   and the vector L1 retires lines, not bytes: that path tops out near
//   2.5 TB/s.)  DMA costs no VGPRs.
// * A (the few activation rows) is loaded ONCE per workgroup into registers in
//   MFMA fragment layout: each of the 4 waves owns a quarter of the workgroup's
//   K range (at most 8 K tiles = 64 VGPRs per 16 rows of A) and streams only
//   that quarter of every B row.
// * Every wave runs a private three-deep pipeline over 16-row B tiles: two
//   tiles live in its LDS buffers and, as soon as a tile has landed, all of its
//   fragments are pulled into registers, which frees the buffer for the DMA of
//   the tile after next BEFORE the MFMAs run.  Two tiles (32 KB per wave,
//   128 KB per CU) are therefore always in flight; waiting is by counted
//   vmcnt, never for an empty queue.  The waves meet only to add their four
//   partial 16x16 tiles through LDS, once per 16 rows of B.
// * A workgroup walks a contiguous range of 16-row B tiles, so the grid is one
//   workgroup per CU and all CUs pull from HBM for the whole kernel.
// * B's scales for a 16-row tile and the wave's K quarter travel by the same
//   DMA (1 KB per tile, 2 KB for the e8m0_shuffle layout whose 32-row blocks
//   interleave both halves) and are picked out of LDS per lane with v_perm.
//
// v_mfma_scale_f32_16x16x128_f8f6f4 is used (16 rows of B per tile balances
// N = 28672 over 256 CUs; MFMA rate is irrelevant here).  Operand order is
// swapped (B rows on the first port) so a lane holds 4 consecutive N of one M
// row.  The reference has no skinny kernel (it runs M = 1 through its generic
// tile kernel, tests/kernel/wave_gemm_mxfp_test.py:296); the contract is the
// same C = dequant(A) . dequant(B)^T.
#include <type_traits>

#include "mxfp4_tile_common.h"

namespace wave_mxfp4 {

constexpr int kStreamWaves = 4;
constexpr int kStreamKtPerWave = 8;                                // K tiles per wave: resident A, 1 KB of a B row
constexpr int kStreamMaxKTiles = kStreamWaves * kStreamKtPerWave;  // per workgroup (K <= 8192)
constexpr int kStreamRowBytes = kStreamKtPerWave * kTileKBytes;    // 1 KB of one B row per DMA instruction
constexpr int kStreamRowPitch = kStreamRowBytes + 32;              // LDS pitch (measured: fragment reads are conflict-free at 32 mod 64)
constexpr int kStreamTileBytes = 16 * kStreamRowPitch;             // one 16-row B tile, one wave's K range
constexpr int kStreamScaleBytes = 2048;                            // its scale image (1 KB used by two layouts)
// Cache policy of the B data loads (the "nt" bit of the buffer instruction): B is read exactly once, and
// marking it non-temporal keeps it from displacing A and the scales (measured: 25.4 -> 23.0 us at M=16).
constexpr int kStreamOnce = 2;

int stream_max_k_tiles() { return kStreamMaxKTiles; }

struct StreamLds {
  uint8_t tile[kStreamWaves][2][kStreamTileBytes];  // two tiles per wave
  uint8_t scales[kStreamWaves][2][kStreamScaleBytes];
  float red[kStreamWaves - 1][4][64][4];            // partial 16x16 tiles of waves 1..3
};
static_assert(sizeof(StreamLds) <= 160 * 1024, "stream kernel LDS");

// s_waitcnt vmcnt(n) only (gfx9 encoding: vm[3:0], exp[6:4], lgkm[11:8], vm[15:14])
template <int N>
__device__ __forceinline__ void stream_wait_vm() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// FULL: every wave owns the same number (1..8) of whole K tiles and the scale rows are whole
// 16-byte pieces, so every B tile costs the same number of DMA instructions,
// nothing is predicated and waits can be counted.  Otherwise (K tails, fewer
// K tiles) the same pipeline runs with predicated loads and full waits.
template <int MT_M, bool FULL, int KW>
__device__ __forceinline__ void stream_body(const GemmParams &p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
  StreamLds &lds = *reinterpret_cast<StreamLds *>(smem_raw);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int fr = lane & 15, fg = lane >> 4;

  // ---- work split: N tiles over workgroups, K tiles over splits and waves ----
  const int nt_total = (p.n + 15) >> 4;
  const uint32_t nt_q = (uint32_t)nt_total / gridDim.x, nt_r = (uint32_t)nt_total - nt_q * gridDim.x;
  const int nt_begin = (int)(blockIdx.x * nt_q + min(blockIdx.x, nt_r));  // the first nt_r workgroups take one more
  const int nt_end = nt_begin + (int)nt_q + (blockIdx.x < nt_r ? 1 : 0);
  if (nt_begin >= nt_end) return;
  const int split = blockIdx.y;
  const int kt_begin = split * p.tiles_per_split;
  const int nkt = min(p.k_tiles, kt_begin + p.tiles_per_split) - kt_begin;
  // The four waves form kw x nw: kw of them share a B tile along K, nw such
  // groups take consecutive tiles (short K: a wave always fetches up to 1 KB of
  // a row, and the fewer waves share a tile the less there is to add up).
  constexpr int kw = FULL ? KW : kStreamWaves, nw = kStreamWaves / kw;
  constexpr int kw_shift = kw == 4 ? 2 : kw == 2 ? 1 : 0;
  const int kq = wave & (kw - 1), nq = wave >> kw_shift;
  const int ktw = FULL ? nkt / kw : (nkt + kStreamWaves - 1) / kStreamWaves;  // <= kStreamKtPerWave
  const int kt0 = kt_begin + kq * ktw;
  const int ntiles = nt_end - nt_begin, steps = (ntiles + nw - 1) >> (2 - kw_shift);
  // tile of this wave in step s (the last step may repeat the last tile: computed, not stored)
  auto tile_of = [&](int s) { return nt_begin + min(s * nw + nq, ntiles - 1); };
  auto tile_valid = [&](int s) { return s * nw + nq < ntiles; };
  const int my_nkt = FULL ? ktw : max(0, min(ktw, kt_begin + nkt - kt0));

  const int kp = p.kp;
  const v4i zero = {0, 0, 0, 0};
  // row-major scale pieces start 16-byte aligned: 8 bytes in front of the wave's first K tile if that is odd
  const int sc_shift = FULL ? (kt0 & 1) * 8 : 0;
  const int tail_chunks = FULL ? 0 : (p.k & (kTileK - 1)) >> 5;  // valid chunks of a partial last K tile
  auto chunk_ok = [&](int kt, int chunk) {
    return FULL || tail_chunks == 0 || kt != p.k_tiles - 1 || chunk < tail_chunks;
  };

  // ---- B data DMA: one instruction = up to 1 KB contiguous ----
  //   row-major   : row r of the tile, K tiles kt0 .. kt0+7 (lane t: K tile t/8, chunk t%8),
  //                 landing at r*pitch + t*16; a fragment (row fr, K tile j, chunk c) is read
  //                 at fr*pitch + j*128 + c*16 (the pitch is 1 KB + 32 B, with which the 16 rows of a
  //                 fragment read fall on different banks).
  //   preshuffled : K step i = 2*j + s of the 16-row block (already in MFMA order: lane l's
  //                 16 bytes at l*16), landing at i*1024 + l*16 and read back from there.
  const bool bpre = p.b_preshuffled != 0;
  // (every descriptor ends with its tensor: an access past it reads zeros instead of a neighbour's memory)
  const __amdgpu_buffer_rsrc_t b_rsrc =
      make_rsrc_n(p.b + (int64_t)nt_begin * 16 * kp, rsrc_bytes(((int64_t)p.n - (int64_t)nt_begin * 16) * kp));
  const int b_voff = bpre ? lane * 16 : min(lane, ktw * 8 - 1) * 16;
  auto issue_rows = [&](int nt, int buf) {
    uint8_t *dst = lds.tile[wave][buf];
    const int tile_off = (nt - nt_begin) * 16 * kp;
    const int row_lim = p.n - 1 - nt * 16;
    if (FULL) {
      // one instruction per i, no control flow: the two layouts differ in scalars only
      // With fewer than 8 K tiles per wave the lanes (row-major) or instructions
      // (preshuffled) past the wave's range fetch its last chunk or K tile again:
      // always the same 16 instructions, and what lands there meets zeros of A.
      const int pitch = bpre ? 1024 : kStreamRowPitch;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int soff = bpre ? tile_off + ((kt0 + min(i >> 1, ktw - 1)) * 4 + (i & 1) * 2) * 512
                              : tile_off + min(i, row_lim) * kp + kt0 * kTileKBytes;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, WAVE_LDS_PTR(dst + i * pitch), 16, b_voff, soff, 0, kStreamOnce);
      }
    } else if (bpre) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int j = i >> 1, s = i & 1;
        if (j < my_nkt) {
          if (chunk_ok(kt0 + j, s * 4 + fg))
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, WAVE_LDS_PTR(dst + i * 1024), 16, lane * 16,
                                                     tile_off + ((kt0 + j) * 4 + s * 2) * 512, 0, kStreamOnce);
          else
            *(v4i *)(dst + i * 1024 + lane * 16) = zero;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        if ((lane >> 3) < my_nkt) {
          if (chunk_ok(kt0 + (lane >> 3), lane & 7))
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, WAVE_LDS_PTR(dst + i * kStreamRowPitch), 16, lane * 16,
                                                     tile_off + min(i, row_lim) * kp + kt0 * kTileKBytes, 0, kStreamOnce);
          else
            *(v4i *)(dst + i * kStreamRowPitch + lane * 16) = zero;
        }
      }
    }
  };
  const uint32_t frag_base = bpre ? (uint32_t)(lane * 16) : (uint32_t)(fr * kStreamRowPitch + fg * 16);
  const uint32_t frag_j = bpre ? 2048u : (uint32_t)kTileKBytes;  // per K tile
  const uint32_t frag_s = bpre ? 1024u : 64u;                    // per K step

  // ---- B scales: an image of the source bytes per B tile and wave ----
  //   row-major : 16 rows x 64 bytes starting at group kt0*8, stored piece-major (lane t -> row
  //               t%16, 16-byte piece t/16, so the 16 rows of a piece are 256 contiguous bytes and
  //               the reads below are conflict-free); K tiles 2q, 2q+1 of row fr are the 16 bytes
  //               at q*256 + fr*16, step s of K tile j byte fg of dword (j%2)*2 + s (one pair of
  //               dwords later when the wave's first K tile is odd: see the alignment note below).
  //   MFMA32    : of each of the 8 consecutive 256-byte blocks (32 rows x one K tile) the two
  //               64-byte runs that hold this tile's 16 rows (lane t -> block t/8, piece t%8);
  //               K tile j of row r is the dword at j*128 + (fg&1)*64 + (r%16)*4, whose bytes
  //               are (step 0, fg/2 = 0), (0, 1), (1, 0), (1, 1).
  //   shuffled  : the 8 whole blocks (both 16-row halves share every dword): K tile j of row r
  //               is the dword at j*256 + fg*64 + (r%16)*4, bytes (step 0, half 0), (0, 1),
  //               (1, 0), (1, 1) with half = (r/16)%2.
  // One v_perm per K tile then forms the MFMA scale operand (step 0 in byte 0, step 1 in byte 1).
  const int bsl = p.b_scale_layout;
  const int sc_block_row_bytes = (p.ksp >> 3) * 256;  // one 32-row tile, all K tiles
  const bool sc_pieces = (p.ks & 15) == 0;
  const __amdgpu_buffer_rsrc_t bs_rsrc =
      make_rsrc_n(p.b_scale, rsrc_bytes(scale_tensor_bytes(p.b_scale_layout, p.n, p.ks, p.ksp)));
  auto issue_scales = [&](int nt, int buf) {
    uint8_t *dst = lds.scales[wave][buf];
    const int n0 = nt * 16;
    const int blocked_off = (n0 >> 5) * sc_block_row_bytes + kt0 * 256;
    if (FULL) {
      // one instruction whatever the layout, a second one for the shuffled blocks
      // (pieces and blocks past the wave's K tiles repeat its last one, and nothing is read past the tensor)
      const int row = min(n0 + (lane & 15), p.n - 1);
      // (the DMA wants 16-byte aligned sources: an odd first K tile starts its image 8 bytes early)
      // (the last wave's pieces end exactly at the end of the row, so nothing is read past the tensor)
      const int off_rm = row * p.ks + kt0 * 8 - sc_shift + min(lane >> 4, (sc_shift + ktw * 8 - 1) >> 4) * 16;
      const int off_native = blocked_off + min(lane >> 3, ktw - 1) * 256 + ((lane & 7) >> 2) * 128 +
                             ((n0 >> 4) & 1) * 64 + (lane & 3) * 16;
      const int off_shuf = blocked_off + min(lane >> 4, ktw - 1) * 256 + (lane & 15) * 16;
      const int off = bsl == WAVE_MXFP4_SCALE_ROW_MAJOR ? off_rm : bsl == WAVE_MXFP4_SCALE_MFMA32 ? off_native : off_shuf;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(bs_rsrc, WAVE_LDS_PTR(dst), 16, off, 0, 0, kStreamOnce);
      if (bsl == WAVE_MXFP4_SCALE_E8M0_SHUFFLE) {
        const int off2 = blocked_off + min(4 + (lane >> 4), ktw - 1) * 256 + (lane & 15) * 16;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(bs_rsrc, WAVE_LDS_PTR(dst + 1024), 16, off2, 0, 0, kStreamOnce);
      }
    } else if (bsl == WAVE_MXFP4_SCALE_ROW_MAJOR) {
      const int row = min(n0 + (lane & 15), p.n - 1);
      const int64_t off = (int64_t)row * p.ks + (int64_t)kt0 * 8 + (lane >> 4) * 16;
      if (sc_pieces && off + 16 <= (int64_t)p.n * p.ks) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(bs_rsrc, WAVE_LDS_PTR(dst), 16, (int)off, 0, 0, 0);
      } else {
        // rows that are not 16-byte multiples: byte copies of the groups that exist
        uint8_t *d8 = dst + lane * 16;
        for (int e = 0; e < 16; ++e) {
          const int g = kt0 * 8 + (lane >> 4) * 16 + e;
          d8[e] = g < p.ks ? p.b_scale[(int64_t)row * p.ks + g] : (uint8_t)127;
        }
      }
    } else if (bsl == WAVE_MXFP4_SCALE_MFMA32) {
      const int blk = lane >> 3, piece = lane & 7;
      const int off = blocked_off + blk * 256 + (piece >> 2) * 128 + ((n0 >> 4) & 1) * 64 + (piece & 3) * 16;
      if (kt0 + blk < p.k_tiles) __builtin_amdgcn_raw_ptr_buffer_load_lds(bs_rsrc, WAVE_LDS_PTR(dst), 16, off, 0, 0, kStreamOnce);
    } else {
      const int off = blocked_off + lane * 16;
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        const int blk = d * 4 + (lane >> 4);
        if (kt0 + blk < p.k_tiles)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(bs_rsrc, WAVE_LDS_PTR(dst + d * 1024), 16, off, d * 1024, 0, 0);
      }
    }
  };
  // per-lane position in the image and byte selector for v_perm (0x0c = constant zero byte)
  const bool sc_rowmajor = bsl == WAVE_MXFP4_SCALE_ROW_MAJOR;

  auto issue_tile = [&](int nt, int buf) {
    if (FULL || my_nkt > 0) {
      issue_scales(nt, buf);
      issue_rows(nt, buf);
    }
  };

  // two B tiles in flight from the start (FULL mode is only launched with at
  // least two tiles per workgroup, which keeps this prologue branch-free)
  issue_tile(tile_of(0), 0);

  // ---- A: resident fragments and scales; issued between the first two B tiles ----
  // All vector memory traffic of the kernel is buffer instructions: with a
  // global_load ... lds pending the compiler treats the queue as unordered and
  // turns every counted wait into a wait for an empty queue.
  //
  // FULL mode loads A in whole cache lines (lane t: row t/8, chunk t%8 of one
  // K tile, two instructions per 16 rows and K tile) and turns the registers
  // into MFMA fragments (lane l: row l%16, chunk l/16) through a small LDS
  // stage after the B stream has been started: fragment-shaped loads touch 16
  // half lines per instruction and cost the vector L1 four times the cycles,
  // in front of the stream.  Scales: one 16-byte piece per lane and row quarter
  // redistributed by ds_bpermute (row-major), or the lane's own dword of each
  // 256-byte block (blocked layouts).  a_sc[..][0] then holds the scales of
  // both K steps in bytes 0 and 1.
  // The generic mode loads fragment-shaped, one scale byte per register.
  v4i a_frag[MT_M][kStreamKtPerWave][2];
  uint32_t a_sc[MT_M][kStreamKtPerWave][2];
  constexpr int kOpselA1 = FULL ? 1 : 0;  // op_sel of the A scale for the second K step
  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc_n(p.a, rsrc_bytes((int64_t)p.m * kp));
  const __amdgpu_buffer_rsrc_t as_rsrc =
      make_rsrc_n(p.a_scale, rsrc_bytes(scale_tensor_bytes(p.a_scale_layout, p.m, p.ks, p.ksp)));
  auto load_b128 = [&](__amdgpu_buffer_rsrc_t r, int voff, int soff) -> v4i {
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    const u4 v = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0);
    return v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
  };
  const int asl = p.a_scale_layout;
  v4i a_sq[MT_M];  // row-major scale pieces
  if (FULL) {
#pragma unroll
    for (int i = 0; i < MT_M; ++i) {
      const int ao0 = min(i * 16 + (lane >> 3), p.m - 1) * kp + (lane & 7) * 16;
      const int ao1 = min(i * 16 + 8 + (lane >> 3), p.m - 1) * kp + (lane & 7) * 16;
#pragma unroll
      for (int j = 0; j < kStreamKtPerWave; ++j) {
        a_frag[i][j][0] = load_b128(a_rsrc, ao0, (kt0 + min(j, ktw - 1)) * kTileKBytes);
        a_frag[i][j][1] = load_b128(a_rsrc, ao1, (kt0 + min(j, ktw - 1)) * kTileKBytes);
      }
      // Both scale shapes are loaded, the one that does not apply from offset
      // 0: separate code paths per layout would make the compiler guard the
      // registers of the other path with waits in front of the stream.
      const bool rm = asl == WAVE_MXFP4_SCALE_ROW_MAJOR;
      // row-major: lane t holds row t/4, bytes 16*(t%4) .. +15 of the wave's 64 = K tiles 2*(t%4), 2*(t%4)+1
      // (16-byte aligned like the image of B's scales: 8 bytes early when the wave's first K tile is odd)
      a_sq[i] = load_b128(as_rsrc,
                          rm ? min(i * 16 + (lane >> 2), p.m - 1) * p.ks + kt0 * 8 - sc_shift +
                                   min(lane & 3, (sc_shift + ktw * 8 - 1) >> 4) * 16
                             : 0,
                          0);
      // blocked: the dword of block (row/32, K tile) that holds this lane's two scale bytes
      const int row = i * 16 + fr;  // rows up to the next multiple of 32 exist in blocked layouts
      const int in_blk = asl == WAVE_MXFP4_SCALE_MFMA32 ? (((fg & 1) << 5) | (row & 31)) * 4 : fg * 64 + (row & 15) * 4;
      const int so = rm ? 0 : (row >> 5) * (p.ksp >> 3) * 256 + in_blk;
#pragma unroll
      for (int j = 0; j < kStreamKtPerWave; ++j)
        a_sc[i][j][0] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(as_rsrc, so, rm ? 0 : (kt0 + min(j, ktw - 1)) * 256, 0);
    }
  } else {
#pragma unroll
    for (int i = 0; i < MT_M; ++i) {
      const int row = min(i * 16 + fr, p.m - 1);
      const int ao = row * kp + fg * 16;
      // scale (row, group kt*8 + s*4 + fg): every layout is linear in kt
      const int so0 = (int)scale_offset(asl, row, fg, p.ks, p.ksp);
      const int so1 = (int)scale_offset(asl, row, 4 + fg, p.ks, p.ksp);
      const int so_kt = asl == WAVE_MXFP4_SCALE_ROW_MAJOR ? 8 : 256;
#pragma unroll
      for (int j = 0; j < kStreamKtPerWave; ++j) {
        a_frag[i][j][0] = a_frag[i][j][1] = zero;
        a_sc[i][j][0] = a_sc[i][j][1] = 127u;
        if (j < my_nkt) {
          const int kt = kt0 + j;
          if (chunk_ok(kt, fg)) a_frag[i][j][0] = load_b128(a_rsrc, ao, kt * kTileKBytes);
          if (chunk_ok(kt, 4 + fg)) a_frag[i][j][1] = load_b128(a_rsrc, ao, kt * kTileKBytes + 64);
          if (kt * 8 + fg < p.ks) a_sc[i][j][0] = __builtin_amdgcn_raw_buffer_load_b8(as_rsrc, so0, kt * so_kt, 0);
          if (kt * 8 + 4 + fg < p.ks) a_sc[i][j][1] = __builtin_amdgcn_raw_buffer_load_b8(as_rsrc, so1, kt * so_kt, 0);
        }
      }
    }
  }


  if (FULL || steps > 1) issue_tile(tile_of(1), 1);

  // Wait until tile nt has landed; tile nt+1 stays in flight.  In FULL mode a
  // tile is 17 DMA instructions (18 with e8m0_shuffle scales, whose first then
  // falls under the wait as well), and the youngest in the queue are those of
  // tile nt+1.
  auto wait_tile = [&](int s) {
    if (FULL && s + 1 < steps) {
      stream_wait_vm<17>();
    } else {
      __builtin_amdgcn_s_waitcnt(0);
    }
    asm volatile("" ::: "memory");
  };
  // Workgroup barrier that orders LDS traffic only: DMA stays in flight across
  // it (a __syncthreads() would wait for vmcnt(0)).
  auto lds_barrier = [&]() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt((7 << 4) | (3 << 14) | 15);  // lgkmcnt(0) only
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  if (FULL) {
    // A into fragment shape.  The stage is the wave's share of the partial-tile
    // area, 16 rows of 128 + 32 bytes (fragment reads then spread over all
    // banks); LDS executes a wave's accesses in order, so one K tile after the
    // other can pass through the same 2.5 KB.
    // (uses of the loaded registers stay behind the DMA issue above)
#pragma unroll
    for (int i = 0; i < MT_M; ++i) {
#pragma unroll
      for (int j = 0; j < kStreamKtPerWave; ++j) asm volatile("" : "+v"(a_sc[i][j][0]));
      asm volatile("" : "+v"(a_sq[i]));
    }
    uint8_t *stage = reinterpret_cast<uint8_t *>(lds.red) + wave * (16 * 160);
    static_assert(kStreamWaves * 16 * 160 <= (int)sizeof(lds.red), "A stage fits the partial-tile area");
    const uint32_t wr = (uint32_t)((lane >> 3) * 160 + (lane & 7) * 16), rd = (uint32_t)(fr * 160 + fg * 16);
#pragma unroll
    for (int i = 0; i < MT_M; ++i) {
#pragma unroll
      for (int j = 0; j < kStreamKtPerWave; ++j) {
        *(v4i *)(stage + wr) = a_frag[i][j][0];
        *(v4i *)(stage + 8 * 160 + wr) = a_frag[i][j][1];
        asm volatile("" ::: "memory");
        a_frag[i][j][0] = *(const v4i *)(stage + rd);
        a_frag[i][j][1] = *(const v4i *)(stage + rd + 64);
        asm volatile("" ::: "memory");
        if (j >= ktw) a_frag[i][j][0] = a_frag[i][j][1] = zero;  // K tiles the wave does not own
      }
      {
        // row-major: K tile j, step s of row fr is byte fg of dword (j%2)*2 + s held by lane fr*4 + j/2;
        // blocked: bytes (step 0, h), (step 1, h) of the lane's dword, h = fg/2 (MFMA32) or the
        // 16-row half (shuffled)
        const bool rm = asl == WAVE_MXFP4_SCALE_ROW_MAJOR;
        const uint32_t h = asl == WAVE_MXFP4_SCALE_MFMA32 ? (uint32_t)(fg >> 1) : (uint32_t)(i & 1);
        const uint32_t sel = rm ? (0x0c0c0000u | (uint32_t)fg | ((uint32_t)(4 + fg) << 8)) : (0x0c0c0000u | h | ((2 + h) << 8));
        const int q[4] = {a_sq[i].x, a_sq[i].y, a_sq[i].z, a_sq[i].w};
#pragma unroll
        for (int j = 0; j < kStreamKtPerWave; ++j) {
          // (with the 8-byte shift K tile j is the (j+1)-th pair of dwords; both candidates are
          // fetched and one is picked, so that no register array is indexed by a run-time value)
          const bool sh = sc_shift != 0;
          const int src0 = (fr * 4 + (j >> 1)) * 4, src1 = (fr * 4 + ((j + 1) >> 1)) * 4;
          const uint32_t p0 = (uint32_t)__builtin_amdgcn_ds_bpermute(src0, q[(j & 1) * 2]);
          const uint32_t p1 = (uint32_t)__builtin_amdgcn_ds_bpermute(src0, q[(j & 1) * 2 + 1]);
          const uint32_t m0 = (uint32_t)__builtin_amdgcn_ds_bpermute(src1, q[((j + 1) & 1) * 2]);
          const uint32_t m1 = (uint32_t)__builtin_amdgcn_ds_bpermute(src1, q[((j + 1) & 1) * 2 + 1]);
          const uint32_t d0 = sh ? m0 : p0, d1 = sh ? m1 : p1;
          a_sc[i][j][0] = __builtin_amdgcn_perm(rm ? d1 : a_sc[i][j][0], rm ? d0 : a_sc[i][j][0], sel);
        }
      }
#pragma unroll
      for (int j = 0; j < kStreamKtPerWave; ++j) {
        if (j >= ktw) a_sc[i][j][0] = 0x7F7Fu;
        a_sc[i][j][1] = a_sc[i][j][0];
      }
    }
    lds_barrier();  // the stage becomes the partial-tile area
    stream_wait_vm<17>();  // tile nt_begin has landed
    asm volatile("" ::: "memory");
  } else {
    wait_tile(0);
  }

  auto store_tile = [&](int nt, int i, int l, const v4f &v) {
    const int m = i * 16 + (l & 15);
    const int n = nt * 16 + (l >> 4) * 4;
    if (m >= p.m || n >= p.n) return;
    const int64_t idx = (int64_t)m * p.n + n;
    const bool vec_ok = (p.n & 3) == 0;
    if (p.partial != nullptr) {
      float *dst = p.partial + (int64_t)split * p.m * p.n + idx;
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
  };

  // ---- the stream ----
  // Per tile t: wait until it has landed (tile t+1 stays in flight), pull its
  // fragments and scales into registers, start the DMA of tile t+2 into the
  // buffer just emptied, multiply, add the four partial tiles through LDS.
  // The sum of a group's tile of step t is formed by its wave t % kw and stays
  // in its registers (kHold tiles per wave): C is written at the end of the
  // kernel, by all four waves at once, so that in the common case no write
  // traffic (16 partial lines per tile) is mixed into the read stream.  With
  // more than kw*kHold steps the oldest held tile is stored just before the DMA
  // issue of the iteration that replaces it: the stores are then older than
  // that DMA and the counted waits stay exact.
  constexpr int kHold = FULL && (MT_M < 4 || KW == 4) ? 2 : 1;  // (64 rows of A leave few registers)
  v4f hold[kHold][MT_M];
  for (int t = 0; t < steps; ++t) {
    const int nt = tile_of(t);
    const int buf = t & 1;
    if (t > 0) wait_tile(t);

    const int n_row = min(nt * 16 + fr, p.n - 1);
    const uint8_t *sc_img = lds.scales[wave][buf];
    const uint8_t *tile = lds.tile[wave][buf] + frag_base;
    v4i bfrag[kStreamKtPerWave][2];
    uint32_t scb[kStreamKtPerWave];
#pragma unroll
    for (int j = 0; j < kStreamKtPerWave; ++j) {
      if (FULL || j < my_nkt) {
        bfrag[j][0] = *(const v4i *)(tile + j * frag_j);
        bfrag[j][1] = *(const v4i *)(tile + j * frag_j + frag_s);
      } else {
        bfrag[j][0] = bfrag[j][1] = zero;
      }
    }
    if (sc_rowmajor) {
      const uint32_t sel = 0x0c0c0000u | (uint32_t)fg | ((uint32_t)(4 + fg) << 8);
      uint32_t d[18];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const v4i v = *(const v4i *)(sc_img + q * 256 + fr * 16);
        d[4 * q] = (uint32_t)v.x, d[4 * q + 1] = (uint32_t)v.y, d[4 * q + 2] = (uint32_t)v.z, d[4 * q + 3] = (uint32_t)v.w;
      }
      d[16] = d[17] = 0x7F7F7F7Fu;
      const bool shifted = sc_shift != 0;  // K tile j then sits one dword pair further on
#pragma unroll
      for (int j = 0; j < kStreamKtPerWave; ++j) {
        // (both candidates are formed and one is picked: an index that depends on
        // `shifted` would put the array in scratch memory)
        const uint32_t plain = __builtin_amdgcn_perm(d[2 * j + 1], d[2 * j], sel);
        const uint32_t moved = __builtin_amdgcn_perm(d[2 * j + 3], d[2 * j + 2], sel);
        scb[j] = shifted ? moved : plain;
      }
    } else {
      const bool native = bsl == WAVE_MXFP4_SCALE_MFMA32;
      const uint32_t h = native ? (uint32_t)(fg >> 1) : (uint32_t)((n_row >> 4) & 1);
      const uint32_t sel = 0x0c0c0000u | h | ((2 + h) << 8);
      const uint32_t *img = (const uint32_t *)(sc_img + (native ? (fg & 1) * 64 : fg * 64) + (n_row & 15) * 4);
      const int stride = native ? 32 : 64;  // dwords per K tile
#pragma unroll
      for (int j = 0; j < kStreamKtPerWave; ++j) {
        const uint32_t d = img[j * stride];
        scb[j] = __builtin_amdgcn_perm(d, d, sel);
      }
    }

    if (FULL) {
      // K tiles the wave does not own: A is zero there, the scale must merely be finite
#pragma unroll
      for (int j = 1; j < kStreamKtPerWave; ++j) {
        if (j >= ktw) scb[j] = 0x7F7Fu;
      }
      // (all eight selects here, ahead of the MFMAs: one directly in front of the MFMA that reads it costs wait states)
#pragma unroll
      for (int j = 0; j < kStreamKtPerWave; ++j) asm volatile("" : "+v"(scb[j]));
    }

    const int reducer = t & (kw - 1);  // the wave of the group that adds up the tile of step t
    const int slot = (t >> kw_shift) & (kHold - 1);
    if (t >= kw * kHold && kq == reducer) {
#pragma unroll
      for (int h = 0; h < kHold; ++h) {
        if (h == slot) {
#pragma unroll
          for (int i = 0; i < MT_M; ++i) store_tile(tile_of(t - kw * kHold), i, lane, hold[h][i]);
        }
      }
    }

    // the buffer is free once the reads above have returned
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt((7 << 4) | (3 << 14) | 15);  // lgkmcnt(0)
    asm volatile("" ::: "memory");
    if (t + 2 < steps) issue_tile(tile_of(t + 2), buf);

    v4f acc[MT_M];
#pragma unroll
    for (int i = 0; i < MT_M; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < kStreamKtPerWave; ++j) {
      if (FULL || j < my_nkt) {
        const v8i vb0 = {bfrag[j][0].x, bfrag[j][0].y, bfrag[j][0].z, bfrag[j][0].w, 0, 0, 0, 0};
        const v8i vb1 = {bfrag[j][1].x, bfrag[j][1].y, bfrag[j][1].z, bfrag[j][1].w, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < MT_M; ++i) {
          const v8i va0 = {a_frag[i][j][0].x, a_frag[i][j][0].y, a_frag[i][j][0].z, a_frag[i][j][0].w, 0, 0, 0, 0};
          const v8i va1 = {a_frag[i][j][1].x, a_frag[i][j][1].y, a_frag[i][j][1].z, a_frag[i][j][1].w, 0, 0, 0, 0};
          acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(vb0, va0, acc[i], 4, 4, 0, (int)scb[j], 0,
                                                                     (int)a_sc[i][j][0]);
          acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(vb1, va1, acc[i], 4, 4, 1, (int)scb[j], kOpselA1,
                                                                     (int)a_sc[i][j][1]);
        }
      }
    }

    // add the partial tiles: the other waves of the group hand theirs to the reducer through LDS
    const int red0 = nq * (kw - 1);  // the group's share of the partial-tile area
    if (kq != reducer) {
#pragma unroll
      for (int i = 0; i < MT_M; ++i) *(v4f *)lds.red[red0 + ((kq - reducer - 1) & (kw - 1))][i][lane] = acc[i];
    }
    lds_barrier();  // partials visible
    if (kq == reducer) {
#pragma unroll
      for (int i = 0; i < MT_M; ++i) {
        v4f v = acc[i];
        for (int w = 0; w < kw - 1; ++w) v += *(const v4f *)lds.red[red0 + w][i][lane];
#pragma unroll
        for (int h = 0; h < kHold; ++h) {
          if (h == slot) hold[h][i] = v;
        }
      }
    }
    lds_barrier();  // red is free again
  }
  // the tiles still held: those of the last kw*kHold (or fewer) steps
  for (int t = max(0, steps - kw * kHold); t < steps; ++t) {
    if (kq == (t & (kw - 1)) && tile_valid(t)) {
#pragma unroll
      for (int h = 0; h < kHold; ++h) {
        if (h == ((t >> kw_shift) & (kHold - 1))) {
#pragma unroll
          for (int i = 0; i < MT_M; ++i) store_tile(tile_of(t), i, lane, hold[h][i]);
        }
      }
    }
  }
}

template <int MT_M, bool FULL, int KW>
__global__ void __launch_bounds__(kStreamWaves * 64, 1) stream_gemm_kernel(const GemmParams p) {
  stream_body<MT_M, FULL, KW>(p);
}

template <int MT_M, bool FULL, int KW>
static hipError_t launch_stream_mt(const GemmParams &p, int grid_x, hipStream_t stream) {
  static LdsAttrOnce once;
  const hipError_t e = allow_dynamic_lds(once, (const void *)stream_gemm_kernel<MT_M, FULL, KW>, (int)sizeof(StreamLds));
  if (e != hipSuccess) return e;
  dim3 grid(grid_x, p.splits, 1);
  stream_gemm_kernel<MT_M, FULL, KW><<<grid, dim3(kStreamWaves * 64), sizeof(StreamLds), stream>>>(p);
  return hipGetLastError();
}

template <bool FULL, int KW>
static hipError_t launch_stream_full(const GemmParams &p, int grid_x, hipStream_t stream) {
  switch ((p.m + 15) / 16) {
    case 1: return launch_stream_mt<1, FULL, KW>(p, grid_x, stream);
    case 2: return launch_stream_mt<2, FULL, KW>(p, grid_x, stream);
    case 3: return launch_stream_mt<3, FULL, KW>(p, grid_x, stream);
    case 4: return launch_stream_mt<4, FULL, KW>(p, grid_x, stream);
    default: return hipErrorInvalidValue;
  }
}

// One workgroup per CU (or per 16-row tile of B if there are fewer tiles).
hipError_t launch_stream_gemm(const GemmParams &p, int num_cus, hipStream_t stream) {
  if (p.tiles_per_split > kStreamMaxKTiles) return hipErrorInvalidValue;
  const int nt_total = (p.n + 15) / 16;
  int grid_x = num_cus > 0 ? num_cus : 256;
  if (p.splits > 1) grid_x = grid_x / p.splits;  // all splits resident at once: one workgroup fills a CU's LDS
  if (grid_x > nt_total) grid_x = nt_total;
  if (grid_x < 1) grid_x = 1;
  // 32-bit DMA offsets inside a workgroup's range of B rows
  if (((int64_t)(nt_total + grid_x - 1) / grid_x + 1) * 16 * p.kp >= ((int64_t)1 << 31)) return hipErrorInvalidValue;
  // ... and into A and both scale matrices (padded to 32-row blocks)
  if ((int64_t)p.m * p.kp >= ((int64_t)1 << 31) || ((int64_t)p.n + 32) * (p.ksp + 8) >= ((int64_t)1 << 31))
    return hipErrorInvalidValue;
  // Counted-wait mode: every wave owns the same number (at most 8) of whole K
  // tiles and sees at least two tiles of B.  As few waves as possible share a
  // tile along K.
  int kw = 0;
  if ((p.k & (kTileK - 1)) == 0 && p.k_tiles % p.tiles_per_split == 0) {
    for (int c = 1; c <= kStreamWaves && kw == 0; c *= 2) {
      if (p.tiles_per_split % c == 0 && p.tiles_per_split / c <= kStreamKtPerWave &&
          nt_total >= 2 * (kStreamWaves / c) * grid_x)
        kw = c;
    }
  }
  if (kw != 0) {
    switch (kw) {
      case 1: return launch_stream_full<true, 1>(p, grid_x, stream);
      case 2: return launch_stream_full<true, 2>(p, grid_x, stream);
      default: return launch_stream_full<true, 4>(p, grid_x, stream);
    }
  }
  return launch_stream_full<false, kStreamWaves>(p, grid_x, stream);
}

}  // namespace wave_mxfp4

// Streaming skinny-M (decode shape) MXFP4 GEMM for gfx950: M <= 64, N large.
//
// The operation is bound by reading B once from HBM (2*M*N*K flops against
// N*K/2 bytes), so the kernel is organised around the memory system:
//
// * B goes global -> LDS with 16-byte-per-lane DMA (buffer_load ... lds), one
//   instruction = 8 rows x 128 bytes = 8 whole cache lines.  (Loading MFMA
//   fragments straight from global touches 16 half lines per instruction and
//   the vector L1 retires lines, not bytes: that path tops out near 2.5 TB/s.)
//   DMA costs no VGPRs, so every wave keeps a private ring of 8 K tiles
//   (16 rows x 256 elements = 2 KB each) in flight: 64 KB per CU.
// * A (the few activation rows) is loaded ONCE per workgroup into registers in
//   MFMA fragment layout: each of the 4 waves owns a quarter of the workgroup's
//   K range (at most 8 K tiles = 64 VGPRs per 16 rows of A) and streams only
//   that quarter of every B row.  The waves never wait for each other inside
//   the stream; their four partial 16x16 tiles are added through LDS once per
//   16 rows of B.
// * A workgroup walks a contiguous range of 16-row B tiles, so the grid is one
//   workgroup per CU and all CUs pull from HBM for the whole kernel.
// * B's scales for a 16-row tile and the wave's K quarter travel by the same
//   DMA (2 KB per tile, any layout) and are picked out of LDS per lane.
//
// v_mfma_scale_f32_16x16x128_f8f6f4 is used (16 rows of B per tile balances
// N = 28672 over 256 CUs; MFMA rate is irrelevant here).  Operand order is
// swapped (B rows on the first port) so a lane holds 4 consecutive N of one M
// row.  The reference has no skinny kernel (it runs M = 1 through its generic
// tile kernel, tests/kernel/wave_gemm_mxfp_test.py:296); the contract is the
// same C = dequant(A) . dequant(B)^T.
#include <type_traits>

#include "mxfp4_common.h"

namespace wave_mxfp4 {

constexpr int kStreamWaves = 4;
constexpr int kStreamKtPerWave = 8;                                // K tiles per wave: resident A, 1 KB of a B row
constexpr int kStreamMaxKTiles = kStreamWaves * kStreamKtPerWave;  // per workgroup (K <= 8192)
constexpr int kStreamRowBytes = kStreamKtPerWave * kTileKBytes;    // 1 KB of one B row per DMA instruction
constexpr int kStreamRowPitch = kStreamRowBytes + 16;              // LDS pitch: 16 rows spread over all banks
constexpr int kStreamTileBytes = 16 * kStreamRowPitch;             // one 16-row B tile, one wave's K range
constexpr int kStreamScaleBytes = 2048;                            // its scale image

int stream_max_k_tiles() { return kStreamMaxKTiles; }

struct StreamLds {
  uint8_t tile[kStreamWaves][2][kStreamTileBytes];     // double-buffered per wave
  uint8_t scales[kStreamWaves][2][kStreamScaleBytes];
  float red[kStreamWaves - 1][4][64][4];               // partial 16x16 tiles of waves 1..3
};
static_assert(sizeof(StreamLds) <= 160 * 1024, "stream kernel LDS");

template <int MT_M>
__device__ __forceinline__ void stream_body(const GemmParams &p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
  StreamLds &lds = *reinterpret_cast<StreamLds *>(smem_raw);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int fr = lane & 15, fg = lane >> 4;

  // ---- work split: N tiles over workgroups, K tiles over splits and waves ----
  const int nt_total = (p.n + 15) >> 4;
  const int nt_begin = (int)(((int64_t)blockIdx.x * nt_total) / gridDim.x);
  const int nt_end = (int)(((int64_t)(blockIdx.x + 1) * nt_total) / gridDim.x);
  if (nt_begin >= nt_end) return;
  const int split = blockIdx.y;
  const int kt_begin = split * p.tiles_per_split;
  const int nkt = min(p.k_tiles, kt_begin + p.tiles_per_split) - kt_begin;
  const int ktw = (nkt + kStreamWaves - 1) / kStreamWaves;  // <= kStreamKtPerWave
  const int kt0 = kt_begin + wave * ktw;
  const int my_nkt = max(0, min(ktw, kt_begin + nkt - kt0));

  const int kp = p.kp;
  const v4i zero = {0, 0, 0, 0};
  const int tail_chunks = (p.k & (kTileK - 1)) >> 5;  // valid chunks of a partial last K tile
  auto chunk_ok = [&](int kt, int chunk) { return tail_chunks == 0 || kt != p.k_tiles - 1 || chunk < tail_chunks; };

  // ---- B data DMA: one instruction = up to 1 KB contiguous ----
  //   row-major   : row r of the tile, K tiles kt0 .. kt0+7 (lane t: K tile t/8, chunk t%8),
  //                 landing at r*pitch + t*16; a fragment (row fr, K tile j, chunk c) is read
  //                 at fr*pitch + j*128 + c*16 (the pitch is 1 KB + 16 B, so the 16 rows of a
  //                 fragment read fall on different banks).
  //   preshuffled : K step i = 2*j + s of the 16-row block (already in MFMA order: lane l's
  //                 16 bytes at l*16), landing at i*1024 + l*16 and read back from there.
  const bool bpre = p.b_preshuffled != 0;
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t *>(p.b + (int64_t)nt_begin * 16 * kp), 0, 0x7FFFFFFF, 0x00020000);
  auto issue_rows = [&](int nt, int buf, int i0, int i1) {
    uint8_t *dst = lds.tile[wave][buf];
    const int tile_off = (nt - nt_begin) * 16 * kp;
    const int row_lim = p.n - 1 - nt * 16;
#pragma unroll
    for (int i = i0; i < i1; ++i) {
      if (bpre) {
        const int j = i >> 1, s = i & 1;
        if (j < my_nkt) {
          if (chunk_ok(kt0 + j, s * 4 + fg))
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, WAVE_LDS_PTR(dst + i * 1024), 16, lane * 16,
                                                     tile_off + ((kt0 + j) * 4 + s * 2) * 512, 0, 0);
          else
            *(v4i *)(dst + i * 1024 + lane * 16) = zero;
        }
      } else {
        const int j = lane >> 3;
        if (j < my_nkt) {
          if (chunk_ok(kt0 + j, lane & 7))
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, WAVE_LDS_PTR(dst + i * kStreamRowPitch), 16, lane * 16,
                                                     tile_off + min(i, row_lim) * kp + kt0 * kTileKBytes, 0, 0);
          else
            *(v4i *)(dst + i * kStreamRowPitch + lane * 16) = zero;
        }
      }
    }
  };
  const uint32_t frag_base = bpre ? (uint32_t)(lane * 16) : (uint32_t)(fr * kStreamRowPitch + fg * 16);
  const uint32_t frag_j = bpre ? 2048u : (uint32_t)kTileKBytes;  // per K tile
  const uint32_t frag_s = bpre ? 1024u : 64u;                    // per K step

  // ---- B scales: a 2 KB image of the source bytes per B tile ----
  //   row-major : 16 rows x 128 bytes starting at group kt0*8 (lane t -> row t/8, piece t%8)
  //   shuffled / MFMA32 : the 8 consecutive 256-byte blocks (32-row tile, kt0 .. kt0+7)
  // and, per lane, where its two bytes of K tile j sit in that image.
  const int bsl = p.b_scale_layout;
  const int64_t sc_block_row_bytes = (int64_t)(p.ksp >> 3) * 256;  // one 32-row tile, all K tiles
  auto scale_byte_off = [&](int n_row, int s) -> int {              // offset for K tile 0 of the image
    if (bsl == WAVE_MXFP4_SCALE_ROW_MAJOR) return fr * 128 + s * 4 + fg;
    if (bsl == WAVE_MXFP4_SCALE_E8M0_SHUFFLE) return fg * 64 + (n_row & 15) * 4 + s * 2 + ((n_row >> 4) & 1);
    return (((fg & 1) << 5) | (n_row & 31)) * 4 + s * 2 + (fg >> 1);
  };
  const int sc_kt_stride = bsl == WAVE_MXFP4_SCALE_ROW_MAJOR ? 8 : 256;

  auto issue_scales = [&](int nt, int buf) {
    uint8_t *dst = lds.scales[wave][buf];
    const int n0 = nt * 16;
    if (bsl == WAVE_MXFP4_SCALE_ROW_MAJOR) {
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        const int row = min(n0 + d * 8 + (lane >> 3), p.n - 1);
        const int64_t off = (int64_t)row * p.ks + (int64_t)kt0 * 8 + (lane & 7) * 16;
        // 16-byte pieces past the end of the scale matrix are not read (their groups are past K)
        if ((p.ks & 15) == 0 && off + 16 <= (int64_t)p.n * p.ks) {
          __builtin_amdgcn_global_load_lds(WAVE_GLOBAL_PTR(p.b_scale + off), WAVE_LDS_PTR(dst + d * 1024), 16, 0, 0);
        } else {
          // rows that are not 16-byte multiples: byte copies of the groups that exist
          uint8_t *d8 = dst + d * 1024 + lane * 16;
          for (int e = 0; e < 16; ++e) {
            const int g = kt0 * 8 + (lane & 7) * 16 + e;
            d8[e] = g < p.ks ? p.b_scale[(int64_t)row * p.ks + g] : (uint8_t)127;
          }
        }
      }
    } else {
      // blocks (n0/32, kt0 + t/16), 16-byte piece t%16; blocks past the last K tile are not read
      const uint8_t *src = p.b_scale + (int64_t)(n0 >> 5) * sc_block_row_bytes + (int64_t)kt0 * 256;
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        const int blk = d * 4 + (lane >> 4);
        if (kt0 + blk < p.k_tiles)
          __builtin_amdgcn_global_load_lds(WAVE_GLOBAL_PTR(src + d * 1024 + lane * 16), WAVE_LDS_PTR(dst + d * 1024),
                                           16, 0, 0);
      }
    }
  };

  // first B tile in flight before anything else
  if (my_nkt > 0) {
    issue_scales(nt_begin, 0);
    issue_rows(nt_begin, 0, 0, 16);
  }

  // ---- A: resident fragments and scales (loaded while the first B tile is in flight) ----
  v4i a_frag[MT_M][kStreamKtPerWave][2];
  uint32_t a_sc[MT_M][kStreamKtPerWave];
#pragma unroll
  for (int i = 0; i < MT_M; ++i) {
    const int row = min(i * 16 + fr, p.m - 1);
    const uint8_t *ap = p.a + (int64_t)row * kp + fg * 16;
#pragma unroll
    for (int j = 0; j < kStreamKtPerWave; ++j) {
      a_frag[i][j][0] = a_frag[i][j][1] = zero;
      a_sc[i][j] = 0x7F7Fu;
      if (j < my_nkt) {
        const int kt = kt0 + j;
        if (chunk_ok(kt, fg)) a_frag[i][j][0] = *(const v4i *)(ap + (int64_t)kt * kTileKBytes);
        if (chunk_ok(kt, 4 + fg)) a_frag[i][j][1] = *(const v4i *)(ap + (int64_t)kt * kTileKBytes + 64);
        const int g0 = kt * 8 + fg, g1 = g0 + 4;
        const uint32_t b0 = g0 < p.ks ? p.a_scale[scale_offset(p.a_scale_layout, row, g0, p.ks, p.ksp)] : 127u;
        const uint32_t b1 = g1 < p.ks ? p.a_scale[scale_offset(p.a_scale_layout, row, g1, p.ks, p.ksp)] : 127u;
        a_sc[i][j] = b0 | (b1 << 8);
      }
    }
  }

  // Workgroup barrier that orders LDS traffic only: the DMA of the next tile
  // stays in flight across it (a __syncthreads() would wait for vmcnt(0)).
  auto lds_barrier = [&]() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt((7 << 4) | (3 << 14) | 15);  // lgkmcnt(0) only
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

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

  // ---- the stream: B tile nt is multiplied while tile nt+1 is in flight ----
  // Per tile: wait for this wave's DMA (everything it has in flight), start the
  // DMA of the next tile, finish the previous tile (wave 0 adds the partials of
  // waves 1..3 and stores, so its stores never sit in front of a DMA wait),
  // multiply, hand the partial tile over.
  v4f prev[MT_M];
  for (int nt = nt_begin; nt <= nt_end; ++nt) {
    const int buf = (nt - nt_begin) & 1;
    const bool have = nt < nt_end;
    if (have) {
      __builtin_amdgcn_s_waitcnt(0);  // DMA of tile nt (and the scale image) has landed
      asm volatile("" ::: "memory");
      if (nt + 1 < nt_end && my_nkt > 0) {
        issue_scales(nt + 1, buf ^ 1);
        issue_rows(nt + 1, buf ^ 1, 0, 16);
      }
    }
    if (nt > nt_begin) {
      // finish tile nt-1: partials of waves 1..3 are in LDS (barrier below, previous iteration)
      if (wave == 0) {
#pragma unroll
        for (int i = 0; i < MT_M; ++i) {
          v4f v = prev[i];
#pragma unroll
          for (int w = 0; w < kStreamWaves - 1; ++w) v += *(const v4f *)lds.red[w][i][lane];
          store_tile(nt - 1, i, lane, v);
        }
      }
      lds_barrier();  // red is free again
    }
    if (!have) break;

    const int n_row = min(nt * 16 + fr, p.n - 1);
    const uint8_t *sc_img = lds.scales[wave][buf];
    const uint8_t *tile = lds.tile[wave][buf] + frag_base;
    const int sc0 = scale_byte_off(n_row, 0), sc1 = scale_byte_off(n_row, 1);
    v4f acc[MT_M];
#pragma unroll
    for (int i = 0; i < MT_M; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < kStreamKtPerWave; ++j) {
      if (j < my_nkt) {
        const v4i b0 = *(const v4i *)(tile + j * frag_j);
        const v4i b1 = *(const v4i *)(tile + j * frag_j + frag_s);
        const uint32_t scb = (uint32_t)sc_img[sc0 + j * sc_kt_stride] | ((uint32_t)sc_img[sc1 + j * sc_kt_stride] << 8);
        const v8i vb0 = {b0.x, b0.y, b0.z, b0.w, 0, 0, 0, 0};
        const v8i vb1 = {b1.x, b1.y, b1.z, b1.w, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < MT_M; ++i) {
          const v8i va0 = {a_frag[i][j][0].x, a_frag[i][j][0].y, a_frag[i][j][0].z, a_frag[i][j][0].w, 0, 0, 0, 0};
          const v8i va1 = {a_frag[i][j][1].x, a_frag[i][j][1].y, a_frag[i][j][1].z, a_frag[i][j][1].w, 0, 0, 0, 0};
          acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(vb0, va0, acc[i], 4, 4, 0, (int)scb, 0,
                                                                     (int)a_sc[i][j]);
          acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(vb1, va1, acc[i], 4, 4, 1, (int)scb, 1,
                                                                     (int)a_sc[i][j]);
        }
      }
    }
    // hand over: wave 0 keeps its tile in registers, the others go through LDS
#pragma unroll
    for (int i = 0; i < MT_M; ++i) {
      if (wave == 0)
        prev[i] = acc[i];
      else
        *(v4f *)lds.red[wave - 1][i][lane] = acc[i];
    }
    lds_barrier();  // partials visible
  }
}

template <int MT_M>
__global__ void __launch_bounds__(kStreamWaves * 64, 1) stream_gemm_kernel(const GemmParams p) {
  stream_body<MT_M>(p);
}

template <int MT_M>
static hipError_t launch_stream_mt(const GemmParams &p, int grid_x, hipStream_t stream) {
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute((const void *)stream_gemm_kernel<MT_M>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(StreamLds));
    if (e != hipSuccess) return e;
    attr_done = true;
  }
  dim3 grid(grid_x, p.splits, 1);
  stream_gemm_kernel<MT_M><<<grid, dim3(kStreamWaves * 64), sizeof(StreamLds), stream>>>(p);
  return hipGetLastError();
}

// One workgroup per CU (or per 16-row tile of B if there are fewer tiles).
hipError_t launch_stream_gemm(const GemmParams &p, int num_cus, hipStream_t stream) {
  if (p.tiles_per_split > kStreamMaxKTiles) return hipErrorInvalidValue;
  const int nt_total = (p.n + 15) / 16;
  int grid_x = num_cus > 0 ? num_cus : 256;
  if (p.splits > 1) grid_x = (grid_x + p.splits - 1) / p.splits;
  if (grid_x > nt_total) grid_x = nt_total;
  if (grid_x < 1) grid_x = 1;
  // 32-bit DMA offsets inside a workgroup's range of B rows
  if (((int64_t)(nt_total + grid_x - 1) / grid_x + 1) * 16 * p.kp >= ((int64_t)1 << 31)) return hipErrorInvalidValue;
  const int mt = (p.m + 15) / 16;
  switch (mt) {
    case 1: return launch_stream_mt<1>(p, grid_x, stream);
    case 2: return launch_stream_mt<2>(p, grid_x, stream);
    case 3: return launch_stream_mt<3>(p, grid_x, stream);
    case 4: return launch_stream_mt<4>(p, grid_x, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace wave_mxfp4

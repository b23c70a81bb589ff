// Skinny-M (decode shape) MXFP4 GEMM for gfx950: M <= 64, N large.
//
// The operation is bound by reading B once from HBM (M*N*K flops against
// N*K/2 bytes), so the kernel is a streaming reader: no LDS staging, every
// operand fragment goes global -> VGPR in exactly the MFMA register layout
// (lane l: row l%16, 16 bytes at K chunk l/16), several K tiles in flight per
// wave.  One workgroup owns 16 rows of B (16 columns of C); its four waves
// take K tiles round-robin (so the workgroup as a whole walks each row
// contiguously) and their partial accumulators are added through LDS.
// The reference has no dedicated skinny kernel (it runs M = 1 through its
// generic tile kernel, tests/kernel/wave_gemm_mxfp_test.py:296); the result
// contract is the same C = dequant(A) . dequant(B)^T.
#include <type_traits>

#include "mxfp4_common.h"

namespace wave_mxfp4 {

constexpr int kSkinnyWaves = 4;
constexpr int kSkinnyDepth = 4;  // K tiles in flight per wave
constexpr int kSkinnyMaxM = 64;

int skinny_max_m() { return kSkinnyMaxM; }

template <int MT_M>
struct SkinnyStage {
  v4i b[2];
  v4i a[MT_M][2];
  uint32_t sb[2];
  uint32_t sa[MT_M][2];
};

template <int MT_M>
__global__ void __launch_bounds__(kSkinnyWaves * 64) skinny_gemm_kernel(const GemmParams p) {
  __shared__ v4f red[kSkinnyWaves][MT_M][64];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int fr = lane & 15, fg = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int split = blockIdx.y;
  const int kt_begin = split * p.tiles_per_split;
  const int kt_end = min(p.k_tiles, kt_begin + p.tiles_per_split);

  const int64_t kp = p.kp;
  const int brow = min(n0 + fr, p.n - 1);
  // byte offset of this lane's chunk of K tile kt, K step s: base + kt*stride + s*step
  const uint8_t *b_lane;
  int b_kt_stride, b_s_step;
  if (p.b_preshuffled) {
    // chunk c = kt*8 + s*4 + fg of row n: (n/16)*16*kp + (c/2)*512 + (c%2)*256 + (n%16)*16
    b_lane = p.b + (int64_t)(brow >> 4) * 16 * kp + (fg >> 1) * 512 + (fg & 1) * 256 + (brow & 15) * 16;
    b_kt_stride = 2048;
    b_s_step = 1024;
  } else {
    b_lane = p.b + (int64_t)brow * kp + fg * 16;
    b_kt_stride = kTileKBytes;
    b_s_step = 64;
  }
  const uint8_t *a_lane[MT_M];
  int arow[MT_M];
#pragma unroll
  for (int i = 0; i < MT_M; ++i) {
    arow[i] = min(i * 16 + fr, p.m - 1);
    a_lane[i] = p.a + (int64_t)arow[i] * kp + fg * 16;
  }
  const bool scale_bytes = (p.ks & 7) != 0;
  const int tail_chunks = (p.k & (kTileK - 1)) >> 5;

  auto load_scale_raw = [&](const uint8_t *base, int layout, int row, int kt, uint32_t(&raw)[2]) {
    if (layout == WAVE_MXFP4_SCALE_MFMA32) {
      raw[0] = base[mfma32_scale_offset(row, kt * 8 + fg, p.ksp >> 3)];
      raw[1] = base[mfma32_scale_offset(row, kt * 8 + 4 + fg, p.ksp >> 3)];
    } else if (layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE) {
      const int64_t off = (int64_t)(row >> 5) * ((p.ksp >> 3) * 256) + (int64_t)kt * 256 + fg * 64 +
                          (row & 15) * 4;
      raw[0] = *(const uint32_t *)(base + off);
      raw[1] = 0;
    } else if (!scale_bytes) {
      const v2i v = *(const v2i *)(base + (int64_t)row * p.ks + kt * 8);
      raw[0] = (uint32_t)v.x;
      raw[1] = (uint32_t)v.y;
    } else {
      const int g0 = kt * 8 + fg, g1 = g0 + 4;
      const uint8_t *rp = base + (int64_t)row * p.ks;
      raw[0] = g0 < p.ks ? rp[g0] : 127u;
      raw[1] = g1 < p.ks ? rp[g1] : 127u;
    }
  };
  auto canon_scale = [&](int layout, int row, const uint32_t(&raw)[2]) -> uint32_t {
    if (layout == WAVE_MXFP4_SCALE_MFMA32) {
      return (raw[0] & 0xFFu) | ((raw[1] & 0xFFu) << 8);
    } else if (layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE) {
      const int sh = ((row >> 4) & 1) * 8;
      return ((raw[0] >> sh) & 0xFFu) | (((raw[0] >> (16 + sh)) & 0xFFu) << 8);
    } else if (!scale_bytes) {
      return ((raw[0] >> (fg * 8)) & 0xFFu) | (((raw[1] >> (fg * 8)) & 0xFFu) << 8);
    }
    return (raw[0] & 0xFFu) | ((raw[1] & 0xFFu) << 8);
  };

  auto load_stage = [&](SkinnyStage<MT_M> &st, int kt) {
    const v4i zero = {0, 0, 0, 0};
    const bool tail = tail_chunks != 0 && kt == p.k_tiles - 1;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const bool valid = !tail || (s * 4 + fg) < tail_chunks;
      st.b[s] = valid ? *(const v4i *)(b_lane + (int64_t)kt * b_kt_stride + s * b_s_step) : zero;
#pragma unroll
      for (int i = 0; i < MT_M; ++i)
        st.a[i][s] = valid ? *(const v4i *)(a_lane[i] + (int64_t)kt * kTileKBytes + s * 64) : zero;
    }
    load_scale_raw(p.b_scale, p.b_scale_layout, brow, kt, st.sb);
#pragma unroll
    for (int i = 0; i < MT_M; ++i) load_scale_raw(p.a_scale, p.a_scale_layout, arow[i], kt, st.sa[i]);
  };

  v4f acc[MT_M];
#pragma unroll
  for (int i = 0; i < MT_M; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};

  auto compute_stage = [&](const SkinnyStage<MT_M> &st) {
    const int scb = (int)canon_scale(p.b_scale_layout, brow, st.sb);
    const v8i vb0 = {st.b[0].x, st.b[0].y, st.b[0].z, st.b[0].w, 0, 0, 0, 0};
    const v8i vb1 = {st.b[1].x, st.b[1].y, st.b[1].z, st.b[1].w, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < MT_M; ++i) {
      const int sca = (int)canon_scale(p.a_scale_layout, arow[i], st.sa[i]);
      const v8i va0 = {st.a[i][0].x, st.a[i][0].y, st.a[i][0].z, st.a[i][0].w, 0, 0, 0, 0};
      const v8i va1 = {st.a[i][1].x, st.a[i][1].y, st.a[i][1].z, st.a[i][1].w, 0, 0, 0, 0};
      // first port = B rows (N index), second port = A rows (M index): the
      // lane's 4 results are 4 consecutive N of one M row.
      acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(vb0, va0, acc[i], 4, 4, 0, scb, 0, sca);
      acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(vb1, va1, acc[i], 4, 4, 1, scb, 1, sca);
    }
  };

  // K tiles of this wave: kt_begin + wave, + kSkinnyWaves, ...
  SkinnyStage<MT_M> st[kSkinnyDepth];
  int kt_load = kt_begin + wave;
#pragma unroll
  for (int d = 0; d < kSkinnyDepth; ++d) {
    if (kt_load < kt_end) load_stage(st[d], kt_load);
    kt_load += kSkinnyWaves;
  }
  for (int kt = kt_begin + wave; kt < kt_end; kt += kSkinnyWaves * kSkinnyDepth) {
#pragma unroll
    for (int d = 0; d < kSkinnyDepth; ++d) {
      if (kt + d * kSkinnyWaves < kt_end) {
        compute_stage(st[d]);
        if (kt_load < kt_end) load_stage(st[d], kt_load);
        kt_load += kSkinnyWaves;
      }
    }
  }

  // ---- add the four waves' partial tiles and store ----
#pragma unroll
  for (int i = 0; i < MT_M; ++i) red[wave][i][lane] = acc[i];
  __syncthreads();
  for (int t = threadIdx.x; t < MT_M * 64; t += kSkinnyWaves * 64) {
    const int i = t >> 6, l = t & 63;
    v4f v = red[0][i][l];
#pragma unroll
    for (int w = 1; w < kSkinnyWaves; ++w) v += red[w][i][l];
    const int m = i * 16 + (l & 15);
    const int n = n0 + (l >> 4) * 4;
    if (m >= p.m || n >= p.n) continue;
    const int64_t idx = (int64_t)m * p.n + n;
    const bool vec_ok = (p.n & 3) == 0;
    if (p.partial != nullptr) {
      float *dst = p.partial + (int64_t)split * p.m * p.n + idx;
      if (vec_ok) *(v4f *)dst = v;
      else for (int r = 0; r < 4 && n + r < p.n; ++r) dst[r] = v[r];
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
      if (vec_ok) *(v4f *)dst = v;
      else for (int r = 0; r < 4 && n + r < p.n; ++r) dst[r] = v[r];
    }
  }
}

hipError_t launch_skinny_gemm(const GemmParams &p, hipStream_t stream) {
  const int mt = (p.m + 15) / 16;
  dim3 grid((p.n + 15) / 16, p.splits, 1);
  dim3 block(kSkinnyWaves * 64);
  switch (mt) {
    case 1: skinny_gemm_kernel<1><<<grid, block, 0, stream>>>(p); break;
    case 2: skinny_gemm_kernel<2><<<grid, block, 0, stream>>>(p); break;
    case 3: skinny_gemm_kernel<3><<<grid, block, 0, stream>>>(p); break;
    case 4: skinny_gemm_kernel<4><<<grid, block, 0, stream>>>(p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace wave_mxfp4

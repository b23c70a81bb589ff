// C ABI of the library: argument validation (before any HIP call), kernel
// selection and launch.  Declarations and the reference interfaces they
// replace are in include/wave_mxfp4.h.
#include <stdio.h>
#include <string.h>

#include "mxfp4_common.h"

using namespace wave_mxfp4;

namespace {

thread_local char g_hip_error[256] = "";

int record_hip(hipError_t e) {
  if (e == hipSuccess) return WAVE_MXFP4_OK;
  snprintf(g_hip_error, sizeof(g_hip_error), "%s: %s", hipGetErrorName(e), hipGetErrorString(e));
  return WAVE_MXFP4_ERR_HIP;
}

inline bool aligned(const void *p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }
inline bool bad_enum(int v, int count) { return v < 0 || v >= count; }

constexpr int kAbiVersion = 10;
constexpr int64_t kMaxDim = (int64_t)1 << 30;

// Shape checks shared by the dense and grouped entry points.
int check_common(const void *a, const void *as, const void *b, const void *bs, const void *c, int64_t m,
                 int64_t n, int64_t k, int out_dtype, int asl, int bsl, int bl, int variant) {
  if (m < 0 || n < 0 || k < 0 || m > kMaxDim || n > kMaxDim || k > kMaxDim) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (k % 32 != 0) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (bad_enum(out_dtype, 2) || bad_enum(asl, 4) || bad_enum(bsl, 3) || bad_enum(bl, 2) ||
      bad_enum(variant, WAVE_MXFP4_VARIANT_COUNT_))
    return WAVE_MXFP4_ERR_BAD_ENUM;
  if (bl == WAVE_MXFP4_B_PRESHUFFLE && (n % 16 != 0 || k % 64 != 0)) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (m == 0 || n == 0) return WAVE_MXFP4_OK;  // nothing to read or write
  if (!c) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (k > 0 && (!a || !as || !b || !bs)) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(a, 16) || !aligned(b, 16) || !aligned(bs, 8) || !aligned(c, 16)) return WAVE_MXFP4_ERR_MISALIGNED;
  if (asl != WAVE_MXFP4_SCALE_PER_ROW && !aligned(as, 8)) return WAVE_MXFP4_ERR_MISALIGNED;
  // 32-bit offsets inside a tile: 256 rows of kp bytes must fit in 31 bits.
  if ((k / 2) * 256 >= ((int64_t)1 << 31)) return WAVE_MXFP4_ERR_UNSUPPORTED;
  return 1;  // proceed
}

void fill_params(GemmParams &p, const void *a, const void *as, const void *b, const void *bs, void *c,
                 int64_t m, int64_t n, int64_t k, int out_dtype, int asl, int bsl, int bl) {
  memset(&p, 0, sizeof(p));
  p.a = (const uint8_t *)a;
  p.a_scale = (const uint8_t *)as;
  p.b = (const uint8_t *)b;
  p.b_scale = (const uint8_t *)bs;
  p.c = c;
  p.m = (int)m;
  p.n = (int)n;
  p.k = (int)k;
  p.kp = (int)(k / 2);
  p.ks = (int)(k / 32);
  p.ksp = (p.ks + 7) / 8 * 8;
  p.k_tiles = (int)((k + kTileK - 1) / kTileK);
  p.tiles_per_split = p.k_tiles;
  p.splits = 1;
  p.out_bf16 = out_dtype == WAVE_MXFP4_OUT_BF16;
  p.a_scale_layout = asl;
  p.b_scale_layout = bsl;
  p.b_preshuffled = bl == WAVE_MXFP4_B_PRESHUFFLE;
}

int pick_tile_variant(int64_t m, int64_t n, bool native_scales) {
  // One tile row of at most 128 rows, both scale tensors already in MFMA32 order: 256-row tiles would be half
  // empty, and up to two 128x128 workgroups per CU run side by side (weights from HBM: 128 x 57344 x 8192 68.1 us
  // on 256x256 tiles, 59.9 on 128x128; 64 x 57344 x 4096: 34.5 against 28.1 us).  Measured up to N = 65536.
  if (native_scales && m <= 128 && n <= 65536) return WAVE_MXFP4_VARIANT_T128x128_W2x2;
  const int64_t t256 = ((m + 255) / 256) * ((n + 255) / 256);
  // 129..256 tiles of 128x256: one workgroup per CU on at least half of them, at nearly twice the MFMA duty of
  // the 128x128 kernel (1024 x 5120 x 16000: 72 -> 60 us; 1024 x 8192: 80 -> 76 us).  Also where a ragged M makes
  // that up to 170 tiles of 256x256, which would leave a third of the CUs idle (1100 x 7168 x 8192: 252 tiles of
  // 128x256 against 140 of 256x256, 49.3 -> 41.8 us; x 4096: 31.3 -> 27.0).
  const int64_t t128x256 = ((m + 127) / 128) * ((n + 255) / 256);
  // (an N that leaves the last 256-column tile half empty can make that no more than 256 tiles of 128x128: one round
  // of one workgroup per CU at 0.53-0.62 us per K tile against 0.67-1.0; 2773 x 1408 x 3584: 21.8 -> 17.3 us, x 16128:
  // 54.6 -> 47.2)
  if (t128x256 > 128 && ((m + 127) / 128) * ((n + 127) / 128) <= 256) return WAVE_MXFP4_VARIANT_T128x128_W2x2;
  if (t128x256 > 128 && t128x256 <= 256 && t256 <= 170) return WAVE_MXFP4_VARIANT_T128x256_W2x2;
  // 8 waves: measured 4-5 % ahead of 4 at 8192^3.  Up to 128 tiles of 256x256 leave half the CUs idle; the same
  // problem as up to 512 tiles of 128x128 fills them with two workgroups each (1024 x 8192 x 16384: 87 -> 82 us).
  if (t256 > 128) return WAVE_MXFP4_VARIANT_T256x256_W4x2;
  return WAVE_MXFP4_VARIANT_T128x128_W2x2;
}

// CUs of the current device (cached per device ordinal).
int device_cus() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    cached[dev] = cus;
  }
  return cached[dev];
}

// ---- Estimated duration of a dense problem on the tile kernels and the mid-M kernel ----
// For problems of up to two rounds of 256x256 tiles the kernels are bound by how fast one workgroup streams its
// operands from HBM, not by the matrix pipes, and which tile shape and split along K is fastest follows from a few
// measured quantities (MI355X, B from HBM, called back to back from one host thread; us):
//   a workgroup's time per K tile as a function of the workgroups in flight (flat up to one per CU - 0.72 on
//   128x128 tiles, 1.03 on 128x256, 1.30 on 256x256 -, then rising: the tables below, for 256 CUs);
//   a fixed part per call (launch, first fill, last C tile, and the scale re-layout launch in front when the scales
//   come row-major: 13.5 / 11.5 / 14.0, with scales in MFMA32 order 5.0 / 6.5 / 9.5; the 128x128 kernel on up to
//   8 K tiles of row-major scales stages them itself: 4.4, and 1.19 per K tile);
//   a split's reduction: a launch (2, or 3.5 where no re-layout launch hides it), 0.4 per part for its fill, and 1.3
//   per million f32 partials;
//   the mid-M kernel: 4.5 + K tiles x (0.27 + 0.0025 M) per round of 128-column strips, + N / 14336 (0.335 per K
//   tile up to 32 rows, rising to 0.415 at 64).
// Fitted to 768 shapes (M = 96..4096, N = 2048..14336, K = 4096..14336, both scale layouts, every tile shape with 1-8
// parts by name): the choice by these estimates is within 5 % of the best measured kernel on 95 % of them and
// within 10 % on 98 % (the borders it replaces: 80 % and 87 %).
struct TileChoice {
  int variant, split;
  double us;
};

static double table_step(const double (*tab)[2], int rows, double wgs) {
  if (wgs <= tab[0][0]) return tab[0][1];
  for (int i = 1; i < rows; ++i)
    if (wgs <= tab[i][0]) {
      const double f = (wgs - tab[i - 1][0]) / (tab[i][0] - tab[i - 1][0]);
      return tab[i - 1][1] + f * (tab[i][1] - tab[i - 1][1]);
    }
  return tab[rows - 1][1] * wgs / tab[rows - 1][0];  // (throughput-bound from there on)
}

// us of variant `v` (128x128, 128x256 or 256x256 tiles) with `s` parts along K; negative where `s` is no valid split
static double tile_cost_us(int v, int s, int64_t m, int64_t n, int64_t k, bool native_scales) {
  static const double t128[][2] = {{0, 0.70},    {256, 0.72},  {257, 0.82},  {320, 0.92},  {384, 0.97},
                                   {448, 1.07},  {512, 1.10},  {513, 1.58},  {640, 1.86},  {768, 1.93},
                                   {1024, 2.33}, {1025, 2.71}, {1344, 3.23}, {1792, 4.24}};
  static const double t128x256[][2] = {{0, 1.02},   {192, 1.03}, {256, 1.12}, {257, 1.88}, {320, 2.15},
                                       {384, 2.23}, {512, 2.37}, {513, 3.11}, {688, 3.43}, {896, 4.58}};
  static const double t256[][2] = {{0, 1.30},   {140, 1.30}, {192, 1.49}, {256, 1.80},
                                   {257, 2.18}, {336, 2.98}, {448, 3.39}, {512, 3.60}};
  int bm, bn;
  tile_variant_shape(v, &bm, &bn);
  const int64_t tiles = ((m + bm - 1) / bm) * ((n + bn - 1) / bn);
  const int64_t k_tiles = (k + kTileK - 1) / kTileK, per = (k_tiles + s - 1) / s;
  if (s > 1 && (k_tiles / s < 2 || (s - 1) * per >= k_tiles)) return -1.0;
  const double wgs = (double)(tiles * s) * 256.0 / (double)device_cus();
  double fixed, step;
  if (bm == 128 && bn == 128) {
    fixed = native_scales ? 5.0 : 13.5;
    step = table_step(t128, sizeof(t128) / sizeof(t128[0]), wgs);
    if (native_scales && wgs <= 256) step += 0.08;
    if (!native_scales && wgs <= 256 && per <= 8 && k % kTileK == 0) fixed = 4.4, step = 1.19;
  } else if (bm == 128) {
    fixed = native_scales ? 6.5 : 11.5;
    step = table_step(t128x256, sizeof(t128x256) / sizeof(t128x256[0]), wgs);
  } else {
    fixed = native_scales ? 9.5 : 14.0;
    step = table_step(t256, sizeof(t256) / sizeof(t256[0]), wgs);
    // (beyond one workgroup per CU the table is the persistent kernel's; an N that is not in whole 256-column tiles
    // runs one tile per workgroup in whole rounds: 3072 x 5504 x 8192, 264 tiles, 111 us = 2 x 1.52 per K tile)
    if (n % 256 != 0 && wgs > 256) step = 1.55 * (double)(((int64_t)wgs + 255) / 256);
  }
  const double reduce = s > 1 ? (native_scales ? 3.5 : 2.0) + 0.4 * s + 1.3e-6 * (double)s * (double)m * (double)n : 0.0;
  return fixed + (double)per * step + reduce;
}

static double mid_cost_us(int64_t m, int64_t n, int64_t k) {
  const double rounds = (double)((n + 127) / 128) / (double)device_cus();
  // (up to 64 rows on its 32- and 64-row blocks: 0.335 per K tile up to 32 rows, 0.415 at 64)
  // (the kernel's row blocks are 32 rows high: 68 rows cost what 96 do)
  const int64_t mb = (m + 31) / 32 * 32;
  const double step = mb > 64 ? 0.27 + 0.0025 * (double)mb : mb > 32 ? 0.415 : 0.335;
  return 4.5 + (double)(k / kTileK) * step * (rounds < 1.0 ? 1.0 : rounds) + (double)n / 14336.0;
}

// Where the estimates hold: whole K tiles, at most two rounds of 256x256 tiles, N up to one round of the mid-M
// kernel's strips (fitted on N <= 14336; on 60 random shapes of N = 16512 .. 32768 the choice by them was at 1.012 of
// the best kernel by name in the geometric mean, the borders at 1.026 with a worst case of 1.38).
static bool tile_model_applies(int64_t m, int64_t n, int64_t k) {
  return m > 64 && n >= 2048 && n <= 32768 && k >= 3584 && k % kTileK == 0 && ((m + 255) / 256) * ((n + 255) / 256) <= 512;
}

// The cheapest tile shape and split by the estimates (`only`: 0, or the one variant to find the split for).
static TileChoice best_tile_choice(int64_t m, int64_t n, int64_t k, bool native_scales, int only) {
  static const int variants[] = {WAVE_MXFP4_VARIANT_T128x128_W2x2, WAVE_MXFP4_VARIANT_T128x256_W2x2,
                                 WAVE_MXFP4_VARIANT_T256x256_W4x2};
  TileChoice best = {only ? only : WAVE_MXFP4_VARIANT_T128x128_W2x2, 1, 1e30};
  for (int v : variants) {
    if (only && !(v == only || (v == WAVE_MXFP4_VARIANT_T256x256_W4x2 && only == WAVE_MXFP4_VARIANT_T256x256_W2x2))) continue;
    int bm, bn;
    tile_variant_shape(v, &bm, &bn);
    const int64_t tiles = ((m + bm - 1) / bm) * ((n + bn - 1) / bn);
    for (int s = 1; s <= 8; ++s) {
      if (s > 1 && tiles * s > 640) break;  // (beyond what was measured with a split, and never close)
      const double us = tile_cost_us(v, s, m, n, k, native_scales);
      if (us >= 0.0 && us < best.us) best = {only ? only : v, s, us};
    }
  }
  return best;
}

// The tile shape for a dense problem: by the estimates where they hold, by the borders of pick_tile_variant beyond.
int pick_tile_variant_k(int64_t m, int64_t n, int64_t k, bool native_scales) {
  if (tile_model_applies(m, n, k)) return best_tile_choice(m, n, k, native_scales, 0).variant;
  return pick_tile_variant(m, n, native_scales);
}

constexpr int64_t kGroupedMidMaxAvgRows = 160;  // (one pass of the 192-row block over every expert, as good as always)
// Whether the mid-M kernel is the faster home of a grouped problem (one workgroup per expert and 128-column strip,
// every expert's B streamed once per block of rows).  Up to 160 rows per expert on average it was, on every shape
// measured (4..32 experts, N = 2048..28672, K = 4096..14336, multinomial groups).  Beyond, a group takes several
// passes of 192-row blocks, and what decides is how the tile kernels' rounds come out: a problem of less than two
// rounds of 256x256 tiles, or one that runs on the smaller tiles, leaves CUs idle for whole rounds (8 experts x 4096
// x 14336, 1280..2560 rows: 140..190 us against 67..125 us here), while one of many well-filled rounds does not
// (8 x 28672 x 4096, 1536 rows: 147 against 185 us).  Both sides are priced in K tiles per workgroup and round with
// factors fitted to 49 such measurements (the choice was within 9 % of the better kernel on all of them).
// `bm_cap`: the tallest block the call may use (256 rows with row-major activation scales, 192 with MFMA32 ones);
// `*bm_max`: the block height the estimate was made for.
static bool grouped_mid_pays(int64_t total_rows, int num_groups, int64_t n, int64_t k, int bm_cap = 192,
                             int *bm_max = nullptr) {
  if (bm_max) *bm_max = 192;
  const int64_t cus = device_cus();
  const int64_t strips = (int64_t)num_groups * ((n + 127) / 128);
  if (2 * strips < cus) return false;
  const int64_t avg = (total_rows + num_groups - 1) / num_groups;
  if (avg <= kGroupedMidMaxAvgRows) return true;
  (void)k;  // (both estimates are proportional to K)
  // passes of 192-row blocks, in halves: groups dealt at random spread about a tenth around the average
  const double passes_raw = (double)avg * 1.1 / 192.0;
  double passes = passes_raw < 1.0 ? 1.0 : (double)((int64_t)(passes_raw * 2.0 + 0.999)) / 2.0;
  double per_pass = 0.9;
  // Where one 256-row block still holds every group and the 192-row block needs a second pass, the taller block
  // (a fifth slower per pass) is taken if the call may (8 x 4096 x 14336, 1536 rows, row-major scales: 106 -> 79 us;
  // 8 x 8192 x 8192: 123 -> 90)
  if (bm_cap >= 256 && passes > 1.0 && avg <= 208) {
    passes = 1.0, per_pass = 1.1;
    if (bm_max) *bm_max = 256;
  }
  const double rounds_mid = strips > cus ? (double)strips / (double)cus : 1.0;
  const double t_mid = rounds_mid * passes * per_pass;
  const int v = pick_tile_variant(total_rows, n, false);
  const double n256 = (double)((n + 255) / 256), n128 = (double)((n + 127) / 128);
  double t_alt;
  if (v == WAVE_MXFP4_VARIANT_T256x256_W4x2) {
    const double rounds = ((double)total_rows / 256.0 + num_groups) * n256 / (double)cus;
    if (rounds >= 2.0) return false;
    t_alt = (rounds < 1.0 ? 1.0 : rounds) * 1.9;
  } else if (v == WAVE_MXFP4_VARIANT_T128x256_W2x2) {
    const double tiles = ((double)total_rows / 128.0 + num_groups) * n256;
    t_alt = (double)((int64_t)((tiles + (double)cus - 1.0) / (double)cus)) * 1.1;
  } else {
    const double tiles = ((double)total_rows / 128.0 + num_groups) * n128;
    t_alt = (double)((int64_t)((tiles + 2.0 * (double)cus - 1.0) / (2.0 * (double)cus))) * 1.1;
  }
  return t_mid < t_alt;
}

bool is_tile_variant(int v) {
  int bm, bn;
  tile_variant_shape(v, &bm, &bn);
  return bm != 0;
}

// Grouped problems of at most this many rows per expert on average go to the mid-M kernel.
// Grouped persistent kernel: a group's last M tile of at most this many rows runs as a short tile (all eight waves
// side by side on 64 rows: an eighth of a full tile's MFMAs), after the full ones.
constexpr int kGroupedShortRows = 64;

// What the mid-M kernel takes (the part of it that the shape alone decides).
// (A partial last K tile is taken with both scale tensors in MFMA32 order, whose padding groups hold 0 = 2^-127:
// what the kernel multiplies past the end of K vanishes in f32.)
bool mid_shape_ok(int64_t m, int64_t n, int64_t k) {
  return m >= 1 && m <= mid_max_m() && k % 32 == 0 && k > 3 * kTileK && n % 4 == 0;
}

int auto_split(int64_t m, int64_t n, int64_t k, int variant, bool native_scales = false);

// Whether the streaming kernel would run this K in its counted-wait mode: the library's split leaves every
// workgroup the same number of whole K tiles, and one, two or four waves share them evenly, at most eight each
// (launch_stream_gemm).  Otherwise it runs its predicated mode with full waits, or a split into many parts:
// 16 x 28672 x 14080 (55 K tiles: five parts of eleven) 148.7 us against 36.4 on the mid-M kernel, K = 11008 and
// 13824 (43 and 54 K tiles) alike, where K = 14336 (two parts of 28) takes 27.
static bool stream_runs_counted(int64_t n, int64_t k) {
  if (k % kTileK != 0) return false;
  const int64_t k_tiles = k / kTileK;
  const int s = auto_split(1, n, k, WAVE_MXFP4_VARIANT_SKINNY);
  if (s < 1 || k_tiles % s != 0) return false;
  const int64_t per = k_tiles / s;
  if (per > stream_max_k_tiles()) return false;
  for (int c = 1; c <= 4; c *= 2)
    if (per % c == 0 && per / c <= 8) return true;
  return false;
}

int pick_variant(int64_t m, int64_t n, int64_t k, int variant, bool native_scales, bool b_preshuffled) {
  int v = variant;
  if (v == WAVE_MXFP4_VARIANT_AUTO) {
    // Reading B once from HBM bounds these problems, and the mid-M kernel gives B and A rings of their own.
    // Measured at K = 2048 .. 8192 (us, other kernel -> mid-M):
    //   64 < M <= 192 against the tile kernels: from N = 12288 on (128 x 12288 x 8192: 29.7 -> 23.3,
    //     128 x 24576: 43.4 -> 27.6; 128 x 8192 loses, 19.3 -> 22.8) and, for 96 < M at K <= 4096, from N = 8192 on
    //     (128 x 8192 x 4096: 18.0 -> 13.6); 192 < M <= 256 on one round of strips from N = 20480 on (256 x 24576:
    //     51.5 -> 43.9, 256 x 32768: 59.0 -> 50.5, 256 x 20480: 43.6 -> 37.7 and 24.1 -> 21.4 at K = 4096 since the
    //     256-row block holds three K tiles of A; 256 x 16384 lost before that, 38.3 -> 39.9, 256 x 14336 x 4096
    //     still does, 15.0 -> 20.7, and so does 256 x 40960, 71.5 -> 88.0: two rounds of 256-row blocks against 160
    //     tiles of 256 x 256)
    //   32 < M <= 64 against the streaming kernel: from N = 12288 on (48 x 28672 x 8192: 28.0 -> 22.5), and from
    //     N = 4096 on at K <= 4096 (64 x 8192 x 4096: 14.5 -> 10.7; 48 x 8192 x 8192 loses, 14.4 -> 17.3); with
    //     row-major scales and operand sets that do not fit the memory-side cache also from N = 6144 on up to
    //     K = 8192 (64 x 6144 x 8192: 25.6 -> 17.3, 64 x 6144 x 6400: 21.3 -> 14.4, 64 x 10240 x 8192: 19.9 -> 17.6)
    //   16 < M <= 32: N from 12288 up to 320 columns per CU (32 x 28672 x 8192: 24.8 -> 22.2; past one round of
    //     128-column strips two workgroups share a CU, 32 x 57344 x 8192: 44.6 -> 38.6; 32 x 114688 x 4096 loses,
    //     43.0 -> 44.5)
    //   M <= 16: the same range of N; up to 192 columns per CU only at K <= 4096 (16 x 28672 x 4096: 13.6 -> 13.0;
    //     a tie or 2 % lost at K = 8192: 16 x 40960 29.8 -> 30.3), beyond at any K (16 x 57344 x 8192: 41.4 -> 38.3)
    // More than 64 rows, N up to 32768, at most two rounds of 256x256 tiles: by the estimates above, the mid-M
    // kernel among the candidates up to 256 rows (the borders below were measured at K = 2048 .. 8192 and stay for
    // what lies outside: wider B, fewer rows).
    if (tile_model_applies(m, n, k)) {
      const TileChoice t = best_tile_choice(m, n, k, native_scales, 0);
      // (two tile rows against a B this wide stream it slower per workgroup than the tables say: 256 x 20480 x 8192
      // with scales in MFMA32 order 44.3 us on the 128x128 tiles, estimated 34, against 36.5 on the mid-M kernel)
      if (m > 192 && n >= 20480 && mid_shape_ok(m, n, k)) return WAVE_MXFP4_VARIANT_MID_M;
      if (n >= 3584 && mid_shape_ok(m, n, k) && mid_cost_us(m, n, k) < t.us) return WAVE_MXFP4_VARIANT_MID_M;
      return t.variant;
    }
    // (a partial last K tile on the mid-M kernel wants both scale tensors in MFMA32 order: handed over that way, or
    // re-laid in scratch by the launch in front)
    if (mid_shape_ok(m, n, k)) {
      const int64_t cus = device_cus();
      // (a partial last K tile: the streaming kernel does not take it, and the direct kernel that would serve up to
      // 64 rows loses from N = 4096 on; scales in MFMA32 order, us: 16 x 23040 x 2880 27.5 -> 13.0, 64 x 23040
      // 32.9 -> 13.8, 64 x 5760 15.9 -> 12.2, and 256 x 23040 on the tiles 33.0 -> 20.4)
      // (with row-major scales the launch that re-lays them costs a narrow B more than the kernel saves: 16 x 5760 x
      // 2880 12.2 -> 16.0 us, against 27.5 -> 19.5 at N = 23040; there the borders of whole K tiles hold from N = 12288 on)
      const bool k_tail = k % kTileK != 0 && native_scales;
      const bool rm_tail = k % kTileK != 0 && !native_scales;
      const bool mid = m > 192  ? n >= 20480 && n <= 128 * cus
                       : m > 64 ? n >= 12288 || (k <= 4096 && n >= 8192 && m > 96)
                       : m > 32 ? n >= 12288 || (!rm_tail && ((k <= 4096 && n >= 4096) || (!native_scales && k <= 8192 && n >= 6144)))
                       : m > 16 ? (n >= 12288 && n <= 320 * cus) || (k_tail && n >= 4096)
                                : (n >= 12288 && n <= 320 * cus && (k <= 4096 || n > 192 * cus)) || (k_tail && n >= 4096) ||
                                      // (scales in MFMA32 order, a nearly full single round of strips: 16 x 28672 x
                                      // 8192 23.2 us on the streaming kernel, 21.1 here; level with row-major scales
                                      // and at N = 20480, behind at 40960)
                                      (native_scales && n >= 24576 && n <= 128 * cus);
      // Both scale tensors already in MFMA32 order (static weights, activations from the quantiser): no kernel
      // needs a re-layout launch in front, and the mid-M kernel cannot narrow its strips (a wave's strip is a
      // 32-row scale block), which moves some borders.  Measured with the weights from HBM on a grid of M = 16 ..
      // 256, N = 12288 .. 57344, K = 4096 / 8192 (us, mid-M -> the kernel taken instead):
      //   16 < M <= 48 at K >= 8192 up to N = 16384: the streaming kernel (32 x 12288: 17.4 -> 14.6, 48 x 12288:
      //     19.3 -> 17.8, 32 x 14336: 17.7 -> 16.5; at N = 20480 the mid-M kernel leads, 18.9 against 20.2)
      //   M <= 64 at K >= 8192 with a second round of strips that is at most a quarter full: the streaming kernel
      //     (32 x 40960: 35.6 -> 33.4, 48 x 40960: 40.6 -> 37.1; preshuffled B: 40.5 -> 34.7, 45.1 -> 38.0;
      //     at N = 57344, three quarters full, the mid-M kernel leads again, 40.4 against 45.8)
      //   48 <= M <= 128 at K <= 4096 between one and two rounds of strips, B row-major: the 128x128 tiles
      //     (48 x 40960 x 4096: 25.0 -> 23.1, 128 x 40960: 29.2 -> 27.9, 96 x 57344: 31.0 -> 29.3)
      //   128 < M <= 192 at K <= 4096 up to N = 16384: the tiles (192 x 12288 x 4096: 16.5 -> 13.9)
      // (With one operand set that stays in the 256 MB memory-side cache the tile kernels look 10-30 % better than
      // this on most of the grid; the borders above are for weights that come from HBM.)
      if (mid && native_scales) {
        const int64_t strips = (n + 127) / 128;
        const bool second_round = strips > cus && strips <= 2 * cus;
        // (K = 8192: the streaming kernel's longest K range without a split; up to 16 rows it also leads at
        // K = 4096 on that quarter-full second round, 16 x 40960 x 4096: 19.2 -> 17.4, preshuffled B 21.4 -> 17.6)
        const bool k_whole = k >= 8192 && k <= (int64_t)kTileK * stream_max_k_tiles();
        if (stream_runs_counted(n, k) &&
            ((k_whole && m > 16 && m <= 48 && strips <= 128) ||
             ((k_whole || m <= 16) && m <= 64 && second_round && 4 * strips <= 5 * cus)))
          return WAVE_MXFP4_VARIANT_SKINNY;
        if (k <= 4096 && ((m >= 48 && m <= 128 && second_round && !b_preshuffled) || (m > 128 && m <= 192 && strips <= 128)))
          return pick_tile_variant_k(m, n, k, true);
      }
      if (mid) return WAVE_MXFP4_VARIANT_MID_M;
    }
    // 32 < M <= 64 against a narrow B with a long K: few column tiles, and the streaming kernel's workgroups each
    // walk all of K with four row blocks of accumulators; the 128x128 tiles with the library's split along K put
    // more CUs to work (us, streaming -> tiles; 64 x 1024 x 8192: 20.8 -> 12.2, 48 x 4096 x 8192: 17.9 -> 13.0,
    // 40 x 2048 x 14336: 19.7 -> 18.1, 64 x 3072 x 14336: 25.1 -> 19.8; at N = 4096, K = 14336 the streaming kernel
    // leads again, 16.1 against 19.5, and at K <= 4096 the two are within a microsecond)
    if (m > 32 && m <= skinny_max_m() && k > 4096 && n <= (k <= 8192 ? 4096 : 3072)) return pick_tile_variant_k(m, n, k, native_scales);
    // A K that the streaming kernel cannot deal evenly over its waves (see stream_runs_counted): the mid-M kernel
    // against a wide B, the 128x128 tiles with the library's split against a narrow one (us, streaming -> taken:
    // 16 x 28672 x 12032 69.1 -> 30.9, 1 x 12288 x 9216 22.2 -> 16.7, 16 x 28672 x 6400 35.6 -> 19.2;
    // 16 x 4096 x 14080 30.0 -> 16.2, 64 x 4096 x 12032 28.3 -> 15.7)
    if (m <= skinny_max_m() && k % kTileK == 0 && !stream_runs_counted(n, k)) {
      // (A count of K tiles beyond the streaming kernel's 32 that the library cannot split evenly - 43 is prime -
      // goes to the direct kernel over the whole K, which is ahead of both up to 8 rows against N <= 8192 and up to
      // 16 rows against N <= 4096, weights from HBM: 1 x 4096 x 11008 with scales in MFMA32 order 11.8 us against
      // 16.9 on the tiles, 1 x 8192: 15.3 against 20.2 on the mid-M kernel, 16 x 4096: 13.4 against 17.2; row-major
      // scales 1 x 6144: 17.8 against 23.3; 16 x 10240 loses, 26.4 against 19.6 on the mid-M kernel)
      const bool whole_k_kernel = k / kTileK > stream_max_k_tiles() && auto_split(1, n, k, WAVE_MXFP4_VARIANT_SKINNY) == 1;
      if (whole_k_kernel && (m <= 8 ? n <= 8192 : m <= 16 && n <= 4096)) return WAVE_MXFP4_VARIANT_SKINNY;
      // (between N = 6144 and 12288 by the estimates: with row-major scales the mid-M kernel, 32 x 6144 x 11008 24.6
      // on the tiles against 19.3; with scales in MFMA32 order the tiles, which then need no launch in front,
      // 64 x 8192 x 14080 22.9 against 30.2)
      // (and up to 16 rows with scales in MFMA32 order a K of at most 32 tiles stays with the streaming kernel below
      // N = 12288: one part, 1 x 8192 x 6400 9.9 us against 13.1 on the mid-M kernel; with row-major scales the
      // mid-M kernel leads, 1 x 10240 x 6400 14.5 against 17.8)
      const bool one_part_few_rows = native_scales && k / kTileK <= stream_max_k_tiles() && m <= 16 && n < 12288;
      if (mid_shape_ok(m, n, k) && !one_part_few_rows &&
          (n >= 12288 || (n >= 6144 && mid_cost_us(m, n, k) < best_tile_choice(m, n, k, native_scales, 0).us)))
        return WAVE_MXFP4_VARIANT_MID_M;
      // (up to 32 K tiles one workgroup still streams a narrow B faster than the tiles: 16 x 4096 x 6400 9.1 against 11.7)
      if (k > 8192) return pick_tile_variant_k(m, n, k, native_scales);
    }
    if (m <= skinny_max_m()) return WAVE_MXFP4_VARIANT_SKINNY;
    v = pick_tile_variant_k(m, n, k, native_scales);
  }
  return v;
}

// Kernels that read both scale tensors in MFMA32 order (the library re-lays them out first when it has scratch).
// The mid-M kernel also reads row-major scales and scales in e8m0_shuffle order (the reference's format for
// preshuffled scales) as they are: no pass per call for them.
bool wants_mfma32_scales(int v) {
  return is_tile_variant(v) || v == WAVE_MXFP4_VARIANT_MID_M || v == WAVE_MXFP4_VARIANT_MID_M_BDIRECT;
}
// What the B-direct mid-M kernel takes (the part of it that shape and layout alone decide): K in whole turns of
// its ring of A, 8 K tiles up to 128 rows and 4 beyond.
bool midb_shape_ok(int64_t m, int64_t n, int64_t k, int b_layout) {
  return b_layout == WAVE_MXFP4_B_PRESHUFFLE && m >= 1 && m <= 256 && n % 32 == 0 && k > 0 &&
         k % (m <= 128 ? 2048 : 1024) == 0;
}
bool mid_reads(int layout) {
  return layout == WAVE_MXFP4_SCALE_ROW_MAJOR || layout == WAVE_MXFP4_SCALE_MFMA32 || layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE;
}

// A partial last K tile with scales that are not (or cannot be brought) in MFMA32 order is only built for the
// 128x128 tile kernel.
bool needs_generic_k(const GemmParams &p) {
  return (p.k % kTileK) != 0 &&
         (p.a_scale_layout != WAVE_MXFP4_SCALE_MFMA32 || p.b_scale_layout != WAVE_MXFP4_SCALE_MFMA32);
}

// Split the library takes by itself for a tile kernel: only when the tile
// grid leaves most of the 256 CUs idle and K is long.
int auto_split(int64_t m, int64_t n, int64_t k, int variant, bool native_scales) {
  if (variant == WAVE_MXFP4_VARIANT_SKINNY) {
    // split K so that each workgroup's range fits the streaming kernel's resident A
    const int64_t k_tiles = (k + kTileK - 1) / kTileK, cap = stream_max_k_tiles();
    if (k_tiles <= cap || k % kTileK != 0) return 1;
    int s = (int)((k_tiles + cap - 1) / cap);
    while (s <= 16 && k_tiles % s != 0) ++s;
    return s <= 16 ? s : 1;
  }
  int bm, bn;
  tile_variant_shape(variant, &bm, &bn);
  if (bm == 0 || variant == WAVE_MXFP4_VARIANT_T256x256_W1x4_BDIRECT) return 1;  // (that kernel takes whole K ranges)
  const int64_t tiles = ((m + bm - 1) / bm) * ((n + bn - 1) / bn);
  const int64_t k_tiles = (k + kTileK - 1) / kTileK;  // a partial last K tile belongs to the last split
  // (up to one workgroup per CU without a split: the parts by the estimates; the asymmetric 256x256 kernels of
  // variant 1 share the 8-wave kernel's tables)
  if (tile_model_applies(m, n, k) && tiles <= 256 &&
      (variant == WAVE_MXFP4_VARIANT_T128x128_W2x2 || variant == WAVE_MXFP4_VARIANT_T128x256_W2x2 ||
       variant == WAVE_MXFP4_VARIANT_T256x256_W4x2 || variant == WAVE_MXFP4_VARIANT_T256x256_W2x2))
    return best_tile_choice(m, n, k, native_scales, variant).split;
  if (tiles > 128 || k_tiles < 8) return 1;
  if (bm == 128 && bn == 128) {
    // Estimate in us, fixed launch time left out: a workgroup's K tiles at the measured 0.52 us each while every
    // CU holds at most one workgroup (1.28 us for the two of a CU beyond that), plus, for a split, the launch that
    // sums the parts and their f32 traffic.  (1024 x 1024: K = 2048 stays whole, K = 8192 takes 3 parts, K = 16384 takes 4.)
    int best = 1;
    double best_us = 0.52 * (double)k_tiles;
    for (int s = 2; s <= 8; ++s) {
      const int64_t per = (k_tiles + s - 1) / s;
      if (k_tiles / s < 2 || (s - 1) * per >= k_tiles) continue;  // every part at least one K tile, most two
      const int64_t wgs = tiles * s;
      const double step = wgs <= 256 ? 0.52 : 1.28 * (double)((wgs + 511) / 512);
      const double us = step * (double)per + 3.5 + (double)s * (double)m * (double)n * 4.0 / 8.0e6;
      if (us < 0.9 * best_us) best = s, best_us = us;
    }
    return best;
  }
  if (tiles > 64 && k_tiles < 48) return 1;  // two splits only pay for a long K
  int s = (int)(256 / tiles);
  if (s > 8) s = 8;
  // splits take ceil(k_tiles / s) K tiles each, the last one what is left (at least one)
  while (s > 1 && (k_tiles / s < 2 || (s - 1) * ((k_tiles + s - 1) / s) >= k_tiles)) --s;
  return s < 1 ? 1 : s;
}

// Reference rule for an explicit split (tagged_mxfp4_gemm.py:636-645) with
// BLOCK_K = 256: K per split = ceil(K / splits) must be >= 256 and a multiple
// of 256; and no split may be left without a K tile.
bool split_ok(int64_t k, int splits, int *tiles_per_split) {
  const int64_t per = (k + splits - 1) / splits;
  if (per < kTileK || per % kTileK != 0) return false;
  *tiles_per_split = (int)(per / kTileK);
  // every split must own at least one K tile: ceil() can leave the last ones empty (K = 299 * 256 in 300 splits),
  // and an empty split writes no partial slice for the reduction to read
  if ((int64_t)(splits - 1) * *tiles_per_split >= (k + kTileK - 1) / kTileK) return false;
  return true;
}

// Scratch of wave_mxfp4_gemm_static: a fixed array in the library's device image, one copy per GPU, held until
// the process ends.  On the host the array's name is only a handle for hipGetSymbolAddress: the address a
// kernel can use is looked up once per device and kept here.
constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];
void *g_static_scratch_ptr[kMaxDevices] = {};

int static_scratch_for_current_device(void **ptr) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return record_hip(e);
  if (dev < 0 || dev >= kMaxDevices) return WAVE_MXFP4_ERR_UNSUPPORTED;
  if (g_static_scratch_ptr[dev] == nullptr) {
    void *found = nullptr;
    e = hipGetSymbolAddress(&found, HIP_SYMBOL(g_static_scratch));
    if (e != hipSuccess) return record_hip(e);
    if (found == nullptr) return WAVE_MXFP4_ERR_UNSUPPORTED;
    g_static_scratch_ptr[dev] = found;  // two threads racing here store the same address
  }
  *ptr = g_static_scratch_ptr[dev];
  return WAVE_MXFP4_OK;
}

}  // namespace

extern "C" {

int wave_mxfp4_abi_version(void) { return kAbiVersion; }

const char *wave_mxfp4_status_string(int status) {
  switch (status) {
    case WAVE_MXFP4_OK: return "ok";
    case WAVE_MXFP4_ERR_NULL_POINTER: return "null pointer argument";
    case WAVE_MXFP4_ERR_BAD_SHAPE: return "bad shape (negative dims, K not a multiple of 32, or layout divisibility)";
    case WAVE_MXFP4_ERR_BAD_ENUM: return "dtype, layout or variant out of range";
    case WAVE_MXFP4_ERR_MISALIGNED: return "pointer not aligned as documented";
    case WAVE_MXFP4_ERR_WORKSPACE: return "workspace missing or too small (split-K, per-row scales)";
    case WAVE_MXFP4_ERR_BAD_SPLIT: return "K per split is below 256 or not a multiple of 256";
    case WAVE_MXFP4_ERR_HIP: return "HIP call failed";
    case WAVE_MXFP4_ERR_UNSUPPORTED: return "unsupported argument combination";
    default: return "unknown status";
  }
}

const char *wave_mxfp4_last_hip_error(void) { return g_hip_error; }

// Bytes of one operand's scales in the padded non row-major layouts.
static size_t scale_buffer_bytes(int64_t rows, int64_t k) {
  const int64_t ks = k / 32;
  return (size_t)((rows + 31) / 32 * 32) * (size_t)((ks + 7) / 8 * 8);
}
static size_t round_up_256(size_t v) { return (v + 255) / 256 * 256; }

static size_t workspace_bytes_of(int64_t m, int64_t n, int64_t k, int split_k, int v, bool native_scales) {
  size_t bytes = round_up_256((size_t)m * (size_t)(k / 32));  // per-row A scales spread out to [M, K/32]
  if (v == WAVE_MXFP4_VARIANT_NAIVE) return bytes;
  int splits = split_k;
  if (splits == 0) splits = auto_split(m, n, k, v, native_scales);
  if (splits > 1) bytes += round_up_256((size_t)splits * (size_t)m * (size_t)n * sizeof(float));
  if (wants_mfma32_scales(v)) bytes += round_up_256(scale_buffer_bytes(m, k)) + round_up_256(scale_buffer_bytes(n, k));
  if (v == WAVE_MXFP4_VARIANT_T256x256_W4x2 && n % 256 == 0 && splits <= 1) {
    // the parts of the tiles of a sparsely filled last round (persistent kernel)
    const int grid = device_cus() / 8 * 8;
    const int64_t tiles = ((m + 255) / 256) * (n / 256);
    const int64_t rest = grid > 0 && tiles % grid != 0 ? (tiles + 7) / 8 * 8 - tiles / grid * grid : 0;
    if (tiles > grid && rest != 0 && rest * 2 <= grid) {
      int64_t parts = grid / rest;
      if (parts > 8) parts = 8;
      bytes += (size_t)(rest * parts) * 256 * 256 * sizeof(float);
    }
  }
  return bytes;
}

size_t wave_mxfp4_workspace_bytes(int64_t m, int64_t n, int64_t k, int split_k, int variant) {
  if (m <= 0 || n <= 0 || k <= 0 || split_k < 0 || bad_enum(variant, WAVE_MXFP4_VARIANT_COUNT_)) return 0;
  // the library's own choice of kernel depends on the scale layouts of the call: the larger of the two
  const size_t plain = workspace_bytes_of(m, n, k, split_k, pick_variant(m, n, k, variant, false, false), false);
  const size_t native = workspace_bytes_of(m, n, k, split_k, pick_variant(m, n, k, variant, true, false), true);
  return plain > native ? plain : native;
}

int wave_mxfp4_gemm(const void *a, const void *a_scale, const void *b, const void *b_scale, void *c,
                    int64_t m, int64_t n, int64_t k, int out_dtype, int a_scale_layout,
                    int b_scale_layout, int b_layout, int split_k, void *workspace,
                    size_t workspace_bytes, int variant, void *hip_stream) {
  int rc = check_common(a, a_scale, b, b_scale, c, m, n, k, out_dtype, a_scale_layout, b_scale_layout,
                        b_layout, variant);
  if (rc <= 0) return rc;
  if (split_k < 0) return WAVE_MXFP4_ERR_BAD_SPLIT;
  hipStream_t stream = (hipStream_t)hip_stream;

  GemmParams p;
  fill_params(p, a, a_scale, b, b_scale, c, m, n, k, out_dtype, a_scale_layout, b_scale_layout, b_layout);
  const bool native_scales = a_scale_layout == WAVE_MXFP4_SCALE_MFMA32 && b_scale_layout == WAVE_MXFP4_SCALE_MFMA32;
  int v = pick_variant(m, n, k, variant, native_scales, b_layout == WAVE_MXFP4_B_PRESHUFFLE);
  if (variant == WAVE_MXFP4_VARIANT_AUTO && v == WAVE_MXFP4_VARIANT_MID_M && split_k > 1)  // (it takes whole K ranges)
    v = m <= skinny_max_m() ? WAVE_MXFP4_VARIANT_SKINNY : pick_tile_variant_k(m, n, k, native_scales);
  if (v == WAVE_MXFP4_VARIANT_SKINNY && m > skinny_max_m()) return WAVE_MXFP4_ERR_UNSUPPORTED;
  // the fallback of the library's own choice of the B-direct mid-M kernel, should the scales not reach MFMA32 order
  const int v_plain = v;
  // (measured at N = 28672, K = 8192 against the strip kernel on the same preshuffled B: M = 256 45.8 -> 43.1 us;
  // past one round of strips the 256x256 tiles lead, 256 x 40960 x 8192: 74.0 against 65.6.
  // Up to 128 rows the strip kernel needs neither K in whole turns nor MFMA32 scales; with both scale tensors
  // already in MFMA32 order the B-direct kernel leads there too, weights from HBM: 128 x 28672 x 8192 32.7 -> 28.1,
  // 128 x 20480 29.5 -> 24.4, 96 x 20480 x 4096 15.4 -> 13.5, 48 x 20480 x 8192 23.6 -> 20.7, 128 x 57344 x 8192
  // 63.4 -> 54.9; at N <= 16384, K = 8192 the streaming kernel keeps M < 64: 32 x 12288 14.9 against 18.4.)
  const int64_t cus_n = 128 * (int64_t)device_cus();  // columns of one round of strips
  // (with resident scales and K <= 4096 it leads from N = 8192 on for 48 rows and more: 128 x 8192 x 4096 15.5 -> 12.5,
  // 48 rows 12.4 -> 11.2, 256 rows 20.0 -> 18.0; at N = 4096 the 128x128 tiles are level or ahead)
  const int64_t midb_min_n = native_scales && k <= 4096 && m >= 48 ? 8192 : 12288;
  if (variant == WAVE_MXFP4_VARIANT_AUTO && n >= midb_min_n && split_k <= 1 && midb_shape_ok(m, n, k, b_layout) &&
      (m > 128 ? n <= cus_n
               : native_scales && n <= 2 * cus_n && (m >= 64 || (m >= 32 && n <= cus_n && (n >= 20480 || k <= 4096)))))
    v = WAVE_MXFP4_VARIANT_MID_M_BDIRECT;
  if (variant == WAVE_MXFP4_VARIANT_MID_M_BDIRECT) {
    const bool native = a_scale_layout == WAVE_MXFP4_SCALE_MFMA32 && b_scale_layout == WAVE_MXFP4_SCALE_MFMA32;
    if (!midb_shape_ok(m, n, k, b_layout) || split_k > 1 || (!native && !workspace)) return WAVE_MXFP4_ERR_UNSUPPORTED;
  }
  if (variant == WAVE_MXFP4_VARIANT_MID_M) {
    const bool native = (mid_reads(a_scale_layout) || a_scale_layout == WAVE_MXFP4_SCALE_PER_ROW) && mid_reads(b_scale_layout);
    if (!mid_shape_ok(m, n, k) || split_k > 1 || (!native && !workspace)) return WAVE_MXFP4_ERR_UNSUPPORTED;
  }
  if (v == WAVE_MXFP4_VARIANT_T256x256_W1x4_BDIRECT) {
    // what the B-direct kernel takes, checked before anything is launched: preshuffled B, whole 256-column tiles,
    // an even number (at least 6) of K tiles, no split, scales in MFMA32 order or scratch to bring them there
    const bool native = (a_scale_layout == WAVE_MXFP4_SCALE_MFMA32 && b_scale_layout == WAVE_MXFP4_SCALE_MFMA32) ||
                        (a_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE && b_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE);
    if (b_layout != WAVE_MXFP4_B_PRESHUFFLE || n % 256 != 0 || k % 512 != 0 || k < 1536 || split_k > 1 ||
        (!native && !workspace))
      return WAVE_MXFP4_ERR_UNSUPPORTED;
  }

  if (v == WAVE_MXFP4_VARIANT_T256x192_W4x2) {
    // the 256x192 tiles exist in the persistent kernel only: whole tiles along N, more tiles than CUs, no split
    const bool native = (a_scale_layout == WAVE_MXFP4_SCALE_MFMA32 && b_scale_layout == WAVE_MXFP4_SCALE_MFMA32) ||
                        (a_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE && b_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE &&
                         k % kTileK == 0);
    const int grid = device_cus() / 8 * 8;
    if (n % 192 != 0 || k < 768 || split_k > 1 || (!native && !workspace) || ((m + 255) / 256) * (n / 192) <= grid)
      return WAVE_MXFP4_ERR_UNSUPPORTED;
  }

  if (k == 0) return record_hip(launch_naive_gemm(p, stream));  // empty reduction: C = 0

  int splits = 1;
  if (v != WAVE_MXFP4_VARIANT_NAIVE) {
    if (split_k > 1) {
      int tps;
      if (!split_ok(k, split_k, &tps)) return WAVE_MXFP4_ERR_BAD_SPLIT;
      splits = split_k;
      p.tiles_per_split = tps;
    } else if (split_k == 0) {
      splits = auto_split(m, n, k, v, native_scales);
      // Scratch too small for the parts (and the re-laid scales behind them): fewer parts, down to none.
      const size_t scale_room = wants_mfma32_scales(v) && !native_scales
                                    ? round_up_256(scale_buffer_bytes(m, k)) + round_up_256(scale_buffer_bytes(n, k))
                                    : 0;
      while (splits > 1) {
        const int64_t per = (p.k_tiles + splits - 1) / splits;
        const bool valid = p.k_tiles / splits >= 2 && (int64_t)(splits - 1) * per < p.k_tiles;
        if (valid && workspace && round_up_256((size_t)splits * m * n * sizeof(float)) + scale_room <= workspace_bytes) break;
        --splits;
      }
      if (splits > 1) p.tiles_per_split = (p.k_tiles + splits - 1) / splits;
    }
  }
  size_t ws_used = 0;
  if (workspace && !aligned(workspace, 256)) return WAVE_MXFP4_ERR_MISALIGNED;
  if (splits > 1) {
    const size_t need = (size_t)splits * m * n * sizeof(float);
    if (!workspace || workspace_bytes < need) return WAVE_MXFP4_ERR_WORKSPACE;
    p.splits = splits;
    p.partial = (float *)workspace;
    ws_used = round_up_256(need);
  }

  hipError_t e;
  size_t ws_scales_end = 0;  // first free byte of the workspace behind partials and re-laid scales
  if (p.a_scale_layout == WAVE_MXFP4_SCALE_PER_ROW) {
    // one scale per row: spread it over the row's groups, then it is a row-major scale matrix
    const size_t need = round_up_256((size_t)m * (size_t)p.ks);
    if (!workspace || ws_used + need > workspace_bytes) return WAVE_MXFP4_ERR_WORKSPACE;
    uint8_t *ws = (uint8_t *)workspace + ws_used;
    e = launch_scale_spread_rows(p.a_scale, ws, m, p.ks, stream);
    if (e != hipSuccess) return record_hip(e);
    p.a_scale = ws;
    p.a_scale_layout = WAVE_MXFP4_SCALE_ROW_MAJOR;
    ws_used += need;
  }
  // The tile kernels read MFMA32-ordered scales with one dword per lane and one
  // cache line per wave instruction; row-major scales cost 32 lines per
  // instruction.  With scratch available, re-lay both operands out first
  // (a few MB, microseconds) and run the native-scale kernel.
  // (Not worth a second launch for a short K range on the 128x128 tiles: there the kernel stages the row-major
  // scale rows of its tile through LDS itself.  With the operands from HBM that wins up to 8 K tiles per workgroup,
  // split or not (128 x 4096 x 4096 in 4 parts: 15.6 against 19.4 us; 1024 x 1024 x 2048: 11.3 against 13.6), is
  // level at 12 and loses beyond (16 K tiles: 25.3 against 22.6; 384 x 3584 x 8192 in 3 parts of 11: 34.5 against
  // 25.6).  Nor beyond one workgroup per CU, where it lost to the re-layout on every shape measured: 1280 x 3584 x
  // 4096, 280 tiles, 38.5 us.)
  const bool small_short = v == WAVE_MXFP4_VARIANT_T128x128_W2x2 && p.tiles_per_split <= 8 &&
                           k % kTileK == 0 && ((m + 127) / 128) * ((n + 127) / 128) * splits <= device_cus() &&
                           p.a_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR && p.b_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR;
  // Both tensors in e8m0_shuffle order, the reference's preshuffled format (tagged_mxfp4_gemm.py:334-403,485-536):
  // the 8-wave persistent kernels can read it in place (two dwords and a byte permute per lane instead of one
  // dword), which a caller without scratch gets.  With scratch the re-layout launch stays: the kernel's scale
  // requests are not free (twelve per wave and K tile instead of six: 8192^3 251.9 against 243.9 us), and at
  // 5.2 us the launch costs less than they do.
  const size_t relayout_bytes = round_up_256(scale_buffer_bytes(m, k)) + round_up_256(scale_buffer_bytes(n, k));
  bool shuffled_in_place = false;
  if (p.a_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE && p.b_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE && splits == 1 &&
      !(workspace && ws_used + relayout_bytes <= workspace_bytes) &&
      (v == WAVE_MXFP4_VARIANT_T256x256_W4x2 || v == WAVE_MXFP4_VARIANT_T256x192_W4x2 ||
       v == WAVE_MXFP4_VARIANT_T256x256_W1x4_BDIRECT)) {
    GemmParams q = p;
    int bm, bn;
    tile_variant_shape(v, &bm, &bn);
    q.tiles_m = (int)((m + bm - 1) / bm);
    q.tiles_n = (int)((n + bn - 1) / bn);
    if (v == WAVE_MXFP4_VARIANT_T256x256_W1x4_BDIRECT)
      shuffled_in_place = asym_gemm_applies(q, device_cus(), true);
    else
      shuffled_in_place = (variant == WAVE_MXFP4_VARIANT_AUTO && v == WAVE_MXFP4_VARIANT_T256x256_W4x2 &&
                           asym_gemm_applies(q, device_cus(), false)) ||
                          persist_gemm_applies(q, v, device_cus());
  }
  if (wants_mfma32_scales(v) && workspace && !small_short && !shuffled_in_place) {
    const size_t a_bytes = round_up_256(scale_buffer_bytes(m, k)), b_bytes = round_up_256(scale_buffer_bytes(n, k));
    const bool mid = v == WAVE_MXFP4_VARIANT_MID_M;
    // (the mid-M kernel reads row-major and e8m0_shuffle scales in place, but only with whole K tiles)
    const bool mid_in_place = mid && k % kTileK == 0;
    const size_t a_need = p.a_scale_layout != WAVE_MXFP4_SCALE_MFMA32 && !(mid_in_place && mid_reads(p.a_scale_layout)) ? a_bytes : 0;
    const size_t b_need = p.b_scale_layout != WAVE_MXFP4_SCALE_MFMA32 && !(mid_in_place && mid_reads(p.b_scale_layout)) ? b_bytes : 0;
    if (ws_used + a_need + b_need <= workspace_bytes) {
      uint8_t *ws = (uint8_t *)workspace + ws_used;
      ws_scales_end = ws_used + a_need + b_need;
      // both operands row-major: one launch re-lays both
      if (a_need && b_need && p.a_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR &&
          p.b_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR &&
          launch_scale_pair_to_mfma32(p.a_scale, ws, m, p.b_scale, ws + a_need, n, p.ks, stream) == hipSuccess) {
        p.a_scale = ws;
        p.b_scale = ws + a_need;
        p.a_scale_layout = p.b_scale_layout = WAVE_MXFP4_SCALE_MFMA32;
      } else if (a_need && b_need && p.a_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE &&
                 p.b_scale_layout == WAVE_MXFP4_SCALE_E8M0_SHUFFLE &&
                 launch_scale_pair_shuffle_to_mfma32(p.a_scale, ws, m, p.b_scale, ws + a_need, n, p.ks, stream) ==
                     hipSuccess) {
        p.a_scale = ws;
        p.b_scale = ws + a_need;
        p.a_scale_layout = p.b_scale_layout = WAVE_MXFP4_SCALE_MFMA32;
      } else {
        if (a_need) {
          e = launch_scale_convert(p.a_scale, p.a_scale_layout, ws, WAVE_MXFP4_SCALE_MFMA32, m, p.ks, stream);
          if (e != hipSuccess) return record_hip(e);
          p.a_scale = ws;
          p.a_scale_layout = WAVE_MXFP4_SCALE_MFMA32;
          ws += a_need;
        }
        if (b_need) {
          e = launch_scale_convert(p.b_scale, p.b_scale_layout, ws, WAVE_MXFP4_SCALE_MFMA32, n, p.ks, stream);
          if (e != hipSuccess) return record_hip(e);
          p.b_scale = ws;
          p.b_scale_layout = WAVE_MXFP4_SCALE_MFMA32;
        }
      }
    }
  }

  if (ws_scales_end < ws_used) ws_scales_end = ws_used;
  if (v == WAVE_MXFP4_VARIANT_MID_M && !mid_gemm_applies(p)) {
    // (the library's own choice without scratch for the scales, or offsets beyond 32 bits: the kernels that
    // served these shapes before)
    if (variant == WAVE_MXFP4_VARIANT_MID_M) return WAVE_MXFP4_ERR_UNSUPPORTED;
    v = m <= skinny_max_m() ? WAVE_MXFP4_VARIANT_SKINNY : pick_tile_variant_k(m, n, k, native_scales);
  }
  if (v == WAVE_MXFP4_VARIANT_MID_M_BDIRECT && !midb_gemm_applies(p)) {
    if (variant == WAVE_MXFP4_VARIANT_MID_M_BDIRECT) return WAVE_MXFP4_ERR_UNSUPPORTED;
    v = v_plain == WAVE_MXFP4_VARIANT_MID_M && !mid_gemm_applies(p)
            ? (m <= skinny_max_m() ? WAVE_MXFP4_VARIANT_SKINNY : pick_tile_variant_k(m, n, k, native_scales))
            : v_plain;
  }
  const int vv = v;
  if (vv == WAVE_MXFP4_VARIANT_MID_M_BDIRECT) {
    e = launch_midb_gemm(p, stream);
  } else if (vv == WAVE_MXFP4_VARIANT_MID_M) {
    e = launch_mid_gemm(p, device_cus(), stream);
  } else if (v == WAVE_MXFP4_VARIANT_NAIVE) {
    e = launch_naive_gemm(p, stream);
  } else if (v == WAVE_MXFP4_VARIANT_SKINNY) {
    // The streaming kernel keeps A in registers and serves up to 32 K tiles per
    // workgroup; a longer K range without a split goes to the direct kernel.
    e = p.tiles_per_split <= stream_max_k_tiles() ? launch_stream_gemm(p, device_cus(), stream)
                                                  : hipErrorInvalidValue;
    if (e == hipErrorInvalidValue) e = launch_skinny_gemm(p, stream);
  } else {
    int bm, bn;
    const int tv = needs_generic_k(p) ? WAVE_MXFP4_VARIANT_T128x128_W2x2 : vv;
    tile_variant_shape(tv, &bm, &bn);
    p.tiles_m = (int)((m + bm - 1) / bm);
    p.tiles_n = (int)((n + bn - 1) / bn);
    const bool want_asym = v == WAVE_MXFP4_VARIANT_T256x256_W1x4_BDIRECT;
    if (want_asym && !asym_gemm_applies(p, device_cus(), true)) return WAVE_MXFP4_ERR_UNSUPPORTED;
    if (want_asym || (variant == WAVE_MXFP4_VARIANT_AUTO && tv == WAVE_MXFP4_VARIANT_T256x256_W4x2 &&
                      asym_gemm_applies(p, device_cus(), false))) {
      e = launch_asym_gemm(p, device_cus(), stream);
    } else if (persist_gemm_applies(p, tv, device_cus())) {
      // a last round of tiles that would leave most workgroups idle is cut along K instead, if there is scratch
      size_t part_bytes = 0;
      int parts = persist_tail_parts(p, tv, device_cus(), &part_bytes);
      if (!(parts > 1 && workspace && ws_scales_end + part_bytes <= workspace_bytes)) parts = 1;
      GemmParams p192 = p;
      p192.tiles_n = (int)(n / 192);
      if (variant == WAVE_MXFP4_VARIANT_AUTO && tv == WAVE_MXFP4_VARIANT_T256x256_W4x2 &&
          persist_prefers_192(p, device_cus(), parts) &&
          persist_gemm_applies(p192, WAVE_MXFP4_VARIANT_T256x192_W4x2, device_cus())) {
        // narrower tiles that fill whole rounds over the CUs
        e = launch_persist_gemm(p192, WAVE_MXFP4_VARIANT_T256x192_W4x2, device_cus(), stream);
      } else {
        if (parts > 1) {
          p.tail_parts = parts;
          p.tail_partial = (float *)((uint8_t *)workspace + ws_scales_end);
        }
        e = launch_persist_gemm(p, tv, device_cus(), stream);
      }
    } else if (tv == WAVE_MXFP4_VARIANT_T256x192_W4x2) {
      return WAVE_MXFP4_ERR_UNSUPPORTED;  // (no one-tile-per-workgroup kernel of that shape)
    } else if (GemmParams p192 = p; variant == WAVE_MXFP4_VARIANT_AUTO && tv == WAVE_MXFP4_VARIANT_T256x256_W4x2 &&
                                    persist_192_over_tile_kernel(p, device_cus()) &&
                                    (p192.tiles_n = (int)(n / 192),
                                     persist_gemm_applies(p192, WAVE_MXFP4_VARIANT_T256x192_W4x2, device_cus()))) {
      // N in whole 192-column tiles but not in whole 256-column ones
      e = launch_persist_gemm(p192, WAVE_MXFP4_VARIANT_T256x192_W4x2, device_cus(), stream);
    } else {
      e = launch_tile_gemm(p, tv, stream);
    }
  }
  if (e != hipSuccess) return record_hip(e);
  if (splits > 1) e = launch_splitk_reduce(p.partial, c, m * n, splits, p.out_bf16, stream);
  return record_hip(e);
}

// Also the set-up call: it looks the array's address up for the current device, which may load the library's code
// object and allocate inside the runtime, so that wave_mxfp4_gemm_static itself never does.
size_t wave_mxfp4_static_scratch_bytes(void) {
  void *ignored = nullptr;
  (void)static_scratch_for_current_device(&ignored);
  return kStaticScratchBytes;
}

// Scratch one call needs: wave_mxfp4_workspace_bytes is the most any layout of the same shape can take; scale
// tensors that come in MFMA32 order are read where they are, and only a_scale_layout PER_ROW spreads rows out.
static size_t call_scratch_bytes(int64_t m, int64_t n, int64_t k, int split_k, int variant, int asl, int bsl) {
  size_t need = wave_mxfp4_workspace_bytes(m, n, k, split_k, variant);
  const auto take = [&need](size_t bytes) { need = need > bytes ? need - bytes : 0; };
  if (asl != WAVE_MXFP4_SCALE_PER_ROW) take(round_up_256((size_t)m * (size_t)(k / 32)));
  const bool native_scales = asl == WAVE_MXFP4_SCALE_MFMA32 && bsl == WAVE_MXFP4_SCALE_MFMA32;
  if (wants_mfma32_scales(pick_variant(m, n, k, variant, native_scales, false))) {
    if (asl == WAVE_MXFP4_SCALE_MFMA32) take(round_up_256(scale_buffer_bytes(m, k)));
    if (bsl == WAVE_MXFP4_SCALE_MFMA32) take(round_up_256(scale_buffer_bytes(n, k)));
  }
  return need;
}

int wave_mxfp4_gemm_static(const void *a, const void *a_scale, const void *b, const void *b_scale, void *c, int64_t m,
                           int64_t n, int64_t k, int out_dtype, int a_scale_layout, int b_scale_layout, int b_layout,
                           int split_k, int variant, void *hip_stream) {
  // the same checks as wave_mxfp4_gemm, before the size test, so that a bad argument reports itself
  const int rc = check_common(a, a_scale, b, b_scale, c, m, n, k, out_dtype, a_scale_layout, b_scale_layout, b_layout,
                              variant);
  if (rc <= 0) return rc;
  if (split_k < 0) return WAVE_MXFP4_ERR_BAD_SPLIT;
  // (the library's own split takes fewer parts where the scratch is short: what has to fit is the call without one)
  size_t need = call_scratch_bytes(m, n, k, split_k, variant, a_scale_layout, b_scale_layout);
  if (split_k == 0 && need > kStaticScratchBytes)
    need = call_scratch_bytes(m, n, k, 1, variant, a_scale_layout, b_scale_layout);
  if (need > kStaticScratchBytes) {
    snprintf(g_hip_error, sizeof(g_hip_error),
             "wave_mxfp4_gemm_static: %lld x %lld x %lld with split_k %d needs %zu bytes of scratch, the static "
             "buffer holds %zu", (long long)m, (long long)n, (long long)k, split_k, need, kStaticScratchBytes);
    return WAVE_MXFP4_ERR_WORKSPACE;
  }
  void *scratch = nullptr;
  const int st = static_scratch_for_current_device(&scratch);
  if (st != WAVE_MXFP4_OK) return st;
  // Nothing in the scratch has to start from zero: every byte a kernel of this call reads from it (re-laid
  // scales with their padding, split-K parts) is written earlier in the same call, on the same stream.
  return wave_mxfp4_gemm(a, a_scale, b, b_scale, c, m, n, k, out_dtype, a_scale_layout, b_scale_layout, b_layout,
                         split_k, scratch, kStaticScratchBytes, variant, hip_stream);
}

// Parts along K the library takes for an MXFP8 problem on the 128x128 tiles: few tiles and a long K leave most CUs
// idle, as for MXFP4.  Priced like there (a workgroup's 128-byte K tile 0.7 us while every CU holds at most one
// workgroup, the sum over the parts 3.5 + 0.4 per part + 1.3 per million f32 partials); parts of at least 8 K tiles.
static int mxfp8_auto_split(int64_t m, int64_t n, int64_t k) {
  const int64_t tiles = ((m + 127) / 128) * ((n + 127) / 128), k_tiles = k / 128;
  if (k % 256 != 0 || tiles > 128 || k_tiles < 16) return 1;
  int best = 1;
  double best_us = 0.7 * (double)k_tiles;
  for (int s = 2; s <= 8; ++s) {
    const int64_t per = (k_tiles + s - 1) / s;
    if (per < 8 || (s - 1) * per >= k_tiles || tiles * s > device_cus()) continue;
    const double us = 0.7 * (double)per + 3.5 + 0.4 * s + 1.3e-6 * (double)s * (double)m * (double)n;
    if (us < 0.9 * best_us) best = s, best_us = us;
  }
  return best;
}

size_t wave_mxfp8_workspace_bytes(int64_t m, int64_t n, int64_t k) {
  if (m <= 0 || n <= 0 || k <= 0 || k % 256 != 0) return 0;
  const int s = mxfp8_auto_split(m, n, k);
  return round_up_256(scale_buffer_bytes(m, k)) + round_up_256(scale_buffer_bytes(n, k)) +
         (s > 1 ? round_up_256((size_t)s * (size_t)m * (size_t)n * sizeof(float)) : 0);
}

int wave_mxfp8_gemm(const void *a, const void *a_scale, const void *b, const void *b_scale, void *c,
                    int64_t m, int64_t n, int64_t k, int a_format, int b_format, int out_dtype, void *workspace,
                    size_t workspace_bytes, int variant, void *hip_stream) {
  if (m < 0 || n < 0 || k < 0 || m > kMaxDim || n > kMaxDim || k > kMaxDim || k % 128 != 0)
    return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (bad_enum(a_format, 3) || bad_enum(b_format, 3) || bad_enum(out_dtype, 2) ||
      bad_enum(variant, WAVE_MXFP4_VARIANT_COUNT_))
    return WAVE_MXFP4_ERR_BAD_ENUM;
  if (variant != WAVE_MXFP4_VARIANT_AUTO && variant != WAVE_MXFP4_VARIANT_T256x256_W2x2 &&
      variant != WAVE_MXFP4_VARIANT_T256x256_W4x2 && variant != WAVE_MXFP4_VARIANT_T128x128_W2x2)
    return WAVE_MXFP4_ERR_UNSUPPORTED;
  // (one 4-bit operand at most: two are wave_mxfp4_gemm's)
  if (a_format == WAVE_MXFP8_B_E2M1 && b_format == WAVE_MXFP8_B_E2M1) return WAVE_MXFP4_ERR_UNSUPPORTED;
  if (m == 0 || n == 0) return WAVE_MXFP4_OK;
  if (!c) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (k > 0 && (!a || !a_scale || !b || !b_scale)) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(a, 16) || !aligned(b, 16) || !aligned(a_scale, 4) || !aligned(b_scale, 4) || !aligned(c, 16))
    return WAVE_MXFP4_ERR_MISALIGNED;
  if (k * 256 >= ((int64_t)1 << 31)) return WAVE_MXFP4_ERR_UNSUPPORTED;  // 32-bit offsets inside a tile
  if (workspace && !aligned(workspace, 256)) return WAVE_MXFP4_ERR_MISALIGNED;
  hipStream_t stream = (hipStream_t)hip_stream;
  GemmParams p;
  memset(&p, 0, sizeof(p));
  p.a = (const uint8_t *)a, p.a_scale = (const uint8_t *)a_scale;
  p.b = (const uint8_t *)b, p.b_scale = (const uint8_t *)b_scale;
  p.c = c;
  p.m = (int)m, p.n = (int)n, p.k = (int)k;
  p.kp = (int)k;  // bytes per operand row
  p.ks = (int)(k / 32);
  p.ksp = (p.ks + 7) / 8 * 8;
  p.k_tiles = (int)(k / 128);  // a K tile is 128 bytes of a row
  p.tiles_per_split = p.k_tiles;
  p.splits = 1;
  p.out_bf16 = out_dtype == WAVE_MXFP4_OUT_BF16;
  if (k == 0) {  // empty reduction: C = 0 (the naive kernel never touches the operands)
    p.kp = 0;
    return record_hip(launch_naive_gemm(p, stream));
  }
  int v = variant;
  if (v == WAVE_MXFP4_VARIANT_AUTO) {
    // (up to 512 tiles of 128x128 are one round of two workgroups per CU, where up to 170 tiles of 256x256 leave
    // CUs idle: 2048 x 4096 x 4096 57.2 -> 38.6 us, 1100 x 7168 x 4096 57.0 -> 39.7; from 576 on the two are level)
    // Beyond that, by rounds over the CUs, fitted to 100 random shapes with the weights from HBM (us per 128-byte K
    // tile: 1.05 per round of two 128x128 workgroups per CU, 1.565 per round of 256x256 tiles, 8 waves: 498 -> 476 us
    // at 8192^3): the 256x256 tiles run in whole rounds unless the persistent kernel takes them (N in whole
    // tiles, more tiles than CUs: a last round filled to a fraction f costs 0.4 + 0.6 f), the small ones fill the
    // chip evenly (1387 x 12160 x 3584, 288 tiles of 256x256 in two rounds: 105.7 -> 88.5 us; 3103 x 4992 x 1536:
    // 57.7 -> 38.2; 1532 x 13696 x 6912: 210.7 -> 175.4).
    const int64_t t128 = ((m + 127) / 128) * ((n + 127) / 128), t256 = ((m + 255) / 256) * ((n + 255) / 256);
    const int64_t cus = device_cus();
    v = WAVE_MXFP4_VARIANT_T128x128_W2x2;
    if (t128 > 2 * cus) {
      double rounds256 = (double)((t256 + cus - 1) / cus);
      if (n % 256 == 0 && t256 > cus && t256 % cus != 0) rounds256 = (double)(t256 / cus) + 0.4 + 0.6 * (double)(t256 % cus) / (double)cus;
      const double kt = (double)(k / 128);
      if (24.5 + 1.565 * kt * rounds256 < 29.2 + 1.05 * kt * (double)t128 / (double)(2 * cus)) v = WAVE_MXFP4_VARIANT_T256x256_W4x2;
    }
  }
  int bm, bn;
  tile_variant_shape(v, &bm, &bn);
  p.tiles_m = (int)((m + bm - 1) / bm);
  p.tiles_n = (int)((n + bn - 1) / bn);
  // with scratch, re-lay both scale tensors out in MFMA32 order first (one launch), as the MXFP4 path does
  const size_t a_bytes = round_up_256(scale_buffer_bytes(m, k));
  const size_t scale_bytes = a_bytes + round_up_256(scale_buffer_bytes(n, k));
  if (workspace && k % 256 == 0 && workspace_bytes >= scale_bytes &&
      launch_scale_pair_to_mfma32(p.a_scale, (uint8_t *)workspace, m, p.b_scale, (uint8_t *)workspace + a_bytes, n,
                                  p.ks, stream) == hipSuccess) {
    p.a_scale = (const uint8_t *)workspace;
    p.b_scale = (const uint8_t *)workspace + a_bytes;
    p.a_scale_layout = p.b_scale_layout = WAVE_MXFP4_SCALE_MFMA32;
    // the library's own split along K (128x128 tiles only): f32 parts behind the scales, summed by one more launch
    const int s = v == WAVE_MXFP4_VARIANT_T128x128_W2x2 ? mxfp8_auto_split(m, n, k) : 1;
    if (s > 1 && workspace_bytes >= scale_bytes + round_up_256((size_t)s * m * n * sizeof(float))) {
      p.splits = s;
      p.tiles_per_split = (p.k_tiles + s - 1) / s;
      p.partial = (float *)((uint8_t *)workspace + scale_bytes);
      const hipError_t e = launch_tile_gemm_fp8(p, v, a_format, b_format, stream);
      if (e != hipSuccess) return record_hip(e);
      return record_hip(launch_splitk_reduce(p.partial, c, m * n, s, p.out_bf16, stream));
    }
  }
  // large dense problems on the 8-wave tiles with re-laid scales: the persistent kernel
  if (v == WAVE_MXFP4_VARIANT_T256x256_W4x2 && persist_gemm_fp8_applies(p, device_cus()))
    return record_hip(launch_persist_gemm_fp8(p, device_cus(), a_format, b_format, stream));
  return record_hip(launch_tile_gemm_fp8(p, v, a_format, b_format, stream));
}

int wave_mxfp8_b_preshuffle(const void *b, void *out, int64_t rows, int64_t k, void *hip_stream) {
  if (rows < 0 || k < 0 || rows % 32 != 0 || k % 128 != 0) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (rows == 0 || k == 0) return WAVE_MXFP4_OK;
  if (!b || !out) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (b == out) return WAVE_MXFP4_ERR_UNSUPPORTED;  // not in place
  if (!aligned(b, 16) || !aligned(out, 16)) return WAVE_MXFP4_ERR_MISALIGNED;
  return record_hip(launch_b8_preshuffle((const uint8_t *)b, (uint8_t *)out, rows, k, (hipStream_t)hip_stream));
}

int wave_mxfp8_gemm_b_preshuffled(const void *a, const void *a_scale, const void *b, const void *b_scale, void *c,
                                  int64_t m, int64_t n, int64_t k, int a_format, int b_format, int out_dtype,
                                  int a_scale_layout, int b_scale_layout, void *workspace, size_t workspace_bytes,
                                  void *hip_stream) {
  if (m < 0 || n < 0 || k < 0 || m > kMaxDim || n > kMaxDim || k > kMaxDim || k % 128 != 0 || n % 32 != 0)
    return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (bad_enum(a_format, 3) || bad_enum(b_format, 3) || bad_enum(out_dtype, 2) || bad_enum(a_scale_layout, 4) ||
      bad_enum(b_scale_layout, 4))
    return WAVE_MXFP4_ERR_BAD_ENUM;
  const auto rm_or_native = [](int l) { return l == WAVE_MXFP4_SCALE_ROW_MAJOR || l == WAVE_MXFP4_SCALE_MFMA32; };
  // (A is 8-bit; a 4-bit B comes in the MXFP4 b_preshuffle order; the kernel takes whole 256-column tiles and pairs of
  // K tiles)
  if (a_format == WAVE_MXFP8_E2M1 || !rm_or_native(a_scale_layout) ||
      !rm_or_native(b_scale_layout) || n % 256 != 0 || k % 256 != 0 || k < 768)
    return WAVE_MXFP4_ERR_UNSUPPORTED;
  if (m == 0 || n == 0) return WAVE_MXFP4_OK;
  if (!c || !a || !a_scale || !b || !b_scale) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(a, 16) || !aligned(b, 16) || !aligned(a_scale, 4) || !aligned(b_scale, 4) || !aligned(c, 16))
    return WAVE_MXFP4_ERR_MISALIGNED;
  if (k * 256 >= ((int64_t)1 << 31)) return WAVE_MXFP4_ERR_UNSUPPORTED;  // 32-bit offsets inside a tile
  if (workspace && !aligned(workspace, 256)) return WAVE_MXFP4_ERR_MISALIGNED;
  hipStream_t stream = (hipStream_t)hip_stream;
  GemmParams p;
  memset(&p, 0, sizeof(p));
  p.a = (const uint8_t *)a, p.a_scale = (const uint8_t *)a_scale;
  p.b = (const uint8_t *)b, p.b_scale = (const uint8_t *)b_scale;
  p.c = c;
  p.m = (int)m, p.n = (int)n, p.k = (int)k;
  p.kp = (int)k;  // bytes per operand row
  p.ks = (int)(k / 32);
  p.ksp = p.ks;  // (K % 256 == 0)
  p.k_tiles = (int)(k / 128);
  p.tiles_per_split = p.k_tiles;
  p.splits = 1;
  p.out_bf16 = out_dtype == WAVE_MXFP4_OUT_BF16;
  p.tiles_m = (int)((m + 255) / 256);
  p.tiles_n = (int)(n / 256);
  const bool a_native = a_scale_layout == WAVE_MXFP4_SCALE_MFMA32, b_native = b_scale_layout == WAVE_MXFP4_SCALE_MFMA32;
  if (!a_native || !b_native) {
    // the row-major ones into MFMA32 order first (one launch)
    const size_t a_bytes = round_up_256(scale_buffer_bytes(m, k));
    if (!workspace || workspace_bytes < a_bytes + round_up_256(scale_buffer_bytes(n, k))) return WAVE_MXFP4_ERR_UNSUPPORTED;
    const hipError_t e = launch_scale_pair_to_mfma32(p.a_scale, (uint8_t *)workspace, a_native ? 0 : m, p.b_scale,
                                                     (uint8_t *)workspace + a_bytes, b_native ? 0 : n, p.ks, stream);
    if (e != hipSuccess) return e == hipErrorInvalidValue ? WAVE_MXFP4_ERR_UNSUPPORTED : record_hip(e);
    if (!a_native) p.a_scale = (const uint8_t *)workspace;
    if (!b_native) p.b_scale = (const uint8_t *)workspace + a_bytes;
  }
  p.a_scale_layout = p.b_scale_layout = WAVE_MXFP4_SCALE_MFMA32;
  if (!asym8_gemm_applies(p, device_cus())) return WAVE_MXFP4_ERR_UNSUPPORTED;
  return record_hip(launch_asym8_gemm(p, device_cus(), a_format, b_format, stream));
}

// Scratch of a grouped call: [M tile table | A scales | B scales].
static size_t grouped_table_bytes(int64_t total_rows, int num_groups) {
  return round_up_256((size_t)(1 + total_rows / 256 + num_groups) * 16);
}
static size_t grouped_a_scale_bytes(int64_t total_rows, int64_t k) { return round_up_256(scale_buffer_bytes(total_rows, k)); }
// f32 parts of the tiles of a sparsely filled last round, cut along K (persistent kernel).  Only problems of at
// most four rounds of 256x256 tiles get the room: there the round is a tenth of the call or more, and beyond, the
// launch that sums the parts (which a grouped call cannot know to skip: the tile count is on the device) costs
// more often than the cut pays.  One part per workgroup at most: a 256x256 f32 tile each.
static size_t grouped_tail_bytes(int64_t total_rows, int64_t n, int64_t k, int num_groups) {
  const int64_t grid = device_cus() / 8 * 8;
  const int64_t tiles = (total_rows / 256 + num_groups) * (n / 256);
  if (n % 256 != 0 || k / kTileK < 8 || grid <= 0 || tiles > 4 * grid) return 0;
  return (size_t)grid * 256 * 256 * sizeof(float);
}

size_t wave_mxfp4_grouped_workspace_bytes(int64_t total_rows, int64_t n, int64_t k, int num_groups) {
  if (total_rows <= 0 || n <= 0 || k <= 0 || num_groups <= 0 || k % kTileK != 0 || n % 32 != 0) return 0;
  return grouped_table_bytes(total_rows, num_groups) + grouped_a_scale_bytes(total_rows, k) +
         round_up_256((size_t)num_groups * scale_buffer_bytes(n, k)) + grouped_tail_bytes(total_rows, n, k, num_groups);
}

int wave_mxfp4_gemm_grouped(const void *a, const void *a_scale, const void *b, const void *b_scale,
                            void *c, const int32_t *offsets, int num_groups, int64_t total_rows,
                            int64_t n, int64_t k, int out_dtype, int a_scale_layout,
                            int b_scale_layout, int b_layout, int variant, void *workspace,
                            size_t workspace_bytes, void *hip_stream) {
  if (num_groups < 0 || num_groups > 65536) return WAVE_MXFP4_ERR_BAD_SHAPE;
  int rc = check_common(a, a_scale, b, b_scale, c, total_rows, n, k, out_dtype, a_scale_layout,
                        b_scale_layout, b_layout, variant);
  if (rc <= 0) return rc;
  if (a_scale_layout == WAVE_MXFP4_SCALE_PER_ROW) return WAVE_MXFP4_ERR_UNSUPPORTED;
  if (num_groups == 0) return WAVE_MXFP4_OK;
  if (!offsets) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(offsets, 4)) return WAVE_MXFP4_ERR_MISALIGNED;
  if (k == 0) return WAVE_MXFP4_ERR_UNSUPPORTED;
  hipStream_t stream = (hipStream_t)hip_stream;

  GemmParams p;
  fill_params(p, a, a_scale, b, b_scale, c, total_rows, n, k, out_dtype, a_scale_layout, b_scale_layout,
              b_layout);
  p.offsets = offsets;
  p.num_groups = num_groups;
  p.b_group_stride = n * (k / 2);
  p.b_scale_group_stride = p.b_scale_layout != WAVE_MXFP4_SCALE_ROW_MAJOR
                               ? ((n + 31) / 32 * 32) * (int64_t)p.ksp
                               : n * (int64_t)p.ks;
  // every expert's B and B_scale must keep the base alignment
  if (p.b_group_stride % 16 != 0 || p.b_scale_group_stride % 8 != 0) return WAVE_MXFP4_ERR_MISALIGNED;

  if (variant == WAVE_MXFP4_VARIANT_SKINNY || variant == WAVE_MXFP4_VARIANT_T256x256_W1x4_BDIRECT ||
      variant == WAVE_MXFP4_VARIANT_T256x192_W4x2)
    return WAVE_MXFP4_ERR_UNSUPPORTED;
  // A small batch routed over the experts: every expert's B is read once for a handful of rows, so the call is
  // bound by streaming B, like the dense mid-M problem.  One workgroup per (expert, strip of columns), no table, no
  // re-layout of the scales.  AUTO takes it where grouped_mid_pays() says so: up to 160 rows per expert on average,
  // and beyond where the tile kernels' rounds would come out sparsely filled.
  if (variant == WAVE_MXFP4_VARIANT_MID_M || variant == WAVE_MXFP4_VARIANT_AUTO) {
    const bool fits = mid_grouped_applies(p);
    if (variant == WAVE_MXFP4_VARIANT_MID_M && !fits) return WAVE_MXFP4_ERR_UNSUPPORTED;
    const int64_t avg = (total_rows + num_groups - 1) / num_groups;
    int bm_max = 192;
    const bool pays = grouped_mid_pays(total_rows, num_groups, n, k, p.a_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR ? 256 : 192, &bm_max);
    if (fits && (variant == WAVE_MXFP4_VARIANT_MID_M || pays)) {
      // rows per block: a quarter more than the average group, 32 or in steps of 64, at most the whole batch.  A
      // group of more rows takes a second pass over its expert's B, which costs that expert's share of the call;
      // a block twice the average group, chosen to avoid that, cost every call more than it saved on
      // multinomially dealt rows (8 experts x 14336 x 4096, 24 / 96 / 128 rows per expert: 49.0 -> 42.5,
      // 65.4 -> 63.3, 84.3 -> 72.5 us), because the rings are sized for the block, not for the rows that arrive.
      int64_t bm = (5 * avg + 3) / 4 < total_rows ? (5 * avg + 3) / 4 : total_rows;
      bm = bm > 256 ? 256 : bm <= 32 ? 32 : (bm + 63) / 64 * 64;
      // (the library's own choice beyond one 192-row block per expert is priced on the block height it names)
      if (variant == WAVE_MXFP4_VARIANT_AUTO && bm > 192) bm = bm_max;
      return record_hip(launch_mid_gemm(p, device_cus(), stream, (int)bm));
    }
  }
  const int v = variant == WAVE_MXFP4_VARIANT_AUTO ? pick_tile_variant(total_rows > 64 ? total_rows : 65, n, false)
                                                   : pick_variant(total_rows, n, k, variant, false, false);
  if (v == WAVE_MXFP4_VARIANT_NAIVE) return record_hip(launch_naive_gemm(p, stream));
  int bm, bn;
  auto size_grid = [&](int tile_variant) {
    tile_variant_shape(tile_variant, &bm, &bn);
    // sum over groups of ceil(rows_e / bm) <= total_rows / bm + num_groups
    p.tiles_m = (int)(total_rows / bm + num_groups);
    p.tiles_n = (int)((n + bn - 1) / bn);
  };
  size_grid(v);
  // With scratch: both scale tensors into the MFMA32 order first.  The experts' B scales are one
  // [E * N, K/32] matrix whose 32-row blocks do not straddle experts when N % 32 == 0.
  if (workspace && !aligned(workspace, 256)) return WAVE_MXFP4_ERR_MISALIGNED;
  const size_t ws_need = wave_mxfp4_grouped_workspace_bytes(total_rows, n, k, num_groups);
  if (workspace && ws_need != 0 && workspace_bytes >= ws_need && (int64_t)num_groups * n <= 0x7FFFFFFF) {
    int32_t *table = (int32_t *)workspace;
    uint8_t *ws_a = (uint8_t *)workspace + grouped_table_bytes(total_rows, num_groups);
    uint8_t *ws_b = ws_a + grouped_a_scale_bytes(total_rows, k);
    hipError_t e = hipSuccess;
    // Large problems on the 256x256 tiles: the persistent kernel over a device-built table of M tiles.  The
    // table is built by the launch that re-lays the row-major scales out (by one of its own when both tensors
    // come in MFMA32 order already: activations from the quantiser, resident weights).
    GemmParams q = p;
    q.tile_table = table;
    q.a_scale_layout = q.b_scale_layout = WAVE_MXFP4_SCALE_MFMA32;
    const auto rm_or_native = [](int l) { return l == WAVE_MXFP4_SCALE_ROW_MAJOR || l == WAVE_MXFP4_SCALE_MFMA32; };
    if (rm_or_native(p.a_scale_layout) && rm_or_native(p.b_scale_layout) && persist_gemm_applies(q, v, device_cus())) {
      const bool a_native = p.a_scale_layout == WAVE_MXFP4_SCALE_MFMA32, b_native = p.b_scale_layout == WAVE_MXFP4_SCALE_MFMA32;
      // (a problem of few rounds cuts a sparse last round along K instead: no short tiles then)
      const bool cut_tail = v == WAVE_MXFP4_VARIANT_T256x256_W4x2 && grouped_tail_bytes(total_rows, n, k, num_groups) != 0;
      const int short_rows = v == WAVE_MXFP4_VARIANT_T256x256_W4x2 && !cut_tail ? kGroupedShortRows : 0;
      const GroupTableArgs gt{offsets, num_groups, 256, short_rows, (int)total_rows, table};
      if (a_native && b_native)
        e = launch_grouped_tile_table(offsets, num_groups, 256, short_rows, total_rows, table, stream);
      else
        e = launch_scale_pair_to_mfma32(p.a_scale, ws_a, a_native ? 0 : total_rows, p.b_scale, ws_b,
                                        b_native ? 0 : (int64_t)num_groups * n, p.ks, stream, &gt);
      if (e == hipSuccess) {
        if (!a_native) q.a_scale = ws_a;
        if (!b_native) q.b_scale = ws_b;
        q.b_scale_group_stride = n * (int64_t)p.ksp;
        if (cut_tail)
          q.tail_partial = (float *)(ws_b + round_up_256((size_t)num_groups * scale_buffer_bytes(n, k)));
        return record_hip(launch_persist_gemm(q, v, device_cus(), stream));
      }
      // (the fast re-layout does not apply and has launched nothing: on to the one-tile-per-workgroup kernel)
      e = hipSuccess;
    }
    // both row-major: one launch re-lays both; where that launcher does not apply (it then launches nothing),
    // or for any other pair of layouts, one general conversion per operand
    e = hipErrorInvalidValue;
    if (p.a_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR && p.b_scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR)
      e = launch_scale_pair_to_mfma32(p.a_scale, ws_a, total_rows, p.b_scale, ws_b, (int64_t)num_groups * n, p.ks, stream);
    if (e == hipErrorInvalidValue) {
      e = hipSuccess;
      if (p.a_scale_layout != WAVE_MXFP4_SCALE_MFMA32)
        e = launch_scale_convert(p.a_scale, p.a_scale_layout, ws_a, WAVE_MXFP4_SCALE_MFMA32, total_rows, p.ks, stream);
      else
        ws_a = const_cast<uint8_t *>(p.a_scale);
      if (e == hipSuccess && p.b_scale_layout != WAVE_MXFP4_SCALE_MFMA32)
        e = launch_scale_convert(p.b_scale, p.b_scale_layout, ws_b, WAVE_MXFP4_SCALE_MFMA32, (int64_t)num_groups * n,
                                 p.ks, stream);
      else if (e == hipSuccess)
        ws_b = const_cast<uint8_t *>(p.b_scale);
    }
    if (e != hipSuccess) return record_hip(e);
    p.a_scale = ws_a;
    p.b_scale = ws_b;
    p.a_scale_layout = p.b_scale_layout = WAVE_MXFP4_SCALE_MFMA32;
    p.b_scale_group_stride = n * (int64_t)p.ksp;  // N % 32 == 0: no padding rows between experts
  }
  const int tv = needs_generic_k(p) ? WAVE_MXFP4_VARIANT_T128x128_W2x2 : v;
  size_grid(tv);
  return record_hip(launch_tile_gemm(p, tv, stream));
}

int wave_mxfp4_interleave_gate_up(const void *src, void *dst, int64_t half_rows, int64_t row_bytes, void *hip_stream) {
  if (half_rows < 0 || row_bytes < 0 || half_rows % 32 != 0) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (half_rows == 0 || row_bytes == 0) return WAVE_MXFP4_OK;
  if (!src || !dst) return WAVE_MXFP4_ERR_NULL_POINTER;
  return record_hip(launch_interleave_rows((const uint8_t *)src, (uint8_t *)dst, half_rows, row_bytes, 32, (hipStream_t)hip_stream));
}

int wave_mxfp4_gemm_gated_quantize(const void *a, const void *a_scale, const void *b, const void *b_scale, void *q,
                                   void *scale, const int32_t *offsets, int num_groups, int64_t total_rows, int64_t n,
                                   int64_t k, int a_scale_layout, int b_scale_layout, int act_scale_layout,
                                   void *workspace, size_t workspace_bytes, void *hip_stream) {
  if (num_groups < 0 || num_groups > 65536) return WAVE_MXFP4_ERR_BAD_SHAPE;
  int rc = check_common(a, a_scale, b, b_scale, q, total_rows, n, k, WAVE_MXFP4_OUT_BF16, a_scale_layout, b_scale_layout,
                        WAVE_MXFP4_B_ROW_MAJOR, WAVE_MXFP4_VARIANT_AUTO);
  if (rc <= 0) return rc;
  if (!scale) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (bad_enum(act_scale_layout, 3)) return WAVE_MXFP4_ERR_BAD_ENUM;
  if (act_scale_layout != WAVE_MXFP4_SCALE_MFMA32) return WAVE_MXFP4_ERR_UNSUPPORTED;  // (what the next GEMM reads)
  if (num_groups > 0 && !offsets) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (num_groups > 0 && !aligned(offsets, 4)) return WAVE_MXFP4_ERR_MISALIGNED;
  const auto rm_or_native = [](int l) { return l == WAVE_MXFP4_SCALE_ROW_MAJOR || l == WAVE_MXFP4_SCALE_MFMA32; };
  if (n % 256 != 0 || k % kTileK != 0 || k < 3 * kTileK || !rm_or_native(a_scale_layout) || !rm_or_native(b_scale_layout))
    return WAVE_MXFP4_ERR_UNSUPPORTED;
  if (!workspace || !aligned(workspace, 256)) return workspace ? WAVE_MXFP4_ERR_MISALIGNED : WAVE_MXFP4_ERR_UNSUPPORTED;
  hipStream_t stream = (hipStream_t)hip_stream;
  const int groups = num_groups > 0 ? num_groups : 1;
  if (workspace_bytes < wave_mxfp4_grouped_workspace_bytes(total_rows, n, k, groups) || (int64_t)groups * n > 0x7FFFFFFF)
    return WAVE_MXFP4_ERR_UNSUPPORTED;

  GemmParams p;
  fill_params(p, a, a_scale, b, b_scale, q, total_rows, n, k, WAVE_MXFP4_OUT_BF16, a_scale_layout, b_scale_layout,
              WAVE_MXFP4_B_ROW_MAJOR);
  p.epi_scale = (uint8_t *)scale;
  p.epi_scale_layout = act_scale_layout;
  p.tiles_m = (int)(num_groups > 0 ? total_rows / 256 + num_groups : (total_rows + 255) / 256);
  p.tiles_n = (int)(n / 256);
  int32_t *table = (int32_t *)workspace;
  uint8_t *ws_a = (uint8_t *)workspace + grouped_table_bytes(total_rows, groups);
  uint8_t *ws_b = ws_a + grouped_a_scale_bytes(total_rows, k);
  const bool a_native = a_scale_layout == WAVE_MXFP4_SCALE_MFMA32, b_native = b_scale_layout == WAVE_MXFP4_SCALE_MFMA32;
  if (num_groups > 0) {
    p.offsets = offsets;
    p.num_groups = num_groups;
    p.b_group_stride = n * (k / 2);
    p.b_scale_group_stride = b_native ? ((n + 31) / 32 * 32) * (int64_t)p.ksp : n * (int64_t)p.ks;
    p.tile_table = table;
  }
  // A small batch routed over the experts (the range the grouped call gives to the mid-M kernel): the same
  // epilogue in that kernel, one launch, no table, the scales read as they are.
  if (num_groups > 0 && b_native && mid_gated_applies(p)) {
    const int64_t avg = (total_rows + num_groups - 1) / num_groups;
    if (grouped_mid_pays(total_rows, num_groups, n, k)) {
      int64_t bm = (5 * avg + 3) / 4 < total_rows ? (5 * avg + 3) / 4 : total_rows;
      bm = bm > 192 ? 192 : bm <= 32 ? 32 : (bm + 63) / 64 * 64;
      p.tile_table = nullptr;
      return record_hip(launch_mid_gated(p, device_cus(), stream, (int)bm));
    }
  }
  GemmParams q32 = p;
  q32.a_scale_layout = q32.b_scale_layout = WAVE_MXFP4_SCALE_MFMA32;
  if (!persist_gated_applies(q32, device_cus())) return WAVE_MXFP4_ERR_UNSUPPORTED;
  hipError_t e = hipSuccess;
  const GroupTableArgs gt{offsets, num_groups, 256, 0, (int)total_rows, table};
  if (a_native && b_native) {
    if (num_groups > 0) e = launch_grouped_tile_table(offsets, num_groups, 256, 0, total_rows, table, stream);
  } else {
    e = launch_scale_pair_to_mfma32(p.a_scale, ws_a, a_native ? 0 : total_rows, p.b_scale, ws_b,
                                    b_native ? 0 : (int64_t)groups * n, p.ks, stream, num_groups > 0 ? &gt : nullptr);
  }
  if (e != hipSuccess) return e == hipErrorInvalidValue ? WAVE_MXFP4_ERR_UNSUPPORTED : record_hip(e);
  if (!a_native) q32.a_scale = ws_a;
  if (!b_native) q32.b_scale = ws_b;
  q32.b_scale_group_stride = n * (int64_t)p.ksp;
  return record_hip(launch_persist_gated(q32, device_cus(), stream));
}

int wave_mxfp4_to_f32(const void *q, float *out, int64_t rows, int64_t kp, void *hip_stream) {
  if (rows < 0 || kp < 0) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (rows == 0 || kp == 0) return WAVE_MXFP4_OK;
  if (!q || !out) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(out, 8)) return WAVE_MXFP4_ERR_MISALIGNED;
  return record_hip(launch_to_f32((const uint8_t *)q, out, rows, kp, (hipStream_t)hip_stream));
}

int wave_mxfp4_e8m0_to_f32(const void *s, float *out, int64_t count, void *hip_stream) {
  if (count < 0) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (count == 0) return WAVE_MXFP4_OK;
  if (!s || !out) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(out, 4)) return WAVE_MXFP4_ERR_MISALIGNED;
  return record_hip(launch_e8m0_to_f32((const uint8_t *)s, out, count, (hipStream_t)hip_stream));
}

int wave_mxfp4_dequant(const void *q, const void *scale, float *out, int64_t rows, int64_t k,
                       int scale_layout, void *hip_stream) {
  if (rows < 0 || k < 0 || k % 32 != 0) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (bad_enum(scale_layout, 3)) return WAVE_MXFP4_ERR_BAD_ENUM;
  if (rows == 0 || k == 0) return WAVE_MXFP4_OK;
  if (!q || !scale || !out) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(out, 8)) return WAVE_MXFP4_ERR_MISALIGNED;
  return record_hip(launch_dequant((const uint8_t *)q, (const uint8_t *)scale, out, rows, k, scale_layout,
                                   (hipStream_t)hip_stream));
}

size_t wave_mxfp4_e8m0_shuffle_bytes(int64_t rows, int64_t ks) {
  if (rows <= 0 || ks <= 0) return 0;
  return (size_t)((rows + 31) / 32 * 32) * (size_t)((ks + 7) / 8 * 8);
}

int wave_mxfp4_e8m0_shuffle(const void *scale, void *out, int64_t rows, int64_t ks, void *hip_stream) {
  if (rows < 0 || ks < 0) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (rows == 0 || ks == 0) return WAVE_MXFP4_OK;
  if (!scale || !out) return WAVE_MXFP4_ERR_NULL_POINTER;
  return record_hip(
      launch_e8m0_shuffle((const uint8_t *)scale, (uint8_t *)out, rows, ks, (hipStream_t)hip_stream));
}

int wave_mxfp4_scale_convert(const void *src, int src_layout, void *dst, int dst_layout, int64_t rows,
                             int64_t ks, void *hip_stream) {
  if (rows < 0 || ks < 0) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (bad_enum(src_layout, 3) || bad_enum(dst_layout, 3)) return WAVE_MXFP4_ERR_BAD_ENUM;
  if (rows == 0 || ks == 0) return WAVE_MXFP4_OK;
  if (!src || !dst) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (src == dst) return WAVE_MXFP4_ERR_UNSUPPORTED;  // not in place
  if (dst_layout == WAVE_MXFP4_SCALE_MFMA32 && !aligned(dst, 4)) return WAVE_MXFP4_ERR_MISALIGNED;
  return record_hip(launch_scale_convert((const uint8_t *)src, src_layout, (uint8_t *)dst, dst_layout, rows, ks,
                                         (hipStream_t)hip_stream));
}

int wave_mxfp4_b_preshuffle(const void *b, void *out, int64_t rows, int64_t kp, void *hip_stream) {
  if (rows < 0 || kp < 0 || rows % 16 != 0 || kp % 32 != 0) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (rows == 0 || kp == 0) return WAVE_MXFP4_OK;
  if (!b || !out) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(b, 16) || !aligned(out, 16)) return WAVE_MXFP4_ERR_MISALIGNED;
  return record_hip(
      launch_b_preshuffle((const uint8_t *)b, (uint8_t *)out, rows, kp, (hipStream_t)hip_stream));
}

static int check_quantize(const void *x, int in_dtype, const void *q, const void *scale, int64_t rows, int64_t k,
                          int scale_layout) {
  if (rows < 0 || k < 0 || k % 32 != 0) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (bad_enum(in_dtype, 3) || bad_enum(scale_layout, 3)) return WAVE_MXFP4_ERR_BAD_ENUM;
  if (rows == 0 || k == 0) return WAVE_MXFP4_OK;
  if (!x || !q || !scale) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(x, 16) || !aligned(q, 4) || (scale_layout != WAVE_MXFP4_SCALE_ROW_MAJOR && !aligned(scale, 4)))
    return WAVE_MXFP4_ERR_MISALIGNED;
  if (scale_layout == WAVE_MXFP4_SCALE_ROW_MAJOR && (k / 32) % 4 == 0 && !aligned(scale, 4))
    return WAVE_MXFP4_ERR_MISALIGNED;
  return 1;  // proceed
}

int wave_mxfp4_quantize(const void *x, int in_dtype, void *q, void *scale, int64_t rows, int64_t k,
                        int scale_layout, void *hip_stream) {
  const int rc = check_quantize(x, in_dtype, q, scale, rows, k, scale_layout);
  if (rc <= 0) return rc;
  return record_hip(launch_quantize(x, in_dtype, nullptr, 1, rows, (uint8_t *)q, (uint8_t *)scale, rows, k,
                                    scale_layout, device_cus(), (hipStream_t)hip_stream));
}

int wave_mxfp4_quantize_rows(const void *x, int in_dtype, int64_t src_rows, const int32_t *row_ids, int row_div,
                             void *q, void *scale, int64_t rows, int64_t k, int scale_layout, void *hip_stream) {
  if (src_rows < 0 || row_div < 1) return WAVE_MXFP4_ERR_BAD_SHAPE;
  const int rc = check_quantize(x, in_dtype, q, scale, rows, k, scale_layout);
  if (rc <= 0) return rc;
  if (!row_ids) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(row_ids, 4)) return WAVE_MXFP4_ERR_MISALIGNED;
  if (src_rows * (int64_t)row_div > 0x7FFFFFFF) return WAVE_MXFP4_ERR_UNSUPPORTED;
  return record_hip(launch_quantize(x, in_dtype, row_ids, row_div, src_rows, (uint8_t *)q, (uint8_t *)scale, rows, k,
                                    scale_layout, device_cus(), (hipStream_t)hip_stream));
}

int wave_mxfp4_moe_align_block_size(const void *topk_ids, int ids_int64, int64_t num_entries, int num_experts,
                                    int block_size, int32_t *sorted_ids, int64_t sorted_len, int32_t *expert_ids,
                                    int64_t expert_ids_len, int32_t *num_tokens_post_pad, int32_t *expert_offsets,
                                    void *hip_stream) {
  if (num_entries < 0 || num_experts < 1 || block_size < 1 || sorted_len < num_entries || expert_ids_len < 0)
    return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (num_experts > kMoeMaxExperts) return WAVE_MXFP4_ERR_UNSUPPORTED;
  // the padded total must fit the int32 outputs
  if (num_entries + (int64_t)num_experts * (block_size - 1) > 0x7FFFFFFF || sorted_len > 0x7FFFFFFF ||
      expert_ids_len > 0x7FFFFFFF)
    return WAVE_MXFP4_ERR_UNSUPPORTED;
  if (bad_enum(ids_int64, 2)) return WAVE_MXFP4_ERR_BAD_ENUM;
  if (!num_tokens_post_pad || (num_entries > 0 && !topk_ids) || (sorted_len > 0 && !sorted_ids) ||
      (expert_ids_len > 0 && !expert_ids))
    return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(topk_ids, ids_int64 ? 8 : 4) || !aligned(sorted_ids, 4) || !aligned(expert_ids, 4) ||
      !aligned(num_tokens_post_pad, 4) || !aligned(expert_offsets, 4))
    return WAVE_MXFP4_ERR_MISALIGNED;
  return record_hip(launch_moe_align(topk_ids, ids_int64, num_entries, num_experts, block_size, sorted_ids, sorted_len,
                                     expert_ids, expert_ids_len, num_tokens_post_pad, expert_offsets,
                                     (hipStream_t)hip_stream));
}

static int check_gated(const void *gate, const void *up, int64_t ld_gate, int64_t ld_up, int dtype, int64_t rows,
                       int64_t n, int64_t mult) {
  if (rows < 0 || n < 0 || n % mult != 0 || ld_gate < n || ld_up < n || ld_gate % 8 != 0 || ld_up % 8 != 0)
    return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (dtype != WAVE_MXFP4_IN_BF16 && dtype != WAVE_MXFP4_IN_F16) return WAVE_MXFP4_ERR_BAD_ENUM;
  if (rows == 0 || n == 0) return WAVE_MXFP4_OK;
  if (!gate || !up) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(gate, 16) || !aligned(up, 16)) return WAVE_MXFP4_ERR_MISALIGNED;
  return 1;
}

int wave_mxfp4_silu_and_mul(const void *gate, const void *up, void *out, int64_t ld_gate, int64_t ld_up,
                            int64_t ld_out, int dtype, int64_t rows, int64_t n, void *hip_stream) {
  const int rc = check_gated(gate, up, ld_gate, ld_up, dtype, rows, n, 8);
  if (rc <= 0) return rc;
  if (ld_out < n || ld_out % 8 != 0) return WAVE_MXFP4_ERR_BAD_SHAPE;
  if (!out) return WAVE_MXFP4_ERR_NULL_POINTER;
  if (!aligned(out, 16)) return WAVE_MXFP4_ERR_MISALIGNED;
  return record_hip(launch_silu_and_mul(gate, up, out, ld_gate, ld_up, ld_out, dtype, rows, n, (hipStream_t)hip_stream));
}

int wave_mxfp4_silu_and_mul_quantize(const void *gate, const void *up, int64_t ld_gate, int64_t ld_up, int dtype,
                                     void *q, void *scale, int64_t rows, int64_t n, int scale_layout,
                                     void *hip_stream) {
  int rc = check_gated(gate, up, ld_gate, ld_up, dtype, rows, n, 32);
  if (rc <= 0) return rc;
  rc = check_quantize(gate, dtype, q, scale, rows, n, scale_layout);
  if (rc <= 0) return rc;
  return record_hip(launch_silu_and_mul_quantize(gate, up, ld_gate, ld_up, dtype, (uint8_t *)q, (uint8_t *)scale, rows, n,
                                                 scale_layout, device_cus(), (hipStream_t)hip_stream));
}

}  // extern "C"

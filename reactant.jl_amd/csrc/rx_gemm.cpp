#include "rx_gemm.h"

#include <cstdlib>
#include <algorithm>
#include <sstream>
#include <stdexcept>

namespace rx {

// f64: the register-staged skeleton on v_mfma_f64_16x16x4_f64
static GemmChoice choose_gemm_f64(int64_t batch, int64_t M, int64_t N, int64_t K, bool a_kc, bool b_kc) {
  GemmChoice c;
  const int ve = 2, bk = 16;
  if (K < 1 || ((a_kc || b_kc) && K % ve != 0)) return c;
  if (N % 4 != 0 || M < 1 || N < 4) return c;
  if (!a_kc && M % ve != 0) return c;
  if (!b_kc && N % ve != 0) return c;
  if (M * N < 64 * 64) return c;
  if (M >= ((int64_t)1 << 30) || N >= ((int64_t)1 << 30) || K >= ((int64_t)1 << 30)) return c;
  // 4096^3: 256x128 tiles on 8 wavefronts 60-62 TFLOP/s, 128x128 on 4 wavefronts 47, 64x64 52-54;
  // 1024^3: 64x64 32, 128x128 11
  int BM = 64, BN = 64, WM = 2, WN = 2;
  if (((M + 255) / 256) * ((N + 127) / 128) * batch >= 256) { BM = 256; BN = 128; WM = 4; WN = 2; }
  else if (((M + 127) / 128) * ((N + 127) / 128) * batch >= 512) { BM = 128; BN = 128; }
  if (const char* e = getenv("RX_GEMM_TILE_F64")) {  // "BM,BN,WM,WN" for tuning runs
    int v[4];
    if (sscanf(e, "%d,%d,%d,%d", &v[0], &v[1], &v[2], &v[3]) == 4) { BM = v[0]; BN = v[1]; WM = v[2]; WN = v[3]; }
  }
  int rb = 4, cb = 8;
  const int64_t gm = (M + BM - 1) / BM, gn = (N + BN - 1) / BN;
  if (gm * gn < 64) rb = cb = 0;
  else if (gm < rb) { cb = (int)(rb * cb / gm); rb = (int)gm; }
  else if (gn < cb) { rb = (int)(rb * cb / gn); cb = (int)gn; }
  const int pad = 2;
  const int64_t a_sz = a_kc ? (int64_t)BM * (bk + pad) : (int64_t)bk * (BM + pad);
  const int64_t b_sz = b_kc ? (int64_t)BN * (bk + pad) : (int64_t)bk * (BN + pad);
  c.lds_bytes = (unsigned)(2 * (a_sz + b_sz) * 8);
  if (c.lds_bytes > 160 * 1024) return c;
  c.block = WM * WN * 64;
  c.grid[0] = (unsigned)gemm_grid(gm, gn, rb, cb);
  c.grid[1] = (unsigned)batch;
  std::ostringstream t;
  t << BM << ", " << BN << ", " << bk << ", " << WM << ", " << WN << ", " << (a_kc ? "true" : "false") << ", " << (b_kc ? "true" : "false")
    << ", " << M << ", " << N << ", " << K << ", " << rb << ", " << cb;
  c.targs = t.str();
  c.skeleton = "rx_gemm_body_f64";
  c.stype_a = "double";
  c.kind = "gemm_f64";
  c.ok = true;
  return c;
}

GemmChoice choose_gemm(DT a, DT b, DT out, int64_t batch, int64_t M, int64_t N, int64_t K, bool a_kc, bool b_kc, bool staged_only, int split) {
  GemmChoice c;
  if (a != b) return c;
  if (split > 1 && (staged_only || batch != 1 || a == DT::F64)) return c;
  if (a == DT::F64 && out == DT::F64) return staged_only ? c : choose_gemm_f64(batch, M, N, K, a_kc, b_kc);
  std::string mma;
  int esize = 0, bk = 0;
  if (a == DT::F32 && out == DT::F32) { mma = "rx_mma_f32"; c.kind = "gemm_f32"; esize = 4; bk = 16; }
  else if (a == DT::BF16 && (out == DT::BF16 || out == DT::F32)) { mma = "rx_mma_bf16"; c.kind = "gemm_bf16"; esize = 2; bk = 64; }
  else if (a == DT::F16 && (out == DT::F16 || out == DT::F32)) { mma = "rx_mma_f16"; c.kind = "gemm_f16"; esize = 2; bk = 64; }
  else if (a == DT::F8E4M3FN && (out == DT::F32 || out == DT::BF16 || out == DT::F16)) { mma = "rx_mma_f8"; c.kind = "gemm_f8"; esize = 1; bk = 128; }
  else return c;
  const int ve = 16 / esize;
  // 16-byte loads along the contracted dimension need whole vectors; a tail shorter than the
  // K step is zero-filled by the register-staged skeleton
  if (K < 1 || ((a_kc || b_kc) && K % ve != 0)) return c;
  if (N % 4 != 0) return c;
  if (!a_kc && M % ve != 0) return c;
  if (!b_kc && N % ve != 0) return c;
  if (M < 1 || N < 4) return c;
  if (M * N < 64 * 64) return c;  // tiny products: the scalar loop is as good
  if (M >= ((int64_t)1 << 30) || N >= ((int64_t)1 << 30) || K >= ((int64_t)1 << 30)) return c;
  // Large problems take 256x256 tiles on 8 wavefronts (each wavefront a 128x64 block of the
  // tile: fewer LDS bytes per MFMA); when that would leave compute units idle, 128x128 on 4.
  // Products that leave most compute units without a 128x128 tile take 64x64 tiles (1000^3 f32:
  // 16 -> 48 TFLOP/s, 1024^3 bf16: 130 -> 240); an operand with at most 64 rows (the output
  // features of a convolution) gets a 64-wide tile so that no MFMA works on padding.
  // A tuning override (RX_GEMM_TILE / _BK / _STAGES / _DIRECT) is honoured or refused with an error: a setting that
  // does not fit must not end in the scalar loop unnoticed.
  bool tuned = false;
  auto refuse = [&](const char* why) {
    throw std::runtime_error(std::string("RX_GEMM_* tuning override cannot be honoured for ") + c.kind + " " + std::to_string(M) + "x" + std::to_string(N) + "x" +
                             std::to_string(K) + ": " + why);
  };
  int BM = 128, BN = 128, WM = 2, WN = 2;
  if (M <= 64 && N > 64) { BM = 64; BN = 128; }
  else if (N <= 64 && M > 64) { BM = 128; BN = 64; }
  else if (M > 128 && N > 128 && ((M + 255) / 256) * ((N + 255) / 256) * batch >= 256) { BM = 256; BN = 256; WM = 2; WN = 4; }
  // 16-bit operands whose 256x256 tiles would leave compute units idle but whose 256x128 tiles fill the chip (the
  // 8192 x 1024 x 4096 layer of the MLP: 256 tiles, one per compute unit): 8 wavefronts, each a 128x32 block of the
  // tile, against 128x128 tiles on 4 wavefronts 75 -> 67 us
  else if (esize == 2 && M >= N && M > 128 && N > 64 && ((M + 255) / 256) * ((N + 127) / 128) * batch >= 256) { BM = 256; BN = 128; WM = 2; WN = 4; }
  else if (esize == 2 && N > M && N > 128 && M > 64 && ((M + 127) / 128) * ((N + 255) / 256) * batch >= 256) { BM = 128; BN = 256; WM = 4; WN = 2; }
  else if (((M + 127) / 128) * ((N + 127) / 128) * batch * split < 128) { BM = 64; BN = 64; }
  if (const char* e = getenv("RX_GEMM_TILE")) {  // "BM,BN,WM,WN" for tuning runs
    int v[4];
    if (sscanf(e, "%d,%d,%d,%d", &v[0], &v[1], &v[2], &v[3]) == 4) { BM = v[0]; BN = v[1]; WM = v[2]; WN = v[3]; tuned = true; }
    else refuse("RX_GEMM_TILE wants BM,BN,WM,WN");
    if (BM < 32 || BN < 32 || WM < 1 || WN < 1 || BM % (32 * WM) != 0 || BN % (32 * WN) != 0 || WM * WN > 16) refuse("tile is not a whole number of 32x32 blocks per wavefront");
  }
  const int ks_step = a == DT::F32 ? 8 : (esize == 2 ? 16 : 64);
  if (const char* e = getenv("RX_GEMM_BK")) {
    const int v = atoi(e);
    if (v <= 0 || v % ks_step != 0) refuse("RX_GEMM_BK is not a multiple of the MFMA k step");
    if (K % v == 0) { bk = v; tuned = true; }   // products whose K it does not divide keep the default
  }
  bool direct = !staged_only;   // global -> LDS direct loads through a ring of LDS stages
  bool direct_forced = false;
  if (const char* e = getenv("RX_GEMM_DIRECT")) { direct = atoi(e) != 0 && !staged_only; direct_forced = atoi(e) != 0 && !staged_only; }
  int stages = 2;
  if (const char* e = getenv("RX_GEMM_STAGES")) { if (atoi(e) < 2) refuse("RX_GEMM_STAGES < 2"); stages = atoi(e); }
  int rb = 4, cb = 8;   // tiles of one XCD's block (rows x columns of the tile grid)
  if (const char* e = getenv("RX_GEMM_BLOCK")) { int v[2]; if (sscanf(e, "%d,%d", &v[0], &v[1]) == 2 && v[0] > 0 && v[1] > 0) { rb = v[0]; cb = v[1]; } }
  // a grid of few tiles (per batch entry) is not worth padding to whole XCD blocks
  if (((M + BM - 1) / BM) * ((N + BN - 1) / BN) < 64) rb = cb = 0;
  // a tile grid with fewer rows (columns) than a block: make the block that flat
  else if ((M + BM - 1) / BM < rb) { const int64_t gm = (M + BM - 1) / BM; cb = (int)(rb * cb / gm); rb = (int)gm; }
  else if ((N + BN - 1) / BN < cb) { const int64_t gn = (N + BN - 1) / BN; rb = (int)(rb * cb / gn); cb = (int)gn; }
  const int nt = WM * WN * 64;
  // 8- and 16-bit operands on the eight-wavefront tiles whose wavefronts own 128 rows (256x256, 256x128): the
  // streaming skeleton on the 16x16 MFMA shapes (kernels/rx_gemm_kernels.h, rx_gemm_body_s).  It wants whole K tiles
  // of 128 bytes and operands below 4 GB (32-bit buffer offsets), and has no K-sliced form; RX_GEMM_STREAM=0 keeps the
  // ring skeleton.
  if (direct && (esize == 1 || esize == 2) && BM == 256 && (BN == 256 || BN == 128) && ((WM == 2 && WN == 4) || (WM == 4 && WN == 2 && BN == 128)) && split == 1 && bk * esize == 128 &&
      K % bk == 0 && stages == 2 && M * K * esize < ((int64_t)1 << 32) && N * K * esize < ((int64_t)1 << 32) &&
      !(getenv("RX_GEMM_STREAM") && atoi(getenv("RX_GEMM_STREAM")) == 0) && !(getenv("RX_GEMM_MFMA32") && atoi(getenv("RX_GEMM_MFMA32")) != 0)) {
    const std::string el = a == DT::F8E4M3FN ? "rx_el_f8" : (a == DT::BF16 ? "rx_el_bf16" : "rx_el_f16");
    // 256x128 tiles: wavefronts of 64x64 (4 + 4 fragments per K tile for 16 MFMA blocks) instead of 128x32 (8 + 2):
    // the 8192 x 1024 x 4096 bf16 layer 68.3 -> 66.6 us
    if (BN == 128 && !tuned) { WM = 4; WN = 2; }
    // three LDS stages where they fit (256x128 tiles: 144 KB): a request then has two K tiles to land instead of one
    int sstages = (BM + BN) * 128 * 3 <= 160 * 1024 ? 3 : 2;
    if (const char* e = getenv("RX_GEMM_STREAM_STAGES")) {
      if ((atoi(e) != 2 && atoi(e) != 3) || (BM + BN) * 128 * atoi(e) > 160 * 1024) refuse("RX_GEMM_STREAM_STAGES is 2, or 3 where three stages fit 160 KB");
      sstages = atoi(e);
    }
    c.lds_bytes = (unsigned)(sstages * (BM + BN) * 128);
    c.block = nt;
    c.grid[0] = (unsigned)gemm_grid((M + BM - 1) / BM, (N + BN - 1) / BN, rb, cb);
    c.grid[1] = (unsigned)batch;
    c.split = 1;
    std::ostringstream t;
    t << el << ", " << BM << ", " << BN << ", " << WM << ", " << WN << ", " << (a_kc ? "true" : "false") << ", " << (b_kc ? "true" : "false") << ", " << M
      << ", " << N << ", " << K << ", " << rb << ", " << cb;
    c.targs = t.str();
    c.stype_a = el + "::elem";
    // 256 x 256 tiles with an even number of K tiles: the ping-pong form of the same tiles (rx_gemm_body_pp: one
    // wavefront of a SIMD multiplies a whole K tile while the other reads its fragments) for 16-bit operands, and for
    // 8-bit operands when B is stored [n][k] (then the requests are shared between the two groups of wavefronts; with
    // one group requesting everything the 8-bit form is slower than the interleaved one).  RX_GEMM_PINGPONG=0 keeps
    // the interleaved form, =1 takes the ping-pong form wherever it exists.
    const int pp = getenv("RX_GEMM_PINGPONG") ? atoi(getenv("RX_GEMM_PINGPONG")) : ((esize == 2 || b_kc) ? 1 : 0);
    if (pp != 0 && BM == 256 && BN == 256 && WM == 2 && WN == 4 && (K / bk) % 2 == 0 && !getenv("RX_GEMM_STREAM_STAGES") && !getenv("RX_GEMM_STREAM_DEPTH")) {
      c.lds_bytes = (unsigned)(2 * (BM + BN) * 128);
      c.skeleton = "rx_gemm_body_pp";
      c.ok = true;
      return c;
    }
    c.skeleton = "rx_gemm_body_s";
    c.depth = 2;
    if (const char* e = getenv("RX_GEMM_STREAM_DEPTH")) {
      if (atoi(e) < 1 || atoi(e) > 3) refuse("RX_GEMM_STREAM_DEPTH is 1, 2 or 3");
      c.depth = atoi(e);
    }
    c.stream_stages = sstages;
    c.stype_a = el + "::elem";
    c.ok = true;
    return c;
  }
  if (direct) {
    const int dbk = bk;
    // 16-bit operands take the 16x16x32 MFMA here (kernels/rx_gemm_kernels.h, rx_mma_16b_16): k step 32
    const bool mfma16 = esize == 2 && dbk % 32 == 0 && !(getenv("RX_GEMM_MFMA32") && atoi(getenv("RX_GEMM_MFMA32")) != 0);
    const std::string dmma = mfma16 ? mma + "_16" : mma;
    const int ks = mfma16 ? 32 : ks_step;
    const int64_t a_ch = (int64_t)BM * dbk / ve, b_ch = (int64_t)BN * dbk / ve;
    const int64_t stage_bytes = ((int64_t)BM + BN) * dbk * esize;
    while (stages > 2 && stage_bytes * stages > 160 * 1024) --stages;
    if (dbk % ks == 0 && K % ((int64_t)dbk * split) == 0 && a_ch % nt == 0 && b_ch % nt == 0 && stage_bytes * stages <= 160 * 1024 &&
        (a_kc ? dbk : BM) % ve == 0 && (b_kc ? dbk : BN) % ve == 0) {
      c.lds_bytes = (unsigned)(stage_bytes * stages);
      c.block = nt;
      const int64_t gm = (M + BM - 1) / BM, gn = (N + BN - 1) / BN;
      c.grid[0] = (unsigned)gemm_grid(gm, gn, rb, cb);
      c.grid[1] = (unsigned)(split > 1 ? split : batch);
      c.split = split;
      std::ostringstream t;
      t << dmma << ", " << BM << ", " << BN << ", " << dbk << ", " << WM << ", " << WN << ", " << stages << ", " << (a_kc ? "true" : "false") << ", "
        << (b_kc ? "true" : "false") << ", " << M << ", " << N << ", " << K << ", " << rb << ", " << cb;
      c.targs = t.str();
      c.skeleton = "rx_gemm_body_dl";
      c.bk = dbk;
      c.stype_a = dmma + "::elem";
      c.ok = true;
      return c;
    }
    if (direct_forced) refuse("the direct-to-LDS skeleton does not tile this shape");
    if (tuned && stage_bytes * 2 > 160 * 1024) refuse("two LDS stages of this tile exceed 160 KB");
  }
  if (split > 1) return c;   // only the direct-to-LDS skeleton slices K
  const int pad = a == DT::F32 ? 4 : (esize == 2 ? 8 : 16);
  const int64_t a_sz = a_kc ? (int64_t)BM * (bk + pad) : (int64_t)bk * (BM + pad);
  const int64_t b_sz = b_kc ? (int64_t)BN * (bk + pad) : (int64_t)bk * (BN + pad);
  c.lds_bytes = (unsigned)(2 * (a_sz + b_sz) * esize);
  if (c.lds_bytes > 160 * 1024) {
    if (tuned) refuse("the register-staged skeleton needs more than 160 KB of LDS for this tile and K step");
    return c;
  }
  c.block = WM * WN * 64;
  const int64_t gm = (M + BM - 1) / BM, gn = (N + BN - 1) / BN;
  c.grid[0] = (unsigned)gemm_grid(gm, gn, rb, cb);
  c.grid[1] = (unsigned)batch;
  std::ostringstream t;
  t << mma << ", " << BM << ", " << BN << ", " << bk << ", " << WM << ", " << WN << ", " << (a_kc ? "true" : "false") << ", " << (b_kc ? "true" : "false")
    << ", " << M << ", " << N << ", " << K << ", " << rb << ", " << cb;
  c.targs = t.str();
  c.skeleton = "rx_gemm_body";
  c.stype_a = mma + "::elem";
  c.ok = true;
  return c;
}

std::string gemm_instance(const GemmChoice& c, const std::string& kbase, const std::string& epi_params, const std::string& epi_ctor, bool batched,
                          const GemmOperandFn& fa, const GemmOperandFn& fb) {
  std::ostringstream o;
  o << "// dot_general on MFMA: " << c.kind << " <" << c.targs << ">\n";
  const bool fn = !fa.type.empty() || !fb.type.empty();
  o << "extern \"C\" __global__ __launch_bounds__(" << c.block << ") void " << kbase << "_gemm(";
  // operands that are read from memory come first, then what the operand functors read, then the epilogue's operands
  std::string params;
  if (fa.type.empty()) params += ", const " + c.stype_a + "* __restrict__ A";
  if (fb.type.empty()) params += ", const " + c.stype_a + "* __restrict__ B";
  params += fa.params + fb.params + epi_params;
  o << params.substr(2) << ") {\n";
  if (!fa.type.empty()) o << "  const " << c.stype_a << "* A = nullptr;\n  " << fa.ctor << "\n";
  if (!fb.type.empty()) o << "  const " << c.stype_a << "* B = nullptr;\n  " << fb.ctor << "\n";
  o << "  " << epi_ctor << "\n";
  o << "  " << c.skeleton << "<" << c.targs << ", " << (batched ? "true" : "false") << ", " << kbase << "_epi";
  if (fn) o << ", " << (fa.type.empty() ? "rx_no_fn" : fa.type) << ", " << (fb.type.empty() ? "rx_no_fn" : fb.type);
  if (c.split > 1) o << ", " << c.split;
  if (c.depth > 0) o << ", " << c.depth;
  if (c.stream_stages > 0) o << ", " << c.stream_stages;
  o << ">(A, B, epi";
  if (fn) o << ", " << (fa.type.empty() ? "rx_no_fn()" : "la") << ", " << (fb.type.empty() ? "rx_no_fn()" : "lb");
  o << ");\n}\n\n";
  return o.str();
}

ConvChoice choose_conv(int64_t B, int64_t C, int64_t H, int64_t W, int64_t O, int64_t KH, int64_t KW, int64_t HO, int64_t WO, int64_t pl,
                       int64_t sh, int64_t sw, int64_t dh, int64_t dw) {
  ConvChoice c;
  if (getenv("RX_CONV_DIRECT") && atoi(getenv("RX_CONV_DIRECT")) == 0) return c;
  if (getenv("RX_MFMA") && atoi(getenv("RX_MFMA")) == 0) return c;
  if (B < 1 || C < 1 || O < 1 || HO < 1 || WO < 1 || KH < 1 || KW < 1) return c;
  // four wavefronts of 16 features each: with fewer than 33 features half of them would idle; a tile is whole rows of
  // the result, at most 25 blocks of 16 pixels (100 accumulator registers); taps unroll, so the filter is small
  if (O < 33 || WO > 400 || KH * KW > 49 || KH > H + 64 || KW > W + 64 || sh < 1 || sw < 1 || dh < 1 || dw < 1 || sh > 4 || sw > 4) return c;
  if (B * C * H * W >= ((int64_t)1 << 31) || B * O * HO * WO >= ((int64_t)1 << 31)) return c;
  const int64_t groups = (O + 63) / 64;
  const int slab = C >= 8 ? 8 : 4;
  const int64_t stages = (C + slab - 1) / slab > 1 ? 2 : 1;
  auto lds_of = [&](int64_t tr) {
    const int64_t pr = (tr - 1) * sh + (KH - 1) * dh + 1, off = (pl + 3) / 4 * 4, lastc = (WO - 1) * sw + (KW - 1) * dw - pl;
    const int64_t pw = (off + std::max<int64_t>(lastc + 1, W) + 3) / 4 * 4;
    const int64_t pch = (pr * pw + 47) / 64 * 64 + 16;
    return (stages * slab * pch + stages * KH * KW * (slab / 4) * 4 * 80) * 4;
  };
  // rows per workgroup: least padded work (ragged last tile, ragged last pixel block, workgroups in whole rounds of
  // the 256 compute units) among the tiles that fit
  double best = 0;
  for (int64_t tr = 1; tr <= HO && tr * WO <= 400; ++tr) {
    if (lds_of(tr) > 160 * 1024) break;
    const int64_t tiles = (HO + tr - 1) / tr, npb = (tr * WO + 15) / 16;
    const int64_t wgs = B * tiles * groups;
    const double rounds = (double)((wgs + 255) / 256);
    // time of the slowest compute unit: the MFMAs of its pixel blocks, the filter it reads once per tile (about one pixel block's worth) and the patch loads
    const double cost = rounds * ((double)npb + 1.0) * (1.0 + 0.02 * (double)((tr - 1) * sh + (KH - 1) * dh + 1) / (double)tr);
    if (c.rows == 0 || cost < best) { best = cost; c.rows = (int)tr; }
  }
  if (c.rows == 0) return c;
  if (const char* e = getenv("RX_CONV_ROWS")) {
    const int v = atoi(e);
    if (v >= 1 && v <= HO && (int64_t)v * WO <= 400 && lds_of(v) <= 160 * 1024) c.rows = v;
  }
  // Against the matrix product on the window matrix, whose tiles span images and which can slice the channels: a
  // workgroup of this kernel passes all channels of its 64 features through LDS for one tile of one image, about 1.5 us
  // per slab however few pixels the tile has.  Estimates in microseconds, fitted to 3 x 3 layers of 64 to 512 features
  // on 7 x 7 to 56 x 56 images in batches of 4 and 32 (512 -> 512 on 14 x 14, 4 images: 0.097 ms direct against 0.055;
  // 32 images of 256 -> 256: 0.086 against 0.103): slabs of max(1.5 us, 1.35 x their MFMA time) here; 70 TFLOP/s, a
  // window matrix written and read when there are more than 128 features, a layout map of the result and two more
  // launches there.
  {
    const int64_t tiles = (HO + c.rows - 1) / c.rows, npb = (c.rows * WO + 15) / 16;
    const double rounds = (double)((B * tiles * groups + 255) / 256);
    const double nslab = (double)((C + slab - 1) / slab), nstep = (double)(KH * KW * (slab / 4));
    const double direct_us = rounds * nslab * std::max(1.5, 1.35 * (double)npb * nstep * 32.0 / 2200.0) + 5.0;
    const double flops = 2.0 * (double)B * (double)O * (double)HO * (double)WO * (double)C * (double)(KH * KW);
    const double window_bytes = O > 128 ? 2.0 * 4.0 * (double)B * (double)C * (double)(KH * KW) * (double)HO * (double)WO : 0.0;
    const double product_us = flops / 70e6 + (window_bytes + 2.0 * 4.0 * (double)B * (double)O * (double)HO * (double)WO) / 5e6 + 5.0 + 8.0;   // three launches
    const char* force = getenv("RX_CONV_DIRECT");   // 2: this kernel wherever it covers the case
    if (direct_us > product_us && !(force && atoi(force) == 2)) { c.rows = 0; return c; }
  }
  c.slab = slab;
  c.grid[0] = (unsigned)(B * ((HO + c.rows - 1) / c.rows));
  c.grid[1] = (unsigned)groups;
  c.lds_bytes = (unsigned)lds_of(c.rows);
  c.ok = true;
  return c;
}

}  // namespace rx

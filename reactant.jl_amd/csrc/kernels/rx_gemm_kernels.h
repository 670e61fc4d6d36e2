// MFMA GEMM skeleton for gfx950 (wave64).  One template covers f32, bf16, f16 and
// f8E4M3FN operands with f32 accumulation, both storage orders of each operand,
// an optional batch dimension, and an epilogue functor that the fusion code
// generator writes for each dot_general group (alpha/beta, bias + gelu, dequant...).
//
//   D[m][n] = sum_k A(m,k) * B(k,n)
//   A is stored [M][K] (A_KC, K contiguous) or [K][M];  B is stored [N][K] (B_KC) or [K][N].
//
// Tiling: a workgroup of WM x WN wavefronts computes a BM x BN tile; each wavefront
// owns (BM/WM) x (BN/WN) as a grid of 32x32 MFMA tiles.  K is walked in steps of BK
// through two LDS buffers: while the MFMAs consume buffer i, the global loads for
// the next step are in flight in registers and are written to buffer i^1 afterwards
// (one barrier per step).  LDS rows are padded so that the 16-byte fragment reads
// of 16 consecutive rows fall into distinct banks.  An operand whose K is not the
// contiguous dimension is kept in LDS as [k][m|n] and read with the LDS transpose
// loads (ds_read_b64_tr_b16 / _b8), which hand each lane consecutive-k values.
//
// The MFMA is issued with the B fragment as the row operand, so a lane holds four
// consecutive n for one m: the epilogue then works on 4-element vectors.
//
// The k index inside one MFMA is whatever the hardware assigns to (lane group,
// register byte); A and B fragments are loaded with the same mapping, which is all
// a contraction needs.
#pragma once

typedef float rx_f32x4 __attribute__((ext_vector_type(4)));
typedef float rx_f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 rx_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 rx_bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 rx_f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 rx_f16x4 __attribute__((ext_vector_type(4)));
typedef short rx_i16x4 __attribute__((ext_vector_type(4)));
typedef int rx_i32x8 __attribute__((ext_vector_type(8)));
typedef int rx_i32x4 __attribute__((ext_vector_type(4)));
typedef int rx_i32x2 __attribute__((ext_vector_type(2)));

#define RX_LDS __attribute__((address_space(3)))
#define RX_LDS_PTR(T, p) ((RX_LDS T*)(p))
// LDS tiles are addressed through address_space(3) pointers throughout, so that every access is
// a ds_read / ds_write (a generic pointer would turn them into slower flat accesses).

// ---------------------------------------------------------------------------
// MMA policies.  KS = k extent consumed by one `mma` call; frag = per-lane operand.
//   load_kc: operand tile in LDS as [o][k] (row stride `ld` elements), 32 rows from `row0`
//   load_tr: operand tile in LDS as [k][o] (row stride `ld` elements), 32 columns from `col0`
// ---------------------------------------------------------------------------
struct rx_mma_f32 {
  typedef float elem;
  typedef rx_f32x4 frag;
  static constexpr int KS = 8;
  static constexpr int PAD = 4;   // elements of row padding in LDS
  RX_DEV frag load_kc(const RX_LDS elem* t, int ld, int row0, int kk, int lane) {
    return *(const RX_LDS rx_f32x4*)(t + (row0 + (lane & 31)) * ld + kk + 4 * (lane >> 5));
  }
  RX_DEV frag load_tr(const RX_LDS elem* t, int ld, int col0, int kk, int lane) {
    const RX_LDS elem* p = t + (kk + 4 * (lane >> 5)) * ld + col0 + (lane & 31);
    frag f;
    f[0] = p[0];
    f[1] = p[ld];
    f[2] = p[2 * ld];
    f[3] = p[3 * ld];
    return f;
  }
  RX_DEV void mma(rx_f32x16& c, const frag& rowop, const frag& colop) {
#pragma unroll
    for (int j = 0; j < 4; ++j) c = __builtin_amdgcn_mfma_f32_32x32x2f32(rowop[j], colop[j], c, 0, 0, 0);
  }
};

struct rx_mma_bf16 {
  typedef rx_u16 elem;
  typedef rx_bf16x8 frag;
  static constexpr int KS = 16;
  static constexpr int PAD = 8;
  RX_DEV frag load_kc(const RX_LDS elem* t, int ld, int row0, int kk, int lane) {
    return *(const RX_LDS rx_bf16x8*)(t + (row0 + (lane & 31)) * ld + kk + 8 * (lane >> 5));
  }
  RX_DEV frag load_tr(const RX_LDS elem* t, int ld, int col0, int kk, int lane) {
    // 16-lane blocks: source lane i points at row k + i/4, columns 4*(i%4)..+3; after the
    // transpose lane j of the block holds 4 consecutive k for column j.
    const int i = lane & 15, q = (lane >> 4) & 1, g = lane >> 5;
    const RX_LDS elem* p = t + (kk + 8 * g + (i >> 2)) * ld + col0 + 16 * q + 4 * (i & 3);
    rx_i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(RX_LDS_PTR(rx_i16x4, p));
    rx_i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(RX_LDS_PTR(rx_i16x4, p + 4 * ld));
    struct { rx_i16x4 a, b; } both = {lo, hi};
    return __builtin_bit_cast(rx_bf16x8, both);
  }
  RX_DEV void mma(rx_f32x16& c, const frag& rowop, const frag& colop) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(rowop, colop, c, 0, 0, 0);
  }
};

struct rx_mma_f16 {
  typedef rx_u16 elem;
  typedef rx_f16x8 frag;
  static constexpr int KS = 16;
  static constexpr int PAD = 8;
  RX_DEV frag load_kc(const RX_LDS elem* t, int ld, int row0, int kk, int lane) {
    return *(const RX_LDS rx_f16x8*)(t + (row0 + (lane & 31)) * ld + kk + 8 * (lane >> 5));
  }
  RX_DEV frag load_tr(const RX_LDS elem* t, int ld, int col0, int kk, int lane) {
    const int i = lane & 15, q = (lane >> 4) & 1, g = lane >> 5;
    const RX_LDS elem* p = t + (kk + 8 * g + (i >> 2)) * ld + col0 + 16 * q + 4 * (i & 3);
    rx_i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(RX_LDS_PTR(rx_i16x4, p));
    rx_i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(RX_LDS_PTR(rx_i16x4, p + 4 * ld));
    struct { rx_i16x4 a, b; } both = {lo, hi};
    return __builtin_bit_cast(rx_f16x8, both);
  }
  RX_DEV void mma(rx_f32x16& c, const frag& rowop, const frag& colop) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(rowop, colop, c, 0, 0, 0);
  }
};

// f8E4M3FN x f8E4M3FN (OCP e4m3 on gfx950), 64 k per instruction
struct rx_mma_f8 {
  typedef rx_u8 elem;
  typedef rx_i32x8 frag;
  static constexpr int KS = 64;
  static constexpr int PAD = 16;
  RX_DEV frag load_kc(const RX_LDS elem* t, int ld, int row0, int kk, int lane) {
    const RX_LDS elem* p = t + (row0 + (lane & 31)) * ld + kk + 32 * (lane >> 5);
    struct { rx_i32x4 a, b; } both = {*(const RX_LDS rx_i32x4*)(p), *(const RX_LDS rx_i32x4*)(p + 16)};
    return __builtin_bit_cast(rx_i32x8, both);
  }
  RX_DEV frag load_tr(const RX_LDS elem* t, int ld, int col0, int kk, int lane) {
    // 16-lane blocks: source lane i points at row k + i/2, columns 8*(i%2)..+7; after the
    // transpose lane j of the block holds 8 consecutive k for column j.
    const int i = lane & 15, q = (lane >> 4) & 1, g = lane >> 5;
    const RX_LDS elem* p = t + (kk + 32 * g + (i >> 1)) * ld + col0 + 16 * q + 8 * (i & 1);
    struct { rx_i32x2 a, b, c, d; } all = {
        __builtin_amdgcn_ds_read_tr8_b64_v2i32(RX_LDS_PTR(rx_i32x2, p)),
        __builtin_amdgcn_ds_read_tr8_b64_v2i32(RX_LDS_PTR(rx_i32x2, p + 8 * ld)),
        __builtin_amdgcn_ds_read_tr8_b64_v2i32(RX_LDS_PTR(rx_i32x2, p + 16 * ld)),
        __builtin_amdgcn_ds_read_tr8_b64_v2i32(RX_LDS_PTR(rx_i32x2, p + 24 * ld))};
    return __builtin_bit_cast(rx_i32x8, all);
  }
  RX_DEV void mma(rx_f32x16& c, const frag& rowop, const frag& colop) {
    // formats 0/0 = e4m3 x e4m3; zero scale operands select the unscaled instruction
    c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(rowop, colop, c, 0, 0, 0, 0, 0, 0);
  }
};

// ---------------------------------------------------------------------------
// cooperative copy of one operand tile: global (row-major, leading dim `gld`) ->
// registers -> LDS (row stride `lld`).  ROWS x COLS elements, 16-byte vectors.
// Rows / column vectors past the end of the matrix are clamped to the last valid
// ones (their products are never stored).
// ---------------------------------------------------------------------------
template <typename E, int ROWS, int COLS, int NT>
struct rx_tile_copy {
  static constexpr int VE = 16 / (int)sizeof(E);           // elements per vector
  static constexpr int VPR = COLS / VE;                    // vectors per row
  static constexpr int TOTAL = ROWS * VPR;
  static constexpr int PER = (TOTAL + NT - 1) / NT;        // vectors per thread
  rx_u32x4 r[PER];

  // ZR / ZC: rows / column vectors past the end read as zero instead (the contracted dimension,
  // whose tail must not contribute to the sums)
  template <bool ZR, bool ZC>
  RX_MEM void load(const E* __restrict__ g, long long gld, int row0, int col0, int nrows, int ncols, int tid) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int v = tid + i * NT;
      if (TOTAL % NT == 0 || v < TOTAL) {
        int rr = row0 + v / VPR;
        int cc = col0 + (v % VPR) * VE;
        const bool zero = (ZR && rr >= nrows) || (ZC && cc + VE > ncols);
        rr = rr < nrows ? rr : nrows - 1;
        cc = cc + VE <= ncols ? cc : ncols - VE;
        r[i] = *reinterpret_cast<const rx_u32x4*>(g + (long long)rr * gld + cc);
        if (zero) r[i] = rx_u32x4{0u, 0u, 0u, 0u};
      }
    }
  }
  // The same tile taken from a functor instead of memory: fn(batch, row, col) is element (row, col)
  // of the operand as it would be stored; positions outside the matrix are zero.
  template <class FN>
  RX_MEM void load_fn(const FN& fn, long long batch, int row0, int col0, int nrows, int ncols, int tid) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int v = tid + i * NT;
      if (TOTAL % NT == 0 || v < TOTAL) {
        const int rr = row0 + v / VPR;
        const int cc = col0 + (v % VPR) * VE;
        union { E e[VE]; rx_u32x4 q; } u;
        if constexpr (FN::vec_width == VE) {
          // a whole vector inside the matrix: the functor's vector form shares the index arithmetic between the lanes
          if (rr < nrows && cc + VE <= ncols) {
            fn.vec(batch, rr, cc, u.e);
          } else {
#pragma unroll
            for (int k = 0; k < VE; ++k) u.e[k] = (rr < nrows && cc + k < ncols) ? fn(batch, rr, cc + k) : E(0);
          }
        } else {
#pragma unroll
          for (int k = 0; k < VE; ++k) u.e[k] = (rr < nrows && cc + k < ncols) ? fn(batch, rr, cc + k) : E(0);
        }
        r[i] = u.q;
      }
    }
  }
  RX_MEM void store(RX_LDS E* lds, int lld, int tid) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int v = tid + i * NT;
      if (TOTAL % NT == 0 || v < TOTAL) *(RX_LDS rx_u32x4*)(lds + (v / VPR) * lld + (v % VPR) * VE) = r[i];
    }
  }
};

// ---------------------------------------------------------------------------
// the kernel body
// ---------------------------------------------------------------------------
// Tile order.  Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  The tile
// grid is cut into blocks of RB x CB tiles; XCD k takes blocks k, k+8, ... and the
// tiles of one block run side by side on that XCD, so they share RB row panels of A and CB
// column panels of B in its L2.  The 8 blocks in flight are consecutive in row-major block
// order, which keeps the panels they share in the memory-side cache.  The grid is padded to
// whole blocks on every XCD (rx::gemm_grid on the host computes the same number); a workgroup
// whose tile falls outside the grid returns false.
template <int GM, int GN, int RB, int CB>
RX_DEV bool rx_gemm_tile(unsigned bid, int* bm, int* bn) {
  if constexpr (RB == 0) {   // small tile grids: no blocks, no padding (one workgroup per tile)
    *bm = (int)(bid % (unsigned)GM);
    *bn = (int)(bid / (unsigned)GM);
    return *bn < GN;
  } else {
    constexpr unsigned PER = RB * CB;
    constexpr unsigned NBC = (GN + CB - 1) / CB;
    const unsigned xcd = bid & 7u, j = bid >> 3;
    const unsigned blk = (j / PER) * 8u + xcd, t = j % PER;
    const unsigned br = blk / NBC, bc = blk % NBC;
    *bm = (int)(br * RB + t % RB);
    *bn = (int)(bc * CB + t / RB);
    return *bm < GM && *bn < GN;
  }
}

// An operand can also be a functor (LA / LB other than rx_no_fn): the fusion code generator
// writes one when the operand is a cheap expansion of smaller data (the window matrix of a
// convolution, a broadcast), so that the expanded matrix never exists in memory.
struct rx_no_fn {
  static constexpr bool none = true;
  static constexpr int vec_width = 0;
  static constexpr int C = 0;                 // as a K-offset functor: none
  RX_DEV unsigned at(int) { return 0u; }
  RX_DEV int row(int) { return 0; }
  RX_DEV int col(int) { return 0; }
};

// An epilogue functor that declares `static constexpr bool masks_rows = true` tests the row it is called with itself
// (it guards its stores only): the skeleton then calls it for the rows past the product's last one too, and with whole
// column tiles the epilogue is straight-line code, in which what depends on the column alone is computed once.
template <class E, class = void> struct rx_epi_masks_rows { static constexpr bool value = false; };
template <class E> struct rx_epi_masks_rows<E, decltype((void)E::masks_rows)> { static constexpr bool value = E::masks_rows; };

template <class MMA, int BM, int BN, int BK, int WM, int WN, bool A_KC, bool B_KC, int M, int N, int K, int RB, int CB, bool BATCHED, class Epi,
          class LA = rx_no_fn, class LB = rx_no_fn>
RX_DEV void rx_gemm_body(const typename MMA::elem* __restrict__ A, const typename MMA::elem* __restrict__ B, const Epi& epi, const LA& la = LA(),
                         const LB& lb = LB()) {
  typedef typename MMA::elem E;
  constexpr int NT = WM * WN * 64;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;   // 32x32 tiles per wavefront
  constexpr int A_ROWS = A_KC ? BM : BK, A_COLS = A_KC ? BK : BM;
  constexpr int B_ROWS = B_KC ? BN : BK, B_COLS = B_KC ? BK : BN;
  constexpr int A_LD = A_COLS + MMA::PAD, B_LD = B_COLS + MMA::PAD;
  constexpr int A_SZ = A_ROWS * A_LD, B_SZ = B_ROWS * B_LD;
  extern __shared__ __attribute__((aligned(16))) unsigned char rx_smem[];
  RX_LDS E* lds = (RX_LDS E*)rx_smem;
  constexpr int STAGE = A_SZ + B_SZ;   // buffer s: A at s*STAGE, B at s*STAGE + A_SZ

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  constexpr int GM = (M + BM - 1) / BM, GN = (N + BN - 1) / BN;
  int bm, bn;
  if (!rx_gemm_tile<GM, GN, RB, CB>(blockIdx.x, &bm, &bn)) return;
  const int m0 = bm * BM, n0 = bn * BN;
  const long long batch = BATCHED ? blockIdx.y : 0;
  const E* Ab = A + batch * (long long)M * K;
  const E* Bb = B + batch * (long long)N * K;
  constexpr long long A_GLD = A_KC ? K : M, B_GLD = B_KC ? K : N;

  rx_f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  rx_tile_copy<E, A_ROWS, A_COLS, NT> ca;
  rx_tile_copy<E, B_ROWS, B_COLS, NT> cb;
  auto gload = [&](int k0) {
    constexpr bool TAIL = K % BK != 0;   // only then can a tile reach past the contracted dimension
    if constexpr (!LA::none) {
      if (A_KC) ca.load_fn(la, batch, m0, k0, M, K, tid); else ca.load_fn(la, batch, k0, m0, K, M, tid);
    } else {
      if (A_KC) ca.template load<false, TAIL>(Ab, A_GLD, m0, k0, M, K, tid); else ca.template load<TAIL, false>(Ab, A_GLD, k0, m0, K, M, tid);
    }
    if constexpr (!LB::none) {
      if (B_KC) cb.load_fn(lb, batch, n0, k0, N, K, tid); else cb.load_fn(lb, batch, k0, n0, K, N, tid);
    } else {
      if (B_KC) cb.template load<false, TAIL>(Bb, B_GLD, n0, k0, N, K, tid); else cb.template load<TAIL, false>(Bb, B_GLD, k0, n0, K, N, tid);
    }
  };
  gload(0);
  ca.store(lds, A_LD, tid);
  cb.store(lds + A_SZ, B_LD, tid);
  __syncthreads();

  constexpr int KT = (K + BK - 1) / BK;
  for (int kt = 0; kt < KT; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < KT) gload((kt + 1) * BK);
    const RX_LDS E* sa = lds + cur * STAGE;
    const RX_LDS E* sb = sa + A_SZ;
#pragma unroll
    for (int kk = 0; kk < BK; kk += MMA::KS) {
      typename MMA::frag fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int o = wm * (BM / WM) + 32 * i;
        fa[i] = A_KC ? MMA::load_kc(sa, A_LD, o, kk, lane) : MMA::load_tr(sa, A_LD, o, kk, lane);
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int o = wn * (BN / WN) + 32 * j;
        fb[j] = B_KC ? MMA::load_kc(sb, B_LD, o, kk, lane) : MMA::load_tr(sb, B_LD, o, kk, lane);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) MMA::mma(acc[i][j], fb[j], fa[i]);
    }
    if (kt + 1 < KT) {
      ca.store(lds + (cur ^ 1) * STAGE, A_LD, tid);
      cb.store(lds + (cur ^ 1) * STAGE + A_SZ, B_LD, tid);
    }
    __syncthreads();
  }

  // epilogue: lane holds D[n = 8*(r/4) + 4*(lane/32) + r%4][m = lane%32] of each 32x32 tile
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + wm * (BM / WM) + 32 * i + (lane & 31);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int nb = n0 + wn * (BN / WN) + 32 * j + 4 * (lane >> 5);
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const int n = nb + 8 * rg;
        if (m < M && n < N) {
          const float v[4] = {acc[i][j][4 * rg], acc[i][j][4 * rg + 1], acc[i][j][4 * rg + 2], acc[i][j][4 * rg + 3]};
          if constexpr (BATCHED) epi(v, (int)batch, m, n); else epi(v, m, n);
        }
      }
    }
  }
}

// ===========================================================================
// Second body: operand tiles travel global -> LDS directly (global_load_lds, 16 bytes per
// lane, no VGPR staging) through a ring of S LDS stages, so S-1 K-steps of loads are in
// flight while one is being multiplied.  A wavefront's load fills 1 KB of contiguous LDS in
// lane order, which rules out row padding; bank conflicts are avoided instead by an XOR
// swizzle of the 16-byte chunk index inside each row, applied on the global-address side
// when loading and on the LDS-address side when reading fragments.
// ===========================================================================

// chunk position inside an LDS row of CPR 16-byte chunks
//   KC tiles ([o][k], fragment reads of 16 consecutive rows at one chunk index)
template <int CPR>
RX_DEV int rx_swz_kc(int row, int c) {
  constexpr int R = CPR >= 16 ? 1 : 16 / CPR;          // rows per 256 bytes of LDS
  return c ^ ((row / R) & (CPR - 1));
}
//   TR tiles ([k][o]): which rows are read together depends on the element size
template <int ESIZE, int CPR>
RX_DEV int rx_swz_tr(int row, int c) {
  // 32 lanes of a transpose read touch 4 rows x 64 B (16-bit) or 8 rows x 32 B (8-bit): each row
  // is moved to its own 64 B / 32 B group so that the 32 lanes cover all 64 banks once
  if constexpr (ESIZE == 2) return c ^ (((row & 3) << 2) & (CPR - 1));
  else if constexpr (ESIZE == 1) return c ^ (((row & 7) << 1) & (CPR - 1));
  else return c ^ ((((row >> 2) & 1) << 3) & (CPR - 1));                      // rows k, k+4 read in one instruction
}

//   TR tiles of 16-bit elements read by the 16 x 16 x 32 MFMA's fragments: the four 16-lane blocks of a transpose read
//   take rows k, k+8, k+16, k+24, so one 32-lane phase reads rows k..k+3 and k+8..k+11, 32 bytes of each; every
//   one of those eight rows gets its own 32-byte group of the 256 bytes that the 64 banks hold
template <int CPR>
RX_DEV int rx_swz_tr16(int row, int c) {
  return c ^ ((((row & 3) | (((row >> 3) & 1) << 2)) << 1) & (CPR - 1));
}

template <class MMA> struct rx_frag_sw;

template <> struct rx_frag_sw<rx_mma_f32> {
  template <int LD> RX_DEV rx_mma_f32::frag kc(const RX_LDS float* t, int row0, int kk, int lane) {
    const int r = row0 + (lane & 31), c = (kk + 4 * (lane >> 5)) >> 2;
    return *(const RX_LDS rx_f32x4*)(t + r * LD + rx_swz_kc<LD / 4>(r, c) * 4);
  }
  template <int LD> RX_DEV rx_mma_f32::frag tr(const RX_LDS float* t, int col0, int kk, int lane) {
    const int col = col0 + (lane & 31), k = kk + 4 * (lane >> 5);
    rx_mma_f32::frag f;
#pragma unroll
    for (int j = 0; j < 4; ++j) f[j] = t[(k + j) * LD + rx_swz_tr<4, LD / 4>(k + j, col >> 2) * 4 + (col & 3)];
    return f;
  }
};
template <> struct rx_frag_sw<rx_mma_bf16> {
  template <int LD> RX_DEV rx_bf16x8 kc(const RX_LDS rx_u16* t, int row0, int kk, int lane) {
    const int r = row0 + (lane & 31), c = (kk + 8 * (lane >> 5)) >> 3;
    return *(const RX_LDS rx_bf16x8*)(t + r * LD + rx_swz_kc<LD / 8>(r, c) * 8);
  }
  template <int LD> RX_DEV rx_bf16x8 tr(const RX_LDS rx_u16* t, int col0, int kk, int lane) {
    const int i = lane & 15, q = (lane >> 4) & 1, g = lane >> 5;
    const int k = kk + 8 * g + (i >> 2), col = col0 + 16 * q + 4 * (i & 3);
    const RX_LDS rx_u16* p0 = t + k * LD + rx_swz_tr<2, LD / 8>(k, col >> 3) * 8 + (col & 7);
    const RX_LDS rx_u16* p1 = t + (k + 4) * LD + rx_swz_tr<2, LD / 8>(k + 4, col >> 3) * 8 + (col & 7);
    struct { rx_i16x4 a, b; } both = {__builtin_amdgcn_ds_read_tr16_b64_v4i16(RX_LDS_PTR(rx_i16x4, p0)),
                                      __builtin_amdgcn_ds_read_tr16_b64_v4i16(RX_LDS_PTR(rx_i16x4, p1))};
    return __builtin_bit_cast(rx_bf16x8, both);
  }
};
template <> struct rx_frag_sw<rx_mma_f16> {
  template <int LD> RX_DEV rx_f16x8 kc(const RX_LDS rx_u16* t, int row0, int kk, int lane) {
    return __builtin_bit_cast(rx_f16x8, rx_frag_sw<rx_mma_bf16>::kc<LD>(t, row0, kk, lane));
  }
  template <int LD> RX_DEV rx_f16x8 tr(const RX_LDS rx_u16* t, int col0, int kk, int lane) {
    return __builtin_bit_cast(rx_f16x8, rx_frag_sw<rx_mma_bf16>::tr<LD>(t, col0, kk, lane));
  }
};
template <> struct rx_frag_sw<rx_mma_f8> {
  template <int LD> RX_DEV rx_i32x8 kc(const RX_LDS rx_u8* t, int row0, int kk, int lane) {
    const int r = row0 + (lane & 31), c = (kk + 32 * (lane >> 5)) >> 4;
    struct { rx_i32x4 a, b; } both = {*(const RX_LDS rx_i32x4*)(t + r * LD + rx_swz_kc<LD / 16>(r, c) * 16),
                                      *(const RX_LDS rx_i32x4*)(t + r * LD + rx_swz_kc<LD / 16>(r, c + 1) * 16)};
    return __builtin_bit_cast(rx_i32x8, both);
  }
  template <int LD> RX_DEV rx_i32x8 tr(const RX_LDS rx_u8* t, int col0, int kk, int lane) {
    const int i = lane & 15, q = (lane >> 4) & 1, g = lane >> 5;
    const int k = kk + 32 * g + (i >> 1), col = col0 + 16 * q + 8 * (i & 1);
    rx_i32x2 r[4];
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const int kh = k + 8 * h;
      const RX_LDS rx_u8* p = t + kh * LD + rx_swz_tr<1, LD / 16>(kh, col >> 4) * 16 + (col & 15);
      r[h] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((RX_LDS rx_i32x2*)p);
    }
    struct { rx_i32x2 a, b, c, d; } all = {r[0], r[1], r[2], r[3]};
    return __builtin_bit_cast(rx_i32x8, all);
  }
};

// ---------------------------------------------------------------------------
// 16-bit operands on v_mfma_f32_16x16x32_{bf16,f16}: under the power limit of this part the 16 x 16 x 32
// instruction sustains about 13 % more flops than 32 x 32 x 16 on the same operand data (measured with MFMAs
// alone on register operands), and a GEMM is power-bound.  The skeleton keeps its 32 x 32 bookkeeping: one
// "macro" step is 32 x 32 x 32 as four MFMAs, a fragment is the two 16-row halves of 32 rows (8 k per lane
// each: lane = row % 16 + 16 * k group), and sub-accumulator (a, b) -- rows 16a.. of the column operand, rows
// 16b.. of the row operand -- sits at registers 4 * (2a + b) .. + 3 of the 16.
// ---------------------------------------------------------------------------
typedef float rx_f32x4v __attribute__((ext_vector_type(4)));

template <bool BF>
struct rx_mma_16b_16 {
  typedef rx_u16 elem;
  typedef rx_i32x8 frag;
  static constexpr int KS = 32;
  static constexpr int PAD = 8;
  RX_DEV void mma(rx_f32x16& c, const frag& rowop, const frag& colop) {
    const rx_i32x4 r0 = {rowop[0], rowop[1], rowop[2], rowop[3]}, r1 = {rowop[4], rowop[5], rowop[6], rowop[7]};
    const rx_i32x4 c0 = {colop[0], colop[1], colop[2], colop[3]}, c1 = {colop[4], colop[5], colop[6], colop[7]};
    rx_f32x4v s[4] = {{c[0], c[1], c[2], c[3]}, {c[4], c[5], c[6], c[7]}, {c[8], c[9], c[10], c[11]}, {c[12], c[13], c[14], c[15]}};
    if constexpr (BF) {
      s[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(rx_bf16x8, r0), __builtin_bit_cast(rx_bf16x8, c0), s[0], 0, 0, 0);
      s[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(rx_bf16x8, r1), __builtin_bit_cast(rx_bf16x8, c0), s[1], 0, 0, 0);
      s[2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(rx_bf16x8, r0), __builtin_bit_cast(rx_bf16x8, c1), s[2], 0, 0, 0);
      s[3] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(rx_bf16x8, r1), __builtin_bit_cast(rx_bf16x8, c1), s[3], 0, 0, 0);
    } else {
      s[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(rx_f16x8, r0), __builtin_bit_cast(rx_f16x8, c0), s[0], 0, 0, 0);
      s[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(rx_f16x8, r1), __builtin_bit_cast(rx_f16x8, c0), s[1], 0, 0, 0);
      s[2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(rx_f16x8, r0), __builtin_bit_cast(rx_f16x8, c1), s[2], 0, 0, 0);
      s[3] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(rx_f16x8, r1), __builtin_bit_cast(rx_f16x8, c1), s[3], 0, 0, 0);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) c[4 * q + e] = s[q][e];
  }
};
typedef rx_mma_16b_16<true> rx_mma_bf16_16;
typedef rx_mma_16b_16<false> rx_mma_f16_16;

template <bool BF> struct rx_frag_sw<rx_mma_16b_16<BF>> {
  template <int LD> RX_DEV rx_i32x8 kc(const RX_LDS rx_u16* t, int row0, int kk, int lane) {
    const int r0 = row0 + (lane & 15), r1 = r0 + 16, c = (kk >> 3) + (lane >> 4);
    struct { rx_i32x4 a, b; } both = {*(const RX_LDS rx_i32x4*)(t + r0 * LD + rx_swz_kc<LD / 8>(r0, c) * 8),
                                      *(const RX_LDS rx_i32x4*)(t + r1 * LD + rx_swz_kc<LD / 8>(r1, c) * 8)};
    return __builtin_bit_cast(rx_i32x8, both);
  }
  template <int LD> RX_DEV rx_i32x8 tr(const RX_LDS rx_u16* t, int col0, int kk, int lane) {
    // a 16-lane block is one k group: source lane i points at row k + i/4, columns 4*(i%4)..+3; after the transpose
    // lane j of the block holds 4 consecutive k for column j
    const int i = lane & 15, g = lane >> 4;
    const int k = kk + 8 * g + (i >> 2);
    rx_i16x4 r[4];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int col = col0 + 16 * h + 4 * (i & 3);
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int kq = k + 4 * q;
        r[2 * h + q] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(RX_LDS_PTR(rx_i16x4, t + kq * LD + rx_swz_tr16<LD / 8>(kq, col >> 3) * 8 + (col & 7)));
      }
    }
    struct { rx_i16x4 a, b, c, d; } all = {r[0], r[1], r[2], r[3]};
    return __builtin_bit_cast(rx_i32x8, all);
  }
};

// What differs between the MFMA shapes outside the fragment readers: the swizzle of [k][o] tiles, the instruction
// counts that the schedule hints use, and where register group rg (four consecutive n) of a 32 x 32 tile lies.
template <class MMA> struct rx_mma_traits {
  static constexpr int TR_SWZ = 0;        // rx_swz_tr
  static constexpr int MFMA_PER_MMA = sizeof(typename MMA::elem) == 4 ? 4 : 1;
  static constexpr int RD_KC = sizeof(typename MMA::elem) == 1 ? 2 : 1;
  static constexpr int RD_TR = sizeof(typename MMA::elem) == 2 ? 2 : 4;
  static constexpr bool RAISE_PRIO = sizeof(typename MMA::elem) == 2;
  RX_DEV void coords(int lane, int rg, int* dm, int* dn) {
    *dm = lane & 31;
    *dn = 8 * rg + 4 * (lane >> 5);
  }
};
template <bool BF> struct rx_mma_traits<rx_mma_16b_16<BF>> {
  static constexpr int TR_SWZ = 1;        // rx_swz_tr16
  static constexpr int MFMA_PER_MMA = 4;
  static constexpr int RD_KC = 2;
  static constexpr int RD_TR = 4;
  static constexpr bool RAISE_PRIO = false;   // measured: raised priority costs this shape 7 % once the epilogue runs
  RX_DEV void coords(int lane, int rg, int* dm, int* dn) {
    *dm = 16 * (rg >> 1) + (lane & 15);
    *dn = 16 * (rg & 1) + 4 * (lane >> 4);
  }
};

template <int V> struct rx_int { static constexpr int value = V; };

// the instruction scheduler may not move anything across this point
#ifndef RX_GEMM_INTERLEAVE
#define RX_GEMM_INTERLEAVE 1
#endif
#ifndef RX_SCHED_FENCE
#define RX_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
#endif

// wait until at most N of this wavefront's vector-memory operations are outstanding
template <int N>
RX_DEV void rx_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// Issue the direct loads of one ROWS x COLS operand tile.  Slot s (16-byte units, lane order)
// of the LDS tile holds global chunk (row = s / CPR, c = swizzle^-1(pos = s % CPR)).
template <typename E, int ROWS, int COLS, int NT, bool KC, int TR_SWZ = 0>
RX_DEV void rx_tile_load_direct(const E* __restrict__ g, long long gld, int row0, int col0, int nrows, int ncols, RX_LDS E* lds, int tid) {
  constexpr int VE = 16 / (int)sizeof(E), CPR = COLS / VE, TOTAL = ROWS * CPR;
  static_assert(TOTAL % NT == 0, "tile must be a whole number of workgroup-wide loads");
  const int wave_base = (tid >> 6) << 6;
#pragma unroll
  for (int i = 0; i < TOTAL / NT; ++i) {
    const int s = i * NT + tid;
    const int row = s / CPR, pos = s % CPR;
    const int c = KC ? rx_swz_kc<CPR>(row, pos) : (TR_SWZ == 1 ? rx_swz_tr16<CPR>(row, pos) : rx_swz_tr<(int)sizeof(E), CPR>(row, pos));   // XOR is its own inverse
    int rr = row0 + row, cc = col0 + c * VE;
    rr = rr < nrows ? rr : nrows - 1;
    cc = cc + VE <= ncols ? cc : ncols - VE;
    // the LDS address is per wavefront: base of this wavefront's 1 KB run; lanes fill it in order
    RX_LDS E* dst = lds + (i * NT + wave_base) * VE;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(g + (long long)rr * gld + cc), (RX_LDS void*)dst, 16, 0, 0);
  }
}

// SPLIT > 1: workgroup (x, y) contracts the y-th of SPLIT equal slices of K and hands the epilogue
// (y, m, n): partial products that a reduction over the leading index adds up (few output tiles, long K).
template <class MMA, int BM, int BN, int BK, int WM, int WN, int S, bool A_KC, bool B_KC, int M, int N, int K, int RB, int CB, bool BATCHED, class Epi,
          int SPLIT = 1, class KOff = rx_no_fn>
RX_DEV void rx_gemm_body_dl(const typename MMA::elem* __restrict__ A, const typename MMA::elem* __restrict__ B, const Epi& epi) {
  typedef typename MMA::elem E;
  typedef rx_mma_traits<MMA> TRAITS;
  constexpr int NT = WM * WN * 64;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int A_ROWS = A_KC ? BM : BK, A_COLS = A_KC ? BK : BM;
  constexpr int B_ROWS = B_KC ? BN : BK, B_COLS = B_KC ? BK : BN;
  constexpr int A_SZ = A_ROWS * A_COLS, B_SZ = B_ROWS * B_COLS, STAGE = A_SZ + B_SZ;
  constexpr int VE = 16 / (int)sizeof(E);
  constexpr int LPS = (A_SZ + B_SZ) / VE / NT;     // loads per thread per stage
  extern __shared__ __attribute__((aligned(16))) unsigned char rx_smem[];
  RX_LDS E* lds = (RX_LDS E*)rx_smem;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  constexpr int GM = (M + BM - 1) / BM, GN = (N + BN - 1) / BN;
  int bm, bn;
  if (!rx_gemm_tile<GM, GN, RB, CB>(blockIdx.x, &bm, &bn)) return;
  const int m0 = bm * BM, n0 = bn * BN;
  const long long batch = BATCHED ? blockIdx.y : 0;
  const E* Ab = A + batch * (long long)M * K;
  const E* Bb = B + batch * (long long)N * K;
  constexpr long long A_GLD = A_KC ? K : M, B_GLD = B_KC ? K : N;
  static_assert(SPLIT >= 1 && K % (SPLIT * BK) == 0 && !(BATCHED && SPLIT > 1), "split of K");
  const int kbase = SPLIT > 1 ? (int)blockIdx.y * (K / SPLIT) : 0;

  rx_f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  auto issue = [&](int kt) {
    RX_LDS E* st = lds + (kt % S) * STAGE;
    const int k0 = kbase + kt * BK;
    if constexpr (!KOff::none) {
      // row shifts (rx_tap_shift): the first operand has KOff::C columns; a shifted row beyond its last one belongs to a
      // result that the epilogue does not keep, so the clamped read is as good as a zero
      static_assert(A_KC && !BATCHED && SPLIT == 1 && BK * (int)sizeof(E) == 128, "row shifts: [row][k] operand, K tiles of 128 bytes");
      rx_tile_load_direct<E, A_ROWS, A_COLS, NT, true>(Ab, (long long)KOff::C, m0 + KOff::row(kt), KOff::col(kt), M, KOff::C, st, tid);
    } else if (A_KC) rx_tile_load_direct<E, A_ROWS, A_COLS, NT, true>(Ab, A_GLD, m0, k0, M, K, st, tid);
    else rx_tile_load_direct<E, A_ROWS, A_COLS, NT, false, TRAITS::TR_SWZ>(Ab, A_GLD, k0, m0, K, M, st, tid);
    if (B_KC) rx_tile_load_direct<E, B_ROWS, B_COLS, NT, true>(Bb, B_GLD, n0, k0, N, K, st + A_SZ, tid);
    else rx_tile_load_direct<E, B_ROWS, B_COLS, NT, false, TRAITS::TR_SWZ>(Bb, B_GLD, k0, n0, K, N, st + A_SZ, tid);
  };
  constexpr int KT = K / SPLIT / BK;
  constexpr int NS = BK / MMA::KS;   // MFMA k-steps per tile
  // Fragments are double-buffered in registers: the LDS reads of step s+1 are issued before the
  // MFMAs of step s.  The barrier that publishes tile kt+1 sits before the LAST step of tile kt:
  // by then every wavefront holds its last fragments of tile kt in registers, so stage kt%S is
  // free for tile kt+S, and the first fragments of tile kt+1 load under the last MFMAs of tile kt.
  typename MMA::frag fa[2][TM], fb[2][TN];
  auto load_frags = [&](int buf, const RX_LDS E* sa, int kk) {
    const RX_LDS E* sb = sa + A_SZ;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int o = wm * (BM / WM) + 32 * i;
      if constexpr (A_KC) fa[buf][i] = rx_frag_sw<MMA>::template kc<A_COLS>(sa, o, kk, lane);
      else fa[buf][i] = rx_frag_sw<MMA>::template tr<A_COLS>(sa, o, kk, lane);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int o = wn * (BN / WN) + 32 * j;
      if constexpr (B_KC) fb[buf][j] = rx_frag_sw<MMA>::template kc<B_COLS>(sb, o, kk, lane);
      else fb[buf][j] = rx_frag_sw<MMA>::template tr<B_COLS>(sb, o, kk, lane);
    }
  };
  auto mma_all = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) MMA::mma(acc[i][j], fb[buf][j], fa[buf][i]);
  };
  // Ask the scheduler for the pattern "one MFMA, one LDS read, ..." over a step: the reads of the
  // next step trickle out under this step's MFMAs instead of going out in one burst.
  constexpr int RD_A = A_KC ? TRAITS::RD_KC : TRAITS::RD_TR;
  constexpr int RD_B = B_KC ? TRAITS::RD_KC : TRAITS::RD_TR;
  constexpr int NRD = TM * RD_A + TN * RD_B;
  constexpr int NMF = TM * TN * TRAITS::MFMA_PER_MMA;
  auto interleave = [&]() {
#if RX_GEMM_INTERLEAVE
    constexpr int PAIRS = NRD < NMF ? NRD : NMF;
    constexpr int MPP = NMF / PAIRS;   // MFMAs per LDS read when there are more MFMAs than reads
#pragma unroll
    for (int k = 0; k < PAIRS; ++k) {
      __builtin_amdgcn_sched_group_barrier(0x008, MPP, 0);   // MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);     // DS read
    }
    if constexpr (NMF > PAIRS * MPP) __builtin_amdgcn_sched_group_barrier(0x008, NMF - PAIRS * MPP, 0);
    if constexpr (NRD > PAIRS) __builtin_amdgcn_sched_group_barrier(0x100, NRD - PAIRS, 0);
#endif
  };
  auto publish = [&]() {
    asm volatile("" ::: "memory");   // compiler-only fences: LDS reads must not move across the barrier
    __builtin_amdgcn_s_barrier();    // bare barrier: __syncthreads() would also wait for the younger loads
    asm volatile("" ::: "memory");
  };
#pragma unroll
  for (int s = 0; s < S; ++s)
    if (s < KT) issue(s);
  if (KT >= S) rx_wait_vmcnt<(S - 1) * LPS>(); else rx_wait_vmcnt<0>();
  publish();
  load_frags(0, lds, 0);

  // P = register buffer that holds step 0 of this tile (compile-time, so that the fragment
  // arrays are never indexed dynamically); the next tile starts in buffer (P + NS) & 1.
  auto tile = [&](auto P, int kt) {
    constexpr int p = decltype(P)::value;
    const RX_LDS E* sa = lds + (kt % S) * STAGE;
    // 16-bit operands: the wavefronts of the main loop run at raised priority (measured: the 8192 x 4096 x 4096 bf16
    // layer 5 % faster; 8-bit operands 2 % slower, so they keep the default)
    if constexpr (TRAITS::RAISE_PRIO) __builtin_amdgcn_s_setprio(3);
#pragma unroll
    for (int s = 0; s + 1 < NS; ++s) {
      // keep the order "LDS reads of the next step, then the MFMAs of this step": the reads then
      // complete under a full step of MFMAs instead of being waited for right after issue
      load_frags((p + s + 1) & 1, sa, (s + 1) * MMA::KS);
      mma_all((p + s) & 1);
      interleave();
    }
    if (kt + 1 < KT) {
      // tile kt+1 has landed once only the (S-2) tiles after it are still in flight
      if (kt + S - 1 < KT) rx_wait_vmcnt<(S - 2) * LPS>(); else rx_wait_vmcnt<0>();
      publish();
      if (kt + S < KT) issue(kt + S);
      load_frags((p + NS) & 1, lds + ((kt + 1) % S) * STAGE, 0);
    }
    mma_all((p + NS - 1) & 1);
    if (kt + 1 < KT) interleave(); else RX_SCHED_FENCE();
  };
  if constexpr (NS % 2 == 0) {
    for (int kt = 0; kt < KT; ++kt) tile(rx_int<0>{}, kt);
  } else {
    for (int kt = 0; kt < KT; kt += 2) {
      tile(rx_int<0>{}, kt);
      if (kt + 1 < KT) tile(rx_int<1>{}, kt + 1);
    }
  }

#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        int dm, dn;
        TRAITS::coords(lane, rg, &dm, &dn);
        const int m = m0 + wm * (BM / WM) + 32 * i + dm;
        const int n = n0 + wn * (BN / WN) + 32 * j + dn;
        constexpr bool WHOLE = (M % BM == 0 || rx_epi_masks_rows<Epi>::value) && N % BN == 0;   // no bounds test: the epilogue becomes straight-line code
        if (WHOLE || (m < M && n < N)) {
          const float v[4] = {acc[i][j][4 * rg], acc[i][j][4 * rg + 1], acc[i][j][4 * rg + 2], acc[i][j][4 * rg + 3]};
          if constexpr (BATCHED) epi(v, (int)batch, m, n);
          else if constexpr (SPLIT > 1) epi(v, (int)blockIdx.y, m, n);
          else epi(v, m, n);
        }
      }
    }
  }
}

// ===========================================================================
// 8- and 16-bit operands on the 16 x 16 MFMA shapes, one operand streamed.
// Under the power limit of this part v_mfma_f32_16x16x128_f8f6f4 sustains about 8 % more flops than 32 x 32 x 64
// on the same data (16 x 16 x 32 against 32 x 32 x 16 for 16-bit operands: 13 %), but 16 x 16 x 128 fragments (16
// rows x 128 bytes of k: 8 registers) do not fit the skeleton above twice.  Here the wavefront's (BM/WM) x (BN/WN)
// tile is NA x NB blocks of 16 x 16 and a K tile is 128 bytes deep -- one 8-bit MFMA, two 16-bit ones: the NB
// fragments of the B operand stay in registers for the whole K tile (two sets: the next tile's are read under the
// last MFMAs of this one), the NA fragments of A stream through four buffers, block i + D being read from LDS while
// block i is multiplied.  128 accumulator + 64 + 32 fragment registers.
// Operand tiles go global -> LDS as buffer loads: the per-thread part of an address is one 32-bit offset that never
// changes (two where the swizzle alternates between loads), the K tile and the row block of load i go into the scalar
// offset, and rows past the end of the operand are outside the buffer's range and read as zero: no address
// arithmetic and no clamping in the main loop.  Two LDS stages per operand (three for the 256 x 128 tiles, where they
// fit), A stages first so that one address register per operand reaches all of its stages.
// Measured against the skeleton above on the same devices: 8192^3 e4m3 484-491 us against 538-560; bf16
// 8192 x 4096 x 4096 with bias + GELU 235-238 us against 245-257 ([m][k] x [k][n]; no difference for [m][k] x [n][k]),
// K = 1024: 74 against 77; 256 x 128 tiles of 8192 x 1024 x 4096: 65 against 66.5.  128 x 128 tiles on four wavefronts
// gain nothing and stay with the skeleton above.
// ===========================================================================
template <int I, int N, class F>
RX_DEV void rx_static_for(F&& f) {
  if constexpr (I < N) {
    f(rx_int<I>{});
    rx_static_for<I + 1, N>(f);
  }
}

//   [k][o] tiles read by the 16 x 16 fragments.  8-bit: one 32-lane phase of a transpose read takes rows k..k+7 and
//   k+16..k+23, 16 bytes of each; 16-bit: rows k..k+3 and k+8..k+11, 32 bytes of each.  Every one of those rows gets
//   its own group of the 256 bytes that the 64 banks hold.
template <int ESZ, int CPR>
RX_DEV int rx_swz_tr_s(int row, int c) {
  if constexpr (ESZ == 1) return c ^ (((row & 7) | (((row >> 4) & 1) << 3)) & (CPR - 1));
  else return rx_swz_tr16<CPR>(row, c);
}

// Element policies: the MFMAs of one 16 x 16 x (128 bytes of k) product, and the row bit that the [k][o] swizzle takes
// beyond the low ones.  The first operand's rows become the rows of the 16 x 16 result: a lane ends with four
// consecutive rows of one column.
struct rx_el_f8 {
  typedef rx_u8 elem;
  static constexpr int VARBIT = 4, NMF = 1;
  RX_DEV void mma(rx_f32x4v& c, const rx_i32x8& rowop, const rx_i32x8& colop) {
    // formats 0/0 = e4m3 x e4m3; zero scale operands select the unscaled instruction
    c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(rowop, colop, c, 0, 0, 0, 0, 0, 0);
  }
};
template <bool BF> struct rx_el_16 {
  typedef rx_u16 elem;
  static constexpr int VARBIT = 3, NMF = 2;
  RX_DEV void mma(rx_f32x4v& c, const rx_i32x8& rowop, const rx_i32x8& colop) {
    // a lane's first 16 bytes are k = 8g .. 8g+7 (g = lane / 16) for the first MFMA, its second 16 bytes
    // k = 32 + 8g .. for the second
    const rx_i32x4 r0 = {rowop[0], rowop[1], rowop[2], rowop[3]}, r1 = {rowop[4], rowop[5], rowop[6], rowop[7]};
    const rx_i32x4 c0 = {colop[0], colop[1], colop[2], colop[3]}, c1 = {colop[4], colop[5], colop[6], colop[7]};
    if constexpr (BF) {
      c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(rx_bf16x8, r0), __builtin_bit_cast(rx_bf16x8, c0), c, 0, 0, 0);
      c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(rx_bf16x8, r1), __builtin_bit_cast(rx_bf16x8, c1), c, 0, 0, 0);
    } else {
      c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(rx_f16x8, r0), __builtin_bit_cast(rx_f16x8, c0), c, 0, 0, 0);
      c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(rx_f16x8, r1), __builtin_bit_cast(rx_f16x8, c1), c, 0, 0, 0);
    }
  }
};
typedef rx_el_16<true> rx_el_bf16;
typedef rx_el_16<false> rx_el_f16;

// Fragments of 16 rows x 128 bytes of k.  LDS addresses and LD (one LDS row) are in bytes.  A lane (row % 16, g = lane
// / 16) holds the 16 bytes at 16 g and the 16 bytes at 64 + 16 g of its row: the four 16-lane blocks of one 16-byte
// read then take neighbouring chunks, which the XOR swizzle keeps on different banks (blocks two chunks apart, as 32
// contiguous bytes per lane would have it, collide two ways: measured with SQ_LDS_BANK_CONFLICT).  Which k a lane holds
// does not matter to a contraction as long as both operands agree, and the transposing reads below do.
template <class EL> struct rx_frag_s {
  // [o][k] tiles
  template <int LD> RX_DEV rx_i32x8 kc(const RX_LDS rx_u8* t, int row0, int lane) {
    const int r = row0 + (lane & 15), c = lane >> 4;
    struct { rx_i32x4 a, b; } both = {*(const RX_LDS rx_i32x4*)(t + r * LD + rx_swz_kc<LD / 16>(r, c) * 16),
                                      *(const RX_LDS rx_i32x4*)(t + r * LD + rx_swz_kc<LD / 16>(r, c + 4) * 16)};
    return __builtin_bit_cast(rx_i32x8, both);
  }
  // [k][o] tiles, col0 in elements: transpose reads, four per fragment
  template <int LD> RX_DEV rx_i32x8 tr(const RX_LDS rx_u8* t, int col0, int lane) {
    const int i = lane & 15, g = lane >> 4;
    if constexpr (sizeof(typename EL::elem) == 1) {
      // source lane i of a 16-lane block points at row k + i/2, columns 8*(i%2)..+7; after the transpose lane j of the
      // block holds 8 consecutive k for column j.  Read h covers k = 16g + 8(h%2) + 64(h/2) .. + 7.
      const int k = 16 * g + (i >> 1), col = col0 + 8 * (i & 1);
      rx_i32x2 r[4];
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        const int kh = k + 8 * (h & 1) + 64 * (h >> 1);
        r[h] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((RX_LDS rx_i32x2*)(t + kh * LD + rx_swz_tr_s<1, LD / 16>(kh, col >> 4) * 16 + (col & 15)));
      }
      struct { rx_i32x2 a, b, c, d; } all = {r[0], r[1], r[2], r[3]};
      return __builtin_bit_cast(rx_i32x8, all);
    } else {
      // source lane i of a 16-lane block points at row k + i/4, columns 4*(i%4)..+3; after the transpose lane j of the
      // block holds 4 consecutive k for column j.  Read h covers k = 8g + 4(h%2) + 32(h/2) .. + 3.
      const int k = 8 * g + (i >> 2), colb = (col0 + 4 * (i & 3)) * 2;
      rx_i16x4 r[4];
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        const int kh = k + 4 * (h & 1) + 32 * (h >> 1);
        r[h] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((RX_LDS rx_i16x4*)(t + kh * LD + rx_swz_tr_s<2, LD / 16>(kh, colb >> 4) * 16 + (colb & 15)));
      }
      struct { rx_i16x4 a, b, c, d; } all = {r[0], r[1], r[2], r[3]};
      return __builtin_bit_cast(rx_i32x8, all);
    }
  }
};

// Direct loads of one operand's tile of ROWS rows x COLS bytes per K tile.  Slot s (16-byte units, lane order) of the
// LDS tile holds global chunk (row = s / CPR, c = swizzle^-1(pos = s % CPR)); load i of a thread covers rows
// i * RSTEP.. of the tile.  The swizzle of a thread's slot is the same for every i, except that the [k][o] swizzle
// takes row bit VARBIT, which i * RSTEP may toggle: then there are two offsets.
template <class EL, int ROWS, int COLS, int NT, bool KC>
struct rx_dma_s {
  static constexpr int ESZ = sizeof(typename EL::elem);
  static constexpr int CPR = COLS / 16, NL = ROWS * CPR / NT, RSTEP = NT / CPR;
  // the [o][k] swizzle takes row bits 1..3, the [k][o] swizzles row bits below 3 and bit VARBIT
  static_assert(ROWS * CPR % NT == 0 && RSTEP % (KC ? 16 : 8) == 0, "tile must be a whole number of workgroup-wide loads");
  static constexpr int VSTEP = 1 << EL::VARBIT;
  static constexpr int NVAR = (KC || RSTEP > VSTEP || NL * RSTEP <= VSTEP) ? 1 : 2;
  static constexpr int I1 = VSTEP / RSTEP;     // first load whose rows have the bit set
  __amdgpu_buffer_rsrc_t rsrc;
  unsigned voff[NVAR];
  unsigned gldb;   // bytes per operand row
  // base: the operand (of this batch entry), ldb: bytes per row of it, o0b: first row of the tile ([o][k]) or byte
  // offset of its first column ([k][o]), bytes: operand size
  __device__ __forceinline__ void init(const void* base, unsigned ldb, int o0b, unsigned bytes, int tid) {
    rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, bytes, 0x00020000);
    gldb = ldb;
#pragma unroll
    for (int v = 0; v < NVAR; ++v) {
      const int i0 = v * I1;
      const int s = i0 * NT + tid;
      const int row = s / CPR, pos = s % CPR;
      if constexpr (KC) voff[v] = (unsigned)(o0b + row) * ldb + rx_swz_kc<CPR>(row, pos) * 16;
      else voff[v] = (unsigned)(row - i0 * RSTEP) * ldb + o0b + rx_swz_tr_s<ESZ, CPR>(row, pos) * 16;
    }
  }
  // kbyte: scalar byte offset of the K tile (k0 bytes for [o][k] operands, k0 rows for [k][o]); wave: wavefront index, scalar
  __device__ __forceinline__ void issue(unsigned kbyte, RX_LDS rx_u8* lds, int wave) const {
#pragma unroll
    for (int i = 0; i < NL; ++i) one(i, kbyte, lds, wave);
  }
  // load i alone (i is a constant wherever this is called: the offsets fold)
  __device__ __forceinline__ void one(int i, unsigned kbyte, RX_LDS rx_u8* lds, int wave) const {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (RX_LDS void*)(lds + (i * NT + wave * 64) * 16), 16, voff[NVAR == 1 ? 0 : ((i * RSTEP / VSTEP) & 1)],
                                             kbyte + i * RSTEP * gldb, 0, 0);
  }
};

// Clock probe for measurements (the library's RxGemmClockProbe; the kernels of compiled programs never carry it): in
// the middle of the K loop of its tile, wavefront 0 of every 16th workgroup sleeps 8 x s_sleep 127 -- 65024 shader
// cycles by the instruction's definition -- and records what the shader-cycle counter and the 100 MHz real-time
// counter advanced meanwhile.  cycles / real time is the clock the compute unit ran at while the rest of the chip
// kept multiplying; the same two counters over a workgroup's whole lifetime read lower, because the cycle counter
// does not advance while the compute unit has nothing to issue.
struct rx_clock_probe {
  static constexpr bool none = false;
  unsigned long long* out;   // per workgroup: [0] cycles, [1] real-time ticks over the sleep
  RX_MEM void mid(int kt, int at, int wave, int lane) const {
    if (kt == at && (blockIdx.x & 15) == 0 && wave == 0) {
      const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
#pragma unroll
      for (int q = 0; q < 8; ++q) __builtin_amdgcn_s_sleep(127);
      const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
      if (lane == 0) { out[blockIdx.x * 2] = c1 - c0; out[blockIdx.x * 2 + 1] = r1 - r0; }
    }
  }
};

// Probe of the ping-pong body (RxGemmClockProbe, kind 2): what the shader-cycle counter and the real-time counter
// advance over the compute phases of wavefronts 0 and 4 of every workgroup -- stretches in which a wavefront issues
// nothing but MFMAs, back to back.  cycles / phases says whether the MFMAs issue at their full rate (16 cycles each for
// the 16 x 16 x 32 shapes), cycles / real time is the clock the compute unit runs at while its MFMA pipes are full.
struct rx_phase_probe {
  static constexpr bool none = false;
  unsigned long long* out;   // per workgroup and group: [0] cycles, [1] real-time ticks, [2] phases
  unsigned long long c = 0, t = 0, c0 = 0, t0 = 0, n = 0;
  RX_MEM void begin() { c0 = __builtin_readcyclecounter(); t0 = __builtin_amdgcn_s_memrealtime(); }
  RX_MEM void end() { c += __builtin_readcyclecounter() - c0; t += __builtin_amdgcn_s_memrealtime() - t0; ++n; }
  RX_MEM void flush(int wave, int lane) const {
    if ((wave & 3) == 0 && lane == 0) { unsigned long long* o = out + (blockIdx.x * 2 + (wave >> 2)) * 3; o[0] = c; o[1] = t; o[2] = n; }
  }
};

// An epilogue functor may supply the accumulators' first values (`has_init`, `init(v, n)`: what it would otherwise add
// to every row of columns n .. n + NV - 1, a bias): the products are then summed onto them, and the epilogue saves the
// addition and the operand's loads and conversions for every block of rows (an eighth of its instructions for bias + GELU).
template <class E, class = void> struct rx_epi_has_init { static constexpr bool value = false; };
template <class E> struct rx_epi_has_init<E, decltype((void)E::has_init)> { static constexpr bool value = E::has_init; };

// A product whose first operand is read through row shifts (KOff of the streaming bodies): K is cut into taps of C
// elements, and tap t = (ty, tx) of a KW-wide window contracts rows m + ty * SY + tx * SX of a matrix of C columns with
// columns t * C .. t * C + C - 1 of the second operand; rows beyond the matrix read as zeros.  With the matrix a zero-
// padded image in [image, row, column, channel] order and SY the padded row length this is a convolution with unit
// strides, evaluated on the padded grid: no window matrix exists, the operand tiles still arrive as plain buffer loads
// with a scalar offset per K tile.
template <int C_, int KW_, int SY_, int SX_, int ESZ_>
struct rx_tap_shift {
  static constexpr bool none = false;
  static constexpr int C = C_;                                // elements per row of the first operand
  static constexpr int CT = C_ * ESZ_ / 128;                  // K tiles per tap
  static_assert(C_ * ESZ_ % 128 == 0, "a tap is whole K tiles");
  // byte offset of K tile kt, to be added to (row of the tile) * C * ESZ
  RX_DEV unsigned at(int kt) {
    const int tap = kt / CT, part = kt % CT;
    return (unsigned)((tap / KW_) * SY_ + (tap % KW_) * SX_) * (unsigned)(C_ * ESZ_) + (unsigned)part * 128u;
  }
  // the same as a row shift and a first column (elements)
  RX_DEV int row(int kt) { const int tap = kt / CT; return (tap / KW_) * SY_ + (tap % KW_) * SX_; }
  RX_DEV int col(int kt) { return (kt % CT) * (128 / ESZ_); }
};

template <class EL, int BM, int BN, int WM, int WN, bool A_KC, bool B_KC, int M, int N, int K, int RB, int CB, bool BATCHED, class Epi, int D = 2, int NSTG = 2, class Probe = rx_no_fn, class KOff = rx_no_fn>
RX_DEV void rx_gemm_body_s(const typename EL::elem* __restrict__ A, const typename EL::elem* __restrict__ B, const Epi& epi, const Probe& probe = Probe()) {
  constexpr int ESZ = sizeof(typename EL::elem);
  constexpr int BKB = 128, BK = BKB / ESZ, NBUF = 4;
  constexpr int NT = WM * WN * 64;
  constexpr int NA = BM / WM / 16, NB = BN / WN / 16;
  static_assert(NA % NBUF == 0 && D >= 1 && D < NBUF && D <= NA, "streaming depth");
  static_assert(NSTG == 2 || NSTG == 3, "LDS stages per operand");
  constexpr int A_ROWS = A_KC ? BM : BK, A_COLS = A_KC ? BKB : BM * ESZ;   // LDS tiles: rows x bytes
  constexpr int B_ROWS = B_KC ? BN : BK, B_COLS = B_KC ? BKB : BN * ESZ;
  constexpr int A_SZ = BM * BKB, B_SZ = BN * BKB;
  typedef rx_dma_s<EL, A_ROWS, A_COLS, NT, A_KC> DMA_A;
  typedef rx_dma_s<EL, B_ROWS, B_COLS, NT, B_KC> DMA_B;
  constexpr int NLT = DMA_A::NL + DMA_B::NL;   // direct loads per thread and K tile
  constexpr long long AROW = KOff::none ? (long long)K : (long long)KOff::C;   // elements per row of the first operand as stored
  static_assert(KOff::none || (A_KC && !BATCHED), "row shifts: the first operand is [row][k]");
  static_assert((long long)M * AROW * ESZ < (1ll << 31) * (KOff::none ? 2 : 1) && (long long)N * K * ESZ < (1ll << 32), "32-bit operand offsets");
  static_assert(K % BK == 0, "whole K tiles");
  extern __shared__ __attribute__((aligned(16))) unsigned char rx_smem[];
  RX_LDS rx_u8* const ldsa = (RX_LDS rx_u8*)rx_smem;
  RX_LDS rx_u8* const ldsb = ldsa + NSTG * A_SZ;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  constexpr int GM = (M + BM - 1) / BM, GN = (N + BN - 1) / BN;
  int bm, bn;
  if (!rx_gemm_tile<GM, GN, RB, CB>(blockIdx.x, &bm, &bn)) return;
  const int m0 = bm * BM, n0 = bn * BN;
  const long long batch = BATCHED ? blockIdx.y : 0;
  constexpr unsigned A_GLDB = (A_KC ? (unsigned)AROW : M) * ESZ, B_GLDB = (B_KC ? K : N) * ESZ;
  constexpr int KT = K / BK;
  constexpr unsigned KA = A_KC ? BKB : BK * A_GLDB, KB = B_KC ? BKB : BK * B_GLDB;   // byte step of one K tile

  rx_f32x4v acc[NA][NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    float v0[4] = {0.f, 0.f, 0.f, 0.f};
    if constexpr (rx_epi_has_init<Epi>::value && !BATCHED) epi.init(v0, n0 + wn * (BN / WN) + 16 * j + 4 * (lane >> 4));
#pragma unroll
    for (int i = 0; i < NA; ++i) acc[i][j] = rx_f32x4v{v0[0], v0[1], v0[2], v0[3]};
  }

  DMA_A dma_a;
  DMA_B dma_b;
  dma_a.init(A + batch * (long long)M * K, A_GLDB, A_KC ? m0 : m0 * ESZ, (unsigned)((long long)M * AROW * ESZ), tid);
  dma_b.init(B + batch * (long long)N * K, B_GLDB, B_KC ? n0 : n0 * ESZ, (unsigned)((long long)N * K * ESZ), tid);
  // tile kt lies in stage kt % NSTG of both operands
  // (st is a constant at every call, so the stage's offset folds into the instruction)
  auto issue = [&](int kt, int st) __attribute__((always_inline)) {
    if constexpr (KOff::none) dma_a.issue((unsigned)kt * KA, ldsa + st * A_SZ, wave);
    else dma_a.issue(KOff::at(kt), ldsa + st * A_SZ, wave);
    dma_b.issue((unsigned)kt * KB, ldsb + st * B_SZ, wave);
  };
  rx_i32x8 fa[NBUF], fb[2][NB];
  auto read_a = [&](auto BUF, auto ST, int blk) {
    const RX_LDS rx_u8* st = ldsa + decltype(ST)::value * A_SZ;
    const int o = wm * (BM / WM) + 16 * blk;
    if constexpr (A_KC) fa[decltype(BUF)::value] = rx_frag_s<EL>::template kc<A_COLS>(st, o, lane);
    else fa[decltype(BUF)::value] = rx_frag_s<EL>::template tr<A_COLS>(st, o, lane);
  };
  // the B fragments of tile kt live in register set kt % 2
  auto read_b = [&](auto J, auto PAR, auto ST) {
    constexpr int j = decltype(J)::value, par = decltype(PAR)::value, st = decltype(ST)::value;
    const int o = wn * (BN / WN) + 16 * j;
    if constexpr (B_KC) fb[par][j] = rx_frag_s<EL>::template kc<B_COLS>(ldsb + st * B_SZ, o, lane);
    else fb[par][j] = rx_frag_s<EL>::template tr<B_COLS>(ldsb + st * B_SZ, o, lane);
  };
  auto publish = [&]() {
    asm volatile("" ::: "memory");   // compiler-only fences: LDS reads must not move across the barrier
    __builtin_amdgcn_s_barrier();    // bare barrier: __syncthreads() would also wait for the younger loads
    asm volatile("" ::: "memory");
  };

  rx_static_for<0, NSTG>([&](auto S) { if constexpr (decltype(S)::value < KT) issue(decltype(S)::value, decltype(S)::value); });
  if constexpr (KT >= NSTG) rx_wait_vmcnt<(NSTG - 1) * NLT>(); else rx_wait_vmcnt<0>();
  publish();
  rx_static_for<0, NB>([&](auto J) { read_b(J, rx_int<0>{}, rx_int<0>{}); });
  rx_static_for<0, D>([&](auto I) { read_a(I, rx_int<0>{}, decltype(I)::value); });

  // The barrier that publishes tile kt+1 sits before the first read of it, D blocks before the end of tile kt: by
  // then every wavefront has issued its last reads of tile kt, so the stages of tile kt take tile kt+NSTG.  The B
  // fragments of tile kt+1 are read with its first D blocks of A, BPB of them per block.  With three stages a request
  // has two K tiles to land instead of one (tiles of 256 x 128, whose K tile is half as long as that of 256 x 256:
  // the wait for the requests of the 8192 x 1024 x 4096 bf16 layer 9.4 -> 0.5 us per workgroup, 62.3 -> 59.9 us).
  constexpr int BPB = (NB + D - 1) / D;
  constexpr int RDS_A = A_KC ? 2 : 4, RDS_B = B_KC ? 2 : 4;   // LDS read instructions per fragment
  constexpr int NMB = NB * EL::NMF;                           // MFMAs per block of A
  // MODE 0: tile kt+NSTG exists, 1: it does not but tile kt+1 does, 2: last tile
  auto tile = [&](auto P, auto ST, auto MODE, int kt) {
    constexpr int p = decltype(P)::value, mode = decltype(MODE)::value;
    constexpr bool last = mode == 2;
    typedef decltype(ST) CUR;                                   // stage of this tile
    typedef rx_int<(decltype(ST)::value + 1) % NSTG> NXT;       // stage of the next one
    rx_static_for<0, NA>([&](auto I) {
      constexpr int i = decltype(I)::value;
      constexpr int t = i + D;                   // block whose read goes out now
      constexpr int nb0 = t >= NA ? (t - NA) * BPB : 0;
      constexpr int nb1 = t >= NA ? (nb0 + BPB < NB ? nb0 + BPB : NB) : 0;
      if constexpr (t < NA) {
        read_a(rx_int<t % NBUF>{}, CUR{}, t);
      } else if constexpr (!last) {
        if constexpr (t == NA) {
          if constexpr (!Probe::none) probe.mid(kt, KT / 2, wave, lane);
          // tile kt+1 has landed once only the NSTG-2 tiles after it are still in flight
          if constexpr (mode == 0) rx_wait_vmcnt<(NSTG - 2) * NLT>(); else rx_wait_vmcnt<0>();
          publish();
          if constexpr (mode == 0) issue(kt + NSTG, CUR::value);
        }
        read_a(rx_int<t % NBUF>{}, NXT{}, t - NA);
        rx_static_for<nb0, nb1>([&](auto J) { read_b(J, rx_int<p ^ 1>{}, NXT{}); });
      }
      // the B fragment is the row operand: a lane ends with four consecutive n of one m
      rx_static_for<0, NB>([&](auto J) {
        constexpr int j = decltype(J)::value;
        EL::mma(acc[i][j], fb[p][j], fa[i % NBUF]);
      });
      // ask the scheduler to let this block's LDS reads trickle out between its MFMAs
      constexpr int nrd = t < NA ? RDS_A : (last ? 0 : RDS_A + (nb1 - nb0) * RDS_B);
      if constexpr (nrd == 0) {
        __builtin_amdgcn_sched_group_barrier(0x008, NMB, 0);
      } else if constexpr (nrd <= NMB) {
        constexpr int mpr = NMB / nrd;           // MFMAs per read
        rx_static_for<0, nrd>([&](auto Q) {
          __builtin_amdgcn_sched_group_barrier(0x008, mpr, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        });
        if constexpr (NMB > nrd * mpr) __builtin_amdgcn_sched_group_barrier(0x008, NMB - nrd * mpr, 0);
      } else {
        constexpr int per = (nrd + NMB - 1) / NMB;
        rx_static_for<0, NMB>([&](auto Q) {
          constexpr int q = decltype(Q)::value;
          constexpr int n = (q + 1) * per <= nrd ? per : (q * per < nrd ? nrd - q * per : 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x100, n, 0);
        });
      }
    });
  };
  // The steady state has no branches inside a tile: it is unrolled over one period of (stage, B register set), and the
  // tiles that cannot request a successor any more are written out one by one (KT is a compile-time constant).
  constexpr int U = NSTG % 2 == 0 ? NSTG : 2 * NSTG;
  constexpr int NSTEADY = KT > NSTG ? ((KT - NSTG) / U) * U : 0;
  for (int kt = 0; kt < NSTEADY; kt += U)
    rx_static_for<0, U>([&](auto UU) {
      constexpr int u = decltype(UU)::value;
      tile(rx_int<u % 2>{}, rx_int<u % NSTG>{}, rx_int<0>{}, kt + u);
    });
  rx_static_for<NSTEADY, KT>([&](auto KK) {
    constexpr int k = decltype(KK)::value;
    tile(rx_int<k % 2>{}, rx_int<k % NSTG>{}, rx_int<(k + NSTG < KT ? 0 : (k + 1 < KT ? 1 : 2))>{}, k);
  });
  RX_SCHED_FENCE();

#pragma unroll
  for (int i = 0; i < NA; ++i) {
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int m = m0 + wm * (BM / WM) + 16 * i + (lane & 15);
      const int n = n0 + wn * (BN / WN) + 16 * j + 4 * (lane >> 4);
      // Whole tiles need no bounds test, and without it the epilogue is straight-line code: the compiler then requests
      // what the functor reads (a bias, the C operand) for all blocks ahead of the arithmetic instead of one
      // request, one wait and one store per block.
      constexpr bool WHOLE = (M % BM == 0 || rx_epi_masks_rows<Epi>::value) && N % BN == 0;
      if (WHOLE || (m < M && n < N)) {
        const float v[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
        if constexpr (BATCHED) epi(v, (int)batch, m, n);
        else epi(v, m, n);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Ping-pong form of the streaming tiles (256 x 256 on eight wavefronts, same LDS tiles, swizzles, fragments and
// MFMAs as rx_gemm_body_s, and the same order of additions into every accumulator: results are bit-identical).
// The two wavefronts of a SIMD -- w and w + 4 -- alternate between a memory phase and a compute phase, half a K tile
// apart: in its memory phase a wavefront reads all its fragments of one K tile from LDS (8 of A, 4 of B: 96
// registers), in its compute phase it issues that tile's 64 (16-bit) or 32 (8-bit) MFMAs back to back at raised
// priority, with nothing in between that could wait for memory, while the other wavefront of the SIMD is in its
// memory phase.  Two barriers per K tile keep the phases apart (the results do not depend on which wavefronts share a
// SIMD, only the overlap does).  Requests go out in memory phases only, between the LDS reads, where a request that has
// to wait for the load path delays no MFMA.
//   interval 2t:   group 0 (wavefronts 0-3) reads tile t (stage t % 2) and requests tile t + 1 into the other stage,
//                  group 1 multiplies tile t - 1
//   interval 2t+1: group 0 multiplies tile t and then waits for tile t + 1 to land, group 1 reads tile t
// The stage of tile t - 1 is free when interval 2t begins (group 1 read it in interval 2t - 1), and tile t + 1 is first
// read in interval 2t + 2.  With B stored [k][n] group 0 requests both operands (256 threads cover a tile).  With B
// stored [n][k] a wavefront's request fills eight whole rows of the LDS tile, and rows 64 wn .. 64 wn + 63 of B are
// read by wavefronts wn and wn + 4 alone: group 0 requests A only, and every wavefront of group 1 requests its 64 rows
// of B of tile t + 2 in its own memory phase of tile t, into the stage it is reading, once its B fragments have
// arrived (wavefront wn read them an interval earlier); that halves the requests of group 0, whose memory phase is
// otherwise as long as a compute phase for 8-bit operands.
// Measured after 150 ms under load (the first 20 ms after an idle period run up to 20 % slower, whatever the kernel):
// bf16 8192 x 4096 x 4096 [m][k] x [k][n] with bias + GELU 199.7 -> 190.0 us, K = 1024: 65.6 -> 64.6 us; e4m3 8192^3
// [m][k] x [n][k] 386 -> 360 us (with group 0 requesting both operands: 411).
// ---------------------------------------------------------------------------
template <class EL, int BM, int BN, int WM, int WN, bool A_KC, bool B_KC, int M, int N, int K, int RB, int CB, bool BATCHED, class Epi, class Probe = rx_no_fn, class KOff = rx_no_fn>
RX_DEV void rx_gemm_body_pp(const typename EL::elem* __restrict__ A, const typename EL::elem* __restrict__ B, const Epi& epi, Probe probe = Probe()) {
  constexpr int ESZ = sizeof(typename EL::elem);
  constexpr int BKB = 128, BK = BKB / ESZ, NSTG = 2;
  constexpr int NTL = 256;                                   // threads of group 0
  constexpr int NA = BM / WM / 16, NB = BN / WN / 16;
  constexpr int A_ROWS = A_KC ? BM : BK, A_COLS = A_KC ? BKB : BM * ESZ;
  constexpr int B_ROWS = B_KC ? BN : BK, B_COLS = B_KC ? BKB : BN * ESZ;
  constexpr int A_SZ = BM * BKB, B_SZ = BN * BKB;
  constexpr int BSL = BN / WN;                               // rows of B that one wavefront column reads
  typedef rx_dma_s<EL, A_ROWS, A_COLS, NTL, A_KC> DMA_A;
  typedef rx_dma_s<EL, B_ROWS, B_COLS, NTL, B_KC> DMA_B;     // B requested by group 0 ([k][n])
  constexpr int NLA = DMA_A::NL;
  constexpr int NLB = B_KC ? BSL * 8 / 64 : DMA_B::NL;       // [n][k]: a wavefront's request covers 8 rows of 128 bytes
  constexpr int NL0 = B_KC ? NLA : NLA + NLB;                // requests per thread of group 0 and K tile
  constexpr int NFR = NA + NB;                               // fragments per wavefront and K tile
  static_assert(WM == 2 && WN == 4, "wavefronts w and w + 4 share a SIMD and a column of B");
  constexpr long long AROW = KOff::none ? (long long)K : (long long)KOff::C;   // elements per row of the first operand as stored
  static_assert(KOff::none || (A_KC && !BATCHED), "row shifts: the first operand is [row][k]");
  static_assert((long long)M * AROW * ESZ < (1ll << 31) * (KOff::none ? 2 : 1) && (long long)N * K * ESZ < (1ll << 32), "32-bit operand offsets");
  constexpr int KT = K / BK;
  static_assert(K % BK == 0 && KT >= 2 && KT % 2 == 0, "an even number of whole K tiles");
  extern __shared__ __attribute__((aligned(16))) unsigned char rx_smem[];
  RX_LDS rx_u8* const ldsa = (RX_LDS rx_u8*)rx_smem;
  RX_LDS rx_u8* const ldsb = ldsa + NSTG * A_SZ;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int grp = wave >> 2;                                 // wavefronts w and w + 4 share a SIMD
  constexpr int GM = (M + BM - 1) / BM, GN = (N + BN - 1) / BN;
  int bm, bn;
  if (!rx_gemm_tile<GM, GN, RB, CB>(blockIdx.x, &bm, &bn)) return;
  const int m0 = bm * BM, n0 = bn * BN;
  const long long batch = BATCHED ? blockIdx.y : 0;
  constexpr unsigned A_GLDB = (A_KC ? (unsigned)AROW : M) * ESZ, B_GLDB = (B_KC ? K : N) * ESZ;
  constexpr unsigned KA = A_KC ? BKB : BK * A_GLDB, KB = B_KC ? BKB : BK * B_GLDB;

  rx_f32x4v acc[NA][NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    float v0[4] = {0.f, 0.f, 0.f, 0.f};
    if constexpr (rx_epi_has_init<Epi>::value && !BATCHED) epi.init(v0, n0 + wn * (BN / WN) + 16 * j + 4 * (lane >> 4));
#pragma unroll
    for (int i = 0; i < NA; ++i) acc[i][j] = rx_f32x4v{v0[0], v0[1], v0[2], v0[3]};
  }
  DMA_A dma_a;
  DMA_B dma_b;
  dma_a.init(A + batch * (long long)M * K, A_GLDB, A_KC ? m0 : m0 * ESZ, (unsigned)((long long)M * AROW * ESZ), tid & (NTL - 1));
  // [n][k]: slot `lane` of a wavefront's request q is row 8 q + lane / 8 of its rows, position lane % 8, and the swizzle
  // puts chunk c of row r at position c ^ ((r / 2) & 7): for odd q (row bit 3 set) bit 2 of the chunk flips
  unsigned slab0 = 0, slab1 = 0;
  if constexpr (B_KC) {
    dma_b.rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(B + batch * (long long)N * K), 0, (unsigned)((long long)N * K * ESZ), 0x00020000);
    slab0 = (unsigned)(n0 + wn * BSL + (lane >> 3)) * B_GLDB + (unsigned)(((lane & 7) ^ (lane >> 4)) * 16);
    slab1 = slab0 ^ 64u;
  } else {
    dma_b.init(B + batch * (long long)N * K, B_GLDB, n0 * ESZ, (unsigned)((long long)N * K * ESZ), tid & (NTL - 1));
  }
  rx_i32x8 fa[NA], fb[NB];
  // request q of a tile by group 0: those of A first (st and q are constants at every call)
  auto request = [&](int kt, int st, int q) __attribute__((always_inline)) {
    if (q < NLA) {
      if constexpr (KOff::none) dma_a.one(q, (unsigned)kt * KA, ldsa + st * A_SZ, wave);
      else dma_a.one(q, KOff::at(kt), ldsa + st * A_SZ, wave);
    }
    else if constexpr (!B_KC) dma_b.one(q - NLA, (unsigned)kt * KB, ldsb + st * B_SZ, wave);
  };
  // request q of this wavefront's rows of B ([n][k])
  auto request_rows = [&](int kt, int st, int q) __attribute__((always_inline)) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(dma_b.rsrc, (RX_LDS void*)(ldsb + st * B_SZ + wn * BSL * BKB + q * 1024), 16, (q & 1) ? slab1 : slab0,
                                             (unsigned)kt * KB + (unsigned)q * 8u * B_GLDB, 0, 0);
  };
  // [row][k] fragments (what rx_frag_s::kc reads) from two addresses per lane and operand: its row within a block of 16
  // and its two chunks, which the swizzle keeps 64 bytes apart; stage and block fold into the instruction's offset
  const unsigned lane_off = (unsigned)(lane & 15) * 128u + (unsigned)(((lane >> 4) ^ ((lane & 15) >> 1)) * 16);
  RX_LDS rx_u8* const pa0 = ldsa + (unsigned)(wm * (BM / WM)) * 128u + lane_off;
  RX_LDS rx_u8* const pa1 = ldsa + (unsigned)(wm * (BM / WM)) * 128u + (lane_off ^ 64u);
  RX_LDS rx_u8* const pb0 = ldsb + (unsigned)(wn * BSL) * 128u + lane_off;
  RX_LDS rx_u8* const pb1 = ldsb + (unsigned)(wn * BSL) * 128u + (lane_off ^ 64u);
  // fragment f of a tile: those of B first
  auto read = [&](auto ST, auto F) {
    constexpr int st = decltype(ST)::value, f = decltype(F)::value;
    if constexpr (f < NB) {
      if constexpr (B_KC) {
        struct { rx_i32x4 a, b; } both = {*(const RX_LDS rx_i32x4*)(pb0 + (st * B_SZ + f * 2048)), *(const RX_LDS rx_i32x4*)(pb1 + (st * B_SZ + f * 2048))};
        fb[f] = __builtin_bit_cast(rx_i32x8, both);
      } else {
        fb[f] = rx_frag_s<EL>::template tr<B_COLS>(ldsb + st * B_SZ, wn * BSL + 16 * f, lane);
      }
    } else {
      constexpr int i = f - NB;
      if constexpr (A_KC) {
        struct { rx_i32x4 a, b; } both = {*(const RX_LDS rx_i32x4*)(pa0 + (st * A_SZ + i * 2048)), *(const RX_LDS rx_i32x4*)(pa1 + (st * A_SZ + i * 2048))};
        fa[i] = __builtin_bit_cast(rx_i32x8, both);
      } else {
        fa[i] = rx_frag_s<EL>::template tr<A_COLS>(ldsa + st * A_SZ, wm * (BM / WM) + 16 * i, lane);
      }
    }
  };
  // end of a phase: nothing moves across it, neither in the compiler's schedule nor at run time
  auto phase_end = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  auto fragments_in = [&]() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); };
  auto multiply = [&]() {
    if constexpr (!Probe::none) probe.begin();
    __builtin_amdgcn_s_setprio(1);
    rx_static_for<0, NA>([&](auto I) {
      constexpr int i = decltype(I)::value;
      // the B fragment is the row operand: a lane ends with four consecutive n of one m
      rx_static_for<0, NB>([&](auto J) { EL::mma(acc[i][decltype(J)::value], fb[decltype(J)::value], fa[i]); });
    });
    __builtin_amdgcn_s_setprio(0);
    if constexpr (!Probe::none) { __builtin_amdgcn_sched_barrier(0); probe.end(); }
  };

  if (grp == 0) {
#pragma unroll
    for (int q = 0; q < NL0; ++q) request(0, 0, q);
    rx_wait_vmcnt<0>();
  } else if constexpr (B_KC) {
    // its rows of B of tiles 0 and 1: group 1 requests two tiles ahead
#pragma unroll
    for (int q = 0; q < NLB; ++q) request_rows(0, 0, q);
#pragma unroll
    for (int q = 0; q < NLB; ++q) request_rows(1, 1, q);
    rx_wait_vmcnt<NLB>();
  }
  phase_end();                 // tile 0 is in LDS
  if (grp == 1) phase_end();   // group 1 runs one interval behind

  if (grp == 0) {
    // REQ: tile k + 1 exists
    auto step = [&](auto UU, auto REQ, int k) {
      constexpr int u = decltype(UU)::value;
      if constexpr (decltype(REQ)::value != 0) {
        rx_static_for<0, NL0>([&](auto Q) {
          constexpr int q = decltype(Q)::value;
          request(k + 1, (u + 1) % 2, q);
          rx_static_for<q * NFR / NL0, (q + 1) * NFR / NL0>([&](auto F) { read(rx_int<u>{}, F); });
          __builtin_amdgcn_sched_barrier(0);
        });
      } else {
        rx_static_for<0, NFR>([&](auto F) { read(rx_int<u>{}, F); });
      }
      fragments_in();
      phase_end();
      multiply();
      __builtin_amdgcn_sched_barrier(0);
      rx_wait_vmcnt<0>();      // what this group requested of tile k + 1 has landed
      phase_end();
    };
    for (int kt = 0; kt < KT - 2; kt += 2) {
      step(rx_int<0>{}, rx_int<1>{}, kt);
      step(rx_int<1>{}, rx_int<1>{}, kt + 1);
    }
    step(rx_int<0>{}, rx_int<1>{}, KT - 2);
    step(rx_int<1>{}, rx_int<0>{}, KT - 1);
  } else {
    // REQ: tile k + 2 exists ([n][k] only); LAST: group 0 has left the loop, its last barrier was the one in this step
    auto step = [&](auto UU, auto REQ, auto LAST, int k) {
      constexpr int u = decltype(UU)::value;
      constexpr bool req = B_KC && decltype(REQ)::value != 0;
      rx_static_for<0, NB>([&](auto F) { read(rx_int<u>{}, F); });
      if constexpr (req) {
        fragments_in();        // this wavefront's B fragments of tile k are in registers: its rows of the stage are free
        __builtin_amdgcn_sched_barrier(0);
      }
      rx_static_for<0, NA>([&](auto I) {
        constexpr int i = decltype(I)::value;
        if constexpr (req) {
#pragma unroll
          for (int q = i * NLB / NA; q < (i + 1) * NLB / NA; ++q) request_rows(k + 2, u, q);
        }
        read(rx_int<u>{}, rx_int<NB + i>{});
        if constexpr (req) __builtin_amdgcn_sched_barrier(0);
      });
      fragments_in();
      // its rows of B of tile k + 1, requested a K tile ago, have landed; the requests just made may still be under way
      if constexpr (B_KC) { if constexpr (req) rx_wait_vmcnt<NLB>(); else rx_wait_vmcnt<0>(); }
      phase_end();
      multiply();
      if constexpr (decltype(LAST)::value == 0) phase_end();
    };
    for (int kt = 0; kt < KT - 2; kt += 2) {
      step(rx_int<0>{}, rx_int<1>{}, rx_int<0>{}, kt);
      step(rx_int<1>{}, rx_int<1>{}, rx_int<0>{}, kt + 1);
    }
    step(rx_int<0>{}, rx_int<0>{}, rx_int<0>{}, KT - 2);
    step(rx_int<1>{}, rx_int<0>{}, rx_int<1>{}, KT - 1);
  }
  RX_SCHED_FENCE();
  if constexpr (!Probe::none) probe.flush(wave, lane);

#pragma unroll
  for (int i = 0; i < NA; ++i) {
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int m = m0 + wm * (BM / WM) + 16 * i + (lane & 15);
      const int n = n0 + wn * (BN / WN) + 16 * j + 4 * (lane >> 4);
      constexpr bool WHOLE = (M % BM == 0 || rx_epi_masks_rows<Epi>::value) && N % BN == 0;
      if (WHOLE || (m < M && n < N)) {
        const float v[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
        if constexpr (BATCHED) epi(v, (int)batch, m, n);
        else epi(v, m, n);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// f64 operands: v_mfma_f64_16x16x4_f64, f64 accumulation.  Same tiling, tile order, operand
// layouts and epilogue interface as rx_gemm_body; a wavefront owns (BM/WM) x (BN/WN) as a grid of
// 16x16 MFMA tiles.  One fragment is two k values per lane (one 16-byte LDS read where k is
// contiguous): lane group g = lane / 16 takes k = 2g for the first MFMA of a pair and k = 2g + 1
// for the second; A and B use the same assignment, which is all a contraction needs.  The B
// fragment is the row operand, with its rows permuted so that a lane ends with four consecutive n of one m.
// ---------------------------------------------------------------------------
typedef double rx_f64x2 __attribute__((ext_vector_type(2)));
typedef double rx_f64x4 __attribute__((ext_vector_type(4)));

template <int BM, int BN, int BK, int WM, int WN, bool A_KC, bool B_KC, int M, int N, int K, int RB, int CB, bool BATCHED, class Epi>
RX_DEV void rx_gemm_body_f64(const double* __restrict__ A, const double* __restrict__ B, const Epi& epi) {
  typedef double E;
  constexpr int NT = WM * WN * 64;
  constexpr int TM = BM / WM / 16, TN = BN / WN / 16;   // 16x16 tiles per wavefront
  constexpr int PAD = 2, KS = 8;
  static_assert(BK % KS == 0 && (BM / WM) % 16 == 0 && (BN / WN) % 16 == 0, "tile shape");
  constexpr int A_ROWS = A_KC ? BM : BK, A_COLS = A_KC ? BK : BM;
  constexpr int B_ROWS = B_KC ? BN : BK, B_COLS = B_KC ? BK : BN;
  constexpr int A_LD = A_COLS + PAD, B_LD = B_COLS + PAD;
  constexpr int A_SZ = A_ROWS * A_LD, B_SZ = B_ROWS * B_LD;
  extern __shared__ __attribute__((aligned(16))) unsigned char rx_smem[];
  RX_LDS E* lds = (RX_LDS E*)rx_smem;
  constexpr int STAGE = A_SZ + B_SZ;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  constexpr int GM = (M + BM - 1) / BM, GN = (N + BN - 1) / BN;
  int bm, bn;
  if (!rx_gemm_tile<GM, GN, RB, CB>(blockIdx.x, &bm, &bn)) return;
  const int m0 = bm * BM, n0 = bn * BN;
  const long long batch = BATCHED ? blockIdx.y : 0;
  const E* Ab = A + batch * (long long)M * K;
  const E* Bb = B + batch * (long long)N * K;
  constexpr long long A_GLD = A_KC ? K : M, B_GLD = B_KC ? K : N;

  rx_f64x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = rx_f64x4{0.0, 0.0, 0.0, 0.0};

  rx_tile_copy<E, A_ROWS, A_COLS, NT> ca;
  rx_tile_copy<E, B_ROWS, B_COLS, NT> cb;
  auto gload = [&](int k0) {
    constexpr bool TAIL = K % BK != 0;
    if (A_KC) ca.template load<false, TAIL>(Ab, A_GLD, m0, k0, M, K, tid); else ca.template load<TAIL, false>(Ab, A_GLD, k0, m0, K, M, tid);
    if (B_KC) cb.template load<false, TAIL>(Bb, B_GLD, n0, k0, N, K, tid); else cb.template load<TAIL, false>(Bb, B_GLD, k0, n0, K, N, tid);
  };
  // The two k values of this lane for the fragment at k offset kk, operand row/column o + idx.
  // The instruction leaves row 4*r + lane/16 of its row operand in accumulator register r; feeding
  // it row 4*(i%4) + i/4 of the B tile from lane i makes those four rows consecutive n.
  const int idx_a = lane & 15, idx_b = 4 * (lane & 3) + ((lane & 15) >> 2);
  auto frag = [&](const RX_LDS E* t, int ld, bool kc, int o, int kk, int idx) {
    const int r = o + idx, k = kk + 2 * (lane >> 4);
    if (kc) return *(const RX_LDS rx_f64x2*)(t + r * ld + k);
    rx_f64x2 f;
    f[0] = t[k * ld + r];
    f[1] = t[(k + 1) * ld + r];
    return f;
  };
  gload(0);
  ca.store(lds, A_LD, tid);
  cb.store(lds + A_SZ, B_LD, tid);
  __syncthreads();

  constexpr int KT = (K + BK - 1) / BK;
  for (int kt = 0; kt < KT; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < KT) gload((kt + 1) * BK);
    const RX_LDS E* sa = lds + cur * STAGE;
    const RX_LDS E* sb = sa + A_SZ;
#pragma unroll
    for (int kk = 0; kk < BK; kk += KS) {
      rx_f64x2 fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[i] = frag(sa, A_LD, A_KC, wm * (BM / WM) + 16 * i, kk, idx_a);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[j] = frag(sb, B_LD, B_KC, wn * (BN / WN) + 16 * j, kk, idx_b);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fb[j][0], fa[i][0], acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fb[j][1], fa[i][1], acc[i][j], 0, 0, 0);
        }
    }
    if (kt + 1 < KT) {
      ca.store(lds + (cur ^ 1) * STAGE, A_LD, tid);
      cb.store(lds + (cur ^ 1) * STAGE + A_SZ, B_LD, tid);
    }
    __syncthreads();
  }

  // epilogue: lane holds D[n = 4*(lane/16) + r][m = lane%16] of each 16x16 tile
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + wm * (BM / WM) + 16 * i + (lane & 15);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wn * (BN / WN) + 16 * j + 4 * (lane >> 4);
      if (m < M && n < N) {
        const double v[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
        if constexpr (BATCHED) epi(v, (int)batch, m, n); else epi(v, m, n);
      }
    }
  }
}

// ===========================================================================
// Direct convolution of f32 images on v_mfma_f32_16x16x4_f32: x [B][C][H][W], w [O][C][KH][KW], out [B][O][HO][WO],
// strides SH / SW, filter dilations DH / DW, zero padding PT / PL rows and columns before the image (what lies after it
// follows from HO and WO).  A workgroup of four wavefronts computes TR whole rows of the result of one image for 64 output
// features, wavefront v the features 16 v .. 16 v + 15 of the group; blockIdx.y is the group of features.  The
// channels pass through LDS in slabs of CB, two stages (one if there is one slab): the patch of the image that the tile
// reads, [CB][(TR - 1) SH + (KH - 1) DH + 1][PW] with the image's column 0 at column OFF and zeros around it, and the slab's weights as [tap][quad of channels]
// [channel of the quad][80] features.  One k step of the MFMA is four channels of one tap: the pixel operand of lane
// (pixel % 16, channel = lane / 16) is patch[channel][row SH + dy DH][column SW + dx DW], i.e. one address per lane and pixel block
// plus a constant per step; the feature operand is one LDS word per step.  Every element of the image is read from
// memory once per tile (and per group of features) instead of once per tap.  The channel pitch of the patch is
// 16 mod 64 words, so that the four channels of a step read different banks.
// The result goes through the generated epilogue functor (bias, activation, store), four consecutive columns at a time.
// Measured: 3 x 3, 64 -> 64 features on 32 images of 56 x 56, padding 1: 75 us (98 TFLOP/s) with bias and ReLU, against
// 119 us for the same product as an implicit GEMM (the window matrix evaluated while its tiles are loaded) plus 9 us for
// the map that brings its [feature][image, pixel] result into this layout.
// ===========================================================================
template <int B, int C, int H, int W, int O, int KH, int KW, int SH, int SW, int DH, int DW, int PT, int PL, int HO, int WO, int TR, int CB, class Epi>
RX_DEV void rx_conv_body(const float* __restrict__ x, const float* __restrict__ w, const Epi& epi) {
  constexpr int TAPS = KH * KW;
  constexpr int PR = (TR - 1) * SH + (KH - 1) * DH + 1;             // rows of the patch
  constexpr int OFF = (PL + 3) / 4 * 4;                             // column of the image's column 0
  constexpr int LASTC = (WO - 1) * SW + (KW - 1) * DW - PL;         // last column of the image that a tile reads (may lie in the padding)
  constexpr int PW = (OFF + (LASTC + 1 > W ? LASTC + 1 : W) + 3) / 4 * 4;   // row pitch
  constexpr int PCH = (PR * PW + 47) / 64 * 64 + 16;                // channel pitch, 16 mod 64
  constexpr int NPX = TR * WO, NPB = (NPX + 15) / 16;               // pixels and blocks of 16 pixels of a tile
  constexpr int NQ = CB / 4, NSTEP = TAPS * NQ;                     // k steps per slab
  constexpr int WST = 80;
  constexpr int PATCH = CB * PCH, WSLAB = NSTEP * 4 * WST;
  constexpr int NSLAB = (C + CB - 1) / CB;
  constexpr int TILES = (HO + TR - 1) / TR;
  static_assert(CB % 4 == 0 && OFF >= PL && PW >= OFF + W, "patch layout");
  extern __shared__ __attribute__((aligned(16))) unsigned char rx_smem[];
  constexpr int NSTG = NSLAB > 1 ? 2 : 1;                           // one slab needs no second stage
  float* const patch = (float*)rx_smem;                             // [NSTG][PATCH]
  float* const wl = patch + NSTG * PATCH;                           // [NSTG][WSLAB]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = blockIdx.x / TILES, y0 = (blockIdx.x % TILES) * TR;
  const int og = blockIdx.y * 64;

  // Loaders.  Patch: the CB * PR rows of a slab, W words each, as 16-byte vectors where the rows are aligned; weights:
  // thread (feature tid % 64, quarter tid / 64) takes a quarter of the feature's CB * TAPS consecutive words.
  constexpr bool VEC = W % 4 == 0;
  constexpr int EPR = VEC ? W / 4 : W;                              // loads per row
  constexpr int NLD = CB * PR * EPR, NLP = (NLD + 255) / 256;
  constexpr int WPT = (CB * TAPS + 3) / 4;
  rx_f32x4 pstage[VEC ? NLP : 1];
  float pstage1[VEC ? 1 : NLP];
  float wstage[WPT];
  auto load_slab = [&](int c0) {
#pragma unroll
    for (int i = 0; i < NLP; ++i) {
      const int v = i * 256 + tid;
      const int row = v / EPR, q = v % EPR;                         // row = channel of the slab * PR + row of the patch
      const int c = c0 + row / PR, y = y0 * SH - PT + row % PR;
      const bool in = v < NLD && c < C && y >= 0 && y < H;
      const float* src = x + (((long long)b * C + c) * H + y) * W;
      if constexpr (VEC) pstage[i] = in ? *(const rx_f32x4*)(src + 4 * q) : rx_f32x4{0.f, 0.f, 0.f, 0.f};
      else pstage1[i] = in ? src[q] : 0.f;
    }
    const int o = og + (tid & 63), part = tid >> 6;
    // whole slabs, whole groups of 64 features and whole quarters: plain consecutive loads, which the compiler widens;
    // else loads at clamped positions inside the filter array and a select (a load under a branch of its own is not
    // combined with its neighbours and costs the kernel 12 %)
    constexpr bool WFULL = C % CB == 0 && O % 64 == 0 && CB * TAPS % 4 == 0;
    const float* wsrc = w + ((long long)(o < O ? o : O - 1) * C + c0) * TAPS;
    const int left = (C - c0) * TAPS;                               // words of this feature from channel c0 on
#pragma unroll
    for (int i = 0; i < WPT; ++i) {
      const int e = part * WPT + i;                                 // (channel of the slab, tap)
      if constexpr (WFULL) {
        wstage[i] = wsrc[e];
      } else {
        const float v = wsrc[e < left ? e : left - 1];
        wstage[i] = (e < CB * TAPS && e < left && o < O) ? v : 0.f;
      }
    }
  };
  auto store_slab = [&](int st) {
#pragma unroll
    for (int i = 0; i < NLP; ++i) {
      const int v = i * 256 + tid;
      const int row = v / EPR, q = v % EPR;
      float* dst = patch + st * PATCH + (row / PR) * PCH + (row % PR) * PW + OFF;
      if (v < NLD) {
        if constexpr (VEC) *(rx_f32x4*)(dst + 4 * q) = pstage[i];
        else dst[q] = pstage1[i];
      }
    }
    const int part = tid >> 6;
#pragma unroll
    for (int i = 0; i < WPT; ++i) {
      const int e = part * WPT + i;
      const int c_l = e / TAPS, tap = e % TAPS;
      if (e < CB * TAPS) wl[st * WSLAB + ((tap * NQ + c_l / 4) * 4 + (c_l & 3)) * WST + (tid & 63)] = wstage[i];
    }
  };

  // a lane's address of each pixel block: its pixel (lane % 16) and its channel of the quad (lane / 16); the tap and the
  // quad are constants of the step
  const int kk = lane >> 4, li = lane & 15;
  int poff[NPB];
#pragma unroll
  for (int pb = 0; pb < NPB; ++pb) {
    int p = pb * 16 + li;
    if (p >= NPX) p = NPX - 1;                                      // ragged last block: those rows of the result are not stored
    poff[pb] = kk * PCH + (p / WO) * SH * PW + (p % WO) * SW + OFF - PL;
  }
  const int woff = kk * WST + wave * 16 + li;
  rx_f32x4 acc[NPB];
#pragma unroll
  for (int pb = 0; pb < NPB; ++pb) acc[pb] = rx_f32x4{0.f, 0.f, 0.f, 0.f};

  load_slab(0);
  // the patch stages start as zeros (the columns around the image are never written afterwards), under the first loads
  for (int i = tid; i < NSTG * PATCH; i += 256) patch[i] = 0.f;
  __syncthreads();
  store_slab(0);
  __syncthreads();
  // One wavefront per SIMD: nothing else hides the LDS latency, so the operands of k step ks + 1 are read into a second
  // register set while the MFMAs of step ks run, one read between two MFMAs (a scheduling barrier after every pair keeps
  // that order: left alone the compiler reads a whole step's operands and then waits for them with the MFMA pipe idle).  The next slab goes
  // into the other stage in the middle of a slab, between two barriers (every wavefront has left the previous slab; the
  // stage is complete), so that the last step of a slab can already read the first operands of the next one.
  float pa[2][NPB], fw[2];
  // operand `pb` of step KS into register set BUF (pb = -1: the filter word)
  auto fetch = [&](auto BUF, auto KS, int pb, const float* pp, const float* ww) __attribute__((always_inline)) {
    constexpr int buf = decltype(BUF)::value, ks = decltype(KS)::value, tap = ks / NQ, q = ks % NQ;
    constexpr int koff = q * 4 * PCH + (tap / KW) * DH * PW + (tap % KW) * DW;
    if (pb < 0) fw[buf] = ww[ks * 4 * WST + woff];
    else pa[buf][pb] = pp[poff[pb] + koff];
  };
  auto fetch_all = [&](auto BUF, auto KS, const float* pp, const float* ww) __attribute__((always_inline)) {
#pragma unroll
    for (int pb = -1; pb < NPB; ++pb) fetch(BUF, KS, pb, pp, ww);
  };
  constexpr bool AHEAD = NSTEP % 2 == 0 && NSTEP >= 4;              // the register sets alternate in step with the slabs
  if constexpr (AHEAD) fetch_all(rx_int<0>{}, rx_int<0>{}, patch, wl);
  for (int s = 0; s < NSLAB; ++s) {
    const int st = s & 1;
    const bool more = s + 1 < NSLAB;
    if (more) load_slab((s + 1) * CB);
    const float* pp = patch + st * PATCH;
    const float* ww = wl + st * WSLAB;
    if constexpr (!AHEAD) fetch_all(rx_int<0>{}, rx_int<0>{}, pp, ww);
    rx_static_for<0, NSTEP>([&](auto KS) {
      constexpr int ks = decltype(KS)::value;
      if constexpr (AHEAD && ks == NSTEP / 2) {
        if (more) {
          __syncthreads();
          store_slab(st ^ 1);
          __syncthreads();
        }
      }
      // where the next step's operands come from: this slab, or (last step) the first step of the next one
      constexpr bool last = ks + 1 == NSTEP;
      const float* np = last ? patch + (st ^ 1) * PATCH : pp;
      const float* nw = last ? wl + (st ^ 1) * WSLAB : ww;
      const bool rd = last ? (AHEAD && more) : true;
      typedef rx_int<last ? 0 : (ks + 1) % 2> NB_;
      typedef rx_int<last ? 0 : ks + 1> NK_;
      if (rd) fetch(NB_{}, NK_{}, -1, np, nw);
      constexpr int GRP = 5;
#pragma unroll
      for (int g = 0; g < NPB; g += GRP) {
#pragma unroll
        for (int pb = g; pb < g + GRP && pb < NPB; ++pb) if (rd) fetch(NB_{}, NK_{}, pb, np, nw);
#pragma unroll
        for (int pb = g; pb < g + GRP && pb < NPB; ++pb) acc[pb] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[ks % 2][pb], fw[ks % 2], acc[pb], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);                     // a few reads, a few MFMAs: the order of the groups stays as written
      }
    });
    if constexpr (!AHEAD) {
      if (more) store_slab(st ^ 1);
      __syncthreads();
    }
  }
  // a lane holds pixels 4 (lane / 16) .. + 3 of each block for feature lane % 16 of its wavefront; the epilogue functor
  // (bias, activation, store) takes them at (image, feature, row, first column)
  const int o = og + wave * 16 + li;
  if (o < O) {
#pragma unroll
    for (int pb = 0; pb < NPB; ++pb) {
      const int p = pb * 16 + 4 * kk;
      // (a functor that declares masks_rows takes the test as its last argument and guards its store with it: its
      // arithmetic is then straight-line code over all the blocks of the lane, whose feature is the same in all of them)
      if constexpr (WO % 4 == 0) {
        // whole vectors: a row of the result and the rows left in the image are multiples of 4 words
        const bool inside = p < NPX && y0 * WO + p < HO * WO;
        if constexpr (rx_epi_masks_rows<Epi>::value) {
          const float v[4] = {acc[pb][0], acc[pb][1], acc[pb][2], acc[pb][3]};
          epi(v, b, o, y0 + p / WO, p % WO, inside);
        } else if (inside) {
          const float v[4] = {acc[pb][0], acc[pb][1], acc[pb][2], acc[pb][3]};
          epi(v, b, o, y0 + p / WO, p % WO);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const bool inside = p + r < NPX && y0 * WO + p + r < HO * WO;
          if constexpr (rx_epi_masks_rows<Epi>::value) {
            const float v[1] = {acc[pb][r]};
            epi(v, b, o, y0 + (p + r) / WO, (p + r) % WO, inside);
          } else if (inside) {
            const float v[1] = {acc[pb][r]};
            epi(v, b, o, y0 + (p + r) / WO, (p + r) % WO);
          }
        }
      }
    }
  }
}

// Choice and instantiation of the MFMA GEMM skeletons (kernels/rx_gemm_kernels.h).
#pragma once
#include <string>

#include "rx_ir.h"

namespace rx {

struct GemmChoice {
  bool ok = false;
  std::string kind;         // "gemm_f32" | "gemm_bf16" | "gemm_f16" | "gemm_f8"
  std::string skeleton;     // template name in rx_gemm_kernels.h
  std::string targs;        // template arguments before the epilogue type
  unsigned grid[3] = {1, 1, 1};
  unsigned block = 256;
  unsigned lds_bytes = 0;   // dynamic LDS (0: the skeleton declares static LDS)
  std::string stype_a, stype_b;
  int split = 1;            // slices of K, one per blockIdx.y (partial products; rx_gemm_body_dl only)
  int depth = 0;            // rx_gemm_body_s: blocks of the streamed operand read ahead (0: the skeleton's default)
  int stream_stages = 0;    // rx_gemm_body_s: LDS stages per operand (0: not that skeleton)
  int bk = 0;               // rx_gemm_body_dl: elements of K per tile
};

// Workgroups to launch for a gm x gn grid of tiles: the kernels walk the tiles in blocks of 4 x 8,
// eight blocks (one per XCD) at a time, and the grid is padded to whole rounds of eight blocks
// (rx_gemm_tile in kernels/rx_gemm_kernels.h decodes the same order).
inline int64_t gemm_grid(int64_t gm, int64_t gn, int rb = 4, int cb = 8) {
  if (rb == 0) return gm * gn;   // plain order for small tile grids
  const int64_t blocks = ((gm + rb - 1) / rb) * ((gn + cb - 1) / cb);
  return (blocks + 7) / 8 * 8 * rb * cb;
}

// Returns ok=false when no skeleton covers the case (the caller then writes a scalar loop).
// `staged_only`: an operand is a functor, which only the register-staged skeleton can read.
GemmChoice choose_gemm(DT a, DT b, DT out, int64_t batch, int64_t M, int64_t N, int64_t K, bool a_k_contig, bool b_k_contig,
                       bool staged_only = false, int split = 1);

// Text of the `extern "C"` kernel <kbase>_gemm that runs the skeleton with epilogue type <kbase>_epi.
// `epi_params` is the tail of the parameter list (epilogue operands and out0), `epi_ctor` builds `epi`.
// An operand computed by a functor: `type` names the functor struct ("" = read from memory), `params` the
// kernel parameters it needs (", const T* name" ...), `ctor` the statement that builds it as `la` / `lb`.
struct GemmOperandFn {
  std::string type, params, ctor;
};
std::string gemm_instance(const GemmChoice& c, const std::string& kbase, const std::string& epi_params, const std::string& epi_ctor, bool batched,
                          const GemmOperandFn& fa = {}, const GemmOperandFn& fb = {});

// Tiling of the direct-convolution kernel (rx_conv_body in kernels/rx_gemm_kernels.h): f32 images [B, C, H, W], filters
// [O, C, KH, KW], result [B, O, HO, WO], strides sh / sw, filter dilations dh / dw, `pl` zero columns before the image.  ok = false
// when the kernel does not cover the case (the convolution is then lowered to a matrix product on the window matrix).
struct ConvChoice {
  bool ok = false;
  int rows = 0;             // rows of the result per workgroup
  int slab = 0;             // channels per LDS stage
  unsigned grid[2] = {1, 1};
  unsigned lds_bytes = 0;
};
ConvChoice choose_conv(int64_t B, int64_t C, int64_t H, int64_t W, int64_t O, int64_t KH, int64_t KW, int64_t HO, int64_t WO, int64_t pl,
                       int64_t sh = 1, int64_t sw = 1, int64_t dh = 1, int64_t dw = 1);

}  // namespace rx

// Ahead-of-time build check of the GEMM skeletons: instantiates every MMA policy and
// both operand orders with a plain store epilogue, so that device-code errors show up
// when the library is built rather than when a module is compiled at run time.
#include <hip/hip_runtime.h>
#include "rx_preamble.h"
#include "rx_gemm_kernels.h"

template <typename OUT, int N>
struct rx_check_epi {
  OUT* out;
  template <int NV>
  __device__ __forceinline__ void operator()(const float (&acc)[NV], int m, int n) const {
#pragma unroll
    for (int l = 0; l < NV; ++l) out[(long long)m * N + n + l] = (OUT)acc[l];
  }
};

#define RX_CHECK(NAME, MMA, BK, AKC, BKC)                                                                          \
  extern "C" __global__ __launch_bounds__(256) void NAME(const MMA::elem* A, const MMA::elem* B, float* out) {      \
    rx_check_epi<float, 512> epi{out};                                                                             \
    rx_gemm_body<MMA, 128, 128, BK, 2, 2, AKC, BKC, 512, 512, 512, 4, 8, false, rx_check_epi<float, 512>>(A, B, epi);     \
  }

RX_CHECK(rx_check_f32_nn, rx_mma_f32, 16, true, false)
RX_CHECK(rx_check_f32_tt, rx_mma_f32, 16, false, true)
RX_CHECK(rx_check_bf16_nn, rx_mma_bf16, 64, true, false)
RX_CHECK(rx_check_bf16_nt, rx_mma_bf16, 64, true, true)
RX_CHECK(rx_check_bf16_tn, rx_mma_bf16, 64, false, false)
RX_CHECK(rx_check_f16_nt, rx_mma_f16, 64, true, true)
RX_CHECK(rx_check_f16_tn, rx_mma_f16, 64, false, false)
RX_CHECK(rx_check_f8_nt, rx_mma_f8, 128, true, true)
RX_CHECK(rx_check_f8_nn, rx_mma_f8, 128, true, false)

// the direct-to-LDS body, with the 32x32 and the 16x16 MFMA shapes of 16-bit operands and the 8-bit one
#define RX_CHECK_DL(NAME, MMA, BM, BN, BK, WM, WN, AKC, BKC)                                                              \
  extern "C" __global__ __launch_bounds__(WM * WN * 64) void NAME(const MMA::elem* A, const MMA::elem* B, float* out) {     \
    rx_check_epi<float, 512> epi{out};                                                                                     \
    rx_gemm_body_dl<MMA, BM, BN, BK, WM, WN, 2, AKC, BKC, 512, 512, 512, 0, 0, false, rx_check_epi<float, 512>>(A, B, epi);  \
  }
RX_CHECK_DL(rx_check_dl_bf16_nn, rx_mma_bf16, 256, 256, 64, 2, 4, true, false)
RX_CHECK_DL(rx_check_dl_bf16x16_nn, rx_mma_bf16_16, 256, 256, 64, 2, 4, true, false)
RX_CHECK_DL(rx_check_dl_bf16x16_nt, rx_mma_bf16_16, 256, 128, 64, 2, 4, true, true)
RX_CHECK_DL(rx_check_dl_bf16x16_tn, rx_mma_bf16_16, 128, 256, 64, 4, 2, false, false)
RX_CHECK_DL(rx_check_dl_f16x16_tt, rx_mma_f16_16, 128, 128, 64, 2, 2, false, true)
RX_CHECK_DL(rx_check_dl_f8_nt, rx_mma_f8, 256, 256, 128, 2, 4, true, true)

// the streaming body (16x16 MFMA shapes), 8- and 16-bit operands, all four operand layouts, 256x256 tiles (wavefronts of 128x64) and 256x128 tiles (64x64; 128x32 by request)
#define RX_CHECK_S(NAME, EL, BM, BN, WM, WN, AKC, BKC, K)                                                                \
  extern "C" __global__ __launch_bounds__(512) void NAME(const EL::elem* A, const EL::elem* B, float* out) {              \
    rx_check_epi<float, 512> epi{out};                                                                                     \
    rx_gemm_body_s<EL, BM, BN, WM, WN, AKC, BKC, 512, 512, K, 0, 0, false, rx_check_epi<float, 512>>(A, B, epi);            \
  }
RX_CHECK_S(rx_check_s_f8_nt, rx_el_f8, 256, 256, 2, 4, true, true, 512)
RX_CHECK_S(rx_check_s_f8_nn, rx_el_f8, 256, 256, 2, 4, true, false, 384)
RX_CHECK_S(rx_check_s_f8_tn, rx_el_f8, 256, 128, 4, 2, false, false, 128)
RX_CHECK_S(rx_check_s_f8_tt, rx_el_f8, 256, 256, 2, 4, false, true, 256)
RX_CHECK_S(rx_check_s_bf16_nn, rx_el_bf16, 256, 256, 2, 4, true, false, 512)
RX_CHECK_S(rx_check_s_bf16_nt, rx_el_bf16, 256, 128, 4, 2, true, true, 64)
RX_CHECK_S(rx_check_s_bf16_nt24, rx_el_bf16, 256, 128, 2, 4, true, true, 64)
RX_CHECK_S(rx_check_s_f16_tn, rx_el_f16, 256, 256, 2, 4, false, false, 192)
RX_CHECK_S(rx_check_s_f16_tt, rx_el_f16, 256, 128, 4, 2, false, true, 128)

// the ping-pong form of the 256x256 streaming tiles
#define RX_CHECK_PP(NAME, EL, AKC, BKC, K)                                                                               \
  extern "C" __global__ __launch_bounds__(512) void NAME(const EL::elem* A, const EL::elem* B, float* out) {              \
    rx_check_epi<float, 512> epi{out};                                                                                     \
    rx_gemm_body_pp<EL, 256, 256, 2, 4, AKC, BKC, 512, 512, K, 0, 0, false, rx_check_epi<float, 512>>(A, B, epi);           \
  }
RX_CHECK_PP(rx_check_pp_bf16_nn, rx_el_bf16, true, false, 512)
RX_CHECK_PP(rx_check_pp_bf16_nt, rx_el_bf16, true, true, 128)
RX_CHECK_PP(rx_check_pp_f16_tn, rx_el_f16, false, false, 256)
RX_CHECK_PP(rx_check_pp_f16_tt, rx_el_f16, false, true, 256)
RX_CHECK_PP(rx_check_pp_f8_nt, rx_el_f8, true, true, 512)
RX_CHECK_PP(rx_check_pp_f8_tn, rx_el_f8, false, false, 256)

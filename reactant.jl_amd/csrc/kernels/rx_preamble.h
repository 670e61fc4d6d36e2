// Device-side helpers shared by every fusion-group kernel (gfx950, wave64).
// This header is embedded into the library and handed to hiprtc together with the
// kernel text that the fusion code generator writes for one module.
#pragma once

typedef unsigned char rx_u8;
typedef unsigned short rx_u16;
typedef unsigned int rx_u32;
typedef unsigned long long rx_u64;
typedef signed char rx_i8;
typedef short rx_i16;
typedef int rx_i32;
typedef long long rx_i64;

#define RX_DEV static __device__ __forceinline__
#define RX_MEM __device__ __forceinline__

template <typename T, int N>
struct __attribute__((aligned(sizeof(T) * N))) rx_vec {
  T v[N];
};

// ---------------------------------------------------------------------------
// vector loads / stores.  The non-temporal forms mark data that is touched once
// (streamed inputs, map outputs) so that it does not displace reusable lines.
// ---------------------------------------------------------------------------
typedef rx_u32 rx_u32x4 __attribute__((ext_vector_type(4)));
typedef rx_u32 rx_u32x2 __attribute__((ext_vector_type(2)));

template <typename V, typename T>
static __device__ __forceinline__ V rx_load(const T* p) {
  return *reinterpret_cast<const V*>(p);
}
template <typename V, typename T>
static __device__ __forceinline__ V rx_load_nt(const T* p) {
  if constexpr (sizeof(V) == 16) {
    return __builtin_bit_cast(V, __builtin_nontemporal_load(reinterpret_cast<const rx_u32x4*>(p)));
  } else if constexpr (sizeof(V) == 8) {
    return __builtin_bit_cast(V, __builtin_nontemporal_load(reinterpret_cast<const rx_u32x2*>(p)));
  } else if constexpr (sizeof(V) == 4) {
    return __builtin_bit_cast(V, __builtin_nontemporal_load(reinterpret_cast<const rx_u32*>(p)));
  } else {
    return *reinterpret_cast<const V*>(p);
  }
}
// a vector at an address that is a multiple of the element size only (padded rows start anywhere)
template <typename V, typename T>
static __device__ __forceinline__ V rx_load_unaligned(const T* p) {
  struct __attribute__((packed, aligned(alignof(T)))) U { V v; };
  return reinterpret_cast<const U*>(p)->v;
}
template <typename T, typename V>
static __device__ __forceinline__ void rx_store(T* p, const V& v) {
  *reinterpret_cast<V*>(p) = v;
}
template <typename T, typename V>
static __device__ __forceinline__ void rx_store_nt(T* p, const V& v) {
  if constexpr (sizeof(V) == 16) {
    __builtin_nontemporal_store(__builtin_bit_cast(rx_u32x4, v), reinterpret_cast<rx_u32x4*>(p));
  } else if constexpr (sizeof(V) == 8) {
    __builtin_nontemporal_store(__builtin_bit_cast(rx_u32x2, v), reinterpret_cast<rx_u32x2*>(p));
  } else if constexpr (sizeof(V) == 4) {
    __builtin_nontemporal_store(__builtin_bit_cast(rx_u32, v), reinterpret_cast<rx_u32*>(p));
  } else {
    *reinterpret_cast<V*>(p) = v;
  }
}
template <typename I>
static __device__ __forceinline__ I rx_clamp_idx(I i, I hi) {
  return i < 0 ? (I)0 : (i > hi ? hi : i);
}

// ---------------------------------------------------------------------------
// bit casts
// ---------------------------------------------------------------------------
RX_DEV rx_u32 rx_f2u(float f) { return __builtin_bit_cast(rx_u32, f); }
RX_DEV float rx_u2f(rx_u32 u) { return __builtin_bit_cast(float, u); }

// ---------------------------------------------------------------------------
// bf16: storage is the upper half of binary32; conversion rounds to nearest even
// ---------------------------------------------------------------------------
RX_DEV float rx_bf16_to_f32(rx_u16 b) { return rx_u2f(((rx_u32)b) << 16); }
// gfx950 converts in hardware (v_cvt_pk_bf16_f32, round to nearest even, NaN stays NaN)
RX_DEV rx_u16 rx_f32_to_bf16(float f) { return __builtin_bit_cast(rx_u16, (__bf16)f); }
RX_DEV float rx_round_bf16(float f) { return rx_bf16_to_f32(rx_f32_to_bf16(f)); }

// ---------------------------------------------------------------------------
// f16
// ---------------------------------------------------------------------------
RX_DEV float rx_f16_to_f32(rx_u16 b) { return (float)__builtin_bit_cast(_Float16, b); }
RX_DEV rx_u16 rx_f32_to_f16(float f) { return __builtin_bit_cast(rx_u16, (_Float16)f); }
RX_DEV float rx_round_f16(float f) { return (float)(_Float16)f; }

// ---------------------------------------------------------------------------
// f8E4M3FN (OCP e4m3: bias 7, no inf, S.1111.111 = NaN, max 448)
// f8E5M2   (bias 15, inf and NaN as in binary16)
// Round to nearest even; a value that rounds above the largest finite number
// becomes NaN (e4m3fn) or inf (e5m2).
// ---------------------------------------------------------------------------
RX_DEV float rx_e4m3_to_f32(rx_u8 b) {
  rx_u32 s = ((rx_u32)(b & 0x80u)) << 24;
  rx_u32 e = (b >> 3) & 0xfu;
  rx_u32 m = b & 7u;
  if (e == 0xfu && m == 7u) return rx_u2f(s | 0x7fc00000u);
  if (e == 0) {
    float v = (float)m * 0.001953125f;  // m * 2^-9
    return rx_u2f(rx_f2u(v) | s);
  }
  return rx_u2f(s | ((e + 120u) << 23) | (m << 20));
}
RX_DEV rx_u8 rx_f32_to_e4m3_sw(float f);
// gfx950 converts f32 -> OCP e4m3 in hardware (round to nearest even).  Only finite values with
// |x| <= 448 are given to it, so its overflow mode never matters: (448, 464] rounds to 448 and
// everything above (or NaN) is the NaN code, as the format without infinity requires.
RX_DEV rx_u8 rx_f32_to_e4m3(float f) {
  const rx_u32 u = rx_f2u(f);
  const rx_u32 a = u & 0x7fffffffu;
  const float c = rx_u2f(a < 0x43e00000u ? a : 0x43e00000u);   // min(|x|, 448); NaN payloads compare above it too
  const rx_u32 packed = (rx_u32)__builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false);
  const rx_u32 code = a > 0x43e80000u ? 0x7fu : (packed & 0x7fu);
  return (rx_u8)(((u >> 24) & 0x80u) | code);
}
// The same for a value known to be finite with |x| <= 448, or NaN: the hardware conversion alone.  A NaN becomes the
// code 0xff whatever its sign (rx_f32_to_e4m3 keeps the sign: 0x7f or 0xff; both are NaN).
RX_DEV rx_u8 rx_f32_to_e4m3_inrange(float f) { return (rx_u8)__builtin_amdgcn_cvt_pk_fp8_f32(f, f, 0, false); }
RX_DEV rx_u8 rx_f32_to_e4m3_sw(float f) {
  rx_u32 u = rx_f2u(f);
  rx_u8 s = (rx_u8)((u >> 24) & 0x80u);
  rx_u32 a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (rx_u8)(s | 0x7fu);       // NaN
  if (a > 0x43e80000u) return (rx_u8)(s | 0x7fu);       // |x| > 464 rounds past 448 (inf too)
  if (a < 0x3c800000u) {                                // |x| < 2^-6: subnormal range
    float v = rx_u2f(a) * 512.0f;                       // in units of 2^-9
    float r = __builtin_rintf(v);                       // ties to even
    return (rx_u8)(s | (rx_u8)(int)r);                  // r == 8 lands on the first normal
  }
  rx_u32 r = a + 0x7ffffu + ((a >> 20) & 1u);           // RNE at 3 mantissa bits
  rx_u32 e = (r >> 23) - 120u;
  rx_u32 m = (r >> 20) & 7u;
  return (rx_u8)(s | (e << 3) | m);
}
RX_DEV float rx_round_e4m3(float f) { return rx_e4m3_to_f32(rx_f32_to_e4m3(f)); }

RX_DEV float rx_e5m2_to_f32(rx_u8 b) {
  rx_u16 h = (rx_u16)(((rx_u16)b) << 8);
  return (float)__builtin_bit_cast(_Float16, h);
}
RX_DEV rx_u8 rx_f32_to_e5m2(float f) {
  rx_u32 u = rx_f2u(f);
  rx_u8 s = (rx_u8)((u >> 24) & 0x80u);
  rx_u32 a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (rx_u8)(s | 0x7fu);
  if (a >= 0x47700000u) return (rx_u8)(s | 0x7cu);      // >= 61440 rounds to inf
  if (a < 0x38800000u) {                                // |x| < 2^-14: subnormal range
    float v = rx_u2f(a) * 65536.0f;                     // units of 2^-16
    float r = __builtin_rintf(v);
    return (rx_u8)(s | (rx_u8)(int)r);
  }
  rx_u32 r = a + 0xfffffu + ((a >> 21) & 1u);
  rx_u32 e = (r >> 23) - 112u;
  rx_u32 m = (r >> 21) & 3u;
  return (rx_u8)(s | (e << 2) | m);
}
RX_DEV float rx_round_e5m2(float f) { return rx_e5m2_to_f32(rx_f32_to_e5m2(f)); }

// ---------------------------------------------------------------------------
// elementwise math with StableHLO semantics
// ---------------------------------------------------------------------------
template <typename T> RX_DEV T rx_max(T a, T b) { return (a > b || a != a) ? a : b; }
template <typename T> RX_DEV T rx_min(T a, T b) { return (a < b || a != a) ? a : b; }
// clamp between two constants lo <= hi (neither NaN); a NaN operand stays NaN
RX_DEV float rx_clamp_ordered(float x, float lo, float hi) {
  const float m = __builtin_amdgcn_fmed3f(x, lo, hi);
  return x != x ? x : m;
}
template <typename T> RX_DEV T rx_sign(T a) {
  return a != a ? a : (T)((a > (T)0) - (a < (T)0));
}
// tanh for results that are rounded to a 16-bit or 8-bit float: 1 - 2/(e^{2x}+1) on the
// hardware exp2 / reciprocal (absolute error ~1e-7, far below half an ulp of bf16 at 1).
// e^{2x} saturates to 0 or inf at the ends, which gives exactly -1 and 1; NaN propagates.
RX_DEV float rx_tanh_fast(float x) {
  const float e = __builtin_amdgcn_exp2f(x * 2.8853900817779268f);
  return __builtin_fmaf(-2.0f, __builtin_amdgcn_rcpf(e + 1.0f), 1.0f);
}
// e^x for results that are rounded to a 16-bit or 8-bit float: the hardware's 2^y on y = x log2(e) (relative error
// about |x| 2^-24 + 2^-23, far below half an ulp of f16); saturates to 0 and inf like expf; results below the smallest
// normal float32 (which only a bf16 result can hold) are flushed to zero.
RX_DEV float rx_exp_fast(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
// 1 / (1 + e^-x) for results that are rounded to a 16-bit or 8-bit float, on the hardware's 2^y and reciprocal
// (absolute error about 1e-7); exactly 0 and 1 at the ends, NaN propagates.
RX_DEV float rx_logistic_fast(float x) { return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f)); }
// 0.5 x (1 + tanh(a (x + b x^3))) = x / (1 + e^(-2 a (x + b x^3))) for results that are rounded to a 16-bit or 8-bit
// float; k1 = -2 a log2(e), k3 = k1 b.  The exponential saturates to 0 or inf at the ends, which gives x and -0 as the
// chain does; x = -inf gives NaN as the chain does (-inf * 0); NaN propagates.  Where 1 + tanh cancels (x < -3) the
// chain in float32 is off by up to |x| 2^-23 in absolute terms; this form is not.
RX_DEV float rx_gelu_chain_fast(float x, float k1, float k3) {
  const float e = __builtin_amdgcn_exp2f(x * __builtin_fmaf(k3, x * x, k1));
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}
// x / y for a divisor that is the same for every element.  1/y in double is loop-invariant; the
// double product is within 2^-52 of the exact quotient, and the quotient of two 24-bit numbers is
// never closer than about 2^-49 (relative) to a midpoint between two floats, so rounding the
// product to float gives the correctly rounded quotient.  Zero, infinite and NaN operands
// behave as in the division (1/0 = inf, 0 * inf = NaN, ...); double has the range for
// subnormal divisors.
RX_DEV float rx_div_uniform(float x, float y) { return (float)((double)x * (1.0 / (double)y)); }
// Marks a value as used here: the compiler then computes it at this point instead of moving the whole computation
// into a conditional store that follows (where equal subexpressions of neighbouring calls could no longer be merged).
template <class V>
RX_DEV void rx_keep_value(V& v) {
  if constexpr (sizeof(V) % 4 == 0) {
    unsigned w[sizeof(V) / 4];
    __builtin_memcpy(w, &v, sizeof(V));
#pragma unroll
    for (unsigned k = 0; k < sizeof(V) / 4; ++k) asm volatile("" : "+v"(w[k]));
    __builtin_memcpy(&v, w, sizeof(V));
  }
}
// A read of memory that nothing writes while the kernel runs (a bias, batch-norm statistics), through the constant
// address space: the compiler may then merge equal reads across the kernel's stores, which for a struct member that is
// only declared __restrict__ it does not.
template <class T>
RX_DEV T rx_load_const(const T* p, long long i) {
  return ((const __attribute__((address_space(4))) T*)p)[i];
}
// x / y for a result that is rounded to a narrow float, where y does not vary along the minor dimension (the sum of a
// softmax row): x times the reciprocal of y, a division that is computed once per row.  The reciprocal of a divisor
// below 2^-128 would overflow although the quotient is finite (1e-20 / 1e-39), so divisors below 2^-64 are scaled by
// 2^64 first and the product is scaled back: both scalings are exact, the result stays within an ulp of float32 of
// the quotient, and zero, infinite and NaN operands behave as in the division.
RX_DEV float rx_div_minor_uniform(float x, float y) {
  const float s = __builtin_fabsf(y) < 0x1p-64f ? 0x1p64f : 1.0f;
  return (x * (1.0f / (y * s))) * s;
}
RX_DEV float rx_logistic(float x) { return 1.0f / (1.0f + expf(-x)); }
RX_DEV double rx_logistic(double x) { return 1.0 / (1.0 + exp(-x)); }
RX_DEV float rx_rsqrt(float x) { return 1.0f / sqrtf(x); }
RX_DEV double rx_rsqrt(double x) { return 1.0 / sqrt(x); }
RX_DEV float rx_gelu_tanh(float x) {
  return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
}
RX_DEV float rx_gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.7071067811865476f)); }
RX_DEV float rx_gelu_sigmoid(float x) { return x / (1.0f + expf(-1.702f * x)); }
RX_DEV double rx_gelu_tanh(double x) {
  return 0.5 * x * (1.0 + tanh(0.7978845608028654 * (x + 0.044715 * x * x * x)));
}
RX_DEV double rx_gelu_erf(double x) { return 0.5 * x * (1.0 + erf(x * 0.7071067811865476)); }
RX_DEV double rx_gelu_sigmoid(double x) { return x / (1.0 + exp(-1.702 * x)); }
// Integer division as XLA defines the cases C++ leaves undefined: x / 0 = all ones, x % 0 = x, and
// for signed types x / -1 = -x with wrap-around (so MIN / -1 = MIN) and x % -1 = 0.  For an unsigned
// type (T)-1 is the largest value, an ordinary divisor.
template <typename T> RX_DEV T rx_idiv(T a, T b) {
  if (b == 0) return (T)-1;
  if constexpr ((T)-1 < (T)0) {
    if (b == (T)-1) return (T)(0 - a);
  }
  return a / b;
}
template <typename T> RX_DEV T rx_irem(T a, T b) {
  if (b == 0) return a;
  if constexpr ((T)-1 < (T)0) {
    if (b == (T)-1) return (T)0;
  }
  return a % b;
}
// float -> integer conversion: truncation toward zero; values beyond the type's range give the
// nearest limit and NaN gives 0 (a plain C++ cast is undefined for those).
template <typename T, typename F> RX_DEV T rx_f2i(F x) {
  constexpr bool sgn = (T)-1 < (T)0;
  constexpr T hi = sgn ? (T)(((unsigned long long)1 << (8 * sizeof(T) - 1)) - 1) : (T)~(T)0;
  constexpr T lo = sgn ? (T)(-(long long)hi - 1) : (T)0;
  if (!(x == x)) return (T)0;
  if (x <= (F)lo) return lo;
  if (x >= (F)hi) return hi;   // (F)hi may round up to 2^k: such x are out of range as well
  return (T)x;
}
template <typename T> RX_DEV T rx_ipow(T a, T b) {
  if (b < 0) return (a == 1) ? (T)1 : ((a == (T)-1) ? ((b & 1) ? (T)-1 : (T)1) : (T)0);
  T r = 1;
  while (b) {
    if (b & 1) r *= a;
    a *= a;
    b >>= 1;
  }
  return r;
}

// ---------------------------------------------------------------------------
// wavefront (64 lanes) reductions.  32-bit payloads move through DPP row
// operations; 64-bit payloads are moved as two halves.  The combined value
// ends up in every lane.
// ---------------------------------------------------------------------------
template <int CTRL, int ROW_MASK>
RX_DEV rx_i32 rx_dpp(rx_i32 v) {
  return __builtin_amdgcn_update_dpp(v, v, CTRL, ROW_MASK, 0xf, false);
}
template <typename T, int CTRL, int ROW_MASK>
RX_DEV T rx_dpp_t(T v) {
  if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, rx_dpp<CTRL, ROW_MASK>(__builtin_bit_cast(rx_i32, v)));
  } else if constexpr (sizeof(T) == 8) {
    rx_u64 u = __builtin_bit_cast(rx_u64, v);
    rx_u32 lo = (rx_u32)rx_dpp<CTRL, ROW_MASK>((rx_i32)(rx_u32)u);
    rx_u32 hi = (rx_u32)rx_dpp<CTRL, ROW_MASK>((rx_i32)(rx_u32)(u >> 32));
    return __builtin_bit_cast(T, ((rx_u64)hi << 32) | lo);
  } else {
    rx_i32 w = (rx_i32)v;
    return (T)rx_dpp<CTRL, ROW_MASK>(w);
  }
}
template <typename T>
RX_DEV T rx_readlane63(T v) {
  if constexpr (sizeof(T) == 8) {
    rx_u64 u = __builtin_bit_cast(rx_u64, v);
    rx_u32 lo = (rx_u32)__builtin_amdgcn_readlane((rx_i32)(rx_u32)u, 63);
    rx_u32 hi = (rx_u32)__builtin_amdgcn_readlane((rx_i32)(rx_u32)(u >> 32), 63);
    return __builtin_bit_cast(T, ((rx_u64)hi << 32) | lo);
  } else if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, __builtin_amdgcn_readlane(__builtin_bit_cast(rx_i32, v), 63));
  } else {
    return (T)__builtin_amdgcn_readlane((rx_i32)v, 63);
  }
}

// digamma: reflection below zero, the recurrence psi(x) = psi(x + 1) - 1 / x up to x >= 10, then the
// asymptotic series; carried in double (poles at the non-positive integers give NaN)
template <typename T>
RX_DEV T rx_digamma(T xin) {
  double x = (double)xin, r = 0.0;
  if (x <= 0.0 && floor(x) == x) return (T)__builtin_nan("");
  if (x < 0.0) {
    r = -3.14159265358979323846 / tan(3.14159265358979323846 * x);
    x = 1.0 - x;
  }
  while (x < 10.0) { r -= 1.0 / x; x += 1.0; }
  const double f = 1.0 / (x * x);
  r += log(x) - 0.5 / x -
       f * (1.0 / 12.0 - f * (1.0 / 120.0 - f * (1.0 / 252.0 - f * (1.0 / 240.0 - f * (1.0 / 132.0 - f * (691.0 / 32760.0 - f * (1.0 / 12.0)))))));
  return (T)r;
}
// bits set / leading zero bits of an integer of any width (the value's own width counts)
template <typename T>
RX_DEV int rx_popcnt(T v) {
  if constexpr (sizeof(T) == 8) return __popcll((unsigned long long)v);
  else if constexpr (sizeof(T) == 4) return __popc((unsigned)v);
  else if constexpr (sizeof(T) == 2) return __popc((unsigned)(unsigned short)v);
  else return __popc((unsigned)(unsigned char)v);
}
template <typename T>
RX_DEV int rx_clz(T v) {
  if constexpr (sizeof(T) == 8) return v == 0 ? 64 : __clzll((long long)v);
  else if constexpr (sizeof(T) == 4) return v == 0 ? 32 : __clz((int)v);
  else if constexpr (sizeof(T) == 2) return (unsigned short)v == 0 ? 16 : __clz((int)(unsigned)(unsigned short)v) - 16;
  else return (unsigned char)v == 0 ? 8 : __clz((int)(unsigned)(unsigned char)v) - 24;
}

struct rx_op_add { template <typename T> RX_MEM T operator()(T a, T b) const { return a + b; } };
struct rx_op_mul { template <typename T> RX_MEM T operator()(T a, T b) const { return a * b; } };
struct rx_op_div { template <typename T> RX_MEM T operator()(T a, T b) const { return a / b; } };
struct rx_op_max { template <typename T> RX_MEM T operator()(T a, T b) const { return rx_max(a, b); } };
struct rx_op_min { template <typename T> RX_MEM T operator()(T a, T b) const { return rx_min(a, b); } };
struct rx_op_and { template <typename T> RX_MEM T operator()(T a, T b) const { return (T)(a & b); } };
struct rx_op_or { template <typename T> RX_MEM T operator()(T a, T b) const { return (T)(a | b); } };

// Combine over the 64 lanes of a wavefront; the result is uniform.
// Rows of 16 lanes are folded with quad permutes and row mirrors, then the row
// totals travel down with row_bcast:15 / row_bcast:31 and lane 63 holds the total.
template <typename T, typename OP>
RX_DEV T rx_wave_reduce(T v, OP op) {
  v = op(v, rx_dpp_t<T, 0xB1, 0xf>(v));   // quad_perm [1,0,3,2]
  v = op(v, rx_dpp_t<T, 0x4E, 0xf>(v));   // quad_perm [2,3,0,1]
  v = op(v, rx_dpp_t<T, 0x141, 0xf>(v));  // row_half_mirror
  v = op(v, rx_dpp_t<T, 0x140, 0xf>(v));  // row_mirror: every lane holds its row total
  T t = rx_dpp_t<T, 0x142, 0xa>(v);       // row_bcast:15 into rows 1 and 3
  rx_u32 lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  if ((lane >> 4) & 1u) v = op(v, t);
  t = rx_dpp_t<T, 0x143, 0xc>(v);         // row_bcast:31 into rows 2 and 3
  if (lane >= 32u) v = op(v, t);
  return rx_readlane63(v);
}

// Value of lane (lane ^ 16): the one exchange that crosses rows of 16 lanes
template <typename T>
RX_DEV T rx_xor16(T v) {
  const rx_i32 addr = (rx_i32)(((__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u))) ^ 16u) << 2);
  if constexpr (sizeof(T) == 8) {
    rx_u64 u = __builtin_bit_cast(rx_u64, v);
    rx_u32 lo = (rx_u32)__builtin_amdgcn_ds_bpermute(addr, (rx_i32)(rx_u32)u);
    rx_u32 hi = (rx_u32)__builtin_amdgcn_ds_bpermute(addr, (rx_i32)(rx_u32)(u >> 32));
    return __builtin_bit_cast(T, ((rx_u64)hi << 32) | lo);
  } else if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, __builtin_amdgcn_ds_bpermute(addr, __builtin_bit_cast(rx_i32, v)));
  } else {
    return (T)__builtin_amdgcn_ds_bpermute(addr, (rx_i32)v);
  }
}
// Combine over aligned groups of W lanes (W a power of two up to 32); every lane of a group
// ends up with its group's result.  Groups of a wavefront are independent: a group whose lanes
// have all left the kernel is simply not there.
template <int W, typename T, typename OP>
RX_DEV T rx_group_reduce(T v, OP op) {
  static_assert(W == 1 || W == 2 || W == 4 || W == 8 || W == 16 || W == 32, "group width");
  if constexpr (W >= 2) v = op(v, rx_dpp_t<T, 0xB1, 0xf>(v));    // quad_perm [1,0,3,2]
  if constexpr (W >= 4) v = op(v, rx_dpp_t<T, 0x4E, 0xf>(v));    // quad_perm [2,3,0,1]
  if constexpr (W >= 8) v = op(v, rx_dpp_t<T, 0x141, 0xf>(v));   // row_half_mirror
  if constexpr (W >= 16) v = op(v, rx_dpp_t<T, 0x140, 0xf>(v));  // row_mirror
  if constexpr (W >= 32) v = op(v, rx_xor16(v));
  return v;
}

// Makes the compiler have `x` in a register at this point of the program (so whatever it was computed from can
// be dropped here, instead of the computation moving to where `x` is used).
template <typename T>
RX_DEV void rx_pin(T& x) {
  if constexpr (sizeof(T) == 4 || sizeof(T) == 8) asm volatile("" : "+v"(x));
}

// Value held by lane `src` (0..63) of this wavefront.
template <typename T>
RX_DEV T rx_lane_from(T v, rx_u32 src) {
  const rx_i32 addr = (rx_i32)(src << 2);
  if constexpr (sizeof(T) == 8) {
    rx_u64 u = __builtin_bit_cast(rx_u64, v);
    rx_u32 lo = (rx_u32)__builtin_amdgcn_ds_bpermute(addr, (rx_i32)(rx_u32)u);
    rx_u32 hi = (rx_u32)__builtin_amdgcn_ds_bpermute(addr, (rx_i32)(rx_u32)(u >> 32));
    return __builtin_bit_cast(T, ((rx_u64)hi << 32) | lo);
  } else if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, __builtin_amdgcn_ds_bpermute(addr, __builtin_bit_cast(rx_i32, v)));
  } else {
    return (T)__builtin_amdgcn_ds_bpermute(addr, (rx_i32)v);
  }
}
// Inclusive prefix combine over the 64 lanes of a wavefront (lane order).
template <typename T, typename OP>
RX_DEV T rx_wave_scan(T v, OP op) {
  const rx_u32 lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
#pragma unroll
  for (rx_u32 d = 1; d < 64u; d <<= 1) {
    const T t = rx_lane_from(v, (lane - d) & 63u);
    if (lane >= d) v = op(t, v);
  }
  return v;
}

// Combine over a workgroup of NWAVES wavefronts through LDS; result uniform.
template <typename T, typename OP, int NWAVES>
RX_DEV T rx_block_reduce(T v, OP op, T* lds /* NWAVES entries */) {
  v = rx_wave_reduce(v, op);
  if constexpr (NWAVES == 1) return v;
  const int w = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[w] = v;
  __syncthreads();
  T r = lds[0];
#pragma unroll
  for (int i = 1; i < NWAVES; ++i) r = op(r, lds[i]);
  return r;
}

// true for every thread of the workgroup if p is true for any of them (w: one word of LDS)
RX_DEV bool rx_block_any(bool p, int* w) {
  if (threadIdx.x == 0) *w = 0;
  __syncthreads();
  if (p) *w = 1;
  __syncthreads();
  const bool r = *w != 0;
  __syncthreads();
  return r;
}

// A workgroup's partial result handed to another workgroup of the same launch without a fence: the value travels in
// 32-bit pieces, each in the low half of a 64-bit word whose high half is a flag, and each word is written by one
// relaxed device-scope atomic store -- a reader that sees the flag sees the piece.  Slots are zero before the launch;
// the reader clears what it has read.  The wait is bounded (2^20 polls of about 1.5 us): no correct run exhausts it.
// A flag is a nonzero 32-bit epoch: readers that clear what they read use epoch 1 throughout; where a slot has several
// readers nothing is cleared, and the epoch changes from launch to launch instead.
template <typename T>
RX_DEV void rx_publish_partial(unsigned long long* slot, T v, rx_u32 epoch = 1u) {
  constexpr int NW = (sizeof(T) + 3) / 4;
  rx_u32 w[NW] = {};
  __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
  for (int k = 0; k < NW; ++k) __hip_atomic_store(slot + k, ((unsigned long long)epoch << 32) | w[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// the same wait for a partial that several workgroups read: the slot keeps its value.  `limit` polls (about 1.5 us each:
// 2^16 polls are about 0.1 s); a wait that expires sets the fault word (pinned host memory, checked by the host) and
// *bad, and continues with what the slot holds
template <typename T>
RX_DEV T rx_peek_partial(unsigned long long* slot, rx_u32 epoch, int limit, unsigned* fault, bool* bad) {
  constexpr int NW = (sizeof(T) + 3) / 4;
  rx_u32 w[NW];
#pragma unroll
  for (int k = 0; k < NW; ++k) {
    unsigned long long x = __hip_atomic_load(slot + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int spin = 0; (rx_u32)(x >> 32) != epoch && spin < limit; ++spin) {
      __builtin_amdgcn_s_sleep(2);
      x = __hip_atomic_load(slot + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if ((rx_u32)(x >> 32) != epoch) {
      __hip_atomic_store(fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      *bad = true;
    }
    w[k] = (rx_u32)x;
  }
  T v;
  __builtin_memcpy(&v, w, sizeof(T));
  return v;
}
template <typename T>
RX_DEV T rx_await_partial(unsigned long long* slot) {
  constexpr int NW = (sizeof(T) + 3) / 4;
  rx_u32 w[NW];
#pragma unroll
  for (int k = 0; k < NW; ++k) {
    unsigned long long x = __hip_atomic_load(slot + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int spin = 0; (x >> 32) == 0 && spin < (1 << 20); ++spin) {
      __builtin_amdgcn_s_sleep(2);
      x = __hip_atomic_load(slot + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    w[k] = (rx_u32)x;
    __hip_atomic_store(slot + k, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  T v;
  __builtin_memcpy(&v, w, sizeof(T));
  return v;
}

// Read-modify-write on one element in global memory (scatter with a combining update).  Sums of
// 32/64-bit integers and floats use the hardware atomics; everything else is a compare-and-swap
// loop on the 32- or 64-bit word (or, for 8/16-bit integers, on the aligned word that holds it).
template <typename T, typename OP>
RX_DEV void rx_atomic_rmw(T* p, T v, OP op) {
  if constexpr (sizeof(T) == 4) {
    rx_u32* w = (rx_u32*)p;
    rx_u32 old = __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), want;
    do {
      want = __builtin_bit_cast(rx_u32, (T)op(__builtin_bit_cast(T, old), v));
    } while (!__hip_atomic_compare_exchange_weak(w, &old, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  } else if constexpr (sizeof(T) == 8) {
    rx_u64* w = (rx_u64*)p;
    rx_u64 old = __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), want;
    do {
      want = __builtin_bit_cast(rx_u64, (T)op(__builtin_bit_cast(T, old), v));
    } while (!__hip_atomic_compare_exchange_weak(w, &old, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  } else {
    const unsigned long long addr = (unsigned long long)p;
    rx_u32* w = (rx_u32*)(addr & ~3ull);
    const unsigned shift = (unsigned)(addr & 3ull) * 8u;
    const rx_u32 mask = (sizeof(T) == 1 ? 0xffu : 0xffffu) << shift;
    rx_u32 old = __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), want;
    do {
      T cur;
      if constexpr (sizeof(T) == 1) cur = __builtin_bit_cast(T, (rx_u8)((old & mask) >> shift));
      else cur = __builtin_bit_cast(T, (rx_u16)((old & mask) >> shift));
      const T nv = (T)op(cur, v);
      rx_u32 bits;
      if constexpr (sizeof(T) == 1) bits = (rx_u32)__builtin_bit_cast(rx_u8, nv);
      else bits = (rx_u32)__builtin_bit_cast(rx_u16, nv);
      want = (old & ~mask) | (bits << shift);
    } while (!__hip_atomic_compare_exchange_weak(w, &old, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  }
}
template <typename T> RX_DEV void rx_atomic_add(T* p, T v) {
  if constexpr (sizeof(T) >= 4) (void)__hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else rx_atomic_rmw(p, v, rx_op_add());
}
template <typename T> RX_DEV void rx_atomic_mul(T* p, T v) { rx_atomic_rmw(p, v, rx_op_mul()); }
template <typename T> RX_DEV void rx_atomic_div(T* p, T v) { rx_atomic_rmw(p, v, rx_op_div()); }
template <typename T> RX_DEV void rx_atomic_max(T* p, T v) { rx_atomic_rmw(p, v, rx_op_max()); }
template <typename T> RX_DEV void rx_atomic_min(T* p, T v) { rx_atomic_rmw(p, v, rx_op_min()); }
template <typename T> RX_DEV void rx_atomic_and(T* p, T v) { rx_atomic_rmw(p, v, rx_op_and()); }
template <typename T> RX_DEV void rx_atomic_or(T* p, T v) { rx_atomic_rmw(p, v, rx_op_or()); }

// Workgroup barrier for data exchanged through LDS only: waits for this wavefront's LDS
// operations, not for its outstanding global loads (a __syncthreads() drains those too, which
// would serialize register prefetch with the compute phase that follows the barrier).
RX_DEV void rx_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// XCD-aware placement: workgroups are dealt round-robin to the 8 XCDs, each with
// its own L2.  This maps hardware workgroup id -> logical tile so that each XCD
// walks one contiguous range of tiles.
RX_DEV rx_u32 rx_xcd_remap(rx_u32 bid, rx_u32 nblocks) {
  const rx_u32 per = nblocks >> 3;
  const rx_u32 main = per << 3;
  if (bid >= main) return bid;
  return (bid & 7u) * per + (bid >> 3);
}

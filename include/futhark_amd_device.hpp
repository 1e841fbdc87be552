// Device-side building blocks shared by the gfx950 SegOp kernels: scalar
// operators, wave64 cross-lane primitives built on DPP, 128-bit memory access
// helpers and launch-side utilities.
//
// Scalar semantics follow rts/c/scalar.h of the reference: integer add wraps
// (scalar.h:29-30), smax/smin (scalar.h:488-503), float max/min ignore NaN like
// fmaxf/fminf (scalar.h:931-934).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <float.h>
#include <limits.h>
#include <math.h>
#include <type_traits>

#include "futhark_amd_kernels.h"

namespace fa {

constexpr int WAVE = 64;
constexpr int NUM_CUS_HINT = 256;  // MI355X: 8 XCDs x 32 CUs

// ---------------------------------------------------------------- operators

template <class T> struct OpAdd {
  static constexpr bool commutative = true;
  static __host__ __device__ __forceinline__ T identity() { return T(0); }
  static __host__ __device__ __forceinline__ T apply(T a, T b) {
    if constexpr (std::is_integral<T>::value) {
      using U = typename std::make_unsigned<T>::type;
      return (T)((U)a + (U)b);
    } else {
      return a + b;
    }
  }
};

template <class T> struct Limits;
template <> struct Limits<int32_t> {
  static __host__ __device__ int32_t lowest() { return INT32_MIN; }
  static __host__ __device__ int32_t highest() { return INT32_MAX; }
};
template <> struct Limits<int64_t> {
  static __host__ __device__ int64_t lowest() { return INT64_MIN; }
  static __host__ __device__ int64_t highest() { return INT64_MAX; }
};
template <> struct Limits<uint32_t> {
  static __host__ __device__ uint32_t lowest() { return 0u; }
  static __host__ __device__ uint32_t highest() { return UINT32_MAX; }
};
template <> struct Limits<uint64_t> {
  static __host__ __device__ uint64_t lowest() { return 0ull; }
  static __host__ __device__ uint64_t highest() { return UINT64_MAX; }
};
template <> struct Limits<float> {
  static __host__ __device__ float lowest() { return -INFINITY; }
  static __host__ __device__ float highest() { return INFINITY; }
};
template <> struct Limits<double> {
  static __host__ __device__ double lowest() { return -(double)INFINITY; }
  static __host__ __device__ double highest() { return (double)INFINITY; }
};

template <class T> struct OpMax {
  static constexpr bool commutative = true;
  static __host__ __device__ __forceinline__ T identity() { return Limits<T>::lowest(); }
  static __host__ __device__ __forceinline__ T apply(T a, T b) {
    if constexpr (std::is_same<T, float>::value) return fmaxf(a, b);
    else if constexpr (std::is_same<T, double>::value) return fmax(a, b);
    else return a < b ? b : a;
  }
};

template <class T> struct OpMin {
  static constexpr bool commutative = true;
  static __host__ __device__ __forceinline__ T identity() { return Limits<T>::highest(); }
  static __host__ __device__ __forceinline__ T apply(T a, T b) {
    if constexpr (std::is_same<T, float>::value) return fminf(a, b);
    else if constexpr (std::is_same<T, double>::value) return fmin(a, b);
    else return a < b ? a : b;
  }
};

// Bitwise operators, integer types only (rts/c/scalar.h:521-534).
template <class T> struct OpAnd {
  static_assert(std::is_integral<T>::value, "bitwise and: integers only");
  static constexpr bool commutative = true;
  static __host__ __device__ __forceinline__ T identity() { return (T)~(T)0; }
  static __host__ __device__ __forceinline__ T apply(T a, T b) { return a & b; }
};
template <class T> struct OpOr {
  static_assert(std::is_integral<T>::value, "bitwise or: integers only");
  static constexpr bool commutative = true;
  static __host__ __device__ __forceinline__ T identity() { return (T)0; }
  static __host__ __device__ __forceinline__ T apply(T a, T b) { return a | b; }
};
template <class T> struct OpXor {
  static_assert(std::is_integral<T>::value, "bitwise xor: integers only");
  static constexpr bool commutative = true;
  static __host__ __device__ __forceinline__ T identity() { return (T)0; }
  static __host__ __device__ __forceinline__ T apply(T a, T b) { return a ^ b; }
};

// x -> a*x + b modulo 2^32.  compose(f, g) is "f, then g": associative, not
// commutative, so a scan that swaps or reorders operands gives wrong results.
struct AffineI32 {
  int32_t a, b;
};
struct OpCompose {
  static constexpr bool commutative = false;
  static __host__ __device__ __forceinline__ AffineI32 identity() { return AffineI32{1, 0}; }
  static __host__ __device__ __forceinline__ AffineI32 apply(AffineI32 f, AffineI32 g) {
    return AffineI32{(int32_t)((uint32_t)f.a * (uint32_t)g.a),
                     (int32_t)((uint32_t)g.a * (uint32_t)f.b + (uint32_t)g.b)};
  }
};

// ------------------------------------------------------- bit reinterpretation

template <class To, class From>
__host__ __device__ __forceinline__ To bit_cast(const From &f) {
  static_assert(sizeof(To) == sizeof(From), "bit_cast size mismatch");
  To t;
  __builtin_memcpy(&t, &f, sizeof(To));
  return t;
}

// ------------------------------------------------------------ wave64 lanes

__device__ __forceinline__ int lane_id() {
  return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// DPP control words (GFX9 encoding).
constexpr int DPP_ROW_SHR1 = 0x111;
constexpr int DPP_ROW_SHR2 = 0x112;
constexpr int DPP_ROW_SHR4 = 0x114;
constexpr int DPP_ROW_SHR8 = 0x118;
constexpr int DPP_WAVE_SHR1 = 0x138;
constexpr int DPP_ROW_BCAST15 = 0x142;
constexpr int DPP_ROW_BCAST31 = 0x143;

// Move a value between lanes with a DPP control; lanes whose source is
// outside the pattern (or masked off by ROW_MASK) receive `old`.
template <int CTRL, int ROW_MASK, class T>
__device__ __forceinline__ T dpp_move(T old, T src) {
  if constexpr (sizeof(T) == 4) {
    int r = __builtin_amdgcn_update_dpp(bit_cast<int>(old), bit_cast<int>(src), CTRL,
                                        ROW_MASK, 0xf, false);
    return bit_cast<T>(r);
  } else {
    static_assert(sizeof(T) == 8, "dpp_move: 4- or 8-byte types only");
    uint64_t o = bit_cast<uint64_t>(old), s = bit_cast<uint64_t>(src);
    int lo = __builtin_amdgcn_update_dpp((int)(uint32_t)o, (int)(uint32_t)s, CTRL, ROW_MASK,
                                         0xf, false);
    int hi = __builtin_amdgcn_update_dpp((int)(uint32_t)(o >> 32), (int)(uint32_t)(s >> 32),
                                         CTRL, ROW_MASK, 0xf, false);
    uint64_t r = ((uint64_t)(uint32_t)hi << 32) | (uint32_t)lo;
    return bit_cast<T>(r);
  }
}

template <class T> __device__ __forceinline__ T read_lane(T v, int lane) {
  if constexpr (sizeof(T) == 4) {
    return bit_cast<T>(__builtin_amdgcn_readlane(bit_cast<int>(v), lane));
  } else {
    uint64_t s = bit_cast<uint64_t>(v);
    uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)s, lane);
    uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(s >> 32), lane);
    return bit_cast<T>(((uint64_t)hi << 32) | lo);
  }
}

// Inclusive scan over the 64 lanes of a wave; all lanes must be active.
// Four row_shr steps scan each row of 16 lanes, row_bcast15 joins rows into
// halves and row_bcast31 joins the halves.
template <class T, class Op> __device__ __forceinline__ T wave_incl_scan(T x) {
  const T id = Op::identity();
  x = Op::apply(dpp_move<DPP_ROW_SHR1, 0xf>(id, x), x);
  x = Op::apply(dpp_move<DPP_ROW_SHR2, 0xf>(id, x), x);
  x = Op::apply(dpp_move<DPP_ROW_SHR4, 0xf>(id, x), x);
  x = Op::apply(dpp_move<DPP_ROW_SHR8, 0xf>(id, x), x);
  x = Op::apply(dpp_move<DPP_ROW_BCAST15, 0xa>(id, x), x);
  x = Op::apply(dpp_move<DPP_ROW_BCAST31, 0xc>(id, x), x);
  return x;
}

// Value of the previous lane (identity in lane 0).
template <class T, class Op> __device__ __forceinline__ T wave_shift_up1(T x) {
  return dpp_move<DPP_WAVE_SHR1, 0xf>(Op::identity(), x);
}

// Reduction over the wave, result valid in every lane.
template <class T, class Op> __device__ __forceinline__ T wave_reduce(T x) {
  return read_lane(wave_incl_scan<T, Op>(x), 63);
}

// Segmented pair (flag, value) under the flag-tuple operator of
// Pass/Flatten/Builtins.hs:374-393.
template <class T> struct SegPair {
  T v;
  uint32_t f;
};

template <class T, class Op>
__device__ __forceinline__ SegPair<T> seg_apply(SegPair<T> a, SegPair<T> b) {
  SegPair<T> r;
  r.f = a.f | b.f;
  r.v = b.f ? b.v : Op::apply(a.v, b.v);
  return r;
}

template <int CTRL, int ROW_MASK, class T, class Op>
__device__ __forceinline__ SegPair<T> seg_dpp_step(SegPair<T> x) {
  SegPair<T> y;
  y.v = dpp_move<CTRL, ROW_MASK>(Op::identity(), x.v);
  y.f = dpp_move<CTRL, ROW_MASK>(0u, x.f);
  return seg_apply<T, Op>(y, x);
}

template <class T, class Op>
__device__ __forceinline__ SegPair<T> wave_incl_scan_seg(SegPair<T> x) {
  x = seg_dpp_step<DPP_ROW_SHR1, 0xf, T, Op>(x);
  x = seg_dpp_step<DPP_ROW_SHR2, 0xf, T, Op>(x);
  x = seg_dpp_step<DPP_ROW_SHR4, 0xf, T, Op>(x);
  x = seg_dpp_step<DPP_ROW_SHR8, 0xf, T, Op>(x);
  x = seg_dpp_step<DPP_ROW_BCAST15, 0xa, T, Op>(x);
  x = seg_dpp_step<DPP_ROW_BCAST31, 0xc, T, Op>(x);
  return x;
}

// ------------------------------------------------------------ 128-bit access

template <class T> struct Vec16 {
  static constexpr int N = 16 / sizeof(T);
  T e[N];
};

template <class T> __device__ __forceinline__ Vec16<T> load_vec16(const T *p) {
  uint4 raw = *reinterpret_cast<const uint4 *>(p);
  return bit_cast<Vec16<T>>(raw);
}

template <class T> __device__ __forceinline__ void store_vec16(T *p, const Vec16<T> &v) {
  *reinterpret_cast<uint4 *>(p) = bit_cast<uint4>(v);
}

// Non-temporal variants for data that is streamed exactly once.
template <class T> __device__ __forceinline__ Vec16<T> load_vec16_nt(const T *p) {
  using V4 = __attribute__((ext_vector_type(4))) uint32_t;
  V4 raw = __builtin_nontemporal_load(reinterpret_cast<const V4 *>(p));
  return bit_cast<Vec16<T>>(raw);
}

// Streaming stores: written once, not read again by the kernel.  Besides the
// non-temporal policy they carry the write-through scope bits (sc0 sc1), which
// the compiler's non-temporal store does not set; with them the segmented scan
// of 2^26 f32 takes 93.0 instead of 98.0 us, the scan of rows 81.9 instead of
// 87.6 us.  The instruction is followed by one idle issue slot, which a store
// of more than eight bytes needs before a vector instruction may overwrite its
// data registers (the compiler cannot see into the statement to add it).  For
// 4-byte stores (the C tile of the matmul) the extra bits change nothing.
template <class T> __device__ __forceinline__ void store_vec16_nt(T *p, const Vec16<T> &v) {
  using V4 = __attribute__((ext_vector_type(4))) uint32_t;
  const V4 raw = bit_cast<V4>(v);
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 0" ::"v"(p), "v"(raw) : "memory");
}
// ------------------------------------------------------------ device atomics
// Relaxed, agent-scope accesses for the look-back descriptors and counters.

__device__ __forceinline__ uint64_t ld_relaxed_u64(const uint64_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_relaxed_u64(uint64_t *p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ld_relaxed_u32(const uint32_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_relaxed_u32(uint32_t *p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ------------------------------------------------------------------- host

static inline bool is_aligned(const void *p, size_t a) { return ((uintptr_t)p % a) == 0; }

static inline __host__ __device__ int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Launch check: returns the positive hipError_t value on failure.
static inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

}  // namespace fa

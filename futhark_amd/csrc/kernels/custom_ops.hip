// Per-program operators: SegOps instantiated with operators and fused maps
// that are not in the library's fixed set, written against the public
// template header alone (include/futhark_amd_segops.hpp).  Each stands for
// what the reference's code generators emit when a program brings its own
// lambda:
//   * an operator over a tuple -- argmax over (value, index) pairs, reduce and
//     scan (tuples in SegBinOps: src/Futhark/IR/SegOp.hs:138-155);
//   * a map fused in front of a reduction -- reduce (+) 0 (map (\x -> x*x) xs),
//     and argmax over zip xs (iota n), where the pair is made on the way in;
//   * maps fused on both sides of a scan (the SegPostOp of
//     SegScan/SinglePass.hs:841-876) -- map sqrt (scan (+) 0 (map (\x -> x*x) xs));
//   * a reduction whose operator does not commute (SegRed.hs:836-921) --
//     composition of affine maps;
//   * reduce_by_index with a tuple operator, which has to lock its bins
//     (ImpGen/GPU/Base.hs:769-842) -- argmax per bin;
//   * the same operators in the segmented forms -- argmax and composition per
//     row (SegRed.hs:396-636), argmax scanned per row, argmax per irregular
//     segment (Pass/Flatten/Builtins.hs:570-602).
#include "futhark_amd_segops.hpp"

namespace {

using namespace fa;

// (value, index) under "the larger value wins, the smaller index among equal
// values": commutative and associative; neutral (lowest, highest).
struct ValIdx {
  int32_t v, i;
};
struct OpArgmax {
  static constexpr bool commutative = true;
  static __host__ __device__ __forceinline__ ValIdx identity() { return ValIdx{INT32_MIN, INT32_MAX}; }
  static __host__ __device__ __forceinline__ ValIdx apply(ValIdx a, ValIdx b) {
    const bool take_a = a.v > b.v || (a.v == b.v && a.i < b.i);
    return take_a ? a : b;
  }
};
struct ZipIndex {  // zip xs (iota n)
  static __device__ __forceinline__ ValIdx apply(int32_t x, int64_t i) { return ValIdx{x, (int32_t)i}; }
};
struct PairAsIs {
  static __device__ __forceinline__ ValIdx apply(ValIdx p, int64_t) { return p; }
};
struct AffineAsIs {
  static __device__ __forceinline__ AffineI32 apply(AffineI32 f, int64_t) { return f; }
};
struct SquareF32 {
  static __device__ __forceinline__ float apply(float x, int64_t) { return x * x; }
  static __device__ __forceinline__ float apply(float x) { return x * x; }
};
struct SqrtF32 {
  static __device__ __forceinline__ float apply(float x) { return __builtin_sqrtf(x); }
};

// The same operator on the {a, b} pair the locked histogram works with.
struct ValIdxAB {
  int32_t a, b;
};
struct OpArgmaxAB {
  static constexpr bool commutative = true;
  static __host__ __device__ __forceinline__ ValIdxAB identity() { return ValIdxAB{INT32_MIN, INT32_MAX}; }
  static __host__ __device__ __forceinline__ ValIdxAB apply(ValIdxAB x, ValIdxAB y) {
    const bool take_x = x.a > y.a || (x.a == y.a && x.b < y.b);
    return take_x ? x : y;
  }
};
struct ZipIndexAB {
  static __device__ __forceinline__ ValIdxAB apply(int32_t x, int64_t i) { return ValIdxAB{x, (int32_t)i}; }
};

// [H][2]i32 from the two component arrays.
__global__ void zip_pairs_kernel(const int32_t *a, const int32_t *b, int32_t *out, int64_t H) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < H) {
    out[2 * i] = a[i];
    out[2 * i + 1] = b[i];
  }
}
__global__ void unzip_pairs_kernel(const int32_t *in, int32_t *a, int32_t *b, int64_t H) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < H) {
    a[i] = in[2 * i];
    b[i] = in[2 * i + 1];
  }
}

}  // namespace

// Two operators in one SegRed (a reduction with several SegBinOps is one
// kernel in the reference too, SegRed.hs:157-199: the operators' accumulators
// sit side by side and every element is read once): sum and maximum of xs.
namespace {
struct SumMax {
  float sum, max;
};
struct OpSumMax {
  static constexpr bool commutative = true;
  static __host__ __device__ __forceinline__ SumMax identity() { return SumMax{0.0f, -INFINITY}; }
  static __host__ __device__ __forceinline__ SumMax apply(SumMax a, SumMax b) {
    return SumMax{a.sum + b.sum, OpMax<float>::apply(a.max, b.max)};
  }
};
struct Twice {
  static __device__ __forceinline__ SumMax apply(float x, int64_t) { return SumMax{x, x}; }
};
}  // namespace

extern "C" int fa_reduce_summax_f32(fa_stream_t stream, const float *xs, int64_t n, float *out2,
                                    void *scratch, size_t scratch_bytes, uint32_t epoch) {
  return launch_reduce<float, SumMax, Twice, OpSumMax>((hipStream_t)stream, xs, n, (SumMax *)out2,
                                                      scratch, scratch_bytes, epoch);
}

extern "C" int fa_reduce_argmax_i32(fa_stream_t stream, const int32_t *xs, int64_t n, int32_t *out2,
                                    void *scratch, size_t scratch_bytes, uint32_t epoch) {
  return launch_reduce<int32_t, ValIdx, ZipIndex, OpArgmax>((hipStream_t)stream, xs, n, (ValIdx *)out2,
                                                            scratch, scratch_bytes, epoch);
}

extern "C" int fa_reduce_compose_i32(fa_stream_t stream, const int32_t *abs, int64_t n, int32_t *out2,
                                     void *scratch, size_t scratch_bytes, uint32_t epoch) {
  if (!is_aligned(abs, 8)) return FA_EALIGN;
  return launch_reduce<AffineI32, AffineI32, AffineAsIs, OpCompose>(
      (hipStream_t)stream, (const AffineI32 *)abs, n, (AffineI32 *)out2, scratch, scratch_bytes, epoch);
}

extern "C" int fa_sumsq_f32(fa_stream_t stream, const float *xs, int64_t n, float *out,
                            void *scratch, size_t scratch_bytes, uint32_t epoch) {
  return launch_reduce<float, float, SquareF32, OpAdd<float>>((hipStream_t)stream, xs, n, out, scratch,
                                                              scratch_bytes, epoch);
}

extern "C" int fa_scan_argmax_i32(fa_stream_t stream, const int32_t *pairs, const uint8_t *flags,
                                  int64_t n, int exclusive, int32_t *out, void *scratch,
                                  size_t scratch_bytes, uint32_t epoch) {
  if (n < 0 || (n > 0 && (pairs == nullptr || out == nullptr || scratch == nullptr))) return FA_EINVAL;
  if (epoch == 0 || epoch >= (1u << 28)) return FA_EINVAL;
  return launch_scan<ValIdx, OpArgmax>((hipStream_t)stream, pairs, flags, (int64_t)0, n, exclusive, out,
                                       scratch, scratch_bytes, epoch);
}

extern "C" int fa_scan_norm_f32(fa_stream_t stream, const float *xs, int64_t n, float *out,
                                void *scratch, size_t scratch_bytes, uint32_t epoch) {
  if (n < 0 || (n > 0 && (xs == nullptr || out == nullptr || scratch == nullptr))) return FA_EINVAL;
  if (epoch == 0 || epoch >= (1u << 28)) return FA_EINVAL;
  return launch_scan<float, OpAdd<float>, SquareF32, SqrtF32>((hipStream_t)stream, xs, nullptr,
                                                              (int64_t)0, n, 0, out, scratch,
                                                              scratch_bytes, epoch);
}

// ---- the segmented forms with the same operators
// map (\row -> reduce argmax ne (zip row (iota k))) xss: a regular segmented
// reduction (SegRed.hs:396-636) with a tuple operator and the pair made on the
// way in; out: [m][2]i32.
extern "C" int fa_segreduce_argmax_i32(fa_stream_t stream, const int32_t *xss, int64_t m, int64_t k,
                                       int32_t *out) {
  return launch_segreduce<int32_t, ValIdx, ZipIndex, OpArgmax>((hipStream_t)stream, xss, m, k,
                                                               (ValIdx *)out);
}

// map (reduce compose (1, 0)) over rows of k affine maps: the operator does not
// commute, every row is folded in element order (SegRed.hs:836-921 per segment).
extern "C" int fa_segreduce_compose_i32(fa_stream_t stream, const int32_t *abss, int64_t m, int64_t k,
                                        int32_t *out) {
  if (!is_aligned(abss, 8) || !is_aligned(out, 8)) return FA_EALIGN;
  return launch_segreduce<AffineI32, AffineI32, AffineAsIs, OpCompose>(
      (hipStream_t)stream, (const AffineI32 *)abss, m, k, (AffineI32 *)out);
}

// map (scan argmax ne) over rows of k (value, index) pairs: the single-pass scan
// with segment starts computed from the row length (SegScan with segment
// dimensions, SegScan/SinglePass.hs:327-361).
extern "C" int fa_scanrows_argmax_i32(fa_stream_t stream, const int32_t *pairs, int64_t m, int64_t k,
                                      int32_t *out, void *scratch, size_t scratch_bytes,
                                      uint32_t epoch) {
  if (m < 0 || k < 0 || (m > 0 && k > INT64_MAX / m)) return FA_EINVAL;
  const int64_t n = m * k;
  if (n == 0) return 0;
  if (pairs == nullptr || out == nullptr || scratch == nullptr) return FA_EINVAL;
  if (epoch == 0 || epoch >= (1u << 28)) return FA_EINVAL;
  return launch_scan<ValIdx, OpArgmax>((hipStream_t)stream, pairs, nullptr, k, n, 0, out, scratch,
                                       scratch_bytes, epoch);
}

// Irregular segments (Pass/Flatten/Builtins.hs:570-602) with the tuple operator:
// out[i] = argmax over the pairs of segment i, the neutral pair when it is empty.
extern "C" size_t fa_segred_argmax_workspace_bytes(int64_t n) {
  return n < 0 ? 0 : segreduce_irregular_workspace_bytes<ValIdx>(n);
}
extern "C" int fa_segred_argmax_i32(fa_stream_t stream, const int64_t *offsets, const int64_t *lens,
                                    int64_t m, const int32_t *pairs, int64_t n, int32_t *out,
                                    void *workspace, size_t workspace_bytes, void *scratch,
                                    size_t scratch_bytes, uint32_t epoch) {
  if (epoch == 0 || epoch >= (1u << 28)) return FA_EINVAL;
  if (n > 0 && scratch == nullptr) return FA_EINVAL;
  return launch_segreduce_irregular<ValIdx, OpArgmax>(
      (hipStream_t)stream, offsets, lens, m, (const ValIdx *)pairs, n, (ValIdx *)out, workspace,
      workspace_bytes, scratch, scratch_bytes, epoch);
}

extern "C" size_t fa_hist_argmax_workspace_bytes(int64_t H) {
  if (H < 0) return 0;
  return (size_t)(3 * H) * 4 + 256;  // two component arrays and the lock words
}

// Bins beyond what a block's LDS holds are updated in place under locks in
// global memory; what bounds H is the 32-bit grid of the helper kernels.
extern "C" int64_t fa_hist_argmax_max_bins(void) { return (int64_t)1 << 31; }

// dest: [H][2]i32 (value, index) pairs, updated in place.
extern "C" int fa_hist_argmax_i32(fa_stream_t stream, const int32_t *is, const int32_t *xs, int64_t n,
                                  int32_t *dest, int64_t H, void *workspace, size_t workspace_bytes) {
  if (n < 0 || H < 0 || H > fa_hist_argmax_max_bins()) return FA_EINVAL;
  if (H == 0) return 0;
  if (dest == nullptr || workspace == nullptr || (n > 0 && (is == nullptr || xs == nullptr)))
    return FA_EINVAL;
  if (workspace_bytes < fa_hist_argmax_workspace_bytes(H)) return FA_ESCRATCH;
  hipStream_t st = (hipStream_t)stream;
  int32_t *a = (int32_t *)workspace, *b = a + H;
  uint32_t *locks = (uint32_t *)(b + H);
  const dim3 grid((unsigned)ceil_div(H, (int64_t)256));
  hipLaunchKernelGGL(unzip_pairs_kernel, grid, dim3(256), 0, st, dest, a, b, H);
  int rc = launch_status();
  if (rc != 0) return rc;
  rc = fa_replicate(stream, 4, locks, H, 0);
  if (rc != 0) return rc;
  rc = launch_hist_locked<int32_t, int32_t, int32_t, ValIdxAB, ZipIndexAB, OpArgmaxAB, int32_t>(
      st, is, xs, n, a, b, locks, H);
  if (rc != 0) return rc;
  hipLaunchKernelGGL(zip_pairs_kernel, grid, dim3(256), 0, st, a, b, dest, H);
  return launch_status();
}

// ===========================================================================
// SegOps inside a block (the reference's intra-block level,
// ImpGen/GPU/Block.hs:357-615: a SegRed, a SegScan and a SegMap over one row,
// all run by the threads of the block that owns the row, the row's values never
// leaving the CU between them):
//   map (\r -> let t = reduce (+) 0 r in map (/ t) (scan (+) 0 r)) xss
// One block per row at a time.  The row's sum is a block reduction; the scan
// walks the row in chunks of IB_CHUNK elements, four consecutive elements per
// thread, with a wave scan of the threads' sums, the waves' sums combined
// through LDS, and the carry of the chunks before kept by every thread.
constexpr int IB_BLOCK = 256;
constexpr int IB_VEC = 4;
constexpr int IB_CHUNK = IB_BLOCK * IB_VEC;

struct IbScan {
  float excl;   // sum of the values of the threads before this one
  float total;  // sum over the block
};
__device__ __forceinline__ IbScan ib_block_scan(float v, float *lds) {
  const int lane = lane_id(), wave = threadIdx.x / WAVE;
  const float incl = wave_incl_scan<float, OpAdd<float>>(v);
  const float excl = wave_shift_up1<float, OpAdd<float>>(incl);
  if (lane == WAVE - 1) lds[wave] = incl;
  __syncthreads();
  float before = 0.0f, total = 0.0f;
#pragma unroll
  for (int w = 0; w < IB_BLOCK / WAVE; w++) {
    const float s = lds[w];
    if (w < wave) before += s;
    total += s;
  }
  __syncthreads();  // lds is free again
  return IbScan{before + excl, total};
}

__global__ __launch_bounds__(IB_BLOCK) void rows_fraction_kernel(const float *__restrict__ xss,
                                                                 int64_t m, int64_t k,
                                                                 float *__restrict__ out) {
  __shared__ float lds[IB_BLOCK / WAVE];
  const bool vectors = k % IB_VEC == 0 && ((uintptr_t)xss | (uintptr_t)out) % 16 == 0;
  for (int64_t row = blockIdx.x; row < m; row += gridDim.x) {
    const float *r = xss + row * k;
    float *o = out + row * k;
    float part = 0.0f;
    if (vectors) {
      for (int64_t i = (int64_t)threadIdx.x * IB_VEC; i < k; i += IB_CHUNK) {
        const Vec16<float> v = load_vec16(r + i);
        part += (v.e[0] + v.e[1]) + (v.e[2] + v.e[3]);
      }
    } else {
      for (int64_t i = threadIdx.x; i < k; i += IB_BLOCK) part += r[i];
    }
    const float total = ib_block_scan(part, lds).total;
    float carry = 0.0f;
    for (int64_t c0 = 0; c0 < k; c0 += IB_CHUNK) {
      const int64_t i0 = c0 + (int64_t)threadIdx.x * IB_VEC;
      // the second read of the row comes from cache; rows of whole 16-byte
      // vectors are read and written as such
      const bool whole = vectors && i0 + IB_VEC <= k;
      float x[IB_VEC];
      if (whole) {
        const Vec16<float> v = load_vec16(r + i0);
#pragma unroll
        for (int e = 0; e < IB_VEC; e++) x[e] = v.e[e];
      } else {
#pragma unroll
        for (int e = 0; e < IB_VEC; e++) x[e] = i0 + e < k ? r[i0 + e] : 0.0f;
      }
#pragma unroll
      for (int e = 1; e < IB_VEC; e++) x[e] += x[e - 1];
      const IbScan s = ib_block_scan(x[IB_VEC - 1], lds);
      if (whole) {
        Vec16<float> v;
#pragma unroll
        for (int e = 0; e < IB_VEC; e++) v.e[e] = (carry + s.excl + x[e]) / total;
        store_vec16_nt(o + i0, v);
      } else {
#pragma unroll
        for (int e = 0; e < IB_VEC; e++)
          if (i0 + e < k) o[i0 + e] = (carry + s.excl + x[e]) / total;
      }
      carry += s.total;
    }
  }
}

// Rows of at most IB_WAVE_ROW_MAX elements: one wave per row, four rows to a
// block, no barrier at all (a block per 256-byte row spends its time in the
// four barriers of ib_block_scan: [2^20][64] took 833 us).
constexpr int IB_WAVE_ROW_MAX = 256;  // at 1024 the block kernel is faster (81 against 96 us for [65536][1024])
__global__ __launch_bounds__(IB_BLOCK) void rows_fraction_wave_kernel(const float *__restrict__ xss,
                                                                      int64_t m, int64_t k,
                                                                      float *__restrict__ out) {
  const int lane = lane_id();
  const int64_t waves = (int64_t)gridDim.x * (IB_BLOCK / WAVE);
  const bool vectors = k % IB_VEC == 0 && ((uintptr_t)xss | (uintptr_t)out) % 16 == 0;
  for (int64_t row = (int64_t)blockIdx.x * (IB_BLOCK / WAVE) + threadIdx.x / WAVE; row < m;
       row += waves) {
    const float *r = xss + row * k;
    float *o = out + row * k;
    // pass one: the row's sum; pass two: scan and divide (the row comes from cache)
    float part = 0.0f;
    for (int64_t i = (int64_t)lane * IB_VEC; i < k; i += WAVE * IB_VEC) {
#pragma unroll
      for (int e = 0; e < IB_VEC; e++) part += i + e < k ? r[i + e] : 0.0f;
    }
    const float total = read_lane(wave_incl_scan<float, OpAdd<float>>(part), WAVE - 1);
    float carry = 0.0f;
    for (int64_t c0 = 0; c0 < k; c0 += WAVE * IB_VEC) {
      const int64_t i0 = c0 + (int64_t)lane * IB_VEC;
      const bool whole = vectors && i0 + IB_VEC <= k;
      float x[IB_VEC];
      if (whole) {
        const Vec16<float> v = load_vec16(r + i0);
#pragma unroll
        for (int e = 0; e < IB_VEC; e++) x[e] = v.e[e];
      } else {
#pragma unroll
        for (int e = 0; e < IB_VEC; e++) x[e] = i0 + e < k ? r[i0 + e] : 0.0f;
      }
#pragma unroll
      for (int e = 1; e < IB_VEC; e++) x[e] += x[e - 1];
      const float incl = wave_incl_scan<float, OpAdd<float>>(x[IB_VEC - 1]);
      const float excl = wave_shift_up1<float, OpAdd<float>>(incl);
      if (whole) {
        Vec16<float> v;
#pragma unroll
        for (int e = 0; e < IB_VEC; e++) v.e[e] = (carry + excl + x[e]) / total;
        store_vec16_nt(o + i0, v);
      } else {
#pragma unroll
        for (int e = 0; e < IB_VEC; e++)
          if (i0 + e < k) o[i0 + e] = (carry + excl + x[e]) / total;
      }
      carry += read_lane(incl, WAVE - 1);
    }
  }
}

// Inclusive scan inside every group of LPR consecutive lanes (a power of two):
// the steps of the wave scan that stay inside a group.  Up to 16 lanes the row
// shifts must not cross into the group before; 32 and 64 lanes are whole rows
// of 16 joined by one or both broadcasts.
template <class T, class Op, int LPR>
__device__ __forceinline__ T lane_group_incl_scan(T x, int lane) {
  static_assert(LPR >= 1 && LPR <= WAVE && (LPR & (LPR - 1)) == 0, "a power of two");
  const T id = Op::identity();
  if constexpr (LPR >= 32) {
    x = Op::apply(dpp_move<DPP_ROW_SHR1, 0xf>(id, x), x);
    x = Op::apply(dpp_move<DPP_ROW_SHR2, 0xf>(id, x), x);
    x = Op::apply(dpp_move<DPP_ROW_SHR4, 0xf>(id, x), x);
    x = Op::apply(dpp_move<DPP_ROW_SHR8, 0xf>(id, x), x);
    x = Op::apply(dpp_move<DPP_ROW_BCAST15, 0xa>(id, x), x);
    if constexpr (LPR == 64) x = Op::apply(dpp_move<DPP_ROW_BCAST31, 0xc>(id, x), x);
  } else {
    const int j = lane & (LPR - 1);
    if constexpr (LPR > 1) {
      const T t = dpp_move<DPP_ROW_SHR1, 0xf>(id, x);
      x = j >= 1 ? Op::apply(t, x) : x;
    }
    if constexpr (LPR > 2) {
      const T t = dpp_move<DPP_ROW_SHR2, 0xf>(id, x);
      x = j >= 2 ? Op::apply(t, x) : x;
    }
    if constexpr (LPR > 4) {
      const T t = dpp_move<DPP_ROW_SHR4, 0xf>(id, x);
      x = j >= 4 ? Op::apply(t, x) : x;
    }
    if constexpr (LPR > 8) {
      const T t = dpp_move<DPP_ROW_SHR8, 0xf>(id, x);
      x = j >= 8 ? Op::apply(t, x) : x;
    }
  }
  return x;
}

// Rows of 4 LPR elements, LPR = 1, 2, ... 64 lanes per row: a wave-wide 16-byte
// load is 64 / LPR whole rows, each scanned by its group of lanes; the row's
// sum is the last lane's scan value, so the row is read once, and a wave has
// IB_PACKED_LOADS loads in flight.  ([2^20][64] f32 with a wave per row, the
// row read twice: 258 us.)
constexpr int IB_PACKED_LOADS = 4;
template <int LPR>
__global__ __launch_bounds__(IB_BLOCK) void rows_fraction_packed_kernel(const float *__restrict__ xss,
                                                                        int64_t m,
                                                                        float *__restrict__ out) {
  constexpr int G = WAVE / LPR;  // rows per load
  constexpr int U = IB_PACKED_LOADS;
  const int lane = lane_id();
  const int64_t n = m * (LPR * IB_VEC);
  const int64_t loads = ceil_div(m, (int64_t)G);
  const int64_t waves = (int64_t)gridDim.x * (IB_BLOCK / WAVE);
  for (int64_t l0 = ((int64_t)blockIdx.x * (IB_BLOCK / WAVE) + threadIdx.x / WAVE) * U; l0 < loads;
       l0 += waves * U) {
    Vec16<float> v[U];
    int64_t at[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      // rows are whole groups of lanes, so a group lies inside the array or
      // beyond it; lanes beyond load the first element and store nothing
      at[u] = ((l0 + u) * WAVE + lane) * IB_VEC;
      v[u] = load_vec16_nt(xss + (at[u] < n ? at[u] : 0));
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      float x[IB_VEC];
#pragma unroll
      for (int e = 0; e < IB_VEC; e++) x[e] = v[u].e[e];
#pragma unroll
      for (int e = 1; e < IB_VEC; e++) x[e] += x[e - 1];
      const float incl = lane_group_incl_scan<float, OpAdd<float>, LPR>(x[IB_VEC - 1], lane);
      float excl = wave_shift_up1<float, OpAdd<float>>(incl);
      if ((lane & (LPR - 1)) == 0) excl = 0.0f;
      const float total = __shfl(incl, lane | (LPR - 1), WAVE);
      Vec16<float> o;
#pragma unroll
      for (int e = 0; e < IB_VEC; e++) o.e[e] = (excl + x[e]) / total;
      if (at[u] < n) store_vec16_nt(out + at[u], o);
    }
  }
}

template <int LPR>
static int launch_rows_fraction_packed(hipStream_t st, const float *xss, int64_t m, float *out) {
  const int64_t loads = ceil_div(m, (int64_t)(WAVE / LPR));
  const int64_t blocks = ceil_div(loads, (int64_t)(IB_BLOCK / WAVE) * IB_PACKED_LOADS);
  const int64_t grid = blocks < 256 * 8 ? blocks : 256 * 8;
  hipLaunchKernelGGL(rows_fraction_packed_kernel<LPR>, dim3((unsigned)grid), dim3(IB_BLOCK), 0, st,
                     xss, m, out);
  return launch_status();
}

extern "C" int fa_rows_fraction_f32(fa_stream_t stream, const float *xss, int64_t m, int64_t k,
                                    float *out) {
  if (m < 0 || k < 0) return FA_EINVAL;
  if (m == 0 || k == 0) return 0;
  if (xss == nullptr || out == nullptr) return FA_EINVAL;
  if (k % IB_VEC == 0 && k <= WAVE * IB_VEC && (k & (k - 1)) == 0 &&
      ((uintptr_t)xss | (uintptr_t)out) % 16 == 0) {
    hipStream_t st = (hipStream_t)stream;
    switch ((int)(k / IB_VEC)) {
      case 1: return launch_rows_fraction_packed<1>(st, xss, m, out);
      case 2: return launch_rows_fraction_packed<2>(st, xss, m, out);
      case 4: return launch_rows_fraction_packed<4>(st, xss, m, out);
      case 8: return launch_rows_fraction_packed<8>(st, xss, m, out);
      case 16: return launch_rows_fraction_packed<16>(st, xss, m, out);
      case 32: return launch_rows_fraction_packed<32>(st, xss, m, out);
      default: return launch_rows_fraction_packed<64>(st, xss, m, out);
    }
  }
  if (k <= IB_WAVE_ROW_MAX) {
    const int64_t blocks = ceil_div(m, (int64_t)(IB_BLOCK / WAVE));
    const int64_t grid = blocks < 256 * 8 ? blocks : 256 * 8;
    hipLaunchKernelGGL(rows_fraction_wave_kernel, dim3((unsigned)grid), dim3(IB_BLOCK), 0,
                       (hipStream_t)stream, xss, m, k, out);
    return launch_status();
  }
  const int64_t grid = m < 256 * 8 ? m : 256 * 8;
  hipLaunchKernelGGL(rows_fraction_kernel, dim3((unsigned)grid), dim3(IB_BLOCK), 0,
                     (hipStream_t)stream, xss, m, k, out);
  return launch_status();
}

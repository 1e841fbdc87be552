// SegHist for gfx950: reduce_by_index with LDS-privatised sub-histograms.
//
// What is computed follows src/Futhark/CodeGen/ImpGen/GPU/SegHist.hs: for every
// element whose bin lies in [0,H) the destination bin is combined with the value
// (out-of-range bins are skipped, SegHist.hs:450-458,750-755); each block keeps
// sub-histograms in LDS, spreads threads over several copies of a bin to cut
// contention (SegHist.hs:654-656) and the copies are combined into the
// destination at the end (SegHist.hs:770-828,1137-1186).
//
// Measured on MI355X: device-scope atomics on HBM complete at about 27 G/s for
// scattered addresses and collapse under contention, while LDS atomics keep up
// with the HBM input stream.  So every element update is an LDS atomic:
//   * one block of 1024 threads per CU holds a bin range of up to 128 KiB in LDS
//     (up to 32768 four-byte bins);
//   * small ranges are replicated C times, copy index = lane mod C, laid out
//     bin-major ([bin][copy]) so the lanes of a wave hit distinct banks;
//   * H larger than one range is covered by P ranges in ONE launch: P blocks
//     that sit on the same XCD read the same input chunk at about the same time
//     (the second read is an L2 hit) and each keeps the updates of its range;
//   * blocks flush with coalesced device-scope atomics, skipping neutral bins.
// H beyond the multi-range limit (up to 255 ranges) first partitions the
// (index, value) pairs by bin range with one pass of the radix kernels (a
// stable ranked scatter, radix.hip.h), then runs LDS histograms over the
// partitions; out-of-range indices land in a partition that is never read.
// Only H beyond 255 ranges falls back to one device atomic per element.
//
// Sums of floats are the exception: the LDS f32 atomic runs at a third to a
// quarter of the integer rate.  f32 sums read the cell, add in a register and
// put the sum back with an integer compare-and-swap (lds_update); float sums
// keep twice the copies of a small range; [H0][m] bins of float vectors
// between 8 and 40 KiB are kept once per wave and updated with ordinary LDS
// reads and writes (seghist_wave_private_vec_kernel).
#include "radix.hip.h"

namespace fa {

// Choices of the float-sum paths (the measurements stand where each is used).
constexpr int HIST_CAS_FEW = 1;   // compare-and-swap attempts of an f32 sum before the float atomic ...
constexpr int HIST_CAS_MANY = 4;  // ... and where a bin has at least 2^HIST_CAS_MANY_COPIES_LOG2 copies
constexpr int HIST_CAS_MANY_COPIES_LOG2 = 2;
constexpr int HIST_COPY_BYTES = 32 * 1024;  // a bin range is replicated while its copies fit in this
constexpr int HIST_VEC_MIN_BYTES = 8192;    // bytes of cells up to which float vector bins stay with the LDS kernel
constexpr int HIST_VEC_UNROLL = 8;          // 16-byte loads a lane of the vector-bin kernel keeps in flight
constexpr int HIST_BLOCK = 1024;
constexpr int HIST_LDS_BYTES = 128 * 1024;  // bin storage per block
constexpr int HIST_MAX_RANGES = 4;          // ranges covered by one launch
constexpr int NUM_XCDS = 8;

// ------------------------------------------------------------ element types
// Bins of 8- and 16-bit element types are accumulated in LDS as 32-bit cells
// (integers sign- or zero-extended, f16 as f32): LDS atomics exist for 32 and 64
// bits only, and src/Futhark/CodeGen/ImpGen/GPU/Base.hs:735-767 with
// rts/c/atomics8.h / atomics16.h emulates the narrow ones by compare-and-swap on
// the containing word for every update.  Here only the flush of a bin to the
// destination does that.  For the integer operators the narrowed wide result
// equals the narrow evaluation (add wraps modulo 2^8 / 2^16 either way; max,
// min, and, or, xor commute with the extension); f16 sums are rounded once per
// block and bin instead of once per element.
template <class T> struct HistAcc { using A = T; };
template <> struct HistAcc<int8_t> { using A = int32_t; };
template <> struct HistAcc<uint8_t> { using A = uint32_t; };
template <> struct HistAcc<int16_t> { using A = int32_t; };
template <> struct HistAcc<uint16_t> { using A = uint32_t; };
template <> struct HistAcc<_Float16> { using A = float; };

template <class Op, class A> struct RebindOp;
template <class T, class A> struct RebindOp<OpAdd<T>, A> { using type = OpAdd<A>; };
template <class T, class A> struct RebindOp<OpMax<T>, A> { using type = OpMax<A>; };
template <class T, class A> struct RebindOp<OpMin<T>, A> { using type = OpMin<A>; };
template <class T, class A> struct RebindOp<OpAnd<T>, A> { using type = OpAnd<A>; };
template <class T, class A> struct RebindOp<OpOr<T>, A> { using type = OpOr<A>; };
template <class T, class A> struct RebindOp<OpXor<T>, A> { using type = OpXor<A>; };

// ------------------------------------------------------------ atomic updates
// `Scope` is __HIP_MEMORY_SCOPE_WORKGROUP for LDS and _AGENT for HBM.

template <class T> struct SameSizeInt;
template <> struct SameSizeInt<float> { using S = int32_t; using U = uint32_t; };
template <> struct SameSizeInt<double> { using S = int64_t; using U = uint64_t; };

template <class T, class Op, int Scope> struct AtomicUpdate;

template <class T, int Scope> struct AtomicUpdate<T, OpAdd<T>, Scope> {
  static __device__ __forceinline__ void apply(T *p, T v) {
    if constexpr (std::is_integral<T>::value) {
      using U = typename std::make_unsigned<T>::type;
      __hip_atomic_fetch_add(reinterpret_cast<U *>(p), (U)v, __ATOMIC_RELAXED, Scope);
    } else {
      __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, Scope);
    }
  }
};

// Float max/min through the integer view: non-negative floats order like signed
// integers, negative floats order inversely like unsigned integers.  NaN inputs
// are dropped (fmax(x, NaN) = x).  Valid while the cell itself is not NaN.
template <class T, int Scope, bool IS_MAX>
__device__ __forceinline__ void float_minmax_update(T *p, T v) {
  using S = typename SameSizeInt<T>::S;
  using U = typename SameSizeInt<T>::U;
  if (v != v) return;
  const S bits = bit_cast<S>(v);
  if (IS_MAX) {
    if (bits >= 0) __hip_atomic_fetch_max(reinterpret_cast<S *>(p), bits, __ATOMIC_RELAXED, Scope);
    else __hip_atomic_fetch_min(reinterpret_cast<U *>(p), (U)bits, __ATOMIC_RELAXED, Scope);
  } else {
    if (bits >= 0) __hip_atomic_fetch_min(reinterpret_cast<S *>(p), bits, __ATOMIC_RELAXED, Scope);
    else __hip_atomic_fetch_max(reinterpret_cast<U *>(p), (U)bits, __ATOMIC_RELAXED, Scope);
  }
}

template <class T, int Scope> struct AtomicUpdate<T, OpMax<T>, Scope> {
  static __device__ __forceinline__ void apply(T *p, T v) {
    if constexpr (std::is_integral<T>::value) __hip_atomic_fetch_max(p, v, __ATOMIC_RELAXED, Scope);
    else float_minmax_update<T, Scope, true>(p, v);
  }
};
template <class T, int Scope> struct AtomicUpdate<T, OpAnd<T>, Scope> {
  static __device__ __forceinline__ void apply(T *p, T v) {
    __hip_atomic_fetch_and(p, v, __ATOMIC_RELAXED, Scope);
  }
};
template <class T, int Scope> struct AtomicUpdate<T, OpOr<T>, Scope> {
  static __device__ __forceinline__ void apply(T *p, T v) {
    __hip_atomic_fetch_or(p, v, __ATOMIC_RELAXED, Scope);
  }
};
template <class T, int Scope> struct AtomicUpdate<T, OpXor<T>, Scope> {
  static __device__ __forceinline__ void apply(T *p, T v) {
    __hip_atomic_fetch_xor(p, v, __ATOMIC_RELAXED, Scope);
  }
};
template <class T, int Scope> struct AtomicUpdate<T, OpMin<T>, Scope> {
  static __device__ __forceinline__ void apply(T *p, T v) {
    if constexpr (std::is_integral<T>::value) __hip_atomic_fetch_min(p, v, __ATOMIC_RELAXED, Scope);
    else float_minmax_update<T, Scope, false>(p, v);
  }
};

// Update of a bin in LDS.  For max and min the cell is read first and the
// atomic issued only if the value would change it: bins are monotone, so a
// stale read can only cause a redundant atomic, and after the first few
// elements of a bin almost no update changes it (LDS atomics run at about a
// quarter of the rate of LDS reads).  NaN values never change a bin (fmax/fmin
// ignore them), and bins start from the identity, so they never hold NaN.
template <class T, class Op, int CAS = 0>
__device__ __forceinline__ void lds_update(T *p, T v) {
  constexpr bool minmax = std::is_same<Op, OpMax<T>>::value || std::is_same<Op, OpMin<T>>::value;
  if constexpr (CAS > 0) {
    // Sums of f32: the cell is read, the sum formed in a register and put back
    // with an integer compare-and-swap, which LDS runs at the rate of its
    // integer atomics; the float atomic, at a third of that rate, takes what
    // is left after CAS attempts (lanes of one wave on one cell: one of them
    // succeeds per attempt).
    static_assert(std::is_same<T, float>::value && std::is_same<Op, OpAdd<T>>::value, "f32 sums");
    uint32_t *q = reinterpret_cast<uint32_t *>(p);
    uint32_t seen = *reinterpret_cast<volatile uint32_t *>(q);
    bool done = false;
#pragma unroll
    for (int attempt = 0; attempt < CAS; attempt++) {
      if (!done) {
        const uint32_t want = bit_cast<uint32_t>(bit_cast<float>(seen) + v);
        done = __hip_atomic_compare_exchange_strong(q, &seen, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
    if (!done) AtomicUpdate<T, Op, __HIP_MEMORY_SCOPE_WORKGROUP>::apply(p, v);
  } else if constexpr (!minmax) {
    AtomicUpdate<T, Op, __HIP_MEMORY_SCOPE_WORKGROUP>::apply(p, v);
  } else {
    const T cur = *reinterpret_cast<volatile T *>(p);
    const bool changes = std::is_same<Op, OpMax<T>>::value ? (v > cur) : (v < cur);
    if (changes) AtomicUpdate<T, Op, __HIP_MEMORY_SCOPE_WORKGROUP>::apply(p, v);
  }
}

// The same for N cells at once (the elements of one step of a thread).  For max
// and min the reads of all cells are issued before any result is looked at, so
// that a step waits for LDS once instead of once per element (2^27 pairs into
// 65536 bins, f32 max: 344 -> 325 us; the waves were waiting on LDS round trips
// with LDS itself busy for under a tenth of the cycles).  Sums of f32 keep
// read, add, compare-and-swap together per element: with the reads of a step
// hoisted, other lanes get in between read and swap more often, more swaps fail
// and more updates end in the float atomic (256 bins: 172 -> 275 us).
// ok[e] says whether element e has a cell at all; p[e] must be readable either
// way.
template <class T, class Op, int CAS, int N>
__device__ __forceinline__ void lds_update_batch(T *const (&p)[N], const bool (&ok)[N], const T (&v)[N]) {
  constexpr bool minmax = std::is_same<Op, OpMax<T>>::value || std::is_same<Op, OpMin<T>>::value;
  if constexpr (minmax) {
    T cur[N];
#pragma unroll
    for (int e = 0; e < N; e++) cur[e] = *reinterpret_cast<volatile T *>(p[e]);
#pragma unroll
    for (int e = 0; e < N; e++) {
      const bool changes = std::is_same<Op, OpMax<T>>::value ? (v[e] > cur[e]) : (v[e] < cur[e]);
      if (ok[e] && changes) AtomicUpdate<T, Op, __HIP_MEMORY_SCOPE_WORKGROUP>::apply(p[e], v[e]);
    }
  } else {
#pragma unroll
    for (int e = 0; e < N; e++)
      if (ok[e]) lds_update<T, Op, CAS>(p[e], v[e]);
  }
}

// Update of a destination cell in HBM.  For float max/min the integer view is
// enough (one atomic without return) unless the cell holds a NaN, which fmax
// and fmin replace by the other operand
// (src/Futhark/CodeGen/ImpGen/GPU/Base.hs:844-905 uses a compare-and-swap loop
// on the operator for every update).  Nothing here ever writes a NaN, so a cell
// seen without one never holds one later; a cell seen with one goes through a
// compare-and-swap loop on the operator itself.
template <class T, class Op>
__device__ __forceinline__ void global_update(T *p, T v) {
  constexpr bool float_minmax =
      !std::is_integral<T>::value && (std::is_same<Op, OpMax<T>>::value || std::is_same<Op, OpMin<T>>::value);
  if constexpr (float_minmax) {
    using U = typename SameSizeInt<T>::U;
    U *q = reinterpret_cast<U *>(p);
    // An ordinary load is enough for the NaN test: a stale value can only be an
    // earlier one, i.e. show a NaN that is gone by now, never hide one.
    const T seen = *reinterpret_cast<const volatile T *>(p);
    if (seen == seen) {
      AtomicUpdate<T, Op, __HIP_MEMORY_SCOPE_AGENT>::apply(p, v);
      return;
    }
    U old = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    while (true) {
      const T want = Op::apply(bit_cast<T>(old), v);
      const U wbits = bit_cast<U>(want);
      if (wbits == old) break;
      if (__hip_atomic_compare_exchange_strong(q, &old, wbits, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT))
        break;
    }
  } else {
    AtomicUpdate<T, Op, __HIP_MEMORY_SCOPE_AGENT>::apply(p, v);
  }
}

// Destination cells narrower than 32 bits: compare-and-swap on the aligned word
// that contains the cell (rts/c/atomics8.h, atomics16.h do the same); `v` is
// the block's partial result in the accumulation type.
template <class T, class OpA, class A>
__device__ __forceinline__ void global_update_narrow(T *p, A v) {
  static_assert(sizeof(T) < 4, "narrow cells only");
  using B = typename std::conditional<sizeof(T) == 1, uint8_t, uint16_t>::type;
  const uintptr_t addr = reinterpret_cast<uintptr_t>(p);
  uint32_t *word = reinterpret_cast<uint32_t *>(addr & ~(uintptr_t)3);
  const int shift = (int)(addr & 3) * 8;
  const uint32_t mask = (uint32_t)(B)~(B)0 << shift;
  uint32_t old = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  while (true) {
    const T cur = bit_cast<T>((B)(old >> shift));
    const T want = (T)OpA::apply((A)cur, v);
    const uint32_t wbits = (old & ~mask) | ((uint32_t)bit_cast<B>(want) << shift);
    if (wbits == old) break;
    if (__hip_atomic_compare_exchange_strong(word, &old, wbits, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT))
      break;
  }
}

// Combines the partial result `acc` of a block into destination cell *p.
template <class T, class OpA, class A>
__device__ __forceinline__ void flush_bin(T *p, A acc) {
  if constexpr (sizeof(T) < 4) global_update_narrow<T, OpA, A>(p, acc);
  else global_update<T, OpA>(p, acc);
}

template <class T> __device__ __forceinline__ bool bits_equal(T a, T b) {
  if constexpr (sizeof(T) == 4) return bit_cast<uint32_t>(a) == bit_cast<uint32_t>(b);
  else return bit_cast<uint64_t>(a) == bit_cast<uint64_t>(b);
}

// The inputs are read once: non-temporal loads (H = 256, 2^27 elements: 186 ->
// 168 us; no change where several blocks share a chunk through L2).
__device__ __forceinline__ uint4 hist_load_nt(const uint4 *p) {
  using V4 = __attribute__((ext_vector_type(4))) uint32_t;
  return bit_cast<uint4>(__builtin_nontemporal_load(reinterpret_cast<const V4 *>(p)));
}

// Four consecutive elements with the widest loads that fit (src is aligned to
// 4 * sizeof(E) bytes).
template <class E> __device__ __forceinline__ void load_elems4(E (&dst)[4], const E *src) {
  if constexpr (sizeof(E) == 1) {
    const uint32_t raw = *reinterpret_cast<const uint32_t *>(src);
    __builtin_memcpy(dst, &raw, 4);
  } else if constexpr (sizeof(E) == 2) {
    const uint2 raw = *reinterpret_cast<const uint2 *>(src);
    __builtin_memcpy(dst, &raw, 8);
  } else {
    constexpr int NV = (int)(4 * sizeof(E) / 16);
    uint4 raw[NV];
#pragma unroll
    for (int q = 0; q < NV; q++) raw[q] = hist_load_nt(reinterpret_cast<const uint4 *>(src) + q);
    __builtin_memcpy(dst, raw, sizeof(raw));
  }
}

// ------------------------------------------------------------- LDS histogram
// Grid layout: block b sits on XCD b % 8.  j = b / 8; range p = j % P;
// chunk set s = (j / P) * 8 + b % 8 of S = gridDim.x / P sets.  The P blocks of
// one chunk set read the same elements, each keeping the bins of its range.
//
// SEGMENTED: the input is [m][seg_len] and every row has its own H_seg bins
// (`map (hist op ne H_seg) iss vss`, SegHist.hs:1057-1136 with segment
// dimensions): element p belongs to row p / seg_len and its bin b, if inside
// [0, H_seg), is bin row * H_seg + b of the m * H_seg = H bins of dest.  A
// thread keeps (row, column) of its current vector and advances them by the
// grid stride, so there is one division per thread, not per element.
//
// VECTOR: the operator works on whole vectors of seg_len elements
// (`reduce_by_index dest (map2 op) (replicate seg_len ne) is vss`, the HistOp
// with an operator shape, SegHist.hs:1057-1136; tests/hist/array.fut): vs is
// [n / seg_len][seg_len], is has one index per row, and element (r, c) goes
// to bin is[r] * seg_len + c when is[r] lies in [0, H_seg).
//
// PAIRS: two index arrays, is and js, address [H_seg][seg_len] bins
// (`reduce_by_index_2d`, prelude/soacs.fut:149-150): element p goes to bin
// is[p] * seg_len + js[p] when is[p] lies in [0, H_seg) and js[p] in [0, seg_len).
enum { HIST_PLAIN = 0, HIST_ROWS = 1, HIST_VECTOR = 2, HIST_PAIRS = 3 };

template <class T, class Op, class I, int MODE, int CAS = 0>
__global__ __launch_bounds__(HIST_BLOCK) void seghist_lds_kernel(
    const I *__restrict__ is, const I *__restrict__ js, const T *__restrict__ vs, int64_t n, T *dest,
    int64_t bin_base, int64_t H, int range_bins, int P, int log2_copies, int64_t seg_len,
    int64_t H_seg) {
  using A = typename HistAcc<T>::A;
  using OpA = typename RebindOp<Op, A>::type;
  extern __shared__ __align__(16) unsigned char s_raw[];
  A *sh = reinterpret_cast<A *>(s_raw);
  constexpr int VEC = 4;  // elements per thread per step

  const int b = blockIdx.x;
  const int j = b / NUM_XCDS;
  const int p = j % P;
  const int64_t S = gridDim.x / P;
  const int64_t s = (int64_t)(j / P) * NUM_XCDS + b % NUM_XCDS;
  const int64_t lo = bin_base + (int64_t)p * range_bins;
  int64_t hi = lo + range_bins;
  if (hi > bin_base + H) hi = bin_base + H;
  const int nb = (int)(hi > lo ? hi - lo : 0);
  const int C = 1 << log2_copies;
  const int cells = nb * C;

  for (int i = threadIdx.x; i < cells; i += HIST_BLOCK) sh[i] = OpA::identity();
  __syncthreads();

  const int copy = threadIdx.x & (C - 1);
  const int64_t nvec = n / VEC;
  const int64_t stride = S * HIST_BLOCK;
  auto update = [&](int64_t bin, T v) {
    const int64_t r = bin - lo;
    if ((uint64_t)r < (uint64_t)nb)
      lds_update<A, OpA, CAS>(&sh[((int)r << log2_copies) + copy], (A)v);
  };
  // (row, column) of every element is tracked
  constexpr bool SEGMENTED = MODE == HIST_ROWS || MODE == HIST_VECTOR;
  auto pair_bin = [&](int64_t i, int64_t j) -> int64_t {
    return (uint64_t)i < (uint64_t)H_seg && (uint64_t)j < (uint64_t)seg_len ? i * seg_len + j
                                                                           : (int64_t)-1;
  };
  // Bin of dest for (position, raw bin) in a histogram per row.
  auto seg_bin = [&](int64_t row, int64_t b) -> int64_t {
    return (uint64_t)b < (uint64_t)H_seg ? row * H_seg + b : (int64_t)-1;
  };
  if (nb > 0) {
    const int64_t i0 = s * HIST_BLOCK + threadIdx.x;
    int64_t row = 0, col = 0, row_step = 0, col_step = 0;
    if constexpr (SEGMENTED) {
      row = (i0 * VEC) / seg_len;
      col = (i0 * VEC) % seg_len;
      row_step = (stride * VEC) / seg_len;
      col_step = (stride * VEC) % seg_len;
    }
    // Loads are requested two steps ahead of their use, while earlier steps go
    // through LDS (the compiler may not move loads across the atomics): with
    // one 32-byte request per thread the block has 32 KiB in flight and a step
    // lasts a memory latency, whatever LDS does (2^27 pairs into 65536 bins:
    // i32 (+) 220 us, f32 max 341 us, the waves at a wait for 83 % of their
    // cycles and LDS busy for under 10 %).
    constexpr int NJ = MODE == HIST_PAIRS ? VEC : 1;
    struct Step {
      I bi[VEC], bj[NJ];
      T bv[VEC];
    };
    auto request = [&](int64_t at, Step &d) {
      if constexpr (MODE != HIST_VECTOR) load_elems4(d.bi, is + at * VEC);
      load_elems4(d.bv, vs + at * VEC);
      if constexpr (MODE == HIST_PAIRS) load_elems4(d.bj, js + at * VEC);
    };
    // One step: the elements of `st` through LDS.
    auto process = [&](const Step &st) {
      const I(&bi)[VEC] = st.bi;
      const I(&bj)[NJ] = st.bj;
      const T(&bv)[VEC] = st.bv;
      (void)bj;
      if constexpr (MODE == HIST_PAIRS) {
#pragma unroll
        for (int e = 0; e < VEC; e++) update(pair_bin((int64_t)bi[e], (int64_t)bj[e]), bv[e]);
      } else if constexpr (MODE == HIST_VECTOR) {
        int64_t r = row, c = col;
#pragma unroll
        for (int e = 0; e < VEC; e++) {
          while (c >= seg_len) {
            c -= seg_len;
            r++;
          }
          const int64_t b = (int64_t)is[r];
          update((uint64_t)b < (uint64_t)H_seg ? b * seg_len + c : (int64_t)-1, bv[e]);
          c++;
        }
        row += row_step;
        col += col_step;
        if (col >= seg_len) {
          col -= seg_len;
          row++;
        }
      } else if constexpr (SEGMENTED) {
        int64_t r = row, c = col;
#pragma unroll
        for (int e = 0; e < VEC; e++) {
          while (c >= seg_len) {  // at most once when seg_len >= VEC
            c -= seg_len;
            r++;
          }
          update(seg_bin(r, (int64_t)bi[e]), bv[e]);
          c++;
        }
        row += row_step;
        col += col_step;
        if (col >= seg_len) {
          col -= seg_len;
          row++;
        }
      } else {
        A *cell[VEC];
        bool ok[VEC];
        A val[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) {
          const int64_t r = (int64_t)bi[e] - lo;
          ok[e] = (uint64_t)r < (uint64_t)nb;
          cell[e] = &sh[((ok[e] ? (int)r : 0) << log2_copies) + copy];
          val[e] = (A)bv[e];
        }
        lds_update_batch<A, OpA, CAS, VEC>(cell, ok, val);
      }
    };
    // Only where a range has one copy of its bins: ranges small enough to be
    // replicated run at the rate of the LDS atomics, and there the extra
    // registers and moves cost 2 % (2^27 i32 pairs, 256 bins: 167 -> 171 us).
    if (log2_copies != 0) {
      for (int64_t i = i0; i < nvec; i += stride) {
        Step cur;
        request(i, cur);
        process(cur);
      }
    } else {
      // A request beyond the end repeats the last valid one (unconditional: a
      // load under a condition makes the compiler wait for all loads where the
      // paths meet) and is not processed.
      const int64_t last = nvec > 0 ? nvec - 1 : 0;
      auto clamped = [&](int64_t at) { return at < nvec ? at : last; };
      // Updates that wait for LDS (the read of max and min, the read and the
      // swap of an f32 sum) keep two steps' loads in flight, in two sets of
      // registers that take turns; updates that do not (integer atomics) keep
      // one: they run at the rate of the LDS atomics and the second set only
      // costs (2^27 pairs into 65536 bins, one / two steps ahead: i32 (+)
      // 199 / 238 us, f32 (+) 297 / 285, f32 max 324 / 316, i32 max 238 / 231).
      constexpr bool WAITS_FOR_LDS = CAS > 0 || std::is_same<OpA, OpMax<A>>::value ||
                                     std::is_same<OpA, OpMin<A>>::value;
      if constexpr (WAITS_FOR_LDS) {
        Step a, b;
        if (i0 < nvec) {
          request(i0, a);
          request(clamped(i0 + stride), b);
        }
        for (int64_t i = i0; i < nvec; i += 2 * stride) {
          Step cur = a;
          request(clamped(i + 2 * stride), a);
          process(cur);
          cur = b;
          request(clamped(i + 3 * stride), b);
          if (i + stride < nvec) process(cur);
        }
      } else {
        Step a;
        if (i0 < nvec) request(i0, a);
        for (int64_t i = i0; i < nvec; i += stride) {
          const Step cur = a;
          request(clamped(i + stride), a);
          process(cur);
        }
      }
    }
    if (s == 0) {
      const int64_t t = nvec * VEC + threadIdx.x;
      if (threadIdx.x < VEC && t < n) {
        if constexpr (MODE == HIST_PAIRS) {
          update(pair_bin((int64_t)is[t], (int64_t)js[t]), vs[t]);
        } else if constexpr (MODE == HIST_VECTOR) {
          const int64_t b = (int64_t)is[t / seg_len];
          update((uint64_t)b < (uint64_t)H_seg ? b * seg_len + t % seg_len : (int64_t)-1, vs[t]);
        } else if constexpr (SEGMENTED) {
          update(seg_bin(t / seg_len, (int64_t)is[t]), vs[t]);
        } else {
          update((int64_t)is[t], vs[t]);
        }
      }
    }
  }
  __syncthreads();

  // Flush: combine the copies of a bin in copy order, skip untouched bins.
  for (int r = threadIdx.x; r < nb; r += HIST_BLOCK) {
    A acc = sh[r << log2_copies];
    for (int c = 1; c < C; c++) acc = OpA::apply(acc, sh[(r << log2_copies) + c]);
    if (!bits_equal(acc, OpA::identity())) flush_bin<T, OpA, A>(dest + (lo - bin_base) + r, acc);
  }
}

template <class U> struct DigitBinRange {
  using Out = uint16_t;  // the bin inside its range: shift <= 15 bits
  uint64_t H;
  int shift;
  __device__ __forceinline__ uint16_t out(U key) const {
    return (uint16_t)((uint64_t)key & (((uint64_t)1 << shift) - 1));
  }
  __device__ __forceinline__ uint32_t operator()(U key, int) const {
    return (uint64_t)key < H ? (uint32_t)((uint64_t)key >> shift) : 255u;
  }
};

// Input: pairs grouped by bin range; range r starts at offs[r * num_tiles] (the
// digit-major offsets of the partition pass).  Of a pair's bin only the place
// inside its range is left, 16 bits (the range is known from where the pair
// lies), so a pair is 2 + sizeof(T) bytes.  Each block takes a contiguous chunk
// of the valid pairs and, for every range the chunk touches, accumulates in LDS
// and flushes.
template <class T, class Op>
__global__ __launch_bounds__(HIST_BLOCK) void seghist_part_kernel(
    const uint16_t *__restrict__ pis, const T *__restrict__ pvs, const uint32_t *__restrict__ offs,
    int64_t num_tiles, T *dest, int64_t H, int shift) {
  using U = uint16_t;
  using A = typename HistAcc<T>::A;
  using OpA = typename RebindOp<Op, A>::type;
  extern __shared__ __align__(16) unsigned char s_raw[];
  A *sh = reinterpret_cast<A *>(s_raw);
  __shared__ uint32_t s_start[RS_RADIX];
  if (threadIdx.x < RS_RADIX) s_start[threadIdx.x] = offs[(int64_t)threadIdx.x * num_tiles];
  __syncthreads();
  const int64_t n_valid = s_start[RS_RADIX - 1];
  const int64_t chunk = ceil_div(ceil_div(n_valid, (int64_t)gridDim.x), 4) * 4;
  const int64_t c0 = (int64_t)blockIdx.x * chunk;
  const int64_t c1 = c0 + chunk < n_valid ? c0 + chunk : n_valid;
  const int range_bins = 1 << shift;
  const int num_ranges = (int)((H + range_bins - 1) >> shift);
  for (int r = 0; r < num_ranges && c0 < c1; r++) {
    const int64_t r0 = s_start[r], r1 = s_start[r + 1];
    const int64_t lo = r0 > c0 ? r0 : c0, hi = r1 < c1 ? r1 : c1;
    if (lo >= hi) continue;  // uniform over the block
    const int64_t bin0 = (int64_t)r << shift;
    const int nb = (int)((H - bin0) < range_bins ? (H - bin0) : range_bins);
    for (int i = threadIdx.x; i < nb; i += HIST_BLOCK) sh[i] = OpA::identity();
    __syncthreads();
    // f32 sums: one compare-and-swap attempt before the float atomic (no copies here)
    constexpr int CAS = std::is_same<A, float>::value && std::is_same<OpA, OpAdd<A>>::value ? HIST_CAS_FEW : 0;
    auto update = [&](U b, T v) { lds_update<A, OpA, CAS>(&sh[(int)b], (A)v); };
    // [lo, hi) = loose elements up to a multiple of four, groups of four read
    // with 16-byte non-temporal loads (two groups of a thread in flight),
    // loose elements at the end.
    int64_t a = (lo + 3) & ~(int64_t)3;
    if (a > hi) a = hi;
    for (int64_t i = lo + threadIdx.x; i < a; i += HIST_BLOCK) update(pis[i], pvs[i]);
    const int64_t groups = (hi - a) / 4;
    int64_t g = threadIdx.x;
    for (; g + HIST_BLOCK < groups; g += 2 * HIST_BLOCK) {
      U b[2][4];
      T v[2][4];
#pragma unroll
      for (int q = 0; q < 2; q++) {
        load_elems4(b[q], pis + a + (g + q * HIST_BLOCK) * 4);
        load_elems4(v[q], pvs + a + (g + q * HIST_BLOCK) * 4);
      }
#pragma unroll
      for (int q = 0; q < 2; q++)
#pragma unroll
        for (int e = 0; e < 4; e++) update(b[q][e], v[q][e]);
    }
    if (g < groups) {
      U b[4];
      T v[4];
      load_elems4(b, pis + a + g * 4);
      load_elems4(v, pvs + a + g * 4);
#pragma unroll
      for (int e = 0; e < 4; e++) update(b[e], v[e]);
    }
    for (int64_t i = a + groups * 4 + threadIdx.x; i < hi; i += HIST_BLOCK) update(pis[i], pvs[i]);
    __syncthreads();
    for (int q = threadIdx.x; q < nb; q += HIST_BLOCK) {
      const A acc = sh[q];
      if (!bits_equal(acc, OpA::identity())) flush_bin<T, OpA, A>(dest + bin0 + q, acc);
    }
    __syncthreads();
  }
}

// Last resort (more than 255 bin ranges): one device-scope atomic per element.
template <class T, class Op, class I>
__global__ __launch_bounds__(256) void seghist_global_kernel(const I *__restrict__ is,
                                                             const T *__restrict__ vs, int64_t n,
                                                             T *dest, int64_t H) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    const int64_t bin = (int64_t)is[i];
    if ((uint64_t)bin < (uint64_t)H)
      flush_bin<T, typename RebindOp<Op, typename HistAcc<T>::A>::type, typename HistAcc<T>::A>(
          dest + bin, (typename HistAcc<T>::A)vs[i]);
  }
}

// Most bins one LDS range holds for an accumulation type of `acc_bytes`
// (fa_tuning.hist_lds_bins_max counts 4-byte bins).
static int hist_range_bins_max(size_t acc_bytes) {
  fa_tuning t;
  fa_get_tuning(&t);
  const int64_t bytes = t.hist_lds_bins_max * 4;
  return (int)((bytes < HIST_LDS_BYTES ? bytes : HIST_LDS_BYTES) / (int64_t)acc_bytes);
}

static int hist_num_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    cus = NUM_CUS_HINT;
    if (hipGetDevice(&dev) == hipSuccess)
      (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  }
  return cus;
}

template <class T, class Op, class I, int MODE, int CAS>
static int launch_lds_kernel(hipStream_t st, int grid, size_t lds, const I *is, const I *js,
                             const T *vs, int64_t n, T *dest, int64_t H, int range_bins, int P,
                             int log2_copies, int64_t seg_len, int64_t H_seg) {
  auto kernel = seghist_lds_kernel<T, Op, I, MODE, CAS>;
  // Initialised once, under the lock C++ gives function-local statics.
  static const hipError_t raised = hipFuncSetAttribute(
      (const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, HIST_LDS_BYTES);
  if (raised != hipSuccess) return (int)raised;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(HIST_BLOCK), lds, st, is, js, vs, n, dest,
                     (int64_t)0, H, range_bins, P, log2_copies, seg_len, H_seg);
  return launch_status();
}

// Launches the LDS kernel over bins [0,H) of `dest` (H <= max ranges * range size).
template <class T, class Op, class I, int MODE = HIST_PLAIN>
static int launch_lds_hist(hipStream_t st, const I *is, const T *vs, int64_t n, T *dest,
                           int64_t H, int64_t seg_len = 0, int64_t H_seg = 0,
                           const I *js = nullptr) {
  using A = typename HistAcc<T>::A;
  const int max_range = hist_range_bins_max(sizeof(A));
  const int P = (int)ceil_div(H, max_range);
  const int range_bins = (int)ceil_div(H, P);
  // A small range is replicated while its copies fit in 32 KiB; float sums,
  // where every lane that meets another on a cell costs a failed
  // compare-and-swap (f32) or a slow atomic (f64), take 64 KiB, the most that
  // leaves two blocks on a CU (f32, Zipf indices, H = 1024 / 2048 / 4096: 314 /
  // 407 / 471 -> 218 / 301 / 390 us; f64 H = 256: 392 -> 250 us, which is also
  // less than the 282 us of a kernel that kept a histogram per wave and is
  // gone; integer sums gain nothing from it).
  constexpr bool f32_sum = std::is_same<A, float>::value && std::is_same<Op, OpAdd<T>>::value;
  constexpr bool f64_sum = std::is_same<A, double>::value && std::is_same<Op, OpAdd<T>>::value;
  const int64_t copy_bytes = f32_sum || f64_sum ? 2 * HIST_COPY_BYTES : HIST_COPY_BYTES;
  int log2_copies = 0;
  while (log2_copies < 5 && (int64_t)range_bins * (2 << log2_copies) * (int64_t)sizeof(A) <= copy_bytes)
    log2_copies++;
  const size_t lds = (size_t)range_bins * sizeof(A) << log2_copies;
  // One block per CU when the range fills LDS, two when two fit.
  const int per_cu = lds * 2 + 4096 <= 160 * 1024 ? 2 : 1;
  int grid = hist_num_cus() * per_cu;
  grid -= grid % (NUM_XCDS * P);
  if (grid < NUM_XCDS * P) grid = NUM_XCDS * P;
  if constexpr (f32_sum) {
    // f32 sums go through compare-and-swap: several attempts where a bin has
    // many copies (lanes that meet on a cell are few), one where it has not
    if (log2_copies >= HIST_CAS_MANY_COPIES_LOG2)
      return launch_lds_kernel<T, Op, I, MODE, HIST_CAS_MANY>(st, grid, lds, is, js, vs, n, dest, H,
                                                             range_bins, P, log2_copies, seg_len, H_seg);
    return launch_lds_kernel<T, Op, I, MODE, HIST_CAS_FEW>(st, grid, lds, is, js, vs, n, dest, H,
                                                          range_bins, P, log2_copies, seg_len, H_seg);
  }
  return launch_lds_kernel<T, Op, I, MODE, 0>(st, grid, lds, is, js, vs, n, dest, H, range_bins, P,
                                              log2_copies, seg_len, H_seg);
}

// ------------------------------- float sums into few bins that are vectors
// `reduce_by_index dest (map2 (+)) (replicate m 0) is vss` with float elements:
// every wave keeps a histogram of its own in LDS and updates it with ordinary
// reads and writes (LDS operations of one wave complete in order); the four
// histograms of a block are combined at the end and flushed with one device
// atomic per non-zero cell.  A lane takes 16 bytes of a row of vss at a time (m is a multiple of that), so the
// lanes of a step cover consecutive rows; rows of one step with the same index
// are told apart by the tag of the bin (the row number's low byte, written by
// every lane of the row and read back): the row whose tag stayed adds its
// vector with ordinary 16-byte reads and writes, the other rows follow with
// the LDS float atomic.  Blocks of four waves, so that a wave's histogram may
// take up to 40 KiB (H0 * m <= 10 Ki cells of 4 bytes).
constexpr int HIST_VEC_BLOCK = 256;
constexpr int HIST_VEC_LDS_MAX = 160 * 1024;

template <class T, class I>
__global__ __launch_bounds__(HIST_VEC_BLOCK) void seghist_wave_private_vec_kernel(
    const I *__restrict__ is, const T *__restrict__ vss, int64_t n_groups, T *dest, int64_t H0,
    int64_t m) {
  constexpr int G = 16 / (int)sizeof(T);  // elements of a lane per step
  constexpr int WAVES = HIST_VEC_BLOCK / WAVE;
  constexpr int U = HIST_VEC_UNROLL;  // steps of a lane whose loads are in flight together
  using VT = T __attribute__((ext_vector_type(G)));
  extern __shared__ __align__(16) unsigned char s_raw[];
  T *sh = reinterpret_cast<T *>(s_raw);
  const int cells = (int)(H0 * m);
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / WAVE));
  for (int i = threadIdx.x; i < cells * WAVES; i += HIST_VEC_BLOCK) sh[i] = T(0);
  __syncthreads();
  // volatile: the order of the LDS operations below is the algorithm
  volatile T *mine = sh + (size_t)wave * cells;
  volatile uint8_t *tags =
      reinterpret_cast<uint8_t *>(sh + (size_t)WAVES * cells) + (size_t)wave * H0;

  auto add_row_part = [&](bool in, I index, int64_t row, int col, const VT &v) {
    const bool valid = in && (uint64_t)(int64_t)index < (uint64_t)H0;
    const uint32_t bin = valid ? (uint32_t)index : 0u;
    // rows of one step are consecutive and at most 64: the low byte tells them apart
    const uint8_t tag = (uint8_t)row;
    if (valid) tags[bin] = tag;
    __builtin_amdgcn_wave_barrier();
    const bool first = valid && tags[bin] == tag;
    const uint32_t cell = bin * (uint32_t)m + (uint32_t)col;
    if (first) {
      volatile VT *p = reinterpret_cast<volatile VT *>(mine + cell);
      const VT old = *p;
      *p = old + v;
    }
    __builtin_amdgcn_wave_barrier();
    if (valid && !first) {
#pragma unroll
      for (int e = 0; e < G; e++)
        AtomicUpdate<T, OpAdd<T>, __HIP_MEMORY_SCOPE_WORKGROUP>::apply(
            const_cast<T *>(&mine[cell + e]), v[e]);
    }
    __builtin_amdgcn_wave_barrier();
  };

  // group g = elements [g * G, g * G + G) of vss, inside row g * G / m.  A lane
  // takes groups g0, g0 + stride, ... in batches of U whose loads are issued a
  // batch ahead, without a condition (a group past the end reads the last one
  // again and is dropped): loads under a condition would make every batch wait
  // for all that are in flight.
  struct Batch {
    VT v[U];
    I index[U];
    int64_t row[U];
    int col[U];
  };
  const int64_t stride = (int64_t)gridDim.x * HIST_VEC_BLOCK;
  const int64_t last_group = n_groups - 1, last_row = last_group * G / m;
  int64_t next = (int64_t)blockIdx.x * HIST_VEC_BLOCK + threadIdx.x;  // first group not fetched yet
  int64_t row = next * G / m;
  int col = (int)(next * G % m);
  const int64_t row_step = stride * G / m;
  const int col_step = (int)(stride * G % m);
  auto fetch = [&](Batch &b) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int64_t g = next < last_group ? next : last_group;
      b.v[u] = bit_cast<VT>(hist_load_nt(reinterpret_cast<const uint4 *>(vss) + g));
      b.index[u] = is[row < last_row ? row : last_row];
      b.row[u] = row;
      b.col[u] = col;
      next += stride;
      row += row_step;
      col += col_step;
      if (col >= (int)m) {
        col -= (int)m;
        row++;
      }
    }
  };
  int64_t g = next;  // first group of the batch in `cur`
  Batch cur;
  fetch(cur);
  while (g < n_groups) {
    Batch ahead;
    fetch(ahead);
    __builtin_amdgcn_sched_barrier(0);  // keep the loads above what follows
#pragma unroll
    for (int u = 0; u < U; u++)
      add_row_part(g + u * stride < n_groups, cur.index[u], cur.row[u], cur.col[u], cur.v[u]);
    cur = ahead;
    g += U * stride;
  }
  __syncthreads();
  for (int c = threadIdx.x; c < cells; c += HIST_VEC_BLOCK) {
    T acc = T(0);
#pragma unroll
    for (int w = 0; w < WAVES; w++) acc += sh[(size_t)w * cells + c];
    if (!bits_equal(acc, T(0))) global_update<T, OpAdd<T>>(dest + c, acc);
  }
}

// Bytes of LDS a block of seghist_wave_private_vec_kernel needs for [H0][m]
// bins, or 0 when the kernel does not take them.
template <class T> static size_t hist_vec_lds_bytes(int64_t H0, int64_t m) {
  constexpr int64_t G = 16 / (int64_t)sizeof(T);
  if (m % G != 0 || H0 > HIST_VEC_LDS_MAX || m > HIST_VEC_LDS_MAX) return 0;
  const size_t bytes =
      (size_t)(HIST_VEC_BLOCK / WAVE) * ((size_t)H0 * (size_t)m * sizeof(T) + (size_t)H0);
  return bytes <= (size_t)HIST_VEC_LDS_MAX ? (bytes + 15) & ~(size_t)15 : 0;
}

template <class T, class I>
static int launch_wave_private_vec_hist(hipStream_t st, const I *is, const T *vss,
                                        int64_t n_updates, T *dest, int64_t H0, int64_t m) {
  const size_t lds = hist_vec_lds_bytes<T>(H0, m);
  if (lds == 0) return FA_EINVAL;
  const int64_t n_groups = n_updates * m / (16 / (int64_t)sizeof(T));
  int per_cu = (int)((size_t)HIST_VEC_LDS_MAX / lds);
  if (per_cu > 8) per_cu = 8;
  const int64_t grid = std::min<int64_t>((int64_t)hist_num_cus() * per_cu,
                                         ceil_div(n_groups, (int64_t)HIST_VEC_BLOCK));
  auto kernel = seghist_wave_private_vec_kernel<T, I>;
  // Initialised once, under the lock C++ gives function-local statics.
  static const hipError_t raised = hipFuncSetAttribute(
      (const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, HIST_VEC_LDS_MAX);
  if (raised != hipSuccess) return (int)raised;
  hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(HIST_VEC_BLOCK), lds, st, is, vss, n_groups,
                     dest, H0, m);
  return launch_status();
}

// Elements per slice of the partitioned path (a multiple of every alignment).
// Shorter slices would let the partitioned pairs of one slice stay in the
// memory-side cache until they are read, but the fixed cost of four launches
// per slice outweighs that: 2^27 updates into 2^22 bins take 773 us in one
// slice, 781 us in two, 890 us in four, 1132 us in eight.
constexpr int64_t HIST_PART_SLICE = (int64_t)1 << 28;

template <class T> constexpr int hist_part_shift() {
  return sizeof(typename HistAcc<T>::A) == 4 ? 15 : 14;  // 128 KiB of bins per range
}

static size_t hist_align(size_t x) { return (x + 255) & ~(size_t)255; }

template <class T, class Op, class U>
static int launch_part_hist(hipStream_t st, const U *is, const T *vs, int64_t n, T *dest,
                            int64_t H, void *scratch, size_t scratch_bytes) {
  constexpr int shift = hist_part_shift<T>();
  const int64_t tiles = rs_num_tiles(n);
  const size_t rs_bytes = hist_align(rs_scratch_bytes(tiles, false));
  const size_t is_bytes = hist_align((size_t)n * sizeof(uint16_t));
  if (scratch_bytes < rs_bytes + is_bytes + (size_t)n * sizeof(T)) return FA_ESCRATCH;
  if (!is_aligned(scratch, 256)) return FA_EALIGN;
  uint16_t *pis = (uint16_t *)((char *)scratch + rs_bytes);
  T *pvs = (T *)((char *)scratch + rs_bytes + is_bytes);
  RsScratch sc = rs_carve(scratch, tiles, false);
  DigitBinRange<U> fn{(uint64_t)H, shift};
  int rc = rs_prepare(st, sc);
  if (rc != 0) return rc;
  rc = rs_pass<U, (int)sizeof(T)>(st, is, pis, vs, pvs, n, fn, 0, 1u, sc);
  if (rc != 0) return rc;
  auto kernel = seghist_part_kernel<T, Op>;
  // Initialised once, under the lock C++ gives function-local statics.
  static const hipError_t raised = hipFuncSetAttribute(
      (const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, HIST_LDS_BYTES);
  if (raised != hipSuccess) return (int)raised;
  hipLaunchKernelGGL(kernel, dim3(hist_num_cus()), dim3(HIST_BLOCK), HIST_LDS_BYTES, st, pis, pvs,
                     (const uint32_t *)sc.offsets, sc.tiles, dest, H, shift);
  return launch_status();
}

template <class T, class Op>
static int launch_hist(hipStream_t st, const void *is, int is64, const void *vs, int64_t n,
                       void *dest, int64_t H, void *scratch, size_t scratch_bytes) {
  if (H == 0 || n == 0) return 0;
  if (!is_aligned(is, 16) || !is_aligned(vs, 16) || !is_aligned(dest, sizeof(T))) return FA_EALIGN;
  const int64_t lds_limit =
      (int64_t)HIST_MAX_RANGES * hist_range_bins_max(sizeof(typename HistAcc<T>::A));
  if (H <= lds_limit) {
    if (is64) return launch_lds_hist<T, Op, int64_t>(st, (const int64_t *)is, (const T *)vs, n, (T *)dest, H);
    return launch_lds_hist<T, Op, int32_t>(st, (const int32_t *)is, (const T *)vs, n, (T *)dest, H);
  }
  const int64_t part_limit = (int64_t)255 << hist_part_shift<T>();
  if (H <= part_limit) {
    // Histograms of pieces of the input add up, so a long input goes through
    // in slices and the workspace is that of one slice.
    for (int64_t lo = 0; lo < n; lo += HIST_PART_SLICE) {
      const int64_t m = n - lo < HIST_PART_SLICE ? n - lo : HIST_PART_SLICE;
      const int rc =
          is64 ? launch_part_hist<T, Op, uint64_t>(st, (const uint64_t *)is + lo, (const T *)vs + lo,
                                                   m, (T *)dest, H, scratch, scratch_bytes)
               : launch_part_hist<T, Op, uint32_t>(st, (const uint32_t *)is + lo, (const T *)vs + lo,
                                                   m, (T *)dest, H, scratch, scratch_bytes);
      if (rc != 0) return rc;
    }
    return 0;
  }
  const int grid = hist_num_cus() * 8;
  if (is64)
    hipLaunchKernelGGL((seghist_global_kernel<T, Op, int64_t>), dim3(grid), dim3(256), 0, st,
                       (const int64_t *)is, (const T *)vs, n, (T *)dest, H);
  else
    hipLaunchKernelGGL((seghist_global_kernel<T, Op, int32_t>), dim3(grid), dim3(256), 0, st,
                       (const int32_t *)is, (const T *)vs, n, (T *)dest, H);
  return launch_status();
}

// Row-major bins of a segmented histogram for the paths that take plain
// indices: flat[p] = row(p) * H_seg + is[p], or -1 when is[p] is out of range.
template <class I>
__global__ __launch_bounds__(256) void seghist_flatten_kernel(const I *__restrict__ is, int64_t n,
                                                              int64_t seg_len, int64_t H_seg,
                                                              int64_t *__restrict__ flat) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x; p < n; p += stride) {
    const int64_t b = (int64_t)is[p];
    flat[p] = (uint64_t)b < (uint64_t)H_seg ? (p / seg_len) * H_seg + b : (int64_t)-1;
  }
}

template <class T, class Op>
static int launch_hist_segmented(hipStream_t st, const void *is, int is64, const void *vs,
                                 int64_t m, int64_t seg_len, void *dest, int64_t H_seg,
                                 void *scratch, size_t scratch_bytes) {
  const int64_t n = m * seg_len, H = m * H_seg;
  if (H == 0 || n == 0) return 0;
  if (!is_aligned(is, 16) || !is_aligned(vs, 16) || !is_aligned(dest, sizeof(T))) return FA_EALIGN;
  const int64_t lds_limit =
      (int64_t)HIST_MAX_RANGES * hist_range_bins_max(sizeof(typename HistAcc<T>::A));
  if (H <= lds_limit) {
    if (is64)
      return launch_lds_hist<T, Op, int64_t, HIST_ROWS>(st, (const int64_t *)is, (const T *)vs, n,
                                                   (T *)dest, H, seg_len, H_seg);
    return launch_lds_hist<T, Op, int32_t, HIST_ROWS>(st, (const int32_t *)is, (const T *)vs, n,
                                                 (T *)dest, H, seg_len, H_seg);
  }
  // Too many bins for one launch of LDS ranges: flatten the indices, then the
  // unsegmented paths.
  const size_t flat_bytes = hist_align((size_t)n * sizeof(int64_t));
  if (scratch_bytes < flat_bytes || !is_aligned(scratch, 256)) return FA_ESCRATCH;
  int64_t *flat = (int64_t *)scratch;
  const int grid = (int)std::min<int64_t>(ceil_div(n, (int64_t)256), (int64_t)hist_num_cus() * 16);
  if (is64)
    hipLaunchKernelGGL((seghist_flatten_kernel<int64_t>), dim3(grid), dim3(256), 0, st,
                       (const int64_t *)is, n, seg_len, H_seg, flat);
  else
    hipLaunchKernelGGL((seghist_flatten_kernel<int32_t>), dim3(grid), dim3(256), 0, st,
                       (const int32_t *)is, n, seg_len, H_seg, flat);
  const int rc = launch_status();
  if (rc != 0) return rc;
  return launch_hist<T, Op>(st, flat, 1, vs, n, dest, H, (char *)scratch + flat_bytes,
                            scratch_bytes - flat_bytes);
}

// Flat bins for a histogram over [H0][H1] bins of vectors of m elements:
// element e of vss belongs to update u = e / m and goes to bin
// ((is[u] * H1 + js[u]) * m + e % m), or nowhere (-1) when a coordinate is out
// of range.  js == nullptr stands for H1 = 1 and no second coordinate.
template <class I>
__global__ __launch_bounds__(256) void seghist_shape_kernel(const I *__restrict__ is,
                                                            const I *__restrict__ js, int64_t n,
                                                            int64_t H0, int64_t H1, int64_t m,
                                                            int64_t *__restrict__ flat) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < n; e += stride) {
    const int64_t u = e / m;
    const int64_t i = (int64_t)is[u], j = js != nullptr ? (int64_t)js[u] : 0;
    const bool inside = (uint64_t)i < (uint64_t)H0 && (uint64_t)j < (uint64_t)H1;
    flat[e] = inside ? (i * H1 + j) * m + e % m : (int64_t)-1;
  }
}

template <class T, class Op>
static int launch_hist_shaped(hipStream_t st, const void *is, const void *js, int is64,
                              const void *vss, int64_t n_updates, void *dest, int64_t H0,
                              int64_t H1, int64_t m, void *scratch, size_t scratch_bytes) {
  const int64_t n = n_updates * m, H = H0 * H1 * m;
  if (H == 0 || n == 0) return 0;
  if (!is_aligned(is, 16) || !is_aligned(vss, 16) || !is_aligned(dest, sizeof(T)) ||
      (js != nullptr && !is_aligned(js, 16)))
    return FA_EALIGN;
  const int64_t lds_limit =
      (int64_t)HIST_MAX_RANGES * hist_range_bins_max(sizeof(typename HistAcc<T>::A));
  if constexpr (std::is_same<Op, OpAdd<T>>::value && std::is_floating_point<T>::value) {
    // Sums of float vectors into few bins: a histogram per wave, no float atomic
    // per element.  Only above HIST_VEC_MIN_BYTES of cells: below, the LDS
    // kernel has eight or more copies of every cell, lanes rarely meet and its
    // update rarely waits (f32 [64][4] bins: 128 against 287 us; [16][64]: 125
    // against 148; [128][16]: 124 against 136; f64 [64][4]: 107 against 146 us;
    // above: f32 [192][16] 150 against 116 us, [256][16] 148 against 122,
    // [512][16] 236 against 194 in favour of this kernel).
    const bool many_cells = H * (int64_t)sizeof(T) > HIST_VEC_MIN_BYTES;
    if (many_cells && js == nullptr && m > 1 && hist_vec_lds_bytes<T>(H0, m) != 0) {
      if (is64)
        return launch_wave_private_vec_hist<T, int64_t>(st, (const int64_t *)is, (const T *)vss,
                                                        n_updates, (T *)dest, H0, m);
      return launch_wave_private_vec_hist<T, int32_t>(st, (const int32_t *)is, (const T *)vss,
                                                      n_updates, (T *)dest, H0, m);
    }
  }
  if (js == nullptr && m > 1 && H <= lds_limit) {  // one index per vector: no flat indices needed
    if (is64)
      return launch_lds_hist<T, Op, int64_t, HIST_VECTOR>(st, (const int64_t *)is, (const T *)vss,
                                                          n, (T *)dest, H, m, H0);
    return launch_lds_hist<T, Op, int32_t, HIST_VECTOR>(st, (const int32_t *)is, (const T *)vss, n,
                                                        (T *)dest, H, m, H0);
  }
  if (js == nullptr && m == 1)
    return launch_hist<T, Op>(st, is, is64, vss, n, dest, H, scratch, scratch_bytes);
  if (js != nullptr && m == 1 && H <= lds_limit) {  // index pairs: the bin is computed on the fly
    if (is64)
      return launch_lds_hist<T, Op, int64_t, HIST_PAIRS>(st, (const int64_t *)is, (const T *)vss, n,
                                                         (T *)dest, H, H1, H0, (const int64_t *)js);
    return launch_lds_hist<T, Op, int32_t, HIST_PAIRS>(st, (const int32_t *)is, (const T *)vss, n,
                                                       (T *)dest, H, H1, H0, (const int32_t *)js);
  }
  const size_t flat_bytes = hist_align((size_t)n * sizeof(int64_t));
  if (scratch_bytes < flat_bytes || !is_aligned(scratch, 256)) return FA_ESCRATCH;
  int64_t *flat = (int64_t *)scratch;
  const int grid = (int)std::min<int64_t>(ceil_div(n, (int64_t)256), (int64_t)hist_num_cus() * 16);
  if (is64)
    hipLaunchKernelGGL((seghist_shape_kernel<int64_t>), dim3(grid), dim3(256), 0, st,
                       (const int64_t *)is, (const int64_t *)js, n, H0, H1, m, flat);
  else
    hipLaunchKernelGGL((seghist_shape_kernel<int32_t>), dim3(grid), dim3(256), 0, st,
                       (const int32_t *)is, (const int32_t *)js, n, H0, H1, m, flat);
  const int rc = launch_status();
  if (rc != 0) return rc;
  return launch_hist<T, Op>(st, flat, 1, vss, n, dest, H, (char *)scratch + flat_bytes,
                            scratch_bytes - flat_bytes);
}

}  // namespace fa

extern "C" size_t fa_seghist_scratch_bytes(fa_dtype t, int is64, int64_t n, int64_t H) {
  const size_t es = dtype_size(t);
  if (es == 0) return 0;
  const size_t as = es < 4 ? 4 : es;  // size of the accumulation type
  if (n < 0) n = 0;
  const int64_t lds_limit = (int64_t)HIST_MAX_RANGES * hist_range_bins_max(as);
  const int64_t part_limit = (int64_t)255 << (as == 4 ? 15 : 14);
  if (H <= lds_limit || H > part_limit) return 256;
  if (n > HIST_PART_SLICE) n = HIST_PART_SLICE;
  (void)is64;  // the partitioned indices are 16 bits whatever the width of the input's
  return hist_align(rs_scratch_bytes(rs_num_tiles(n), false)) + hist_align((size_t)n * 2) +
         (size_t)n * es + 256;
}

extern "C" int fa_seghist(fa_stream_t stream, fa_dtype t, fa_op op, const void *is, int is64,
                          const void *vs, int64_t n, void *dest, int64_t H, void *scratch,
                          size_t scratch_bytes) {
  if (n < 0 || H < 0 || (H > 0 && dest == nullptr) || (n > 0 && (is == nullptr || vs == nullptr)))
    return FA_EINVAL;
  hipStream_t s = (hipStream_t)stream;
#define FA_HIST_NARROW_INT(T)                                                                      \
  switch (op) {                                                                                    \
    case FA_ADD: return launch_hist<T, OpAdd<T>>(s, is, is64, vs, n, dest, H, scratch, scratch_bytes); \
    case FA_MAX: return launch_hist<T, OpMax<T>>(s, is, is64, vs, n, dest, H, scratch, scratch_bytes); \
    case FA_MIN: return launch_hist<T, OpMin<T>>(s, is, is64, vs, n, dest, H, scratch, scratch_bytes); \
    case FA_AND: return launch_hist<T, OpAnd<T>>(s, is, is64, vs, n, dest, H, scratch, scratch_bytes); \
    case FA_OR: return launch_hist<T, OpOr<T>>(s, is, is64, vs, n, dest, H, scratch, scratch_bytes);  \
    case FA_XOR: return launch_hist<T, OpXor<T>>(s, is, is64, vs, n, dest, H, scratch, scratch_bytes); \
    default: return FA_ENOTSUP;                                                                    \
  }
  switch (t) {
    case FA_I8: FA_HIST_NARROW_INT(int8_t)
    case FA_U8: FA_HIST_NARROW_INT(uint8_t)
    case FA_I16: FA_HIST_NARROW_INT(int16_t)
    case FA_U16: FA_HIST_NARROW_INT(uint16_t)
    case FA_F16:
      switch (op) {
        case FA_ADD: return launch_hist<_Float16, OpAdd<_Float16>>(s, is, is64, vs, n, dest, H, scratch, scratch_bytes);
        case FA_MAX: return launch_hist<_Float16, OpMax<_Float16>>(s, is, is64, vs, n, dest, H, scratch, scratch_bytes);
        case FA_MIN: return launch_hist<_Float16, OpMin<_Float16>>(s, is, is64, vs, n, dest, H, scratch, scratch_bytes);
        default: return FA_ENOTSUP;
      }
    case FA_BF16:
      return FA_ENOTSUP;
    default:
      break;
  }
#undef FA_HIST_NARROW_INT
  FA_DISPATCH_TYPE_OP(launch_hist, t, op, s, is, is64, vs, n, dest, H, scratch, scratch_bytes);
}

extern "C" size_t fa_seghist_segmented_scratch_bytes(fa_dtype t, int64_t m, int64_t seg_len,
                                                     int64_t H_seg) {
  if (m < 0 || seg_len < 0 || H_seg < 0) return 0;
  const int64_t n = m * seg_len;
  return hist_align((size_t)n * sizeof(int64_t)) + fa_seghist_scratch_bytes(t, 1, n, m * H_seg);
}

extern "C" int fa_seghist_segmented(fa_stream_t stream, fa_dtype t, fa_op op, const void *is,
                                    int is64, const void *vs, int64_t m, int64_t seg_len,
                                    void *dest, int64_t H_seg, void *scratch,
                                    size_t scratch_bytes) {
  if (m < 0 || seg_len < 0 || H_seg < 0) return FA_EINVAL;
  if (m > 0 && ((H_seg > 0 && dest == nullptr) || (seg_len > 0 && (is == nullptr || vs == nullptr))))
    return FA_EINVAL;
  // m * seg_len and m * H_seg must be representable
  if (m > 0 && (seg_len > INT64_MAX / m || H_seg > INT64_MAX / m)) return FA_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  switch (t) {
    case FA_I32: case FA_I64: case FA_F32: case FA_F64:
      break;
    default:
      return FA_ENOTSUP;
  }
  FA_DISPATCH_TYPE_OP(launch_hist_segmented, t, op, s, is, is64, vs, m, seg_len, dest, H_seg,
                      scratch, scratch_bytes);
}

extern "C" size_t fa_seghist_shaped_scratch_bytes(fa_dtype t, int is64, int64_t n_updates,
                                                  int64_t H0, int64_t H1, int64_t m) {
  if (n_updates < 0 || H0 < 0 || H1 < 0 || m < 0) return 0;
  const int64_t n = n_updates * m;
  return hist_align((size_t)n * sizeof(int64_t)) + fa_seghist_scratch_bytes(t, 1, n, H0 * H1 * m) +
         fa_seghist_scratch_bytes(t, is64, n, H0 * H1 * m);
}

extern "C" int fa_seghist_shaped(fa_stream_t stream, fa_dtype t, fa_op op, const void *is,
                                 const void *js, int is64, const void *vss, int64_t n_updates,
                                 void *dest, int64_t H0, int64_t H1, int64_t m, void *scratch,
                                 size_t scratch_bytes) {
  if (n_updates < 0 || H0 < 0 || H1 < 0 || m < 0) return FA_EINVAL;
  if (js == nullptr && H1 != 1) return FA_EINVAL;
  // H0 * H1 * m and n_updates * m must be representable
  if (H1 > 0 && H0 > INT64_MAX / H1) return FA_EINVAL;
  if (m > 0 && (H0 * H1 > INT64_MAX / m || n_updates > INT64_MAX / m)) return FA_EINVAL;
  if (H0 * H1 * m > 0 && dest == nullptr) return FA_EINVAL;
  if (n_updates * m > 0 && (is == nullptr || vss == nullptr)) return FA_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  switch (t) {
    case FA_I32: case FA_I64: case FA_F32: case FA_F64:
      break;
    default:
      return FA_ENOTSUP;
  }
  FA_DISPATCH_TYPE_OP(launch_hist_shaped, t, op, s, is, js, is64, vss, n_updates, dest, H0, H1, m,
                      scratch, scratch_bytes);
}

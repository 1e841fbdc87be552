// SegScan for gfx950: single-pass scan with decoupled look-back.
//
// What is computed follows src/Futhark/CodeGen/ImpGen/GPU/SegScan/SinglePass.hs
// (dynamic tile ids :443-461, tile aggregate/prefix publication with status
// X/A/P :128-131,625-777) and, for segments, the flag-tuple operator of
// src/Futhark/Pass/Flatten/Builtins.hs:374-393.  How it is computed is native
// to CDNA4:
//   * blocks stay on their CU and take tiles by ticket; tiles travel from HBM
//     straight into LDS two rounds ahead (global_load_lds_dwordx4);
//   * a thread scans 128 consecutive bytes one element after the other, so a
//     wave needs one DPP scan per tile; the LDS layout that makes this possible
//     costs no barrier, because every wave keeps to its own 8 KiB;
//   * a tile descriptor is a 64-bit word {value bits, epoch, segment flag,
//     status} written and read with single relaxed agent-scope accesses, so no
//     fence separates value and status.  8-byte element types use two such
//     words (low and high half), accepted only when both carry the same status;
//   * descriptors carry a launch epoch, so no kernel clears them between calls;
//   * a wave of its own looks back, one round behind the scan and one round
//     ahead of the stores, so nobody waits for a round trip between CUs;
//   * the waves of a block do not meet at barriers: they pass wave totals,
//     prefixes and tickets through small rings in LDS with progress counters,
//     so their load, compute and store phases drift apart and the CU's memory
//     pipeline always has work.
#include <stdlib.h>

#include <mutex>

#include "dispatch.hip.h"

namespace fa {

// Look-back windows are one descriptor per lane, 64 tiles.  Two or four per
// lane (128 or 256 tiles per round trip) measured slower on 2^26 f32 (93 ->
// 100 -> 121 us), narrower first windows (8, 16, 32 tiles) no faster.
//
// Cache policy, measured on 2^26 f32 with flags: values are loaded with the
// default policy (non-temporal: scan 93 -> 108 us), flag bytes non-temporal
// (default: 113 instead of 98 us), results stored non-temporal (default: 119).

constexpr uint32_t ST_X = 0;  // nothing published
constexpr uint32_t ST_A = 1;  // aggregate of the tile
constexpr uint32_t ST_P = 2;  // inclusive prefix up to the end of the tile

// Scratch: a header, then one descriptor per tile.  Header: 32-bit word 1
// counts the blocks that have left, word 16 is the epoch word of
// fa_segscan_static, and every 64th word (256 bytes apart, so that they sit in
// different memory channels) is a ticket counter: same-address atomics are
// performed one at a time, about 12 ns each on MI355X, and a channel that does
// little else slows every stream that crosses it.  Counter c hands out the
// tiles congruent to c modulo the number of counters in use; a block draws
// from counter (block index mod that number).  Every tile is handed out as
// long as at least that many blocks get to run at the same time, which the
// number (8) is small enough for: a block occupies one CU.
constexpr size_t SCAN_HEADER_BYTES = 8192;
constexpr int SCAN_MAX_COUNTERS = 8;
constexpr int SCAN_COUNTER_STRIDE = 64;  // in 32-bit words
constexpr size_t SCAN_DESC_BYTES = 16;

__device__ __forceinline__ uint32_t desc_meta(uint32_t epoch, uint32_t flag, uint32_t status) {
  return (epoch << 3) | ((flag & 1u) << 2) | status;
}

template <class T>
__device__ __forceinline__ void desc_publish(uint64_t *desc, int64_t tile, uint32_t epoch,
                                             uint32_t status, uint32_t flag, T v) {
  const uint32_t meta = desc_meta(epoch, flag, status);
  if constexpr (sizeof(T) == 4) {
    st_relaxed_u64(desc + 2 * tile, ((uint64_t)bit_cast<uint32_t>(v) << 32) | meta);
  } else {
    const uint64_t b = bit_cast<uint64_t>(v);
    st_relaxed_u64(desc + 2 * tile, ((b & 0xffffffffull) << 32) | meta);
    st_relaxed_u64(desc + 2 * tile + 1, ((b >> 32) << 32) | meta);
  }
}

// Reading a descriptor, in two steps so that a caller can request several
// before it examines the first.  desc_decode returns false while the tile has
// published nothing (for this epoch), or while the two halves of an 8-byte
// value belong to different publications.
struct DescWords {
  uint64_t w0, w1;
};
template <class T> __device__ __forceinline__ DescWords desc_load(const uint64_t *desc, int64_t tile) {
  DescWords d;
  d.w0 = ld_relaxed_u64(desc + 2 * tile);
  d.w1 = sizeof(T) == 4 ? 0ull : ld_relaxed_u64(desc + 2 * tile + 1);
  return d;
}
template <class T>
__device__ __forceinline__ bool desc_decode(const DescWords &d, uint32_t epoch, uint32_t &status,
                                            uint32_t &flag, T &v) {
  const uint32_t m0 = (uint32_t)d.w0;
  if ((m0 >> 3) != epoch || (m0 & 3u) == ST_X) return false;
  if constexpr (sizeof(T) == 4) {
    v = bit_cast<T>((uint32_t)(d.w0 >> 32));
  } else {
    if ((uint32_t)d.w1 != m0) return false;
    v = bit_cast<T>((d.w0 >> 32) | ((d.w1 >> 32) << 32));
  }
  status = m0 & 3u;
  flag = (m0 >> 2) & 1u;
  return true;
}

// Where segments come from: nowhere, a flag byte per element, or rows of equal
// length (`map (scan op ne) xss`: SegScan with segment dimensions,
// SegScan/SinglePass.hs:327-361 -- the reference tests whether two positions
// lie in the same row; here the row starts are computed from the element
// index, so there is no flag array to read).
enum { SEG_NONE = 0, SEG_FLAGS = 1, SEG_ROWS = 2 };

// ===========================================================================
// The kernel.
//
// A block has seven data waves and one protocol wave, and LDS holds two tile
// buffers.  Call the block's q-th tile "tile q".  Nothing waits for something
// requested in the same round:
//   * tile q's bytes (values, and flag bytes of a flag-driven scan) are
//     requested in round q-2, straight from HBM into LDS;
//   * in round q a data wave scans its part of tile q locally and leaves the
//     results in registers; the protocol wave publishes the tile's aggregate;
//   * in round q+1 the protocol wave looks back for the tile's prefix -- its
//     predecessors published their aggregates a round ago, so it finds them;
//   * in round q+2 the data waves complete tile q with that prefix and store it.
//
// Data waves: inside a tile every wave owns 8 KiB of values (and the flag
// bytes that go with them).
//   * It fetches them itself, eight 1 KiB instructions, in a layout that gives
//     each thread 128 consecutive bytes -- 32 four-byte or 16 eight-byte
//     elements.
//   * The results go through the same LDS bytes (free once the tile is in
//     registers) and leave in 1 KiB instructions again.  Only the owning wave
//     ever touches these bytes.
//   * Its only vector memory operations are those loads and stores, so it can
//     wait for exactly the loads it needs by count (vector memory operations
//     of a wave complete in issue order).
// Protocol wave: draws the tickets, publishes aggregates and prefixes, looks
// back.  It moves no data, so its descriptor reads never queue behind bulk
// loads.  A ticket is drawn at the end of a round and used a round later, so
// the atomic's round trip is not waited for either.
//
// The waves talk through rings in LDS (slot = tile number mod 8) with
// monotonic progress counters: a data wave's count of tiles whose wave total
// it has written, the protocol wave's counts of prefixes and of tickets handed
// out.  A reader spins on the counter (rarely: everything is produced a round
// before it is needed).  Eight slots are enough: a data wave enters round q+8
// only after it has completed tile q+5, whose prefix exists only once every
// wave has scanned tile q+5, i.e. is past everything that reads slot q.
//
// LDS layout of the values: thread i owns bytes [128 i, 128 i + 128) of a
// buffer; its k-th 16-byte unit sits in slot k ^ ((i >> 1) & 7), which makes
// the 16 lanes of one phase of a 128-bit access hit all 64 banks once.  A
// 1 KiB instruction (lane l at byte 16 l of LDS block m) thus moves, for
// thread 8 m + (l >> 3), unit (l & 7) ^ ((4 m + (l >> 4)) & 7): a permutation
// inside one 128-byte line of global memory, so global accesses stay whole
// lines.  Flag bytes: thread i owns EPT consecutive bytes; with 32 of them the
// two 16-byte halves are swapped for threads with bit 3 set, for the same reason.
constexpr int SS_WAVES = 7;                                       // data waves
constexpr int SS_DATA_THREADS = SS_WAVES * WAVE;
constexpr int SS_BLOCK = SS_DATA_THREADS + WAVE;                  // + the protocol wave
constexpr int SS_THREAD_BYTES = 128;
constexpr int SS_UNITS = SS_THREAD_BYTES / 16;                    // 16-byte units per thread
constexpr int SS_WAVE_BYTES = WAVE * SS_THREAD_BYTES;             // 8 KiB
constexpr int SS_TILE_BYTES = SS_WAVES * SS_WAVE_BYTES;           // 56 KiB
constexpr int SS_RING = 8;
template <class T> constexpr int ss_tile_elems() { return SS_TILE_BYTES / (int)sizeof(T); }
// One buffer: the values, then (flag-driven scans) one flag byte per element.
template <class T> constexpr int ss_buffer_bytes(bool flags) {
  return SS_TILE_BYTES + (flags ? ss_tile_elems<T>() : 0);
}

// 16 bytes per lane from global memory straight into LDS: lane l's data lands
// at lds_addr + 16 l.  The compiler does not know of this load; whoever reads
// the bytes waits for vmcnt first.
// NT selects the non-temporal cache policy.
template <bool NT>
__device__ __forceinline__ void ss_load_to_lds(const void *gaddr, uint32_t lds_addr) {
  if constexpr (NT)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(
                     __builtin_amdgcn_readfirstlane(lds_addr)),
                 "v"(gaddr)
                 : "memory");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(
                     __builtin_amdgcn_readfirstlane(lds_addr)),
                 "v"(gaddr)
                 : "memory");
}

// Waits until at most `younger` vector memory operations of this wave are
// outstanding (wave-uniform argument; anything unexpected waits for all).
__device__ __forceinline__ void ss_wait_vm(int younger) {
  switch (younger) {
    case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
    case 9: asm volatile("s_waitcnt vmcnt(9)" ::: "memory"); break;
    case 10: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
    case 16: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
    case 17: asm volatile("s_waitcnt vmcnt(17)" ::: "memory"); break;
    case 18: asm volatile("s_waitcnt vmcnt(18)" ::: "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
}

// Progress counters in LDS.  LDS operations of a wave are performed in issue
// order, so a counter stored after the data it announces needs no hardware
// fence, only the compiler kept from reordering (a release or acquire
// operation here would also wait for the wave's outstanding global loads and
// stores, which is exactly what these waves must not do).
__device__ __forceinline__ void ss_signal(uint32_t *counter, uint32_t value) {
  asm volatile("" ::: "memory");
  __hip_atomic_store(counter, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  asm volatile("" ::: "memory");
}
__device__ __forceinline__ void ss_await(const uint32_t *counter, uint32_t at_least) {
  while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < at_least)
    __builtin_amdgcn_s_sleep(2);
  asm volatile("" ::: "memory");
}

// Start flags of a thread's elements: the raw flag bytes (one test per
// element, no unpacking), or a bit mask computed from the row length.
template <int EPT, bool RAW> struct SsFlags {
  uint32_t w[RAW ? EPT / 4 : 1];
  __device__ __forceinline__ bool test(int e) const {
    if constexpr (RAW) return ((w[e >> 2] >> (8 * (e & 3))) & 0xffu) != 0u;
    else return ((w[0] >> e) & 1u) != 0u;
  }
  __device__ __forceinline__ bool any() const {
    uint32_t o = 0u;
#pragma unroll
    for (int i = 0; i < (RAW ? EPT / 4 : 1); i++) o |= w[i];
    return o != 0u;
  }
};

template <class T, class Op, int SEGKIND, bool EXCL>
__global__ __launch_bounds__(SS_BLOCK) void segscan_kernel(
    const T *__restrict__ xs, const uint8_t *__restrict__ flags, int64_t n, T *__restrict__ out,
    uint32_t *header, uint64_t *desc, uint32_t epoch, const uint32_t *epoch_dev, int64_t num_tiles,
    int64_t seg_len) {
  // The epoch of this launch: an argument, or (for callers whose launches may
  // be replayed with the same arguments) a word a preceding kernel advanced.
  if (epoch_dev != nullptr) epoch = *epoch_dev;
  constexpr bool SEG = SEGKIND != SEG_NONE;
  constexpr bool FLAGS = SEGKIND == SEG_FLAGS;
  constexpr int VEC = Vec16<T>::N;
  constexpr int EPT = SS_THREAD_BYTES / (int)sizeof(T);
  constexpr int TILE = ss_tile_elems<T>();
  constexpr int BUFFER = ss_buffer_bytes<T>(FLAGS);
  constexpr int FLAG_LOADS = FLAGS ? EPT / 16 : 0;  // 1 KiB flag loads per wave and tile
  using Pair = SegPair<T>;
  using V4 = __attribute__((ext_vector_type(4))) uint32_t;

  extern __shared__ __align__(16) unsigned char ss_lds[];
  __shared__ uint32_t s_tile[SS_RING];        // tile q of this block (a ticket)
  __shared__ uint32_t s_tiles_known;          // how many of them have been handed out
  __shared__ T s_wv[SS_RING][SS_WAVES];       // wave totals of tile q
  __shared__ uint32_t s_wf[SS_RING][SS_WAVES];
  __shared__ uint32_t s_scanned[SS_WAVES];    // per data wave: tiles whose total is written
  __shared__ T s_pv[SS_RING];                 // exclusive prefix of tile q
  __shared__ uint32_t s_pf[SS_RING];
  __shared__ uint32_t s_prefixes_known;       // how many of them are there
  __shared__ uint32_t s_sink;

  // Ticket v of counter c is tile v * counters + c.
  const uint32_t counters = gridDim.x < (unsigned)SCAN_MAX_COUNTERS ? gridDim.x : (unsigned)SCAN_MAX_COUNTERS;
  const uint32_t my_counter = blockIdx.x % counters;
  uint32_t *ticket = header + my_counter * SCAN_COUNTER_STRIDE;
  const int tid = threadIdx.x;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)ss_lds;

  if (tid < SS_WAVES) s_scanned[tid] = 0u;
  if (tid == 0) {
    s_tiles_known = 0u;
    s_prefixes_known = 0u;
  }
  __syncthreads();  // the only barrier

  // Tile q of this block; waits until its ticket has been handed out.  (Ticket
  // values are the same in all lanes; readfirstlane says so to the compiler.)
  auto tile_of = [&](int q) -> int64_t {
    ss_await(&s_tiles_known, (uint32_t)q + 1u);
    return (int64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)s_tile[q % SS_RING]);
  };

  if (wave == SS_WAVES) {
    // ------------------------------------------------------------ protocol wave
    // Exclusive prefix of `tile` (> 0): folds the descriptors of the tiles
    // before it, newest window first, back to one that has published its prefix
    // (or, in a segmented scan, contains a segment start).
    uint32_t drawn = 0u;      // the ticket drawn in this round (in flight until the next round ends)
    bool ticket_drawn = false;
    auto look_back = [&](int64_t tile) -> Pair {
      Pair acc = {Op::identity(), 0u};
      // A window is the `width` tiles up to tile j, one descriptor per lane, in
      // the highest lanes.
      int64_t j = tile - 1;
      int width = WAVE;
      while (true) {
        const int64_t idx = j - (int64_t)(WAVE - 1 - lane);
        const bool active = lane >= WAVE - width && idx >= 0;
        uint32_t st = idx < 0 ? ST_P : ST_A, fg = 0u;  // before tile 0: an empty prefix
        T v = Op::identity();
        DescWords raw = {0ull, 0ull};
        if (active) raw = desc_load<T>(desc, idx);
        // The round's ticket is drawn behind the first window's loads: vector
        // memory operations return in order, and the loads must not wait for
        // the atomic's round trip.
        if (!ticket_drawn) {
          if (lane == 0) drawn = atomicAdd(ticket, 1u);
          ticket_drawn = true;
        }
        if (active) {
          while (!desc_decode<T>(raw, epoch, st, fg, v)) {
            __builtin_amdgcn_s_sleep(1);
            raw = desc_load<T>(desc, idx);
          }
        }
        // A published prefix (or, in a segmented scan, a segment start) ends the
        // walk: lanes before the last such lane do not count.
        const bool term = lane >= WAVE - width && (st == ST_P || (SEG && fg));
        const uint64_t mask = __ballot(term);
        Pair mine = {v, SEG ? fg : 0u};
        if (mask) {
          const int first = 63 - __builtin_clzll(mask);
          if (lane < first) {
            mine.v = Op::identity();
            mine.f = 0u;
          }
        }
        Pair win;
        if constexpr (SEG) {
          Pair sc = wave_incl_scan_seg<T, Op>(mine);
          win.v = read_lane(sc.v, 63);
          win.f = read_lane(sc.f, 63);
          acc = seg_apply<T, Op>(win, acc);
        } else {
          win.v = read_lane(wave_incl_scan<T, Op>(mine.v), 63);
          acc.v = Op::apply(win.v, acc.v);
        }
        if (mask) break;
        j -= width;
        width = WAVE;
      }
      return acc;
    };

    // Hands ticket `t` out as tile `q`.
    auto hand_out = [&](int q, uint32_t t) {
      if (lane == 0) {
        s_tile[q % SS_RING] = t * counters + my_counter;
        ss_signal(&s_tiles_known, (uint32_t)q + 1u);
      }
    };
    // The first three tickets are drawn one after the other, each after the one
    // before has come back: three tickets drawn at once would be consecutive
    // tiles, and the block next in line would wait two rounds for the aggregate
    // of this block's third tile.  Drawn a round trip apart, the first tickets
    // of all blocks come first, then their second ones, as in every later round.
    uint32_t t0 = 0u, t1 = 0u, t2 = 0u, pending = 0u;
    if (lane == 0) t0 = atomicAdd(ticket, 1u);
    hand_out(0, t0);
    if (lane == 0) t1 = atomicAdd(ticket, 1u + (t0 >> 31));  // (+0) issued after t0 is back
    hand_out(1, t1);
    if (lane == 0) t2 = atomicAdd(ticket, 1u + (t1 >> 31));
    hand_out(2, t2);
    // From here on a ticket is drawn in one round and handed out at the end of
    // the next: by then it has long been back, and nothing waits for the
    // atomic's round trip.  Round q hands out tile q+3, which the data waves
    // request at the end of their round q+1 (they are at least a round behind
    // this wave: a data wave completes tile q-1 in round q+1 with the prefix
    // found here in round q).
    if (lane == 0) pending = atomicAdd(ticket, 1u + (t2 >> 31));

    bool have_p1 = false;
    int64_t p1 = 0;                   // the tile of the round before
    Pair bt1 = {Op::identity(), 0u};  // and its aggregate
    for (int q = 0;; q++) {
      const int64_t cur = (int64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)s_tile[q % SS_RING]);
      const bool have_cur = cur < num_tiles;
      if (!have_cur && !have_p1) break;
      ticket_drawn = false;
      Pair bt = {Op::identity(), 0u};  // tile aggregate
      if (have_cur) {
        // Wave totals of tile q: wait for all seven data waves.
        if (lane < SS_WAVES) ss_await(&s_scanned[lane], (uint32_t)q + 1u);
        __builtin_amdgcn_wave_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int w = 0; w < SS_WAVES; w++) {
          Pair t = {s_wv[q % SS_RING][w], SEG ? s_wf[q % SS_RING][w] : 0u};
          if constexpr (SEG) bt = seg_apply<T, Op>(bt, t);
          else bt.v = Op::apply(bt.v, t.v);
        }
        // The first tile, and a tile that contains a segment start, know their
        // inclusive prefix already: nothing before the start can reach past it.
        const bool final_now = cur == 0 || (SEG && bt.f);
        if (lane == 0) desc_publish<T>(desc, cur, epoch, final_now ? ST_P : ST_A, bt.f, bt.v);
      }
      if (have_p1) {
        Pair acc = {Op::identity(), 0u};
        if (p1 > 0) {
          acc = look_back(p1);
          if (lane == 0 && !(SEG && bt1.f)) {
            Pair inc;
            if constexpr (SEG) inc = seg_apply<T, Op>(acc, bt1);
            else { inc.v = Op::apply(acc.v, bt1.v); inc.f = 0u; }
            desc_publish<T>(desc, p1, epoch, ST_P, inc.f, inc.v);
          }
        }
        if (lane == 0) {
          s_pv[(q - 1) % SS_RING] = acc.v;
          s_pf[(q - 1) % SS_RING] = acc.f;
          ss_signal(&s_prefixes_known, (uint32_t)q);
        }
      }
      if (!ticket_drawn && lane == 0) drawn = atomicAdd(ticket, 1u);
      hand_out(q + 3, pending);
      pending = drawn;
      have_p1 = have_cur;
      p1 = cur;
      bt1 = bt;
    }
    // The last ticket drawn is not used, but its atomic must have been performed
    // before this block reports that it has left: the block that leaves last
    // rearms the counters for the next launch.
    if (lane == 0) {
      s_sink = pending;  // waits for the atomic
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
      const uint32_t left = atomicAdd(header + 1, 1u);
      if (left == gridDim.x - 1) {
        st_relaxed_u32(header + 1, 0u);
        for (uint32_t c = 0; c < counters; c++) st_relaxed_u32(header + c * SCAN_COUNTER_STRIDE, 0u);
      }
    }
    return;
  }

  // ---------------------------------------------------------------- data waves
  // This thread's 128 bytes inside a buffer, and the swizzle of its units.
  const int my_region = tid * SS_THREAD_BYTES;
  const int my_sw = (tid >> 1) & 7;
  // A 1 KiB instruction j of this wave covers LDS block m = 8 wave + j: lane l
  // holds unit (l & 7) ^ ((4 m + (l >> 4)) & 7) of thread 8 m + (l >> 3).  m & 1
  // equals j & 1, so the unit a lane moves alternates between two values.
  const int io_thread = lane >> 3;  // + 8 m
  const int io_unit[2] = {(lane & 7) ^ (lane >> 4), (lane & 7) ^ (4 | (lane >> 4))};
  const bool flags_dma = FLAGS && ((uintptr_t)flags & 15u) == 0;
  const int flag_loads = flags_dma ? FLAG_LOADS : 0;
  // Flag bytes of this thread inside a buffer's flag area: EPT bytes, in 16-byte
  // halves when there are two (swapped for threads with bit 3 set).
  const int my_flag_half = (tid >> 3) & 1;

  // Requests this wave's part of tile `t` into buffer `b`.  Returns true when
  // the data travels by direct-to-LDS loads, which the wave waits for by count;
  // a tile that is not whole is loaded element-wise through registers, neutral
  // elements beyond n.
  auto fetch = [&](int64_t t, int b) -> bool {
    if (t >= num_tiles) return false;
    const int64_t t0 = t * TILE;
    const bool whole = t0 + TILE <= n;
    const bool dma = whole && (!FLAGS || flags_dma);
    const char *src = reinterpret_cast<const char *>(xs + t0);
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int m = 8 * wave + j;
      const int off = (8 * m + io_thread) * SS_THREAD_BYTES + io_unit[j & 1] * 16;
      if (dma) {
        ss_load_to_lds<false>(src + off, lds_base + b * BUFFER + m * 1024);
      } else {
        const int64_t idx = t0 + off / (int)sizeof(T);
        Vec16<T> v;
#pragma unroll
        for (int e = 0; e < VEC; e++) v.e[e] = idx + e < n ? xs[idx + e] : Op::identity();
        *reinterpret_cast<Vec16<T> *>(ss_lds + b * BUFFER + m * 1024 + lane * 16) = v;
      }
    }
    if constexpr (FLAGS) {
      // The wave's flag bytes: WAVE * EPT bytes at wave * WAVE * EPT of the flag area.
      const int fbase = wave * WAVE * EPT;
#pragma unroll
      for (int q = 0; q < EPT / 16; q++) {
        // 1 KiB block q: lane l holds 16 bytes of thread (64 q + l) / (EPT / 16).
        int thread_in_wave, half;
        if constexpr (EPT == 32) {
          thread_in_wave = 32 * q + (lane >> 1);
          half = (lane & 1) ^ ((thread_in_wave >> 3) & 1);
        } else {
          thread_in_wave = lane;
          half = 0;
        }
        const int foff = fbase + thread_in_wave * EPT + half * 16;
        if (dma) {
          ss_load_to_lds<true>(flags + t0 + foff, lds_base + b * BUFFER + SS_TILE_BYTES + fbase + q * 1024);
        } else {
          V4 w4;
#pragma unroll
          for (int c = 0; c < 4; c++) {
            uint32_t w = 0u;
#pragma unroll
            for (int k = 0; k < 4; k++) {
              const int64_t idx = t0 + foff + 4 * c + k;
              if (idx < n && flags[idx] != 0) w |= 1u << (8 * k);
            }
            w4[c] = w;
          }
          *reinterpret_cast<V4 *>(ss_lds + b * BUFFER + SS_TILE_BYTES + fbase + q * 1024 + lane * 16) = w4;
        }
      }
    }
    return dma;
  };

  int64_t cur = tile_of(0);
  bool cur_async = fetch(cur, 0);
  int64_t nxt = tile_of(1);
  bool nxt_async = fetch(nxt, 1);

  // The tiles scanned one and two rounds ago wait in registers for their prefix.
  bool have_p1 = false, have_p2 = false;
  int64_t p1 = 0, p2 = 0;
  T x1[EPT], x2[EPT];
  SsFlags<EPT, FLAGS> fl1, fl2;
  Pair ex1 = {Op::identity(), 0u}, ex2 = {Op::identity(), 0u};  // what precedes the thread in its wave
#pragma unroll
  for (int e = 0; e < EPT; e++) x1[e] = x2[e] = Op::identity();
#pragma unroll
  for (int i = 0; i < (FLAGS ? EPT / 4 : 1); i++) fl1.w[i] = fl2.w[i] = 0u;

  for (int q = 0; cur < num_tiles || have_p1 || have_p2; q++) {
    const int par = q & 1;
    unsigned char *buffer = ss_lds + par * BUFFER;
    unsigned char *region = buffer + my_region;
    const bool have_cur = cur < num_tiles;
    T x[EPT];
    SsFlags<EPT, FLAGS> fl;
    Pair excl = {Op::identity(), 0u};
#pragma unroll
    for (int i = 0; i < (FLAGS ? EPT / 4 : 1); i++) fl.w[i] = 0u;

    if (have_cur) {
      // ---- wait for this wave's part of the tile.  Younger than its loads
      //      are the stores of the round before (none before round 2) and the
      //      loads of the tile after it.
      if (cur_async) {
        if (!nxt_async) ss_wait_vm(0);
        else ss_wait_vm((q < 3 ? 8 : 16) + flag_loads);
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int k = 0; k < SS_UNITS; k++) {
        const Vec16<T> v = *reinterpret_cast<const Vec16<T> *>(region + ((k ^ my_sw) << 4));
#pragma unroll
        for (int e = 0; e < VEC; e++) x[k * VEC + e] = v.e[e];
      }
      if constexpr (FLAGS) {
        const unsigned char *fsrc = buffer + SS_TILE_BYTES + tid * EPT;
#pragma unroll
        for (int h = 0; h < EPT / 16; h++) {
          const int slot = EPT == 32 ? (h ^ my_flag_half) : 0;
          const V4 v = *reinterpret_cast<const V4 *>(fsrc + slot * 16);
#pragma unroll
          for (int c = 0; c < 4; c++) fl.w[4 * h + c] = v[c];
        }
      }
      if constexpr (SEGKIND == SEG_ROWS) {
        // Bit e: element e of this thread opens a row.
        const int64_t pos = (cur * TILE + (int64_t)tid * EPT) % seg_len;
        uint32_t m = 0u;
        if (seg_len >= EPT) {
          const int64_t first = pos == 0 ? 0 : seg_len - pos;
          if (first < EPT) m = 1u << (int)first;
        } else {
          int p = (int)pos;
          const int sl = (int)seg_len;
#pragma unroll
          for (int e = 0; e < EPT; e++) {
            if (p == 0) m |= 1u << e;
            p = p + 1 == sl ? 0 : p + 1;
          }
        }
        fl.w[0] = m;
      }

      // ---- scan inside the thread.
#pragma unroll
      for (int e = 1; e < EPT; e++) {
        if constexpr (SEG) x[e] = fl.test(e) ? x[e] : Op::apply(x[e - 1], x[e]);
        else x[e] = Op::apply(x[e - 1], x[e]);
      }

      // ---- one scan across the lanes of the wave.
      Pair tot = {x[EPT - 1], (SEG && fl.any()) ? 1u : 0u};
      Pair incl = {Op::identity(), 0u};
      if constexpr (SEG) {
        incl = wave_incl_scan_seg<T, Op>(tot);
        excl.f = dpp_move<DPP_WAVE_SHR1, 0xf>(0u, incl.f);
      } else {
        incl.v = wave_incl_scan<T, Op>(tot.v);
      }
      excl.v = wave_shift_up1<T, Op>(incl.v);
      if (lane == 63) {
        s_wv[q % SS_RING][wave] = incl.v;
        s_wf[q % SS_RING][wave] = incl.f;
        ss_signal(&s_scanned[wave], (uint32_t)q + 1u);
      }
    }

    // ---- complete and store the tile of two rounds ago: apply what precedes
    //      the thread, write the results into the thread's LDS bytes (those of
    //      `cur`, which is in registers now) and take the wave's 8 KiB out in
    //      store order.
    if (have_p2) {
      // Its prefix is there once q-1 prefixes are; then all its wave totals are too.
      ss_await(&s_prefixes_known, (uint32_t)q - 1u);
      const int slot = (q - 2) % SS_RING;
      Pair base = {s_pv[slot], SEG ? s_pf[slot] : 0u};
#pragma unroll
      for (int w = 0; w < SS_WAVES; w++) {
        if (w < wave) {
          Pair t = {s_wv[slot][w], SEG ? s_wf[slot][w] : 0u};
          if constexpr (SEG) base = seg_apply<T, Op>(base, t);
          else base.v = Op::apply(base.v, t.v);
        }
      }
      if constexpr (SEG) base = seg_apply<T, Op>(base, ex2);
      else base.v = Op::apply(base.v, ex2.v);
      bool seen = false;
      T before = base.v;
#pragma unroll
      for (int k = 0; k < SS_UNITS; k++) {
        Vec16<T> o;
#pragma unroll
        for (int c = 0; c < VEC; c++) {
          const int e = k * VEC + c;
          const bool f = SEG && fl2.test(e);
          seen = seen || f;
          const T inc = seen ? x2[e] : Op::apply(base.v, x2[e]);
          if constexpr (EXCL) o.e[c] = f ? Op::identity() : before;
          else o.e[c] = inc;
          before = inc;
        }
        *reinterpret_cast<Vec16<T> *>(region + ((k ^ my_sw) << 4)) = o;
      }
      // Same wave wrote these bytes: its LDS operations complete in order.
      __builtin_amdgcn_wave_barrier();
      const int64_t t0 = p2 * TILE;
      const bool whole = t0 + TILE <= n;
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const int m = 8 * wave + j;
        const Vec16<T> v = *reinterpret_cast<const Vec16<T> *>(buffer + m * 1024 + lane * 16);
        const int off = (8 * m + io_thread) * SS_THREAD_BYTES + io_unit[j & 1] * 16;
        const int64_t idx = t0 + off / (int)sizeof(T);
        if (whole) {
          store_vec16_nt(out + idx, v);
        } else {
#pragma unroll
          for (int e = 0; e < VEC; e++)
            if (idx + e < n) out[idx + e] = v.e[e];
        }
      }
    }
    // All LDS reads of this buffer have landed before new loads overwrite it.
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    const int64_t upc = tile_of(q + 2);
    const bool upc_async = fetch(upc, par);

    // ---- the scanned tiles move up in the queue for their prefix.
    have_p2 = have_p1;
    have_p1 = have_cur;
    p2 = p1;
    p1 = cur;
#pragma unroll
    for (int e = 0; e < EPT; e++) {
      x2[e] = x1[e];
      x1[e] = x[e];
    }
    fl2 = fl1;
    fl1 = fl;
    ex2 = ex1;
    ex1 = excl;
    cur = nxt;
    nxt = upc;
    cur_async = nxt_async;
    nxt_async = upc_async;
  }
}

static int scan_grid_limit() {
  static const int limit = [] {
    int dev = 0, cus = NUM_CUS_HINT;
    if (hipGetDevice(&dev) == hipSuccess)
      (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    return cus;
  }();
  return limit;
}

template <class T> static int64_t scan_num_tiles(int64_t n) {
  return ceil_div(n, (int64_t)ss_tile_elems<T>());
}

template <class T, class Op>
static int launch_scan(hipStream_t s, const void *xs, const uint8_t *flags, int64_t seg_len,
                       int64_t n, int exclusive, void *out, void *scratch, size_t scratch_bytes,
                       uint32_t epoch, const uint32_t *epoch_dev = nullptr) {
  if (n == 0) return 0;
  const int64_t tiles = scan_num_tiles<T>(n);
  if (scratch_bytes < SCAN_HEADER_BYTES + (size_t)tiles * SCAN_DESC_BYTES) return FA_ESCRATCH;
  if (!is_aligned(xs, 16) || !is_aligned(out, 16) || !is_aligned(scratch, 16) ||
      (flags && !is_aligned(flags, 4)))
    return FA_EALIGN;
  // Tickets are 32-bit and every block draws a few beyond the last tile.
  if (tiles > INT32_MAX - 65536) return FA_EINVAL;
  uint32_t *header = (uint32_t *)scratch;
  uint64_t *desc = (uint64_t *)((char *)scratch + SCAN_HEADER_BYTES);
  const int64_t limit = scan_grid_limit();
  const dim3 grid((unsigned)(tiles < limit ? tiles : limit)), block(SS_BLOCK);
#define FA_LAUNCH(SEGV, EXV)                                                                   \
  do {                                                                                         \
    auto kernel = segscan_kernel<T, Op, SEGV, EXV>;                                            \
    constexpr int lds_bytes = 2 * ss_buffer_bytes<T>(SEGV == SEG_FLAGS);                       \
    /* Initialised once, under the lock C++ gives function-local statics. */                   \
    static const hipError_t raised = hipFuncSetAttribute(                                      \
        (const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);          \
    if (raised != hipSuccess) return (int)raised;                                              \
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, s, (const T *)xs, flags, n, (T *)out,   \
                       header, desc, epoch, epoch_dev, tiles, seg_len);                        \
  } while (0)
  if (seg_len > 0) {
    if (exclusive) FA_LAUNCH(SEG_ROWS, true);
    else FA_LAUNCH(SEG_ROWS, false);
  } else if (flags) {
    if (exclusive) FA_LAUNCH(SEG_FLAGS, true);
    else FA_LAUNCH(SEG_FLAGS, false);
  } else {
    if (exclusive) FA_LAUNCH(SEG_NONE, true);
    else FA_LAUNCH(SEG_NONE, false);
  }
#undef FA_LAUNCH
  return launch_status();
}

}  // namespace fa

namespace fa {

// ---- scratch for the entry point that allocates nothing
constexpr size_t SCAN_STATIC_BYTES = 256 * 1024;
constexpr int SCAN_STATIC_EPOCH_WORD = 16;  // 32-bit word of the header that holds the epoch

}  // namespace fa

// Look-back scratch of fa_segscan_static: ticket counter, epoch word and tile
// descriptors.  Every GPU the library runs on holds its own copy, zero at
// load time, until the process ends.
static __device__ __align__(256) unsigned char static_scratch[fa::SCAN_STATIC_BYTES];

namespace fa {

// Advances the epoch word; before it would wrap, clears the descriptors.  One block.
__global__ __launch_bounds__(256) void scan_static_epoch_kernel(uint32_t *header, uint64_t *desc,
                                                                int words) {
  const uint32_t next = header[SCAN_STATIC_EPOCH_WORD] + 1u;
  const bool wrap = next >= (1u << 28);
  if (wrap)
    for (int i = threadIdx.x; i < words; i += blockDim.x) desc[i] = 0ull;
  __syncthreads();
  if (threadIdx.x == 0) header[SCAN_STATIC_EPOCH_WORD] = wrap ? 1u : next;
}

// Device address of `static_scratch` on the current device (in host code the array's
// name is only a handle for this query).
static int scan_static_scratch(void **out) {
  constexpr int MAX_DEVICES = 64;
  static std::mutex mu;
  static void *ptrs[MAX_DEVICES];
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= MAX_DEVICES) return FA_EINVAL;
  std::lock_guard<std::mutex> guard(mu);
  if (ptrs[dev] == nullptr) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch));
    if (e != hipSuccess) return (int)e;
    if (p == nullptr) return FA_EINVAL;
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return 0;
}

template <class T, class Op>
static int launch_scan_static(hipStream_t s, const void *xs, const uint8_t *flags, int64_t n,
                              int exclusive, void *out, void *base) {
  uint32_t *header = (uint32_t *)base;
  uint64_t *desc = (uint64_t *)((char *)base + SCAN_HEADER_BYTES);
  hipLaunchKernelGGL(scan_static_epoch_kernel, dim3(1), dim3(256), 0, s, header, desc,
                     (int)((SCAN_STATIC_BYTES - SCAN_HEADER_BYTES) / 8));
  const int rc = launch_status();
  if (rc != 0) return rc;
  return launch_scan<T, Op>(s, xs, flags, (int64_t)0, n, exclusive, out, base, SCAN_STATIC_BYTES, 1u,
                            header + SCAN_STATIC_EPOCH_WORD);
}

}  // namespace fa

extern "C" int64_t fa_segscan_static_max_n(fa_dtype t) {
  const size_t es = dtype_size(t);
  if (es != 4 && es != 8) return 0;
  const int64_t tile = (es == 4) ? ss_tile_elems<int32_t>() : ss_tile_elems<int64_t>();
  return (int64_t)((SCAN_STATIC_BYTES - SCAN_HEADER_BYTES) / SCAN_DESC_BYTES) * tile;
}

extern "C" int fa_segscan_static_init(void) {
  void *base = nullptr;
  return scan_static_scratch(&base);
}

extern "C" int fa_segscan_static(fa_stream_t stream, fa_dtype t, fa_op op, const void *xs,
                                 const uint8_t *flags, int64_t n, int exclusive, void *out) {
  if (n < 0 || (n > 0 && (xs == nullptr || out == nullptr))) return FA_EINVAL;
  const size_t es = dtype_size(t);
  if (es != 4 && es != 8) return FA_ENOTSUP;
  if (n > fa_segscan_static_max_n(t)) return FA_ESCRATCH;  // beyond what the fixed scratch holds
  if (n == 0) return 0;
  void *base = nullptr;
  const int rc = scan_static_scratch(&base);
  if (rc != 0) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (t == FA_I32X2)
    return op == FA_COMPOSE
               ? launch_scan_static<AffineI32, OpCompose>(s, xs, flags, n, exclusive, out, base)
               : FA_ENOTSUP;
  FA_DISPATCH_TYPE_OP(launch_scan_static, t, op, s, xs, flags, n, exclusive, out, base);
}

extern "C" size_t fa_segscan_scratch_bytes(fa_dtype t, int64_t n) {
  const size_t es = dtype_size(t);
  if (es != 4 && es != 8) return 0;
  if (n < 0) n = 0;
  const int64_t tile = (es == 4) ? ss_tile_elems<int32_t>() : ss_tile_elems<int64_t>();
  const int64_t tiles = ceil_div(n, tile);
  return SCAN_HEADER_BYTES + (size_t)(tiles < 1 ? 1 : tiles) * SCAN_DESC_BYTES;
}

extern "C" int fa_segscan(fa_stream_t stream, fa_dtype t, fa_op op, const void *xs,
                          const uint8_t *flags, int64_t n, int exclusive, void *out,
                          void *scratch, size_t scratch_bytes, uint32_t epoch) {
  if (n < 0 || (n > 0 && (xs == nullptr || out == nullptr || scratch == nullptr)))
    return FA_EINVAL;
  if (epoch == 0 || epoch >= (1u << 28)) return FA_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  if (t == FA_I32X2)
    return op == FA_COMPOSE ? launch_scan<AffineI32, OpCompose>(s, xs, flags, (int64_t)0, n, exclusive,
                                                                out, scratch, scratch_bytes, epoch)
                            : FA_ENOTSUP;
  FA_DISPATCH_TYPE_OP(launch_scan, t, op, s, xs, flags, (int64_t)0, n, exclusive, out, scratch,
                      scratch_bytes, epoch);
}

extern "C" int fa_segscan_rows(fa_stream_t stream, fa_dtype t, fa_op op, const void *xss,
                               int64_t m, int64_t k, int exclusive, void *out, void *scratch,
                               size_t scratch_bytes, uint32_t epoch) {
  if (m < 0 || k < 0 || (m > 0 && k > INT64_MAX / m)) return FA_EINVAL;
  const int64_t n = m * k;
  if (n > 0 && (xss == nullptr || out == nullptr || scratch == nullptr)) return FA_EINVAL;
  if (epoch == 0 || epoch >= (1u << 28)) return FA_EINVAL;
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (t == FA_I32X2)
    return op == FA_COMPOSE
               ? launch_scan<AffineI32, OpCompose>(s, xss, (const uint8_t *)nullptr, k, n, exclusive,
                                                   out, scratch, scratch_bytes, epoch)
               : FA_ENOTSUP;
  FA_DISPATCH_TYPE_OP(launch_scan, t, op, s, xss, (const uint8_t *)nullptr, k, n, exclusive, out,
                      scratch, scratch_bytes, epoch);
}

// futhark_amd_segops.hpp -- the SegOp kernels of libfuthark_amd_kernels.so as
// templates, for operators and fused maps the library's fixed operator set
// (fa_op x fa_dtype) does not have.
//
// The reference generates one kernel per SegOp of a program, with the
// program's own operator and the scalar code fused around it inlined
// (src/Futhark/CodeGen/ImpGen/GPU/SegRed.hs, SegScan/SinglePass.hs, SegHist.hs;
// the lambdas are those of src/Futhark/IR/SegOp.hs: SegBinOp :138-155 with its
// neutral element, the map part of the body before it, and SegPostOp after a
// scan).  Here the same role is played by template parameters: a translation
// unit includes this header, names its operator and maps, and gets the gfx950
// kernels (compiled with hipcc --offload-arch=gfx950) behind a launcher.
//
// An operator Op over element type T (4 or 8 bytes, trivially copyable; a tuple
// is a struct) provides
//     static constexpr bool commutative;
//     static __host__ __device__ T identity();       // the neutral element
//     static __host__ __device__ T apply(T a, T b);  // a first, then b; associative
// A map provides  static __device__ T apply(...)  as stated at each launcher.
//
//   launch_scan<T, Op, Pre, Post>      single-pass scan (also segmented by flags or
//                                      in rows of equal length), maps T -> T fused in
//   launch_reduce<Tin, T, Pre, Op>     reduction; Pre maps (element, its index) to T;
//                                      operators that do not commute are folded in
//                                      element order (SegRed.hs:836-921)
//   launch_segreduce<Tin, T, Pre, Op>  the same per row of a [m][k] array (regular
//                                      segments, SegRed.hs:396-636)
//   launch_segreduce_irregular<T, Op>  per (offset, length) segment: a scan with flags
//                                      from the offsets and a gather (Builtins.hs:570-602)
//   launch_hist_locked<...>            reduce_by_index for an operator over a pair of
//                                      values kept in two arrays, which no single
//                                      atomic can update: bins are locked
//                                      (ImpGen/GPU/Base.hs:769-842)
//
// futhark_amd/csrc/kernels/custom_ops.hip is written against this header alone
// and shows each of them.
#pragma once

#include "futhark_amd_device.hpp"

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
// fa_segscan_static, word 512 counts the blocks that have arrived, and every
// 64th word up to there (256 bytes apart, so that they sit in different memory
// channels) is a ticket counter: same-address atomics are performed one at a
// time, about 12 ns each on MI355X, and a channel that does little else slows
// every stream that crosses it.  Counter c hands out the tiles congruent to c
// modulo the number of counters in use, and a block draws from one counter for
// as long as it runs (its tiles then come in increasing order, which the
// pipeline of three tiles inside a block relies on).  Every tile is handed out
// only if every counter has a block drawing from it.  Which counter a block
// takes is the launch's choice (ScanTickets):
//   * BY_ARRIVAL: the block's arrival number (one more atomic, on one address
//     for all blocks) modulo the number of counters.  Whichever blocks the
//     hardware starts first, the first eight cover all eight counters, so the
//     launch finishes as long as eight blocks (or the whole grid, if it is
//     smaller) can be resident at the same time -- on any CUs, of any die.
//     The arrival atomic costs 1.5-2.5 us per launch (256 atomics on one
//     address, and a round trip more before the first ticket): 2^26 f32 with
//     flags 92.9 -> 94.4 us, 2^24 i32 28.8 -> 30.4 us.
//   * BY_BLOCK: block index modulo the number of counters, no arrival atomic,
//     and the first two tiles of a block follow from its index as well, so its
//     first loads wait for nothing.  This needs every block of the launch
//     resident at the same time (the grid has at most one block per CU): true
//     for a launch that has the GPU to itself, not guaranteed under a CU mask,
//     nor when other kernels that themselves wait for something hold CUs.
//     Callers choose it when they know that the launch is alone on the device.
enum class ScanTickets { BY_ARRIVAL = 0, BY_BLOCK = 1 };
constexpr size_t SCAN_HEADER_BYTES = 8192;
constexpr int SCAN_MAX_COUNTERS = 8;
constexpr int SCAN_COUNTER_STRIDE = 64;  // in 32-bit words
constexpr int SCAN_ARRIVAL_WORD = SCAN_MAX_COUNTERS * SCAN_COUNTER_STRIDE;
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
                 : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(
                     __builtin_amdgcn_readfirstlane(lds_addr)),
                 "v"(gaddr)
                 : "memory", "m0");
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

// Pre and Post are the maps fused into the scan: element x enters as
// Pre::apply(x) (the body of the SegScan before its operator) and result r
// leaves as Post::apply(r) (the SegPostOp, src/Futhark/IR/SegOp.hs:138-155).
// Both keep the element type.
struct MapIdentity {
  template <class T> static __device__ __forceinline__ T apply(T x) { return x; }
};

template <class T, class Op, int SEGKIND, bool EXCL, class Pre = MapIdentity, class Post = MapIdentity>
__global__ __launch_bounds__(SS_BLOCK) void segscan_kernel(
    const T *__restrict__ xs, const uint8_t *__restrict__ flags, int64_t n, T *__restrict__ out,
    uint32_t *header, uint64_t *desc, uint32_t epoch, const uint32_t *epoch_dev, int64_t num_tiles,
    int64_t seg_len, uint32_t by_arrival) {
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
  const int tid = threadIdx.x;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)ss_lds;

  // The protocol wave takes the block's arrival number first of all: its round
  // trip runs while the rest of the block sets up.
  uint32_t arrival = 0u;
  if (by_arrival && tid == SS_DATA_THREADS) arrival = atomicAdd(header + SCAN_ARRIVAL_WORD, 1u);
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
    const uint32_t my_counter =
        (by_arrival ? (uint32_t)__builtin_amdgcn_readfirstlane((int)arrival) : blockIdx.x) % counters;
    uint32_t *ticket = header + my_counter * SCAN_COUNTER_STRIDE;
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

    // Hands tile number `t` out as the block's tile `q`.
    auto hand_out = [&](int q, uint32_t t) {
      if (lane == 0) {
        s_tile[q % SS_RING] = t;
        ss_signal(&s_tiles_known, (uint32_t)q + 1u);
      }
    };
    // By block index, the first two tiles of block b are b and b + gridDim.x,
    // without a ticket (every block of such a launch is resident, so each of
    // these tiles has its block): the first loads leave before any atomic has
    // come back.  The counters hand out what follows.
    const uint32_t first_ticketed = by_arrival ? 0u : 2u * gridDim.x;
    auto tile_of_ticket = [&](uint32_t t) { return first_ticketed + t * counters + my_counter; };
    // The first three tickets are drawn one after the other, each after the one
    // before has come back: three tickets drawn at once would be consecutive
    // tiles, and the block next in line would wait two rounds for the aggregate
    // of this block's third tile.  Drawn a round trip apart, the first tickets
    // of all blocks come first, then their second ones, as in every later round.
    uint32_t t0 = 0u, t1 = 0u, t2 = 0u, pending = 0u;
    if (by_arrival) {
      if (lane == 0) t0 = atomicAdd(ticket, 1u);
      hand_out(0, tile_of_ticket(t0));
      if (lane == 0) t1 = atomicAdd(ticket, 1u + (t0 >> 31));  // (+0) issued after t0 is back
      hand_out(1, tile_of_ticket(t1));
    } else {
      hand_out(0, blockIdx.x);
      hand_out(1, blockIdx.x + gridDim.x);
    }
    if (lane == 0) t2 = atomicAdd(ticket, 1u + (t1 >> 31));
    hand_out(2, tile_of_ticket(t2));
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
      hand_out(q + 3, tile_of_ticket(pending));
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
        st_relaxed_u32(header + SCAN_ARRIVAL_WORD, 0u);
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
        for (int e = 0; e < VEC; e++) v.e[e] = idx + e < n ? Pre::apply(xs[idx + e]) : Op::identity();
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
        // (a tile loaded through registers has been mapped on the way in)
#pragma unroll
        for (int e = 0; e < VEC; e++) x[k * VEC + e] = cur_async ? Pre::apply(v.e[e]) : v.e[e];
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
          if constexpr (EXCL) o.e[c] = Post::apply(f ? Op::identity() : before);
          else o.e[c] = Post::apply(inc);
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

template <class T, class Op, class Pre = MapIdentity, class Post = MapIdentity>
static int launch_scan(hipStream_t s, const void *xs, const uint8_t *flags, int64_t seg_len,
                       int64_t n, int exclusive, void *out, void *scratch, size_t scratch_bytes,
                       uint32_t epoch, const uint32_t *epoch_dev = nullptr,
                       ScanTickets tickets = ScanTickets::BY_ARRIVAL) {
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
    auto kernel = segscan_kernel<T, Op, SEGV, EXV, Pre, Post>;                                            \
    constexpr int lds_bytes = 2 * ss_buffer_bytes<T>(SEGV == SEG_FLAGS);                       \
    /* Initialised once, under the lock C++ gives function-local statics. */                   \
    static const hipError_t raised = hipFuncSetAttribute(                                      \
        (const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);          \
    if (raised != hipSuccess) return (int)raised;                                              \
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, s, (const T *)xs, flags, n, (T *)out,   \
                       header, desc, epoch, epoch_dev, tiles, seg_len,                         \
                       tickets == ScanTickets::BY_ARRIVAL ? 1u : 0u);                          \
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

// ===========================================================================
// Reduction with a fused map, for operators over 4- or 8-byte elements.
//
// Stage two as in the library's reduction: every block publishes its partial
// as a {value, epoch} word, the block that drew the last ticket folds them in
// block order.  The scratch buffer and its epochs are shared with the scan,
// whose descriptor words end in (epoch << 3 | flag << 2 | status) with status
// 1 or 2; a partial ends in (epoch << 3 | 3), so no word a scan has left behind
// can be taken for a partial, whatever the two epochs.
constexpr int RED_BLOCK = 1024;
constexpr int RED_MAX_GRID = 1024;
constexpr size_t RED_HEADER_BYTES = 8192;  // the scan's ticket counters live here

__device__ __forceinline__ uint32_t partial_meta(uint32_t epoch) { return (epoch << 3) | 3u; }

template <class T>
__device__ __forceinline__ void partial_publish(uint64_t *desc, int slot, uint32_t epoch, T v) {
  epoch = partial_meta(epoch);
  if constexpr (sizeof(T) == 4) {
    st_relaxed_u64(desc + 2 * slot, ((uint64_t)bit_cast<uint32_t>(v) << 32) | epoch);
  } else {
    const uint64_t b = bit_cast<uint64_t>(v);
    st_relaxed_u64(desc + 2 * slot, ((b & 0xffffffffull) << 32) | epoch);
    st_relaxed_u64(desc + 2 * slot + 1, ((b >> 32) << 32) | epoch);
  }
}

template <class T>
__device__ __forceinline__ T partial_wait(const uint64_t *desc, int slot, uint32_t epoch) {
  epoch = partial_meta(epoch);
  uint64_t w0;
  while ((uint32_t)(w0 = ld_relaxed_u64(desc + 2 * slot)) != epoch) __builtin_amdgcn_s_sleep(1);
  if constexpr (sizeof(T) == 4) {
    return bit_cast<T>((uint32_t)(w0 >> 32));
  } else {
    uint64_t w1;
    while ((uint32_t)(w1 = ld_relaxed_u64(desc + 2 * slot + 1)) != epoch)
      __builtin_amdgcn_s_sleep(1);
    return bit_cast<T>((w0 >> 32) | ((w1 >> 32) << 32));
  }
}

// Fold over the threads of a block in thread order (lane order inside a wave,
// then wave order), result in every thread.
template <class T, class Op, int BLOCK>
__device__ __forceinline__ T block_fold_ordered(T v, T *lds /* BLOCK/64 slots */) {
  v = read_lane(wave_incl_scan<T, Op>(v), 63);
  const int wave = threadIdx.x / WAVE;
  if (lane_id() == 0) lds[wave] = v;
  __syncthreads();
  T r = lds[0];
#pragma unroll
  for (int w = 1; w < BLOCK / WAVE; w++) r = Op::apply(r, lds[w]);
  __syncthreads();
  return r;
}

// out[0] = fold of Pre::apply(xs[i], i) over i < n.  Commutative operators:
// thread t takes elements t, t + T, ... (SegRed.hs:802-832).  Others
// (SegRed.hs:836-921): a block takes a contiguous stretch, a round of the block
// is BLOCK * PER consecutive elements, a thread folds PER consecutive ones, and
// threads, rounds and blocks are combined in order.
template <class Tin, class T, class Pre, class Op>
__global__ __launch_bounds__(RED_BLOCK) void reduce_kernel(const Tin *__restrict__ xs, int64_t n,
                                                           T *__restrict__ out, uint32_t *ticket,
                                                           uint64_t *desc, uint32_t epoch,
                                                           bool vectors) {
  constexpr int PER = 4;
  __shared__ T lds[RED_BLOCK / WAVE];
  __shared__ uint32_t s_ticket;
  uint32_t my_ticket = 0;
  if (gridDim.x > 1 && threadIdx.x == 0) my_ticket = atomicAdd(ticket, 1u);

  T v = Op::identity();
  if constexpr (Op::commutative) {
    // As the library's own reduction reads (segred_nonseg_kernel): 16 bytes per
    // load with the non-temporal policy, two loads in flight per thread, the
    // map applied to every element with its own index.  Inputs whose base is not
    // 16-byte aligned, and element types that do not divide 16 bytes, are read
    // element by element.
    constexpr bool VECTORS = 16 % sizeof(Tin) == 0 && sizeof(Tin) <= 8;
    const int64_t stride = (int64_t)gridDim.x * RED_BLOCK;
    int64_t i = (int64_t)blockIdx.x * RED_BLOCK + threadIdx.x;
    int64_t done = 0;  // elements [0, done) are covered by vector loads
    if constexpr (VECTORS) {
      if (vectors) {
        constexpr int VEC = 16 / (int)sizeof(Tin);
        constexpr int UNROLL = 2;
        const int64_t nvec = n / VEC;
        T acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[e] = Op::identity();
        int64_t j = i;
        for (; j + (UNROLL - 1) * stride < nvec; j += UNROLL * stride) {
          Vec16<Tin> x[UNROLL];
#pragma unroll
          for (int u = 0; u < UNROLL; u++) x[u] = load_vec16_nt(xs + (j + u * stride) * VEC);
#pragma unroll
          for (int u = 0; u < UNROLL; u++)
#pragma unroll
            for (int e = 0; e < VEC; e++)
              acc[e] = Op::apply(acc[e], Pre::apply(x[u].e[e], (j + u * stride) * VEC + e));
        }
        for (; j < nvec; j += stride) {
          const Vec16<Tin> x = load_vec16_nt(xs + j * VEC);
#pragma unroll
          for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], Pre::apply(x.e[e], j * VEC + e));
        }
#pragma unroll
        for (int e = 0; e < VEC; e++) v = Op::apply(v, acc[e]);
        done = nvec * VEC;
      }
    }
    i += done;
    for (; i + (PER - 1) * stride < n; i += PER * stride) {
      Tin x[PER];
#pragma unroll
      for (int u = 0; u < PER; u++) x[u] = xs[i + u * stride];
#pragma unroll
      for (int u = 0; u < PER; u++) v = Op::apply(v, Pre::apply(x[u], i + u * stride));
    }
    for (; i < n; i += stride) v = Op::apply(v, Pre::apply(xs[i], i));
    v = block_fold_ordered<T, Op, RED_BLOCK>(v, lds);
  } else {
    constexpr int64_t ROUND = (int64_t)RED_BLOCK * PER;
    const int64_t rounds = ceil_div(n, ROUND);
    const int64_t per_block = ceil_div(rounds, (int64_t)gridDim.x);
    const int64_t r0 = (int64_t)blockIdx.x * per_block;
    const int64_t r1 = r0 + per_block < rounds ? r0 + per_block : rounds;
    for (int64_t r = r0; r < r1; r++) {
      const int64_t base = r * ROUND + (int64_t)threadIdx.x * PER;
      T t = Op::identity();
#pragma unroll
      for (int u = 0; u < PER; u++)
        if (base + u < n) t = Op::apply(t, Pre::apply(xs[base + u], base + u));
      v = Op::apply(v, block_fold_ordered<T, Op, RED_BLOCK>(t, lds));
    }
  }

  if (gridDim.x == 1) {
    if (threadIdx.x == 0) *out = v;
    return;
  }
  if (threadIdx.x == 0) {
    partial_publish<T>(desc, (int)blockIdx.x, epoch, v);
    s_ticket = my_ticket;
    // Last ticket of this launch: rearm the counter for the next one.
    if (my_ticket == gridDim.x - 1) st_relaxed_u32(ticket, 0u);
  }
  __syncthreads();
  if (s_ticket != gridDim.x - 1) return;
  // Stage two in block order, by one wave: the result does not depend on
  // timing, and operands keep their order.
  if (threadIdx.x < WAVE) {
    T r = Op::identity();
    for (int p0 = 0; p0 < (int)gridDim.x; p0 += WAVE) {
      const int p = p0 + (int)threadIdx.x;
      T mine = p < (int)gridDim.x ? partial_wait<T>(desc, p, epoch) : Op::identity();
      r = Op::apply(r, read_lane(wave_incl_scan<T, Op>(mine), 63));
    }
    if (threadIdx.x == 0) *out = r;
  }
}

// Scratch and epoch as for fa_segred_nonseg (the same buffer may serve).
template <class Tin, class T, class Pre, class Op>
static int launch_reduce(hipStream_t s, const Tin *xs, int64_t n, T *out, void *scratch,
                         size_t scratch_bytes, uint32_t epoch) {
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "4- or 8-byte elements");
  if (n < 0 || out == nullptr || scratch == nullptr || (n > 0 && xs == nullptr)) return FA_EINVAL;
  if (epoch == 0 || epoch >= (1u << 28)) return FA_EINVAL;
  if (scratch_bytes < RED_HEADER_BYTES + (size_t)RED_MAX_GRID * 16) return FA_ESCRATCH;
  if (!is_aligned(scratch, 16)) return FA_EALIGN;
  int dev = 0, cus = NUM_CUS_HINT;
  if (hipGetDevice(&dev) == hipSuccess)
    (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  const int64_t want = ceil_div(n, (int64_t)RED_BLOCK * 16);
  const int limit = cus > RED_MAX_GRID ? RED_MAX_GRID : cus;
  const int grid = (int)(want < 1 ? 1 : (want > limit ? limit : want));
  uint32_t *ticket = (uint32_t *)scratch;
  uint64_t *desc = (uint64_t *)((char *)scratch + RED_HEADER_BYTES);
  hipLaunchKernelGGL((reduce_kernel<Tin, T, Pre, Op>), dim3(grid), dim3(RED_BLOCK), 0, s, xs, n, out,
                     ticket, desc, epoch, is_aligned(xs, 16));
  return launch_status();
}

// ===========================================================================
// Segmented reductions with a fused map, for operators over 4- or 8-byte
// elements.
//
// Regular segments, `map (\row -> reduce op ne (map f row)) xss` with
// xss : [m][k] (SegRed.hs:396-636): a row is folded by a group of G lanes
// (1 to 64, a power of two, chosen from k) or, when it is long, by a block.
// Element j of a row enters as Pre::apply(x, j), j its position in the row.
// Operands keep their order whatever the operator: a round of a group is G
// consecutive elements, folded across the lanes in lane order (an inclusive
// scan over the wave restricted to the group), and rounds are folded in turn;
// operators that commute skip the per-round fold and fold the lanes once at
// the end.
constexpr int SEGRED_T_BLOCK = 256;
constexpr int64_t SEGRED_T_LONG = 16384;  // rows longer than this get a block each

// Fold over the G lanes of a group (groups are aligned, G a power of two),
// result valid in the group's last lane; lane order kept.
template <class T, class Op, int G> __device__ __forceinline__ T group_fold_ordered(T v) {
  const T id = Op::identity();
  if constexpr (G >= 2) v = Op::apply(dpp_move<DPP_ROW_SHR1, 0xf>(id, v), v);
  if constexpr (G >= 4) v = Op::apply(dpp_move<DPP_ROW_SHR2, 0xf>(id, v), v);
  if constexpr (G >= 8) v = Op::apply(dpp_move<DPP_ROW_SHR4, 0xf>(id, v), v);
  if constexpr (G >= 16) v = Op::apply(dpp_move<DPP_ROW_SHR8, 0xf>(id, v), v);
  if constexpr (G >= 32) v = Op::apply(dpp_move<DPP_ROW_BCAST15, 0xa>(id, v), v);
  if constexpr (G >= 64) v = Op::apply(dpp_move<DPP_ROW_BCAST31, 0xc>(id, v), v);
  return v;
}
// The row shifts above pull in the lanes of the group only when the group is a
// whole row of 16 lanes or more; inside a row a shift crosses group borders,
// so smaller groups mask what comes from outside.
template <class T, class Op, int G> __device__ __forceinline__ T small_group_fold_ordered(T v) {
  static_assert(G < 16, "groups below a DPP row");
  const int sub = lane_id() % G;
#pragma unroll
  for (int d = 1; d < G; d *= 2) {
    T other;
    if constexpr (sizeof(T) == 4) {
      other = bit_cast<T>(__shfl_up(bit_cast<int>(v), d, WAVE));
    } else {
      other = bit_cast<T>((unsigned long long)__shfl_up((unsigned long long)bit_cast<uint64_t>(v), d, WAVE));
    }
    if (sub >= d) v = Op::apply(other, v);
  }
  return v;
}

template <class Tin, class T, class Pre, class Op, int G>
__global__ __launch_bounds__(SEGRED_T_BLOCK) void segreduce_group_kernel(const Tin *__restrict__ xss,
                                                                         int64_t m, int64_t k,
                                                                         T *__restrict__ out) {
  const int64_t gthread = (int64_t)blockIdx.x * SEGRED_T_BLOCK + threadIdx.x;
  const int64_t seg = gthread / G;
  const int sub = (int)(gthread % G);
  const bool live = seg < m;
  const Tin *row = xss + (live ? seg : 0) * k;
  T acc = Op::identity();
  auto fold = [](T v) {
    if constexpr (G >= 16) return group_fold_ordered<T, Op, G>(v);
    else if constexpr (G > 1) return small_group_fold_ordered<T, Op, G>(v);
    else return v;
  };
  if constexpr (Op::commutative) {
    if (live)
      for (int64_t j = sub; j < k; j += G) acc = Op::apply(acc, Pre::apply(row[j], j));
    acc = fold(acc);
  } else {
    // Every lane of the wave takes part in every round (the folds move data
    // across lanes), so the trip count is that of the longest row: k for all.
    for (int64_t j0 = 0; j0 < k; j0 += G) {
      const int64_t j = j0 + sub;
      const T mine = live && j < k ? Pre::apply(row[j], j) : Op::identity();
      const T round = fold(mine);  // in the group's last lane: elements j0 .. j0 + G - 1
      acc = Op::apply(acc, round);
    }
  }
  if (live && sub == G - 1) out[seg] = acc;
}

template <class Tin, class T, class Pre, class Op>
__global__ __launch_bounds__(RED_BLOCK) void segreduce_block_kernel(const Tin *__restrict__ xss,
                                                                    int64_t m, int64_t k,
                                                                    T *__restrict__ out) {
  __shared__ T lds[RED_BLOCK / WAVE];
  for (int64_t seg = blockIdx.x; seg < m; seg += gridDim.x) {
    const Tin *row = xss + seg * k;
    T acc = Op::identity();
    if constexpr (Op::commutative) {
      for (int64_t j = threadIdx.x; j < k; j += RED_BLOCK) acc = Op::apply(acc, Pre::apply(row[j], j));
      acc = block_fold_ordered<T, Op, RED_BLOCK>(acc, lds);
    } else {
      for (int64_t j0 = 0; j0 < k; j0 += RED_BLOCK) {
        const int64_t j = j0 + threadIdx.x;
        const T mine = j < k ? Pre::apply(row[j], j) : Op::identity();
        acc = Op::apply(acc, block_fold_ordered<T, Op, RED_BLOCK>(mine, lds));
      }
    }
    if (threadIdx.x == 0) out[seg] = acc;
  }
}

// out[i] = fold of Pre::apply(xss[i][j], j) over j < k, for i < m.  k == 0
// gives m neutral elements.
template <class Tin, class T, class Pre, class Op>
static int launch_segreduce(hipStream_t s, const Tin *xss, int64_t m, int64_t k, T *out) {
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "4- or 8-byte elements");
  if (m < 0 || k < 0) return FA_EINVAL;
  if (m == 0) return 0;
  if (out == nullptr || (k > 0 && xss == nullptr)) return FA_EINVAL;
  if (k > SEGRED_T_LONG) {
    int dev = 0, cus = NUM_CUS_HINT;
    if (hipGetDevice(&dev) == hipSuccess)
      (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    const int64_t most = (int64_t)cus * 2;
    hipLaunchKernelGGL((segreduce_block_kernel<Tin, T, Pre, Op>), dim3((unsigned)(m < most ? m : most)),
                       dim3(RED_BLOCK), 0, s, xss, m, k, out);
    return launch_status();
  }
#define FA_GROUPS(G)                                                                              \
  do {                                                                                            \
    const int64_t blocks = ceil_div(m * (G), (int64_t)SEGRED_T_BLOCK);                            \
    if (blocks > INT32_MAX) return FA_EINVAL;                                                     \
    hipLaunchKernelGGL((segreduce_group_kernel<Tin, T, Pre, Op, G>), dim3((unsigned)blocks),      \
                       dim3(SEGRED_T_BLOCK), 0, s, xss, m, k, out);                               \
  } while (0)
  if (k <= 2) FA_GROUPS(1);
  else if (k <= 8) FA_GROUPS(4);
  else if (k <= 64) FA_GROUPS(16);
  else FA_GROUPS(64);
#undef FA_GROUPS
  return launch_status();
}

// Irregular segments given as (offset, length) pairs, the way flattening
// expresses them (Pass/Flatten/Builtins.hs:570-602): flags are written from
// the offsets, the values are scanned with the flag-tuple operator, and
// segment i takes the scanned value at its last element, or the neutral
// element when it is empty.  Segments must be in order and must not overlap
// (offsets[i] + lens[i] <= offsets[i+1] <= n); elements between two segments
// and behind the last one belong to nobody (they are scanned on as a tail of
// the segment before them, which nobody reads).  workspace: n * (sizeof(T) + 1) bytes rounded up to 16, 16-byte
// aligned; scratch and epoch as for launch_scan.
// Clears `units` 16-byte units (a kernel rather than a memset, so that callers
// may record the launches in a graph).
static __global__ void clear_units_kernel(uint4 *p, int64_t units) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < units; i += stride)
    p[i] = uint4{0u, 0u, 0u, 0u};
}
template <class T>
__global__ void segments_to_flags_kernel(const int64_t *__restrict__ offsets,
                                         const int64_t *__restrict__ lens, int64_t m, int64_t n,
                                         uint8_t *flags) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < m && lens[i] > 0 && offsets[i] >= 0 && offsets[i] < n) flags[offsets[i]] = 1;
}
template <class T, class Op>
__global__ void segments_gather_kernel(const int64_t *__restrict__ offsets,
                                       const int64_t *__restrict__ lens, int64_t m, int64_t n,
                                       const T *__restrict__ scanned, T *__restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= m) return;
  const int64_t last = offsets[i] + lens[i] - 1;
  out[i] = lens[i] > 0 && last >= 0 && last < n ? scanned[last] : Op::identity();
}
template <class T> static size_t segreduce_irregular_workspace_bytes(int64_t n) {
  return (((size_t)n * sizeof(T) + 15) & ~(size_t)15) + (((size_t)n + 15) & ~(size_t)15);
}
template <class T, class Op, class Pre = MapIdentity>
static int launch_segreduce_irregular(hipStream_t s, const int64_t *offsets, const int64_t *lens,
                                      int64_t m, const T *xs, int64_t n, T *out, void *workspace,
                                      size_t workspace_bytes, void *scratch, size_t scratch_bytes,
                                      uint32_t epoch) {
  if (m < 0 || n < 0) return FA_EINVAL;
  if (m == 0) return 0;
  if (offsets == nullptr || lens == nullptr || out == nullptr) return FA_EINVAL;
  if (m > (int64_t)INT32_MAX * 256) return FA_EINVAL;
  const dim3 per_segment((unsigned)ceil_div(m, (int64_t)256));
  if (n > 0) {
    if (xs == nullptr || workspace == nullptr) return FA_EINVAL;
    if (workspace_bytes < segreduce_irregular_workspace_bytes<T>(n)) return FA_ESCRATCH;
    if (!is_aligned(workspace, 16)) return FA_EALIGN;
    T *scanned = (T *)workspace;
    uint8_t *flags = (uint8_t *)workspace + (((size_t)n * sizeof(T) + 15) & ~(size_t)15);
    const int64_t units = ceil_div(n, (int64_t)16);
    const int64_t clear_blocks = ceil_div(units, (int64_t)256);
    hipLaunchKernelGGL(clear_units_kernel, dim3((unsigned)(clear_blocks < 4096 ? clear_blocks : 4096)),
                       dim3(256), 0, s, (uint4 *)flags, units);
    int rc0 = launch_status();
    if (rc0 != 0) return rc0;
    hipLaunchKernelGGL(segments_to_flags_kernel<T>, per_segment, dim3(256), 0, s, offsets, lens, m, n,
                       flags);
    int rc = launch_status();
    if (rc != 0) return rc;
    rc = launch_scan<T, Op, Pre>(s, xs, flags, (int64_t)0, n, 0, scanned, scratch, scratch_bytes, epoch);
    if (rc != 0) return rc;
  }
  hipLaunchKernelGGL((segments_gather_kernel<T, Op>), per_segment, dim3(256), 0, s, offsets, lens, m, n,
                     (const T *)workspace, out);
  return launch_status();
}

// ===========================================================================
// reduce_by_index with an operator over a pair (A, B) whose components live in
// two destination arrays.  No single atomic updates both, so a bin is locked
// while it is updated (the reference's locking update, Base.hs:769-842: try the
// lock with a compare-and-swap, do the update and release inside the branch
// that got it, so that lanes of one wave that want the same lock cannot block
// each other).  Sub-histograms are private to a block and live in LDS, with
// LDS locks; at the end the block merges its non-neutral bins into the
// destination under locks in global memory (one lock word per bin).
// Pre::apply(x, i) makes the pair {a, b} of element i; Op works on that pair.
template <class P> __device__ __forceinline__ bool bits_equal_pair(const P &x, const P &y) {
  static_assert(sizeof(P) == 8, "a pair of two 4-byte components");
  return bit_cast<uint64_t>(x) == bit_cast<uint64_t>(y);
}
constexpr int HL_BLOCK = 512;
constexpr int HL_MAX_BINS = 8192;

// Runs `update` under the lock.  All lanes of the wave that want a lock call
// this together.  The loop runs until no lane of the wave is left waiting (a
// wave-wide vote), so a lane that got its lock updates and releases inside the
// loop body, in the same trip; written as "spin until the lock is mine, then
// update", the compiler places the update behind the spin loop, where lanes
// that hold a lock wait for the lanes of their own wave that spin on it.
// BACKOFF (locks in global memory): a trip in which no lane of the wave got its
// lock is followed by a pause, so that the waves that wait do not keep the
// lock's memory channel busy with attempts while its holder needs it to
// release.
template <class P, class Op, bool BACKOFF = false, class F>
__device__ __forceinline__ void hl_with_lock(uint32_t *lock, F &&update) {
  bool waiting = true;
  while (__ballot(waiting) != 0) {
    bool got = false;
    if (waiting) {
      if (atomicCAS(lock, 0u, 1u) == 0u) {
        update();
        __threadfence();
        atomicExch(lock, 0u);
        waiting = false;
        got = true;
      }
    }
    if constexpr (BACKOFF) {
      if (__ballot(got) == 0) __builtin_amdgcn_s_sleep(32);
    }
  }
}

template <class Tin, class A, class B, class P, class Pre, class Op, class I>
__global__ __launch_bounds__(HL_BLOCK) void hist_locked_kernel(const I *__restrict__ is,
                                                               const Tin *__restrict__ xs, int64_t n,
                                                               A *dest_a, B *dest_b, uint32_t *locks,
                                                               int64_t H) {
  extern __shared__ __align__(16) unsigned char hl_lds[];
  const int nb = (int)H;
  volatile A *sa = reinterpret_cast<volatile A *>(hl_lds);
  volatile B *sb = reinterpret_cast<volatile B *>(hl_lds + (size_t)nb * sizeof(A));
  uint32_t *sl = reinterpret_cast<uint32_t *>(hl_lds + (size_t)nb * (sizeof(A) + sizeof(B)));
  const P ne = Op::identity();
  for (int i = threadIdx.x; i < nb; i += HL_BLOCK) {
    sa[i] = ne.a;
    sb[i] = ne.b;
    sl[i] = 0u;
  }
  __syncthreads();
  const int64_t stride = (int64_t)gridDim.x * HL_BLOCK;
  for (int64_t i = (int64_t)blockIdx.x * HL_BLOCK + threadIdx.x; i < n; i += stride) {
    const int64_t bin = (int64_t)is[i];
    if ((uint64_t)bin >= (uint64_t)H) continue;  // out of range: ignored
    const P mine = Pre::apply(xs[i], i);
    // (lanes that are not here do not vote: a ballot counts active lanes only)
    hl_with_lock<P, Op>(&sl[bin], [&] {
      P cur;
      cur.a = sa[bin];
      cur.b = sb[bin];
      const P r = Op::apply(cur, mine);
      sa[bin] = r.a;
      sb[bin] = r.b;
    });
  }
  __syncthreads();
  for (int bin = threadIdx.x; bin < nb; bin += HL_BLOCK) {
    P mine;
    mine.a = sa[bin];
    mine.b = sb[bin];
    if (bits_equal_pair(mine, ne)) continue;  // untouched
    hl_with_lock<P, Op>(&locks[bin], [&] {
      P cur;
      cur.a = __hip_atomic_load(dest_a + bin, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      cur.b = __hip_atomic_load(dest_b + bin, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      // the block's bin holds later elements than nothing in particular: the
      // operator must commute, as reduce_by_index requires
      const P r = Op::apply(cur, mine);
      __hip_atomic_store(dest_a + bin, r.a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(dest_b + bin, r.b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    });
  }
}

// More bins than a block's LDS holds (the reference's pass over global memory
// with locks, SegHist.hs:377-467 with Base.hs:769-842).  Locking a bin of the
// destination for every update is only bearable while updates to a bin are
// rare: under skewed indices thousands of waves queue on the locks of a few
// bins, and same-address atomics are performed one at a time.  So a block keeps
// HL_MAX_BINS slots in LDS as a cache of the bins it meets: slot bin mod
// HL_MAX_BINS belongs to the first bin that claims it (a tag word, claimed by
// compare-and-swap, never given up), updates of that bin are made in the slot
// under the slot's LDS lock, and only updates of other bins that map to a taken
// slot go to the destination under the bin's global lock.  Frequent bins get
// their slots early and stay out of global memory; at the end the block merges
// its slots into the destination.
template <class Tin, class A, class B, class P, class Pre, class Op, class I>
__global__ __launch_bounds__(HL_BLOCK) void hist_locked_cached_kernel(const I *__restrict__ is,
                                                                      const Tin *__restrict__ xs,
                                                                      int64_t n, A *dest_a, B *dest_b,
                                                                      uint32_t *locks, int64_t H) {
  extern __shared__ __align__(16) unsigned char hl_lds[];
  constexpr int SLOTS = HL_MAX_BINS;
  static_assert((SLOTS & (SLOTS - 1)) == 0, "slot = bin mod a power of two");
  volatile A *sa = reinterpret_cast<volatile A *>(hl_lds);
  volatile B *sb = reinterpret_cast<volatile B *>(hl_lds + (size_t)SLOTS * sizeof(A));
  uint32_t *sl = reinterpret_cast<uint32_t *>(hl_lds + (size_t)SLOTS * (sizeof(A) + sizeof(B)));
  uint32_t *tag = sl + SLOTS;  // bin + 1 of the slot's owner, 0 while free
  const P ne = Op::identity();
  for (int i = threadIdx.x; i < SLOTS; i += HL_BLOCK) {
    sa[i] = ne.a;
    sb[i] = ne.b;
    sl[i] = 0u;
    tag[i] = 0u;
  }
  __syncthreads();
  auto update_global = [&](int64_t bin, const P &mine) {
    hl_with_lock<P, Op, true>(&locks[bin], [&] {
      P cur;
      cur.a = __hip_atomic_load(dest_a + bin, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      cur.b = __hip_atomic_load(dest_b + bin, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const P r = Op::apply(cur, mine);
      __hip_atomic_store(dest_a + bin, r.a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(dest_b + bin, r.b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    });
  };
  const int64_t stride = (int64_t)gridDim.x * HL_BLOCK;
  for (int64_t i = (int64_t)blockIdx.x * HL_BLOCK + threadIdx.x; i < n; i += stride) {
    const int64_t bin = (int64_t)is[i];
    if ((uint64_t)bin >= (uint64_t)H) continue;  // out of range: ignored
    const P mine = Pre::apply(xs[i], i);
    const int slot = (int)(bin & (SLOTS - 1));
    const uint32_t want = (uint32_t)bin + 1u;
    uint32_t owner = __hip_atomic_load(&tag[slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (owner == 0u) {
      const uint32_t seen = atomicCAS(&tag[slot], 0u, want);
      owner = seen == 0u ? want : seen;
    }
    if (owner == want) {
      hl_with_lock<P, Op>(&sl[slot], [&] {
        P cur;
        cur.a = sa[slot];
        cur.b = sb[slot];
        const P r = Op::apply(cur, mine);
        sa[slot] = r.a;
        sb[slot] = r.b;
      });
    } else {
      update_global(bin, mine);
    }
  }
  __syncthreads();
  for (int slot = threadIdx.x; slot < SLOTS; slot += HL_BLOCK) {
    const uint32_t owner = tag[slot];
    if (owner == 0u) continue;
    P mine;
    mine.a = sa[slot];
    mine.b = sb[slot];
    if (bits_equal_pair(mine, ne)) continue;
    update_global((int64_t)owner - 1, mine);
  }
}

// dest_a, dest_b: H bins each, holding the values to combine with (as
// reduce_by_index takes them); locks: H 32-bit words, all zero, zero again
// afterwards.  Up to HL_MAX_BINS bins are accumulated per block in LDS; with
// more, a block caches the bins it meets first in LDS and updates the others
// in place under the locks.
template <class Tin, class A, class B, class P, class Pre, class Op, class I>
static int launch_hist_locked(hipStream_t s, const I *is, const Tin *xs, int64_t n, A *dest_a,
                              B *dest_b, uint32_t *locks, int64_t H) {
  static_assert(Op::commutative, "reduce_by_index needs a commutative operator");
  if (n < 0 || H < 0) return FA_EINVAL;
  if (H == 0 || n == 0) return 0;
  if (is == nullptr || xs == nullptr || dest_a == nullptr || dest_b == nullptr || locks == nullptr)
    return FA_EINVAL;
  int dev = 0, cus = NUM_CUS_HINT;
  if (hipGetDevice(&dev) == hipSuccess)
    (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (H > HL_MAX_BINS) {
    if (H > ((int64_t)1 << 31)) return FA_EINVAL;  // a slot's tag is bin + 1 in 32 bits
    auto cached = hist_locked_cached_kernel<Tin, A, B, P, Pre, Op, I>;
    constexpr int cached_lds = HL_MAX_BINS * (int)(sizeof(A) + sizeof(B) + 8);
    static const hipError_t raised_cached = hipFuncSetAttribute(
        (const void *)cached, hipFuncAttributeMaxDynamicSharedMemorySize, cached_lds);
    if (raised_cached != hipSuccess) return (int)raised_cached;
    const int64_t want = ceil_div(n, (int64_t)HL_BLOCK * 8);
    const int grid = (int)(want < 1 ? 1 : (want > cus ? cus : want));
    hipLaunchKernelGGL(cached, dim3(grid), dim3(HL_BLOCK), cached_lds, s, is, xs, n, dest_a, dest_b,
                       locks, H);
    return launch_status();
  }
  const size_t lds = (size_t)H * (sizeof(A) + sizeof(B) + 4);
  const int64_t want = ceil_div(n, (int64_t)HL_BLOCK * 8);
  const int grid = (int)(want < 1 ? 1 : (want > cus ? cus : want));
  auto kernel = hist_locked_kernel<Tin, A, B, P, Pre, Op, I>;
  static const hipError_t raised = hipFuncSetAttribute(
      (const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
      HL_MAX_BINS * (int)(sizeof(A) + sizeof(B) + 4));
  if (raised != hipSuccess) return (int)raised;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(HL_BLOCK), lds, s, is, xs, n, dest_a, dest_b, locks, H);
  return launch_status();
}

}  // namespace fa

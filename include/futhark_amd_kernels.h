/*
 * futhark_amd_kernels.h -- C ABI of the gfx950 SegOp kernel library
 * (libfuthark_amd_kernels.so).
 *
 * Each launcher below stands where the Futhark GPU backends place one or more
 * generated `gpu_kernel_<name>(ctx, grid..., block..., shared_bytes, args...)`
 * host wrappers (reference: src/Futhark/CodeGen/Backends/GPU.hs:31-69) around
 * kernels emitted by the SegOp code generators
 * (src/Futhark/CodeGen/ImpGen/GPU/{SegRed,SegScan/SinglePass,SegHist,SegMap}.hs).
 * Instead of kernel text compiled at context creation, the kernels are
 * hand-written HIP compiled offline for gfx950; the launcher picks grid, block
 * and LDS sizes itself.
 *
 * Conventions
 *  - plain C: pointers and sizes only.  All data pointers are DEVICE pointers.
 *  - every call is asynchronous on `stream` (a hipStream_t passed as void*).
 *  - scratch memory is supplied by the caller (the runtime's pooled allocator);
 *    `fa_*_scratch_bytes` reports how much a call needs.  No launcher
 *    allocates or frees device memory.
 *  - return value: 0 on success, a positive hipError_t value if a HIP call
 *    failed, or a negative FA_E* code for an argument the library rejects.
 */
#ifndef FUTHARK_AMD_KERNELS_H
#define FUTHARK_AMD_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *fa_stream_t; /* hipStream_t */

/* Element types (Futhark primitive types that occur on the path). */
typedef enum {
  FA_I32 = 0,
  FA_I64 = 1,
  FA_F32 = 2,
  FA_F64 = 3,
  FA_U32 = 4,
  FA_U64 = 5,
  FA_F16 = 6,  /* IEEE binary16 bits in a uint16_t (docs/c-api.rst:229-233) */
  FA_BF16 = 7, /* bfloat16 bits in a uint16_t: f32 = bits << 16 */
  /* 8- and 16-bit integers: element types of fa_seghist only (the types
   * rts/c/atomics8.h and atomics16.h exist for). */
  FA_I8 = 8,
  FA_U8 = 9,
  FA_I16 = 10,
  FA_U16 = 11,
  /* A pair of i32, (a, b), standing for the map x -> a*x + b modulo 2^32
   * (8 bytes, a first): the element type of FA_COMPOSE, scans only. */
  FA_I32X2 = 12,
  FA_DTYPE_COUNT
} fa_dtype;

/* Scalar operators with the neutral element the kernels use for padding:
 * ADD: 0;  MAX: lowest (INT_MIN / -inf);  MIN: highest (INT_MAX / +inf).
 * Semantics are those of rts/c/scalar.h: two's-complement wrap-around add
 * (scalar.h:29-30), smax/smin (scalar.h:488-503), fmaxf/fminf, i.e. NaN-ignoring
 * (scalar.h:931-934). */
/* FA_AND, FA_OR, FA_XOR: integer types only (neutral elements -1, 0, 0).
 * FA_COMPOSE: FA_I32X2 only, (a1, b1) then (a2, b2) = (a1*a2, a2*b1 + b2) with
 * wrap-around arithmetic, neutral (1, 0): composition of affine maps, the
 * operator of linear recurrences.  Associative and NOT commutative; it exists
 * so that the order in which the scans combine their operands is observable
 * (the reference's single-pass scan keeps operand order, so non-commutative
 * operators are legal there: SegScan/SinglePass.hs:738-746). */
typedef enum {
  FA_ADD = 0, FA_MAX = 1, FA_MIN = 2, FA_AND = 3, FA_OR = 4, FA_XOR = 5, FA_COMPOSE = 6, FA_OP_COUNT
} fa_op;

#define FA_EINVAL (-1)   /* bad argument (null pointer, negative size, ...) */
#define FA_ENOTSUP (-2)  /* dtype/op combination not built */
#define FA_ESCRATCH (-3) /* scratch buffer too small */
#define FA_EALIGN (-4)   /* pointer not aligned as the kernel requires */

/* Human-readable text for a return code (static storage). */
const char *fa_strerror(int code);

/* Library/ABI version: major*1000 + minor. */
int fa_version(void);

/* Thresholds behind the launchers' choice of code path, the counterpart of
 * the threshold and shared_memory tuning parameters a compiled program exposes
 * (src/Futhark/CodeGen/ImpGen/GPU/Base.hs:118-120, rts/c/gpu.h:93-135).  They are
 * kept per calling thread (a launcher reads the values of the thread that calls
 * it; a new thread starts with the defaults); a field that is 0 means the
 * built-in default.
 *   segred_small_threshold  rows of a regular segmented reduce up to this many
 *                           elements are folded by groups of lanes, longer
 *                           ones by whole blocks (default 8192)
 *   hist_lds_bins_max       most bins (of 4 bytes; half as many of 8) one LDS
 *                           range of a histogram holds (default and upper
 *                           limit 32768); four ranges fit one launch, more
 *                           bins go through the partitioned path
 *   matmul_pad_min_work     least M*N*K*batch for which shapes off the tile
 *                           grid run on padded copies (default 2^24)
 *   scan_tickets_by_block   how a block of the single-pass scan picks the ticket
 *                           counter it draws tiles from.  0 (default): by the
 *                           order in which blocks start; the scan finishes
 *                           whenever eight of its blocks can be resident at the
 *                           same time, on any CUs.  Nonzero: by block index,
 *                           which saves an atomic on one address per block and
 *                           the wait for the first ticket (2-3 us per launch)
 *                           and needs all blocks of the launch (one per CU at
 *                           most) resident at the same time: for callers that
 *                           know the launch has the device to itself (no CU
 *                           mask, no other kernels that wait for something
 *                           while they hold CUs)
 *   sort_wide_positions     nonzero: the radix sort counts and scatters with
 *                           64-bit positions whatever the number of keys (0:
 *                           only from 2^32 - 1 keys on), so that this path can
 *                           be exercised without 16 GiB of keys */
typedef struct fa_tuning {
  int64_t segred_small_threshold;
  int64_t hist_lds_bins_max;
  int64_t matmul_pad_min_work;
  int64_t scan_tickets_by_block;
  int64_t sort_wide_positions;
} fa_tuning;
void fa_set_tuning(const fa_tuning *t); /* NULL: all defaults */
void fa_get_tuning(fa_tuning *out);     /* the values in effect */

/* ------------------------------------------------------------------ SegRed
 * Non-segmented reduction `reduce op ne xs`.
 * Replaces: segred_nonseg (SegRed.hs:327-394): stage one, per-block partials,
 * last-block-finishes stage two with an atomic counter (SegRed.hs:923-1047).
 * out: one element.  scratch: at least fa_segred_scratch_bytes(), under the
 * zero-once / increasing-epoch protocol described at fa_segscan (the same
 * buffer may serve both). */
size_t fa_segred_scratch_bytes(fa_dtype t);
int fa_segred_nonseg(fa_stream_t stream, fa_dtype t, fa_op op,
                     const void *xs, int64_t n, void *out,
                     void *scratch, size_t scratch_bytes, uint32_t epoch);

/* Regular segmented reduction `map (reduce op ne) xss`, xss : [m][k] row-major.
 * Replaces: segred_small / segred_large (SegRed.hs:396-636).  No scratch. */
int fa_segred_regular(fa_stream_t stream, fa_dtype t, fa_op op,
                      const void *xss, int64_t m, int64_t k, void *out);
/* The same with a workspace of fa_segred_regular_workspace_bytes() bytes
 * (16-byte aligned; 0 bytes for most shapes): a few very long rows are then cut
 * into pieces that fill the chip and folded in two stages, as the reference's
 * large-segments case spreads a segment over several blocks (SegRed.hs:507-636). */
size_t fa_segred_regular_workspace_bytes(fa_dtype t, int64_t m, int64_t k);
int fa_segred_regular_ws(fa_stream_t stream, fa_dtype t, fa_op op,
                         const void *xss, int64_t m, int64_t k, void *out,
                         void *workspace, size_t workspace_bytes);

/* Reduction with a vectorised operator, `reduce (map2 op) (replicate k ne) xss`
 * with xss : [n][k] row-major: out[j] = fold over i of xss[i][j], k results
 * (the reference interchanges the loops of such a SegRed so that each thread
 * folds one element of the vector, SegRed.hs:274-290).  n = 0 gives k neutral
 * elements.  workspace: fa_segred_columns_workspace_bytes() bytes, 16-byte
 * aligned, contents irrelevant; without it one block per column strip folds
 * all rows. */
size_t fa_segred_columns_workspace_bytes(fa_dtype t, int64_t n, int64_t k);
int fa_segred_columns(fa_stream_t stream, fa_dtype t, fa_op op,
                      const void *xss, int64_t n, int64_t k, void *out,
                      void *workspace, size_t workspace_bytes);

/* ----------------------------------------------------------------- SegScan
 * Single-pass scan with decoupled look-back.
 * Replaces: segscan (SegScan/SinglePass.hs:327-879) plus the status-flag fill
 * kernel the reference launches before it (SinglePass.hs:379-389).
 *
 * flags == NULL : `scan op ne xs`.
 * flags != NULL : the flag-tuple operator of Pass/Flatten/Builtins.hs:374-393,
 *   (fx,x) (+) (fy,y) = (fx||fy, if fy then y else x op y), neutral (false,ne);
 *   flags is one byte per element, nonzero = a segment starts here.
 * exclusive != 0: out[i] = (inclusive result)[i-1] within the segment, `ne` at
 *   i == 0 and at segment starts (prelude/soacs.fut:212-215 for the
 *   unsegmented case).
 *
 * scratch protocol: the buffer must have been zero-filled once when it was
 * allocated; after that it may be passed to any number of fa_segscan calls
 * provided `epoch` is strictly larger on every call
 * (1 <= epoch < 2^28; zero-fill again before wrapping).  Tile descriptors
 * carry the epoch, so no per-call clearing kernel is needed. */
size_t fa_segscan_scratch_bytes(fa_dtype t, int64_t n);
/* Elements of type t per tile (the unit of the look-back: one descriptor per
 * tile; the reference's B * chunk elements of a virtual block,
 * SinglePass.hs:32-48).  0 for types the scan does not take. */
int64_t fa_segscan_tile_elems(fa_dtype t);
int fa_segscan(fa_stream_t stream, fa_dtype t, fa_op op,
               const void *xs, const uint8_t *flags, int64_t n, int exclusive,
               void *out, void *scratch, size_t scratch_bytes, uint32_t epoch);

/* The same over rows of equal length, `map (scan op ne) xss` with xss : [m][k]
 * (SegScan with segment dimensions, SegScan/SinglePass.hs:327-361): the scan
 * restarts at every multiple of k.  No flag array exists or is read.  Scratch
 * and epoch as for fa_segscan with n = m * k. */
int fa_segscan_rows(fa_stream_t stream, fa_dtype t, fa_op op,
                    const void *xss, int64_t m, int64_t k, int exclusive,
                    void *out, void *scratch, size_t scratch_bytes, uint32_t epoch);

/* fa_segscan for callers that cannot allocate or pass a workspace: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It
 * has no counterpart in the reference.  The look-back scratch is a fixed
 * array inside the library (a header and 256 KiB of tile descriptors, 16384
 * tiles: 234 881 024 four-byte or 117 440 512 eight-byte elements; one copy per
 * GPU, held until the process
 * ends), its epoch lives in that array and is advanced on the device, so
 * identical launches may be repeated.  No device memory is allocated or
 * freed.  n beyond fa_segscan_static_max_n(t) returns FA_ESCRATCH.  All calls
 * on one GPU share the array: calls that overlap in time on one GPU race.
 * fa_segscan_static_init() resolves the array's address on the current device
 * ahead of the first call (which otherwise does it). */
int64_t fa_segscan_static_max_n(fa_dtype t);
int fa_segscan_static_init(void);
int fa_segscan_static(fa_stream_t stream, fa_dtype t, fa_op op,
                      const void *xs, const uint8_t *flags, int64_t n, int exclusive,
                      void *out);

/* Irregular segmented reduction (Pass/Flatten/Builtins.hs:582-602):
 *   out[i] = lens[i] == 0 ? ne : segscan(flags-from-offsets, vs)[offsets[i]+lens[i]-1]
 * computed without materialising the scan.  Segments must be in order and
 * disjoint (offsets non-decreasing, offsets[i] + lens[i] <= offsets[i+1], all
 * within [0,n]); elements between segments are ignored.  `scratch` is plain
 * workspace of fa_segred_irregular_scratch_bytes(t, n) bytes, 16-byte aligned;
 * its contents on entry do not matter. */
size_t fa_segred_irregular_scratch_bytes(fa_dtype t, int64_t n);
int fa_segred_irregular(fa_stream_t stream, fa_dtype t, fa_op op,
                        const void *vs, int64_t n,
                        const int64_t *offsets, const int64_t *lens, int64_t m,
                        void *out, void *scratch, size_t scratch_bytes);

/* fa_segred_irregular with the check of fa_segments_check (below) done by its
 * first kernel, which reads every offset and length anyway: one launch less
 * than the check followed by the reduction. */
int fa_segred_irregular_checked(fa_stream_t stream, fa_dtype t, fa_op op,
                                const void *vs, int64_t n,
                                const int64_t *offsets, const int64_t *lens, int64_t m,
                                void *out, void *scratch, size_t scratch_bytes,
                                int32_t *failure, int32_t code);

/* Checks what fa_segred_irregular requires of its segments (in order, disjoint,
 * inside [0, n)): stores `code` into *failure (device-visible memory, e.g. a
 * pinned host word) when they are not, and leaves it alone otherwise.  A
 * compiled Futhark program reports an out-of-bounds index at the next
 * synchronisation in the same way (global_failure, rts/c/gpu.h). */
int fa_segments_check(fa_stream_t stream, const int64_t *offsets, const int64_t *lens,
                      int64_t m, int64_t n, int32_t *failure, int32_t code);

/* ----------------------------------------------------------------- SegHist
 * `reduce_by_index dest op ne is vs` (prelude/soacs.fut:132-146): for every i
 * with 0 <= is[i] < H, dest[is[i]] = dest[is[i]] op vs[i]; other indices are
 * ignored (SegHist.hs:450-458,750-755).  dest is updated in place.
 * Replaces: seghist_local / seghist_global and the SegRed over sub-histograms
 * (SegHist.hs:377-467,576-828,1137-1186).  `is` is i32 (is64 == 0) or i64.
 * Element types: every integer type of 8 to 64 bits with add, max, min, and,
 * or, xor; f16, f32, f64 with add, max, min (the table of
 * src/Futhark/CodeGen/ImpGen/GPU.hs:43-90).  Cells narrower than 32 bits are
 * updated by compare-and-swap on the aligned 32-bit word that contains them
 * (rts/c/atomics8.h, atomics16.h), so dest must lie in an allocation that
 * covers whole words.  f16 sums are accumulated in f32 per block and rounded
 * when a block combines its bins into dest.
 * scratch: fa_seghist_scratch_bytes() for the same t, is64, n and H; contents
 * need no initialisation (large H partitions the input into it). */
size_t fa_seghist_scratch_bytes(fa_dtype t, int is64, int64_t n, int64_t H);
int fa_seghist(fa_stream_t stream, fa_dtype t, fa_op op,
               const void *is, int is64, const void *vs, int64_t n,
               void *dest, int64_t H, void *scratch, size_t scratch_bytes);

/* Segmented form, `map2 (hist op ne H_seg) iss vss` over [m][seg_len] inputs
 * (SegHist.hs:1057-1136 with segment dimensions; tests/hist/segmented.fut):
 * dest is [m][H_seg], row r receives the elements of row r whose index lies in
 * [0, H_seg).  t is FA_I32, FA_I64, FA_F32 or FA_F64. */
size_t fa_seghist_segmented_scratch_bytes(fa_dtype t, int64_t m, int64_t seg_len, int64_t H_seg);
int fa_seghist_segmented(fa_stream_t stream, fa_dtype t, fa_op op,
                         const void *is, int is64, const void *vs,
                         int64_t m, int64_t seg_len, void *dest, int64_t H_seg,
                         void *scratch, size_t scratch_bytes);

/* Histograms with a shape: bins laid out as [H0][H1] vectors of m elements.
 * Update u carries the index (is[u], js[u]) and the vector vss[u][0..m); when
 * both coordinates are in range, dest[is[u]][js[u]][c] = op(that, vss[u][c])
 * for every c.  js == NULL (then H1 must be 1) is the one-dimensional
 * `reduce_by_index dest (map2 op) (replicate m ne) is vss` (a HistOp with an
 * operator shape, SegHist.hs:1057-1136; tests/hist/array.fut); m == 1 with js
 * is `reduce_by_index_2d` (prelude/soacs.fut:149-150; tests/hist/hist2d.fut).
 * is and js have the same width (is64).  t is FA_I32, FA_I64, FA_F32 or FA_F64. */
size_t fa_seghist_shaped_scratch_bytes(fa_dtype t, int is64, int64_t n_updates,
                                       int64_t H0, int64_t H1, int64_t m);
int fa_seghist_shaped(fa_stream_t stream, fa_dtype t, fa_op op,
                      const void *is, const void *js, int is64, const void *vss,
                      int64_t n_updates, void *dest, int64_t H0, int64_t H1, int64_t m,
                      void *scratch, size_t scratch_bytes);

/* -------------------------------------------------------------- radix sort
 * Stable LSD radix sort with 8-bit digits: per pass a digit histogram
 * (SegHist), an exclusive scan of the counts (SegScan) and a ranked scatter
 * (cf. tests/issue2234.fut:10-58 for the composition, 2-bit digits there).
 * key_bytes is 4 or 8; keys compare as unsigned.  val_bytes is 0, 4 or 8.
 * keys_in/vals_in are not modified; the result lands in keys_out/vals_out.
 * keys_tmp/vals_tmp are n-element ping-pong buffers.  begin_bit/end_bit select
 * the key bits that take part (multiple of 8 apart).  Positions are unsigned
 * 32-bit numbers below 2^32 - 1 keys and 64-bit ones from there on. */
size_t fa_radix_sort_scratch_bytes(int64_t n);
int fa_radix_sort(fa_stream_t stream, int key_bytes, int val_bytes,
                  const void *keys_in, void *keys_out, void *keys_tmp,
                  const void *vals_in, void *vals_out, void *vals_tmp,
                  int64_t n, int begin_bit, int end_bit,
                  void *scratch, size_t scratch_bytes);

/* ------------------------------------------------- tiled SegMap (matmul)
 * C[b][i][j] = sum_k A[b][i][k] * B[b][k][j], all row-major, f32 output and
 * f32 accumulation.  in_t is FA_F32, FA_F16 or FA_BF16.
 * Replaces: the block/register-tiled segmap_intrablock that
 * mmBlkRegTiling produces (src/Futhark/Optimise/BlkRegTiling.hs:463-621). */
int fa_matmul(fa_stream_t stream, fa_dtype in_t,
              const void *A, const void *B, float *C,
              int64_t batch, int64_t M, int64_t N, int64_t K);
/* The same with a workspace of fa_matmul_workspace_bytes() bytes (256-byte
 * aligned; may be NULL when that is 0).  Shapes the MFMA kernels do not take
 * directly (M or N not a multiple of 256, K not a multiple of 64, or 16 for
 * f32) then run on zero-padded copies of the operands instead of on the scalar
 * kernel, when the padding costs less than that (mmBlkRegTiling guards every
 * load and store instead, BlkRegTiling.hs:219-254). */
size_t fa_matmul_workspace_bytes(fa_dtype in_t, int64_t batch, int64_t M, int64_t N, int64_t K);
int fa_matmul_ws(fa_stream_t stream, fa_dtype in_t,
                 const void *A, const void *B, float *C,
                 int64_t batch, int64_t M, int64_t N, int64_t K,
                 void *workspace, size_t workspace_bytes);

/* Scan with a vector operator: out[i][j] = xss[0][j] op ... op xss[i][j] for
 * xss, out : [n][k], without a transposed copy.  Replaces: the SegScan of
 * `scan (map2 op) (replicate k ne) xss`, which the reference compiles with its
 * two-pass scan (src/Futhark/CodeGen/ImpGen/GPU/SegScan/TwoPass.hs; the
 * single-pass kernel refuses array operators, SegScan/SinglePass.hs
 * canBeSinglePass).  Takes rows of whole 1 KiB strips (k * element size a
 * multiple of 1024) of 4- or 8-byte elements: fa_vecscan_workspace_bytes is 0
 * for every other shape and fa_vecscan then returns FA_ENOTSUP (transpose with
 * fa_map_transpose, scan rows with fa_segscan_rows, transpose back).  The
 * workspace's contents are irrelevant; xss, out and workspace 16-byte aligned. */
size_t fa_vecscan_workspace_bytes(fa_dtype t, int64_t n, int64_t k);
int fa_vecscan(fa_stream_t stream, fa_dtype t, fa_op op, const void *xss, int64_t n, int64_t k,
               void *out, void *workspace, size_t workspace_bytes);

/* ------------------------------------------------ builtin data movement
 * Batched 2-D transpose: dst[b][j][i] = src[b][i][j], src : [batch][rows][cols].
 * Replaces: map_transpose_{1,2,4,8}b and their low_height / low_width / small /
 * large variants (rts/opencl/transpose.cl, chosen in rts/c/gpu.h:333-461). */
int fa_map_transpose(fa_stream_t stream, int elem_bytes,
                     void *dst, const void *src,
                     int64_t batch, int64_t rows, int64_t cols);

/* Copy between two index functions over the same shape:
 *   dst[dst_offset + sum_k i_k*dst_strides[k]] = src[src_offset + sum_k i_k*src_strides[k]]
 * for every index (i_0..i_{rank-1}) of `shape`; offsets and strides count
 * elements of elem_bytes (1, 2, 4, 8) bytes, strides may be negative,
 * rank <= 8.  The regions must not overlap.  The copy runs as a flat device
 * copy, as a batched transpose or element by element, decided as the reference
 * decides (rts/c/copy.h:55-190; lmad_copy_gpu2gpu_{1,2,4,8}b,
 * rts/c/gpu.h:484-586); *path, if not NULL, says which. */
enum { FA_LMAD_NOTHING = 0, FA_LMAD_FLAT = 1, FA_LMAD_TRANSPOSE = 2, FA_LMAD_GENERAL = 3 };
int fa_lmad_copy(fa_stream_t stream, int elem_bytes,
                 void *dst, int64_t dst_offset, const int64_t *dst_strides,
                 const void *src, int64_t src_offset, const int64_t *src_strides,
                 const int64_t *shape, int rank, int *path);

/* Fill n elements of elem_bytes (1,2,4,8) each with the given bit pattern.
 * Replaces: builtin#replicate_* (ImpGen/GPU/Base.hs:1274-1350). */
int fa_replicate(fa_stream_t stream, int elem_bytes, void *dst, int64_t n,
                 uint64_t pattern);

/* dst[i] = start + i*step for i < n, i32/i64 (ImpGen/GPU/Base.hs:1353-1436). */
int fa_iota(fa_stream_t stream, fa_dtype t, void *dst, int64_t n,
            int64_t start, int64_t step);

/* ---------------------------------------------- per-program operators (proofs)
 * SegOps instantiated from include/futhark_amd_segops.hpp with operators and
 * fused maps outside the fixed set above (csrc/kernels/custom_ops.hip); they
 * stand for the kernels the reference generates for a program's own lambdas
 * (SegBinOp with tuples and SegPostOp, src/Futhark/IR/SegOp.hs:138-155).
 * Scratch and epoch as for fa_segred_nonseg / fa_segscan.
 *   argmax on (value, index) pairs of i32: the larger value, the smaller index
 *   among equal values; neutral (INT32_MIN, INT32_MAX).
 *   fa_reduce_argmax_i32: over zip xs (iota n), the pair made on the way in; out2: 2 x i32
 *   fa_scan_argmax_i32:   pairs [n][2]i32 in and out, optionally segmented by flags
 *   fa_reduce_compose_i32: fold of affine maps (FA_COMPOSE, not commutative) in
 *                          element order (SegRed.hs:836-921); out2: 2 x i32
 *   fa_sumsq_f32:         reduce (+) 0 (map (\x -> x*x) xs)
 *   fa_reduce_summax_f32: (reduce (+) 0 xs, reduce f32.max (-inf) xs) in one kernel, two
 *                         operators side by side (SegRed.hs:157-199); out2: 2 x f32
 *   fa_scan_norm_f32:     map sqrt (scan (+) 0 (map (\x -> x*x) xs))
 *   fa_hist_argmax_i32:   reduce_by_index with argmax into dest [H][2]i32 (updated
 *                         in place), bins locked while updated because the tuple's
 *                         components live in two arrays (ImpGen/GPU/Base.hs:769-842):
 *                         up to 8192 bins in sub-histograms in LDS, more in place
 *                         in global memory (SegHist.hs:377-467);
 *                         H <= fa_hist_argmax_max_bins(); workspace of
 *                         fa_hist_argmax_workspace_bytes(H) bytes, contents irrelevant. */
/* The same operators in the segmented forms (a program's own operator in
 * `map (reduce op ne)`, `map (scan op ne)` and in a reduction over irregular
 * segments; SegRed.hs:396-636, SegScan/SinglePass.hs:327-361,
 * Pass/Flatten/Builtins.hs:570-602):
 *   fa_segreduce_argmax_i32:  xss [m][k]i32 -> out [m][2]i32, (max, first column of it)
 *                             per row, (i32.lowest, i32.highest) for k = 0
 *   fa_segreduce_compose_i32: abss [m][k][2]i32 -> out [m][2]i32, the maps of a row
 *                             composed in element order
 *   fa_scanrows_argmax_i32:   pairs [m][k][2]i32 -> out of the same shape, scanned per
 *                             row; scratch and epoch as for fa_segscan with n = m * k
 *   fa_segred_argmax_i32:     pairs [n][2]i32, segments (offsets[i], lens[i]) in order
 *                             and not overlapping -> out [m][2]i32;
 *                             workspace of fa_segred_argmax_workspace_bytes(n) bytes,
 *                             16-byte aligned, contents irrelevant */
int fa_segreduce_argmax_i32(fa_stream_t stream, const int32_t *xss, int64_t m, int64_t k,
                            int32_t *out);
int fa_segreduce_compose_i32(fa_stream_t stream, const int32_t *abss, int64_t m, int64_t k,
                             int32_t *out);
int fa_scanrows_argmax_i32(fa_stream_t stream, const int32_t *pairs, int64_t m, int64_t k,
                           int32_t *out, void *scratch, size_t scratch_bytes, uint32_t epoch);
size_t fa_segred_argmax_workspace_bytes(int64_t n);
int fa_segred_argmax_i32(fa_stream_t stream, const int64_t *offsets, const int64_t *lens, int64_t m,
                         const int32_t *pairs, int64_t n, int32_t *out, void *workspace,
                         size_t workspace_bytes, void *scratch, size_t scratch_bytes,
                         uint32_t epoch);
int fa_reduce_argmax_i32(fa_stream_t stream, const int32_t *xs, int64_t n, int32_t *out2,
                         void *scratch, size_t scratch_bytes, uint32_t epoch);
int fa_scan_argmax_i32(fa_stream_t stream, const int32_t *pairs, const uint8_t *flags, int64_t n,
                       int exclusive, int32_t *out, void *scratch, size_t scratch_bytes,
                       uint32_t epoch);
int fa_reduce_compose_i32(fa_stream_t stream, const int32_t *abs, int64_t n, int32_t *out2,
                          void *scratch, size_t scratch_bytes, uint32_t epoch);
int fa_sumsq_f32(fa_stream_t stream, const float *xs, int64_t n, float *out,
                 void *scratch, size_t scratch_bytes, uint32_t epoch);
int fa_reduce_summax_f32(fa_stream_t stream, const float *xs, int64_t n, float *out2,
                         void *scratch, size_t scratch_bytes, uint32_t epoch);
int fa_scan_norm_f32(fa_stream_t stream, const float *xs, int64_t n, float *out,
                     void *scratch, size_t scratch_bytes, uint32_t epoch);
/* map (\r -> let t = reduce (+) 0 r in map (/ t) (scan (+) 0 r)) xss for
 * xss : [m][k]f32: a reduction, a scan and a map over a row by the block that
 * owns it.  Replaces: the intra-block SegOps of a kernel at block level
 * (src/Futhark/CodeGen/ImpGen/GPU/Block.hs:357-615). */
int fa_rows_fraction_f32(fa_stream_t stream, const float *xss, int64_t m, int64_t k, float *out);
size_t fa_hist_argmax_workspace_bytes(int64_t H);
int64_t fa_hist_argmax_max_bins(void);
int fa_hist_argmax_i32(fa_stream_t stream, const int32_t *is, const int32_t *xs, int64_t n,
                       int32_t *dest, int64_t H, void *workspace, size_t workspace_bytes);

/* Measurement aid (no counterpart in the reference): the rate the matrix cores
 * sustain on registers alone.  `blocks` blocks of four waves each issue `iters`
 * rounds of sixteen independent 32x32x16 MFMAs (f16 or bf16 in, f32 accumulate)
 * on fragments read once from `operands` (8 KiB of 16-bit values, distributed
 * like the caller's matrices: the sustained clock depends on them).  *flop, if
 * not NULL, receives the number of floating-point operations of the launch;
 * `sink` is one float the kernel may write. */
int fa_mfma_probe(fa_stream_t stream, fa_dtype in_t, const void *operands, int blocks,
                  int iters, float *sink, double *flop);

/* Plain device copy kernel used for calibration of bandwidth counters. */
int fa_copy(fa_stream_t stream, void *dst, const void *src, size_t bytes);

#ifdef __cplusplus
}
#endif
#endif /* FUTHARK_AMD_KERNELS_H */

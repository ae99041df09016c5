/* hordead_gpu.h -- C ABI of the MI355X (gfx950) tensor backend for horde-ad.
 *
 * This is the boundary a `Gpu` carrier of horde-ad's tensor classes binds with
 * `foreign import ccall`: one entry point per array primitive that the
 * `BaseTensor Concrete` instance (src/HordeAd/Core/OpsConcrete.hs:97-775)
 * obtains from ox-arrays or from its own Haskell index loops.  Everything is
 * plain C: opaque handles, pointers, sizes, an `int` status.  No exception,
 * no C++ type and no torch type crosses it.
 *
 * Model
 *   - `hgpu_ctx`   one device + one in-order HIP stream + a caching allocator.
 *   - `hgpu_array` an immutable strided VIEW (dtype, rank, shape, element
 *                  strides, element offset) of a reference-counted device
 *                  buffer.  Strides may be 0 (replicate) or negative (reverse),
 *                  exactly the freedom ox-arrays' arrays have
 *                  (src/HordeAd/Core/CarriersConcrete.hs:150-155).
 *   - Logical element order is row-major over `shape`; every compute entry
 *     point returns a dense row-major array.
 *   - All work is enqueued on the context's stream; only `hgpu_download`,
 *     `hgpu_read_scalar`, `hgpu_compare_all` and `hgpu_sync` wait for it.
 *   - `hgpu_release` may be called from any thread (it is what a Haskell
 *     `ForeignPtr` finalizer calls); the buffer returns to the allocator and
 *     may be reused by later enqueued work, which the in-order stream makes
 *     safe.
 *
 * Status codes: 0 = ok; otherwise `hgpu_last_error` holds a message.  Indices
 * out of bounds in index/gather/scatter/onehot are NOT errors: they have the
 * reference's defined semantics (zeros / skipped), see each entry point.
 */
#ifndef HORDEAD_GPU_H
#define HORDEAD_GPU_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct hgpu_ctx hgpu_ctx;
typedef struct hgpu_array hgpu_array;

#define HGPU_MAX_RANK 16

enum hgpu_status {
  HGPU_OK = 0,
  HGPU_ERR_INVALID = 1,     /* shape/dtype/argument mismatch (the reference calls `error`) */
  HGPU_ERR_OOM = 2,         /* device allocation failed */
  HGPU_ERR_DEVICE = 3,      /* a HIP call failed */
  HGPU_ERR_UNSUPPORTED = 4  /* valid request this build has no kernel for */
};

/* Scalar types: the reference's whitelist (src/HordeAd/Core/Types.hs:135-150,
 * OpsConcrete.hs:1043-1058).  Haskell `Int` is I64; `CInt` is I32; Bool is one
 * byte holding 0 or 1. */
enum hgpu_dtype {
  HGPU_F64 = 0, HGPU_F32 = 1, HGPU_I64 = 2, HGPU_I32 = 3,
  HGPU_I16 = 4, HGPU_I8 = 5, HGPU_BOOL = 6
};

/* Unary opcodes: OpCodeNum1 / OpCode1 (src/HordeAd/Core/AstInterpret.hs:394-421). */
enum hgpu_op1 {
  HGPU_NEG = 0, HGPU_ABS, HGPU_SIGNUM,
  HGPU_RECIP, HGPU_EXP, HGPU_LOG, HGPU_SQRT, HGPU_SIN, HGPU_COS, HGPU_TAN,
  HGPU_ASIN, HGPU_ACOS, HGPU_ATAN, HGPU_SINH, HGPU_COSH, HGPU_TANH,
  HGPU_ASINH, HGPU_ACOSH, HGPU_ATANH,
  HGPU_NOT,           /* notB on Bool (AstInterpret.hs:329-335) */
  HGPU_OP1_COUNT
};

/* Binary opcodes: + and * (AstInterpret.hs:187-188), OpCode2 (:423-429),
 * OpCodeIntegral2 (:431-435) with the divisor-0 rule of Types.hs:394-419
 * (quotH a 0 = a on scalars; arrays replace a 0 divisor by 1,
 * CarriersConcrete.hs:40-56,140-144 -- the two rules agree: quot a 1 = a, and
 * differ for remH: scalar remH a 0 = a, array remH a 0 = rem a 1 = 0; the
 * array rule is HGPU_REM, the scalar rule is HGPU_REM_SCALAR). */
enum hgpu_op2 {
  HGPU_ADD = 0, HGPU_MUL, HGPU_SUB,
  HGPU_DIV, HGPU_POW, HGPU_LOGBASE, HGPU_ATAN2,
  HGPU_QUOT, HGPU_REM, HGPU_REM_SCALAR,
  HGPU_MIN, HGPU_MAX,
  HGPU_AND,           /* &&* on Bool (AstInterpret.hs:336-344) */
  HGPU_OP2_COUNT
};

/* Comparison opcodes (Types.hs:442-452). */
enum hgpu_cmp { HGPU_LEQ = 0, HGPU_EQ = 1, HGPU_LT = 2 };

/* Conversion modes for hgpu_convert. */
enum hgpu_conv {
  HGPU_CONV_CAST = 0,   /* realToFrac / fromIntegral (OpsConcrete.hs:456-532) */
  HGPU_CONV_FLOOR = 1   /* floor: float -> integer (OpsConcrete.hs:455) */
};

/* ---------------------------------------------------------------- context */

/* Creates a context on HIP device `device` (one stream, default priority).
 * No reference counterpart: `Concrete` needs no state (OpsConcrete.hs:97). */
int hgpu_init(int device, hgpu_ctx** ctx);
/* Waits for the stream and frees every cached device block.  Arrays still
 * alive keep their buffers until released. */
int hgpu_shutdown(hgpu_ctx* ctx);
/* Blocks until all enqueued work is complete. */
int hgpu_sync(hgpu_ctx* ctx);
/* Message of the last failed call made on this context by any thread. */
const char* hgpu_last_error(hgpu_ctx* ctx);
/* Allocator statistics: bytes held by live arrays, bytes reserved from the
 * device (live + cached), number of device allocations made so far. */
int hgpu_mem_stats(hgpu_ctx* ctx, uint64_t* in_use, uint64_t* reserved, uint64_t* n_device_allocs);
/* The stream all work is enqueued on, as a `hipStream_t` cast to void*.  The
 * call first enqueues whatever launches the library is holding back (see
 * hgpu_contract_sum_map): a caller that puts work of its own on the stream
 * asks for the stream each time, right before it does. */
void* hgpu_stream(hgpu_ctx* ctx);
/* When `limit` >= 0, the next `limit`-th device allocation and all later ones
 * fail with HGPU_ERR_OOM (host-forced fault injection for tests of the error
 * path); a negative value switches it off. */
int hgpu_inject_alloc_failure(hgpu_ctx* ctx, int64_t limit);

/* Per-launch timing for benchmarks: while enabled every kernel launch has a
 * HIP event pair on the context's stream.  The run-time compiled kernels and
 * the staged matrix products carry their pair (it holds the kernel's own begin
 * and end); the other kernels are bracketed by theirs, which also times the
 * dispatch (a few microseconds more per launch).  The report has one
 * line per kernel family: "name launches total_ms algorithmic_bytes
 * algorithmic_flops".  Enabling (or disabling) clears the records.  on = 2
 * makes the matrix-product labels carry the problem shape. */
int hgpu_profile_enable(hgpu_ctx* ctx, int on);
int hgpu_profile_report(hgpu_ctx* ctx, char* buf, size_t n);

/* Calibration for benchmarks (no reference counterpart): a loop of nothing but
 * one matrix-core instruction on independent accumulators, 16 wavefronts per
 * CU, timed with events on the context's stream.  variant 0: v_mfma_f64_16x16x4,
 * 1: v_mfma_f64_4x4x4 (four blocks), 2: v_mfma_f32_16x16x4, 3: v_mfma_f32_32x32x2.
 * Variants 4, 5, 6: v_mfma_f64_16x16x4 fed as a product kernel feeds it (four
 * wavefronts hold a 64 x 64 tile, fragments read from LDS, a barrier per 16 k,
 * nothing loaded from memory) at one, two and four wavefronts per SIMD.
 * *tflops is what the loop sustains on this device: with its way of feeding
 * the instruction, the ceiling of a product kernel built on it.  Waits for
 * the stream. */
int hgpu_mfma_probe(hgpu_ctx* ctx, int variant, int iters, double* tflops);

/* ----------------------------------------------------------------- memory */

/* tkconcrete/tsconcrete/tconcrete (OpsConcrete.hs:120-124): identity on the
 * CPU, an upload here.  `host` holds prod(shape) elements in row-major order
 * and is borrowed for the call only. */
int hgpu_upload(hgpu_ctx* ctx, int dtype, int rank, const int64_t* shape,
                const void* host, hgpu_array** out);
/* Nested.stoVector (OpsConcrete.hs:144-164, `tstoListLinear`): writes the
 * logical row-major contents of the view to `host`; waits for the stream. */
int hgpu_download(hgpu_ctx* ctx, const hgpu_array* a, void* host);
/* Reads the single element of a one-element array (unConcrete on a scalar,
 * `kfromS`); waits for the stream.  `host` receives one value of a's dtype. */
int hgpu_read_scalar(hgpu_ctx* ctx, const hgpu_array* a, void* host);
int hgpu_retain(hgpu_array* a);
int hgpu_release(hgpu_array* a);

/* sshape/rshape/xshape/tftk (OpsConcrete.hs:99-106): host metadata only. */
int hgpu_rank(const hgpu_array* a);
int hgpu_dtype_of(const hgpu_array* a);
int64_t hgpu_size(const hgpu_array* a);
int hgpu_shape(const hgpu_array* a, int64_t* shape_out);
int hgpu_strides(const hgpu_array* a, int64_t* strides_out);
/* 1 when the view is dense row-major (what `stoVector` can return without a copy). */
int hgpu_is_dense(const hgpu_array* a);

/* ------------------------------------------------- views (no element traffic) */

/* tstranspose (OpsConcrete.hs:647-649): result dim i = source dim perm[i] for
 * i < nperm; the remaining dims keep their place. */
int hgpu_transpose(hgpu_ctx* ctx, const hgpu_array* a, int nperm, const int* perm, hgpu_array** out);
/* tsreshape (OpsConcrete.hs:650-652): a view when the strides allow it, else a
 * dense copy. */
int hgpu_reshape(hgpu_ctx* ctx, const hgpu_array* a, int rank, const int64_t* shape, hgpu_array** out);
/* tsslice (OpsConcrete.hs:641-643) generalised to any dim: elements
 * [start, start+len) of dimension `dim`. */
int hgpu_slice(hgpu_ctx* ctx, const hgpu_array* a, int dim, int64_t start, int64_t len, hgpu_array** out);
/* tsreverse (OpsConcrete.hs:644-646) generalised to any dim. */
int hgpu_reverse(hgpu_ctx* ctx, const hgpu_array* a, int dim, hgpu_array** out);
/* tsreplicateN / tsreplicate0N (OpsConcrete.hs:243-246): new leading dims of
 * stride 0. */
int hgpu_replicate(hgpu_ctx* ctx, const hgpu_array* a, int nprefix, const int64_t* prefix_shape, hgpu_array** out);
/* tsindex / tindexZSScalar (OpsConcrete.hs:1477-1490): fixes the first n dims.
 * Any index out of bounds gives an all-zero array of the remaining shape. */
int hgpu_index_prefix(hgpu_ctx* ctx, const hgpu_array* a, int n, const int64_t* ix, hgpu_array** out);
/* A gather whose index function is affine in the position and provably in
 * bounds (tgatherZSScalar, OpsConcrete.hs:1654-1665, with f linear): the result
 * is a view of a's buffer with the given shape, strides (in elements) and
 * offset relative to a's first element.  Refused (HGPU_ERR_INVALID) when any
 * addressed element would lie outside a's buffer. */
int hgpu_as_strided(hgpu_ctx* ctx, const hgpu_array* a, int rank, const int64_t* shape,
                    const int64_t* strides, int64_t offset, hgpu_array** out);

/* ----------------------------------------------------------------- compute */

/* Dense copy of a view in logical order (what ox-arrays does before handing a
 * strided array to a C kernel that wants a vector). */
int hgpu_materialize(hgpu_ctx* ctx, const hgpu_array* a, hgpu_array** out);
/* Zero-extends every dimension d by lo[d] elements in front and hi[d] behind
 * (the zero rows a gather with out-of-bounds indices produces,
 * OpsConcrete.hs:1488-1490; also slice's VJP, DeltaEval.hs:569-575).  Unlike
 * the other compute entry points the result is dense in the operand's own
 * order of dims in memory (a transposed view pads into a transposed array). */
int hgpu_pad(hgpu_ctx* ctx, const hgpu_array* a, const int64_t* lo, const int64_t* hi, hgpu_array** out);

/* Elementwise Num/Fractional/Floating/IntegralH instances of arrays
 * (CarriersConcrete.hs:40-56,333-343), dispatched from AstN1S/AstR1S/AstPlusS/
 * AstTimesS/AstR2S/AstI2S (AstInterpret.hs:187-194).  Operands have equal
 * shape and dtype. */
int hgpu_ewise1(hgpu_ctx* ctx, int op1, const hgpu_array* a, hgpu_array** out);
int hgpu_ewise2(hgpu_ctx* ctx, int op2, const hgpu_array* a, const hgpu_array* b, hgpu_array** out);
/* Elementwise comparison giving a BOOL array: the lane-batched form of
 * AstLeqK / AstLeqS (AstInterpret.hs:345-366). */
int hgpu_compare(hgpu_ctx* ctx, int cmp, const hgpu_array* a, const hgpu_array* b, hgpu_array** out);
/* Whole-array comparison, one Bool: EqH/OrdH Concrete (CarriersConcrete.hs:
 * 310-331) -- lexicographic over the row-major element sequence.  Waits. */
int hgpu_compare_all(hgpu_ctx* ctx, int cmp, const hgpu_array* a, const hgpu_array* b, int* result);
/* Elementwise conditional, cond BOOL: the lane-batched form of kcond / ifH
 * (OpsConcrete.hs:113-119). */
int hgpu_select(hgpu_ctx* ctx, const hgpu_array* cond, const hgpu_array* a, const hgpu_array* b, hgpu_array** out);
/* tsfloor / tsfromIntegral / tscast / tkcast (OpsConcrete.hs:352-368,455-532). */
int hgpu_convert(hgpu_ctx* ctx, const hgpu_array* a, int dtype, int mode, hgpu_array** out);

/* A chain of the elementwise operations above in one pass.  The program is
 * straight-line code over numbered slots: slots 0 .. n_in-1 are the inputs
 * (views of one shape), slot n_in + k is the result of instruction k, whose
 * operands a, b, c name earlier slots.  `kind` selects the family: OP1 (op =
 * hgpu_op1), OP2 (op = hgpu_op2), CMP (op = hgpu_cmp, result BOOL), SELECT
 * (a = BOOL condition, b, c), CONVERT (op = hgpu_conv mode, dtype = target).
 * outs[i] receives slot out_slots[i] as a dense array.  This is what the
 * interpreter's one-call-per-node stream of `+`, `*`, `sin`, ...
 * (AstInterpret.hs:187-194) becomes when the host layer defers it; results
 * equal those of the single entry points applied in program order. */
enum hgpu_fused_kind { HGPU_FUSED_OP1 = 0, HGPU_FUSED_OP2 = 1, HGPU_FUSED_CMP = 2, HGPU_FUSED_SELECT = 3, HGPU_FUSED_CONVERT = 4 };
typedef struct hgpu_fused_instr { int32_t kind, op, dtype, a, b, c; } hgpu_fused_instr;
int hgpu_fused_map(hgpu_ctx* ctx, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog,
                   int n_out, const int* out_slots, hgpu_array** outs);
/* hgpu_fused_map that also sums: outs[i] = slot out_slots[i] as for
 * hgpu_fused_map, and sums[j] = the sum of all elements of slot sum_slots[j]
 * (a rank-0 array of the slot's type, accumulated in double / int64 in an order
 * fixed by the size), all from ONE pass over the inputs.  An objective
 * `ssum0 (f x y z)` and its gradient (test/simplified/TestAdaptorSimplified.hs:
 * 610-624,682) share most of their program: evaluated together they read x, y, z
 * once.  Inputs must be dense or one broadcast element (else
 * HGPU_ERR_UNSUPPORTED: run hgpu_fused_map and hgpu_fused_sum). */
int hgpu_fused_map_sums(hgpu_ctx* ctx, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog,
                        int n_out, const int* out_slots, hgpu_array** outs, int n_sum, const int* sum_slots, hgpu_array** sums);

/* hgpu_fused_map that also sums one slot over every dim but one:
 * sum[c] = the sum of slot sum_slot over all elements whose index along dim
 * keep_dim is c (a rank-1 array of the slot's floating-point type, accumulated
 * in double in an order fixed by the shape), from the pass that writes outs.
 * The convolution layers add their bias as
 * `stranspose @'[0, 3, 1, 2] $ sreplicate $ sreplicate $ sreplicate bias`
 * (example/MnistCnnShaped2.hs:57-63): the bias's cotangent is the layer's
 * cotangent summed over batch, height and width, and that cotangent is written
 * out anyway for the kernel's gradient.  HGPU_ERR_UNSUPPORTED for arrays of
 * fewer than 2^18 or more than 2^31 elements (run hgpu_fused_map and
 * hgpu_contract). */
int hgpu_fused_map_dimsum(hgpu_ctx* ctx, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog,
                          int n_out, const int* out_slots, hgpu_array** outs, int sum_slot, int keep_dim, hgpu_array** sum);
/* tssum0 of such a program's result (OpsConcrete.hs:229-230), evaluated on the
 * fly: the result itself is never written.  Inputs must be dense or one
 * broadcast element (else HGPU_ERR_UNSUPPORTED: write the result out and sum
 * that).  Accumulates in double / int64 in an order fixed by the size. */
int hgpu_fused_sum(hgpu_ctx* ctx, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, int slot, hgpu_array** out);
/* The first extremum of such a program's result along its trailing n_reduce
 * dims (taken together, row-major), evaluated on the fly: the result itself is
 * never written.  values / indices get the leading dims' shape; an index
 * counts positions within the reduced dims (at most 64 of them).  With this,
 * `maxPool2dUnpaddedS (reluS (conv + bias))` (External/CommonShapedOps.hs:
 * 241-260) reads the convolution once and writes only the pooled maxima and
 * their arguments. */
int hgpu_fused_extremum(hgpu_ctx* ctx, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, int slot, int n_reduce,
                        int want_max, hgpu_array** values, hgpu_array** indices);

/* out[o] = sum_r a[o,r] * b[o,r]  (b == NULL: b = 1), o ranging over the first
 * n_keep dims and r over the rest.  With the free views above this one entry
 * point is tssum / tssumN / tssum0 (OpsConcrete.hs:215-230, b NULL, summed dims
 * transposed behind), tsdot0 (:231-232), tsdot1In (:233-235), tsmatvecmul
 * (:236) and tsmatmul2 (:237-242, which the reference itself defines as
 * dot1In over replicated and transposed views).  Floating-point summation
 * order is unspecified (as it is in ox-arrays) but fixed by the shapes;
 * integers are exact.  The launch of a small reduction may be held back like
 * that of a small product (see hgpu_contract_sum_map): reductions that do not
 * read one another's results then leave as one kernel. */
int hgpu_contract(hgpu_ctx* ctx, const hgpu_array* a, const hgpu_array* b, int n_keep, hgpu_array** out);

/* out = sum_t contract(a[t], b[t], n_keep): the same contraction of n pairs of
 * one shape and dtype, summed.  This is what the cotangent of a parameter
 * that is used once per step of an unrolled recurrence amounts to
 * (DeltaEval.hs:391-595 adds the per-use contributions one by one); when all
 * pairs share one layout and the whole is a matrix product it is one launch
 * whose K chunks run over all pairs.  Summation order is fixed by the shapes. */
int hgpu_contract_sum(hgpu_ctx* ctx, int n, const hgpu_array* const* a, const hgpu_array* const* b, int n_keep, hgpu_array** out);
/* A contraction followed, in the same pass, by an elementwise program over its
 * result -- `maxPool2dUnpaddedS (reluS (conv2dPreservingS ker x + bias))`
 * (example/MnistCnnShaped2.hs:45-64, External/CommonShapedOps.hs:33-44,241-260)
 * reaches the backend as a contraction, `+`, a comparison, a conditional, `*`
 * and an arg-maximum over windows; this entry point runs them as one kernel
 * when the shapes allow and never writes the convolution's own result.
 *   C = hgpu_contract(a, b, n_keep)                       (shape: the kept dims)
 *   program: as for hgpu_fused_map; exactly one entry of `in` is NULL and
 *   stands for C, the others are views of the kept shape;
 *   outs[i] = slot out_slots[i], dense, of the kept shape (n_out may be 0);
 *   when `values` is not NULL: V = the view (view_rank, view_shape,
 *   view_strides in elements, offset 0) of the dense row-major result of slot
 *   ext_slot, and values / indices are the first extremum of V over its
 *   trailing n_reduce dims, as for hgpu_fused_extremum.
 * Results equal those of the single entry points applied one after another. */
int hgpu_contract_map(hgpu_ctx* ctx, const hgpu_array* a, const hgpu_array* b, int n_keep,
                      int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog,
                      int n_out, const int* out_slots, hgpu_array** outs,
                      int ext_slot, int view_rank, const int64_t* view_shape, const int64_t* view_strides,
                      int n_reduce, int want_max, hgpu_array** values, hgpu_array** indices);

/* A SUM of contractions followed, in the same pass, by an elementwise program
 * over the sum: a layer of the reference's recurrent network,
 * `tanh (wX `rmatmul2` x + wS `rmatmul2` s + rtr (rreplicate batch_size b))`
 * (example/MnistRnnRanked2.hs:62-75), reaches the backend as two matrix
 * products, two `+` and a `tanh`, and the head of its cotangent as two
 * products, a `+` and `* (1 - h * h)` (DeltaEval.hs:391-595 adds the two uses
 * of a layer's output).  Neither the products nor their sum are written.
 *   C = sum_t hgpu_contract(a[t], b[t], n_keep); the terms agree in dtype and
 *   in their first n_keep dims, the contracted dims may differ from term to term;
 *   program, in, out_slots, outs: as for hgpu_contract_map (exactly one entry
 *   of `in` is NULL and stands for C; n_out >= 1).
 * When the contracted dims are short (together at most 512 elements, 1024 when
 * the result has at most 160,000 elements -- where a product with a K loop
 * would split K to fill the device and add partial results) and the
 * kept shape has two non-unit dims this is one kernel compiled for the shapes,
 * with the whole contracted dim of a term in LDS; otherwise the single entry
 * points run one after another (a single product that is split in two or
 * three along its contracted dim is added up by the pass that runs the
 * program).  Results equal theirs up to the order of the floating-point sums.
 * The compiled kernel's launch may be held back until the next call that
 * needs the stream (any other launch, copy, synchronisation, hgpu_stream, the
 * ends of a graph capture): held-back products that do not read one another's
 * results then go out as one kernel -- step t + 1 of the first layer of an
 * unrolled recurrence with step t of the second.  The order of results as the
 * stream sees it is the order of the calls; a launch error that shows up late
 * is returned by hgpu_sync. */
int hgpu_contract_sum_map(hgpu_ctx* ctx, int n_terms, const hgpu_array* const* a, const hgpu_array* const* b, int n_keep,
                          int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog,
                          int n_out, const int* out_slots, hgpu_array** outs);

/* hgpu_contract whose operands need not exist in memory.  The cotangent of a
 * pooled, rectified convolution -- `sscatter` at the arg-maxima, times the relu
 * mask (test/simplified/TestMnistPP.hs:734-735) -- is an elementwise expression
 * of small arrays, four times their size, that three contractions consume (the
 * bias, kernel and input gradients).  An operand is either a plain array or
 *   E = slot `slot` of an elementwise program over `in` (views of one shape),
 *   P = E, its dims merged to `mshape` (same element count; row-major, so
 *       merging is free), zero-extended by lo / hi per dim (NULL: none),
 *   operand = the view (rank, shape, strides, offset) of P's dense row-major layout,
 * evaluated while the kernel stages it.  b == NULL is a plain sum of a over the
 * dims behind the first n_keep.  flags bit 0: fail with HGPU_ERR_UNSUPPORTED when
 * no kernel takes the operands in this form, instead of writing them out first
 * (what the call otherwise does: results equal hgpu_fused_map, hgpu_reshape,
 * hgpu_pad, hgpu_as_strided and hgpu_contract applied one after another). */
typedef struct hgpu_operand {
  const hgpu_array* array;              /* not NULL: the operand is this array, the rest is ignored */
  int n_in;
  const hgpu_array* const* in;
  int n_instr;
  const hgpu_fused_instr* prog;
  int slot;
  int rank_m;
  const int64_t* mshape;
  const int64_t* lo;
  const int64_t* hi;
  int rank;
  const int64_t* shape;
  const int64_t* strides;
  int64_t offset;
} hgpu_operand;
int hgpu_contract_operands(hgpu_ctx* ctx, const hgpu_operand* a, const hgpu_operand* b, int n_keep, int flags, hgpu_array** out);

/* hgpu_contract for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  The caller brings the result array `out`
 * (dense, of the operands' dtype, of the kept shape, not sharing memory with an
 * operand); this call makes no device allocation and frees none.  It always
 * takes the HBM-bound reduction kernels (never the matrix-product path, which
 * needs tables and partial products of its own), so floating-point sums may be
 * associated differently from hgpu_contract's when that runs a matrix product;
 * for plain sums and dot products the two agree bit for bit as long as both
 * cut the reduction into the same number of chunks.  The partial sums of a
 * split reduction live in one fixed array of 1 MiB per device, held until the
 * process ends: a request whose partial sums (outputs x chunks x 8 bytes) would
 * exceed it runs with as many chunks as fit, or unsplit when not even two fit
 * (then its sums are associated differently from hgpu_contract's: equal for
 * integers, within rounding for floating point); no valid request is refused
 * for its size.  A result array of the wrong shape, dtype or layout, or one
 * that shares memory with an operand, is HGPU_ERR_INVALID.  Every call on a
 * device uses that device's one array: calls that overlap on one device (two
 * contexts, two streams) race; calls on one context are ordered by its stream. */
int hgpu_contract_noalloc(hgpu_ctx* ctx, const hgpu_array* a, const hgpu_array* b, int n_keep, hgpu_array* out);
/* tsargMin / tsargMax (OpsConcrete.hs:533-534, targMinS :1712-1746): index of
 * the first minimal / maximal element along the LAST dim; result I64 of shape
 * init(shape). */
int hgpu_argminmax_last(hgpu_ctx* ctx, const hgpu_array* a, int want_max, hgpu_array** out);
/* The same pass also hands out the extremal VALUES (values may be NULL):
 * `sgather t (\ix -> ix ++ [kargMax (t !$ ix)])`, the maximum of every pooling
 * window (External/CommonShapedOps.hs:241-260), is then no gather at all. */
int hgpu_extremum_last(hgpu_ctx* ctx, const hgpu_array* a, int want_max, hgpu_array** values, hgpu_array** indices);
/* tsiota (OpsConcrete.hs:535-536): [0, 1, ..., n-1] of the given dtype. */
int hgpu_iota(hgpu_ctx* ctx, int64_t n, int dtype, hgpu_array** out);
/* tsappend / trconcat (OpsConcrete.hs:623-625,638-640): concatenation along
 * dim 0 of n arrays that agree on all other dims. */
int hgpu_concat(hgpu_ctx* ctx, int n, const hgpu_array* const* parts, hgpu_array** out);

/* tsgather / tgatherZSScalar (OpsConcrete.hs:1621-1665):
 *   out[m.., n..] = src[ix[0][m..], ..., ix[n_ix-1][m..], n..]
 * where every ix[j] is an I64 array (any view) of shape shm, and shn is the
 * rest of src's shape after its first n_ix dims.  A position with any index
 * out of bounds yields zeros (OpsConcrete.hs:923-926,1488-1490,1504-1506).
 * Pure data movement: bit-exact. */
int hgpu_gather(hgpu_ctx* ctx, const hgpu_array* src, int n_ix, const hgpu_array* const* ix,
                int rank_m, const int64_t* shm, hgpu_array** out);
/* tsscatter / tscatterZSScalar (OpsConcrete.hs:1581-1619):
 *   out = 0;  out[ix[0][m..], ..., ix[n_ix-1][m..], n..] += src[m.., n..]
 * src has shape shm ++ shn (rank_m leading dims are shm), out has shape
 * shp ++ shn with shp given (n_ix dims).  Positions with an index out of
 * bounds are skipped (OpsConcrete.hs:944-950).  Positions that land on one
 * place are added in ascending row-major order of the positions, starting
 * from zero -- the reference's order (`shsEnum`, OpsConcrete.hs:1594,1613) --
 * without atomics (a stable sort by destination, then every run summed front
 * to back): results are the same from run to run, for every element type of
 * the whitelist, and floating-point sums carry the rounding of that order.
 * `flags`: bit 0 = the caller guarantees distinct positions map to distinct
 * destinations (plain stores, no sort). */
int hgpu_scatter_add(hgpu_ctx* ctx, const hgpu_array* src, int n_ix, const hgpu_array* const* ix,
                     int rank_m, const int64_t* shp, int flags, hgpu_array** out);
/* tsscatter (OpsConcrete.hs:1581-1619) for an index function that is AFFINE in
 * the positions and sends distinct positions to distinct places (the caller's
 * promise; a violation leaves one of the colliding values, it corrupts
 * nothing):
 *   out = 0;  out[c0[0] + sum_d coef[d*n_ix+0]*m_d, ..., n..] = src[m.., n..]
 * for all positions m of src's first rank_m dims; out has shape shp ++ shn.
 * Every position must land inside shp (else HGPU_ERR_INVALID: use
 * hgpu_scatter_add, which skips them).  No index arrays are read; the result
 * keeps src's order of dims in memory and may be a transposed view.  Pure data
 * movement: bit-exact. */
int hgpu_scatter_affine(hgpu_ctx* ctx, const hgpu_array* src, int rank_m, int n_ix, const int64_t* c0,
                        const int64_t* coef, const int64_t* shp, hgpu_array** out);
/* tsoneHot / toneHotS (OpsConcrete.hs:1516-1525): zeros of shape shp ++ shape(v)
 * with v written at prefix index ix; all zeros when ix is out of bounds. */
int hgpu_onehot(hgpu_ctx* ctx, const hgpu_array* v, int n, const int64_t* ix, const int64_t* shp, hgpu_array** out);

/* ------------------------------------------------------------- graphs */

/* A gradient program is evaluated again and again on arrays of the same
 * shapes (ADEngine.hs:266-288, revInterpretArtifact: the artifact is built
 * once, interpreted per batch).  Between hgpu_capture_begin and
 * hgpu_capture_end every compute call of this header is RECORDED instead of
 * executed: the arrays it returns have the right shapes but no contents yet.
 * hgpu_graph_launch then runs the whole recorded sequence as one submission
 * (a HIP graph) and refreshes those arrays in place; it may be called any
 * number of times.  Arrays that existed before the capture are read at every
 * launch (refresh them with hgpu_overwrite to feed a new batch).  The graph
 * does NOT retain them: the caller keeps every array the recording read alive
 * until hgpu_graph_destroy -- a released array's block returns to the
 * allocator, and later launches would read whatever was allocated there next.
 * Entry points that need the host -- upload, download, read_scalar,
 * compare_all, sync -- fail with HGPU_ERR_UNSUPPORTED during a capture: make
 * constants beforehand.  Memory handed out during a capture stays reserved for
 * the graph until hgpu_graph_destroy.  One capture at a time per context; the
 * capturing thread is the only one that may use the context meanwhile. */
typedef struct hgpu_graph hgpu_graph;
int hgpu_capture_begin(hgpu_ctx* ctx);
int hgpu_capture_end(hgpu_ctx* ctx, hgpu_graph** out);
int hgpu_graph_launch(hgpu_graph* g);
int hgpu_graph_destroy(hgpu_graph* g);
/* Replaces the contents of a dense array with host data (same shape and
 * dtype).  The one exception to "arrays are immutable": meant for the input
 * arrays of a captured graph, between launches. */
int hgpu_overwrite(hgpu_ctx* ctx, hgpu_array* a, const void* host);
/* Replaces the contents of the dense array dst with the elements of src (same
 * shape and dtype, any view, not of dst's own memory), on the device.  The
 * second exception to "arrays are immutable": the parameter update of a
 * training step (External/OptimizerTools.hs:20-47, 137-225 return new arrays;
 * a recorded step must put them where its next launch reads its parameters).
 * May be recorded into a graph. */
int hgpu_assign(hgpu_ctx* ctx, hgpu_array* dst, const hgpu_array* src);

/* ------------------------------------------------------------- api table */

/* The same entry points as a table of function pointers, so that host code
 * written against the table can be pointed at another provider of this ABI
 * (the test suite points it at a CPU checker). */
typedef struct hgpu_api {
  size_t struct_size;   /* sizeof(hgpu_api) of the provider's build: members beyond it are absent */
  int (*init)(int, hgpu_ctx**);
  int (*shutdown)(hgpu_ctx*);
  int (*sync)(hgpu_ctx*);
  const char* (*last_error)(hgpu_ctx*);
  int (*upload)(hgpu_ctx*, int, int, const int64_t*, const void*, hgpu_array**);
  int (*download)(hgpu_ctx*, const hgpu_array*, void*);
  int (*read_scalar)(hgpu_ctx*, const hgpu_array*, void*);
  int (*retain)(hgpu_array*);
  int (*release)(hgpu_array*);
  int (*rank)(const hgpu_array*);
  int (*dtype_of)(const hgpu_array*);
  int64_t (*size)(const hgpu_array*);
  int (*shape)(const hgpu_array*, int64_t*);
  int (*strides)(const hgpu_array*, int64_t*);
  int (*is_dense)(const hgpu_array*);
  int (*transpose)(hgpu_ctx*, const hgpu_array*, int, const int*, hgpu_array**);
  int (*reshape)(hgpu_ctx*, const hgpu_array*, int, const int64_t*, hgpu_array**);
  int (*slice)(hgpu_ctx*, const hgpu_array*, int, int64_t, int64_t, hgpu_array**);
  int (*reverse)(hgpu_ctx*, const hgpu_array*, int, hgpu_array**);
  int (*replicate)(hgpu_ctx*, const hgpu_array*, int, const int64_t*, hgpu_array**);
  int (*index_prefix)(hgpu_ctx*, const hgpu_array*, int, const int64_t*, hgpu_array**);
  int (*as_strided)(hgpu_ctx*, const hgpu_array*, int, const int64_t*, const int64_t*, int64_t, hgpu_array**);
  int (*materialize)(hgpu_ctx*, const hgpu_array*, hgpu_array**);
  int (*pad)(hgpu_ctx*, const hgpu_array*, const int64_t*, const int64_t*, hgpu_array**);
  int (*ewise1)(hgpu_ctx*, int, const hgpu_array*, hgpu_array**);
  int (*ewise2)(hgpu_ctx*, int, const hgpu_array*, const hgpu_array*, hgpu_array**);
  int (*compare)(hgpu_ctx*, int, const hgpu_array*, const hgpu_array*, hgpu_array**);
  int (*compare_all)(hgpu_ctx*, int, const hgpu_array*, const hgpu_array*, int*);
  int (*select)(hgpu_ctx*, const hgpu_array*, const hgpu_array*, const hgpu_array*, hgpu_array**);
  int (*convert)(hgpu_ctx*, const hgpu_array*, int, int, hgpu_array**);
  int (*contract)(hgpu_ctx*, const hgpu_array*, const hgpu_array*, int, hgpu_array**);
  int (*argminmax_last)(hgpu_ctx*, const hgpu_array*, int, hgpu_array**);
  int (*iota)(hgpu_ctx*, int64_t, int, hgpu_array**);
  int (*concat)(hgpu_ctx*, int, const hgpu_array* const*, hgpu_array**);
  int (*gather)(hgpu_ctx*, const hgpu_array*, int, const hgpu_array* const*, int, const int64_t*, hgpu_array**);
  int (*scatter_add)(hgpu_ctx*, const hgpu_array*, int, const hgpu_array* const*, int, const int64_t*, int, hgpu_array**);
  int (*onehot)(hgpu_ctx*, const hgpu_array*, int, const int64_t*, const int64_t*, hgpu_array**);
  /* optional (may be NULL): a provider without it gets the operations one by one */
  int (*fused_map)(hgpu_ctx*, int, const hgpu_array* const*, int, const hgpu_fused_instr*, int, const int*, hgpu_array**);
  int (*scatter_affine)(hgpu_ctx*, const hgpu_array*, int, int, const int64_t*, const int64_t*, const int64_t*, hgpu_array**);
  int (*capture_begin)(hgpu_ctx*);
  int (*capture_end)(hgpu_ctx*, hgpu_graph**);
  int (*graph_launch)(hgpu_graph*);
  int (*graph_destroy)(hgpu_graph*);
  int (*overwrite)(hgpu_ctx*, hgpu_array*, const void*);
  int (*contract_sum)(hgpu_ctx*, int, const hgpu_array* const*, const hgpu_array* const*, int, hgpu_array**);
  int (*assign)(hgpu_ctx*, hgpu_array*, const hgpu_array*);
  int (*extremum_last)(hgpu_ctx*, const hgpu_array*, int, hgpu_array**, hgpu_array**);
  int (*fused_extremum)(hgpu_ctx*, int, const hgpu_array* const*, int, const hgpu_fused_instr*, int, int, int, hgpu_array**, hgpu_array**);
  int (*fused_sum)(hgpu_ctx*, int, const hgpu_array* const*, int, const hgpu_fused_instr*, int, hgpu_array**);
  int (*contract_map)(hgpu_ctx*, const hgpu_array*, const hgpu_array*, int, int, const hgpu_array* const*, int, const hgpu_fused_instr*,
                      int, const int*, hgpu_array**, int, int, const int64_t*, const int64_t*, int, int, hgpu_array**, hgpu_array**);
  int (*contract_operands)(hgpu_ctx*, const hgpu_operand*, const hgpu_operand*, int, int, hgpu_array**);
  int (*fused_map_sums)(hgpu_ctx*, int, const hgpu_array* const*, int, const hgpu_fused_instr*, int, const int*, hgpu_array**, int, const int*, hgpu_array**);
  int (*contract_sum_map)(hgpu_ctx*, int, const hgpu_array* const*, const hgpu_array* const*, int, int, const hgpu_array* const*, int, const hgpu_fused_instr*, int,
                         const int*, hgpu_array**);
  int (*fused_map_dimsum)(hgpu_ctx*, int, const hgpu_array* const*, int, const hgpu_fused_instr*, int, const int*, hgpu_array**, int, int, hgpu_array**);
} hgpu_api;

/* The table of this library's own entry points. */
const hgpu_api* hgpu_get_api(void);

#ifdef __cplusplus
}
#endif
#endif /* HORDEAD_GPU_H */

/* hordead_host.h -- C ABI of the host layer: the `Gpu` carrier's tensor-class
 * operations as horde-ad's interpreter would call them, one call per AST node.
 *
 * Where hordead_gpu.h is the array library (strided views + kernels), this
 * layer is what `instance BaseTensor Gpu` binds method by method
 * (reference class: src/HordeAd/Core/Ops.hs:297-1255; the instance it stands
 * beside: src/HordeAd/Core/OpsConcrete.hs:97-775).  It adds what an array
 * library cannot know:
 *   - index FUNCTIONS (tsgather / tsscatter / tsindex0 inside them) evaluated
 *     once over all positions with lane-batched scalars (`hh_ix`), so that an
 *     affine index function becomes a strided view and anything else becomes
 *     index arrays (reference: one call of the closure per position,
 *     OpsConcrete.hs:1581-1665, AstInterpret.hs:242-283);
 *   - dual numbers: values carry a tape node, and `hh_backward` transposes the
 *     recorded operations (reference: OpsADVal.hs:44-60, DeltaEval.hs:391-595).
 *
 * Every function returns an hgpu_status code; `hh_last_error` has the message.
 * Shape mismatches are HGPU_ERR_INVALID (the reference calls `error`).
 */
#ifndef HORDEAD_HOST_H
#define HORDEAD_HOST_H

#include "hordead_gpu.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct hh_ctx hh_ctx;   /* a provider context + the tape of the gradient in progress */
typedef struct hh_val hh_val;   /* a tensor value (primal array view + tape node) */
typedef struct hh_ix hh_ix;     /* a lane-batched scalar: `IntOf Gpu` inside an index function */

/* Context on the gfx950 library (device `device`). */
int hh_create_gpu(int device, hh_ctx** out);
/* Context on any provider of the array ABI. */
int hh_create(const hgpu_api* api, int device, hh_ctx** out);
int hh_destroy(hh_ctx* ctx);
const char* hh_last_error(hh_ctx* ctx);
int hh_sync(hh_ctx* ctx);
hgpu_ctx* hh_array_ctx(hh_ctx* ctx);
/* Elementwise operations are deferred and handed to the provider as fused
 * programs (default, when the provider has fused_map); 0 runs them one by one. */
int hh_set_fusion(hh_ctx* ctx, int on);
/* Forgets the recorded operations; values made before stay usable as constants. */
int hh_tape_reset(hh_ctx* ctx);

/* tsconcrete (OpsConcrete.hs:120-124): a value from host data; `requires_grad`
 * makes it a differentiable input (an `ADVal` with a fresh input delta,
 * OpsADVal.hs:62-73). */
int hh_upload(hh_ctx* ctx, int dtype, int rank, const int64_t* shape, const void* host, int requires_grad, hh_val** out);
/* The same from an array already on the device (the array is retained). */
int hh_from_array(hh_ctx* ctx, hgpu_array* a, int requires_grad, hh_val** out);
/* sconcrete (sreplicate sh x): a constant of the given shape, no element traffic. */
int hh_constant(hh_ctx* ctx, int dtype, double value, int rank, const int64_t* shape, hh_val** out);
/* The primal array of a value (a new reference the caller releases). */
int hh_array(hh_val* v, hgpu_array** out);
int hh_download(hh_ctx* ctx, hh_val* v, void* host);
/* ---- evaluating one gradient program many times (ADEngine.hs:266-288) ----
 * revInterpretArtifact interprets a gradient artifact that was built once.
 * Here the operations issued between hh_capture_begin and hh_capture_end are
 * recorded into a device graph instead of being executed; hh_graph_launch runs
 * the recording as one submission and refreshes, in place, every value made
 * inside the capture (results included).  Values that existed before the
 * capture are the program's inputs: they are read at every launch, and
 * hh_overwrite replaces their contents between launches; the caller keeps them
 * alive (not hh_free'd) until hh_graph_free, the graph holds no reference.  Run the same
 * program once without capture first, so that constants and generated kernels
 * exist (nothing may be uploaded or read back during a capture).
 * hh_force writes a deferred value out (inside a capture: records that). */
typedef struct hh_graph hh_graph;
int hh_capture_begin(hh_ctx* ctx);
int hh_capture_end(hh_ctx* ctx, hh_graph** out);
int hh_graph_launch(hh_ctx* ctx, hh_graph* g);
int hh_graph_free(hh_ctx* ctx, hh_graph* g);
int hh_force(hh_ctx* ctx, hh_val* v);
int hh_overwrite(hh_ctx* ctx, hh_val* v, const void* host);
/* The primal part of v as a dense row-major array: a copy when the value is a
 * strided view (an affine gather, a transpose), v's own array otherwise.  The
 * reference's Concrete backend copies in every gather (OpsConcrete.hs:1621-1665);
 * here affine gathers are views, and this is where such a chain is written out
 * when a caller wants the array itself (bench/ConvVjpBench.hs times exactly that). */
int hh_dense(hh_ctx* ctx, hh_val* v, hh_val** out);
/* dst's memory takes src's elements (same shape and type; dst an array made by
 * upload, src not a view of it): how a recorded training step hands the
 * updated parameters to its next launch. */
int hh_assign(hh_ctx* ctx, hh_val* dst, hh_val* src);
int hh_val_rank(hh_val* v);
int hh_val_dtype(hh_val* v);
int hh_val_shape(hh_val* v, int64_t* shape);
int hh_free(hh_val* v);

/* Gradient descent on device arrays (External/OptimizerTools.hs).
 * hh_update_with_gradient: updateWithGradient (:20-47), params - gamma * gradient
 * for one array; arrays of a non-differentiable type come back unchanged.
 * hh_update_with_gradient_adam: updateWithGradientAdam (:137-225) for one array;
 * t_new is the iteration count AFTER this step (tAdam + 1), from which the
 * step size alphat = alpha * sqrt (1 - beta2^t) / (1 - beta1^t) is computed on
 * the host as the reference does.  hh_adam_apply is the same update with
 * alphat given as a rank-0 array (hh_adam_step_size makes one), for a recorded
 * step whose step size changes between launches (hh_overwrite it).
 * defaultArgsAdam (:82-88): alpha 0.001, beta1 0.9, beta2 0.999, epsilon 1e-7. */
int hh_update_with_gradient(hh_ctx* ctx, double gamma, hh_val* params, hh_val* gradient, hh_val** out);
int hh_update_with_gradient_adam(hh_ctx* ctx, double alpha, double beta1, double beta2, double epsilon, int t_new, hh_val* m, hh_val* v,
                                 hh_val* params, hh_val* gradient, hh_val** m_new, hh_val** v_new, hh_val** params_new);
int hh_adam_step_size(hh_ctx* ctx, int dtype, double alpha, double beta1, double beta2, int t_new, hh_val** out);
int hh_adam_apply(hh_ctx* ctx, hh_val* alphat, double beta1, double beta2, double epsilon, hh_val* m, hh_val* v, hh_val* params, hh_val* gradient,
                  hh_val** m_new, hh_val** v_new, hh_val** params_new);

/* gradientFromDelta (DeltaEval.hs:64-78): cotangents of `inputs` for d(out)=dt. */
int hh_backward(hh_ctx* ctx, hh_val* out, hh_val* dt, int n, hh_val* const* inputs, hh_val** grads);

/* Elementwise Num/Floating/IntegralH/RealFloatH methods (AstInterpret.hs:187-194). */
int hh_ewise1(hh_ctx* ctx, int op1, hh_val* a, hh_val** out);
int hh_ewise2(hh_ctx* ctx, int op2, hh_val* a, hh_val* b, hh_val** out);
/* Elementwise comparison -> Bool tensor (AstLeqS, AstInterpret.hs:353-366). */
int hh_compare(hh_ctx* ctx, int cmp, hh_val* a, hh_val* b, hh_val** out);
/* Whole-tensor comparison -> one Bool on the host (AstLeq, EqH/OrdH). */
int hh_compare_all(hh_ctx* ctx, int cmp, hh_val* a, hh_val* b, int* result);
/* Elementwise conditional on a Bool tensor (what tsmap0N/tszipWith0N of ifH compute). */
int hh_select(hh_ctx* ctx, hh_val* cond, hh_val* a, hh_val* b, hh_val** out);
/* tscast / tsfromIntegral (mode HGPU_CONV_CAST), tsfloor (HGPU_CONV_FLOOR). */
int hh_convert(hh_ctx* ctx, hh_val* a, int dtype, int mode, hh_val** out);
int hh_tssumN(hh_ctx* ctx, hh_val* t, int k, hh_val** out);              /* Ops.hs:514; tssum is k = 1 */
int hh_tssum0(hh_ctx* ctx, hh_val* t, hh_val** out);                     /* Ops.hs:517 */
int hh_tsdot0(hh_ctx* ctx, hh_val* a, hh_val* b, hh_val** out);          /* Ops.hs:519 */
int hh_tsdot1In(hh_ctx* ctx, hh_val* a, hh_val* b, hh_val** out);        /* Ops.hs:522 */
/* ssumN @sh (sdot1In a b) as one contraction over the n innermost dims
 * (the shape conv layers reach the backend in, TestMnistPP.hs:735 `t259`). */
int hh_tsdotNIn(hh_ctx* ctx, hh_val* a, hh_val* b, int n, hh_val** out);
/* The same array as a fresh differentiable input of the current tape (what
 * crevOnParams does with the parameters for every gradient, OpsADVal.hs:62-73). */
int hh_as_input(hh_ctx* ctx, hh_val* v, hh_val** out);
/* tprimalPart (OpsConcrete.hs:761): the value without its dual part. */
int hh_tprimalPart(hh_ctx* ctx, hh_val* v, hh_val** out);
/* tD: the primal part of `primal` with the dual part (tape node) of `dual`
 * (lossSoftMaxCrossEntropyS, External/CommonShapedOps.hs:89-111). */
int hh_tD(hh_ctx* ctx, hh_val* primal, hh_val* dual, hh_val** out);
/* ConvertTensor (src/HordeAd/Core/ConvertTensor.hs:25-236; Concrete instance
 * OpsConcrete.hs:777-876, interpretTKConversion :878-904).  The carrier's arrays
 * know their shape at run time and a product is a pair of handles on the host,
 * so kfromS / sfromK / sfromR / rfromS / sfromX / xfromS and nest / unnest are
 * the identity on data and dual part (zip / unzip never reach this layer: the
 * host keeps the two handles).  What remains is the reference's check:
 * K_FROM_S / S_FROM_K need a rank-0 array; S_FROM_R / S_FROM_X need the array's
 * shape to equal (rank, shape), the shape the shaped type names; NEST / UNNEST
 * take in `rank` the number of outer dims (<= the array's rank; `shape`, when
 * not NULL, must equal the leading dims).  A failed check is HGPU_ERR_INVALID
 * (the reference calls `error`). */
enum hh_conversion {
  HH_CONV_K_FROM_S = 0, HH_CONV_S_FROM_K, HH_CONV_S_FROM_R, HH_CONV_R_FROM_S, HH_CONV_S_FROM_X, HH_CONV_X_FROM_S,
  HH_CONV_NEST, HH_CONV_UNNEST
};
int hh_tconvert(hh_ctx* ctx, int conv, hh_val* v, int rank, const int64_t* shape, hh_val** out);
int hh_tsmatvecmul(hh_ctx* ctx, hh_val* m, hh_val* v, hh_val** out);     /* Ops.hs:538 */
int hh_tsmatmul2(hh_ctx* ctx, hh_val* a, hh_val* b, hh_val** out);       /* Ops.hs:543 */
int hh_tsreplicateN(hh_ctx* ctx, hh_val* t, int n, const int64_t* shm, hh_val** out);   /* Ops.hs:552; also tsreplicate0N */
int hh_tsappend(hh_ctx* ctx, hh_val* a, hh_val* b, hh_val** out);        /* Ops.hs:825 */
int hh_tsslice(hh_ctx* ctx, hh_val* t, int64_t i, int64_t n, hh_val** out);   /* Ops.hs:828 */
int hh_tsreverse(hh_ctx* ctx, hh_val* t, hh_val** out);                  /* Ops.hs:831 */
int hh_tstranspose(hh_ctx* ctx, hh_val* t, int n, const int* perm, hh_val** out);   /* Ops.hs:833 */
int hh_tsreshape(hh_ctx* ctx, hh_val* t, int rank, const int64_t* shape, hh_val** out);   /* Ops.hs:837 */
int hh_tsindex(hh_ctx* ctx, hh_val* t, int n, const int64_t* ix, hh_val** out);   /* Ops.hs:667, host indices */
int hh_tsargminmax(hh_ctx* ctx, hh_val* t, int want_max, hh_val** out);  /* Ops.hs:792 */
int hh_tsiota(hh_ctx* ctx, int64_t n, int dtype, hh_val** out);          /* Ops.hs:795 */

/* Index functions.  A position space is a shape `shm`; `hh_ix_var` is its d-th
 * position variable.  All hh_ix of one function must share the space. */
int hh_ix_var(hh_ctx* ctx, int rank_m, const int64_t* shm, int d, hh_ix** out);
int hh_ix_const(hh_ctx* ctx, int rank_m, const int64_t* shm, int dtype, double value, hh_ix** out);
/* A rank-0 tensor value used as a scalar inside an index function. */
int hh_ix_lift(hh_ctx* ctx, int rank_m, const int64_t* shm, hh_val* scalar, hh_ix** out);
int hh_ix_op1(hh_ctx* ctx, int op1, hh_ix* a, hh_ix** out);              /* AstN1K / AstR1K */
int hh_ix_op2(hh_ctx* ctx, int op2, hh_ix* a, hh_ix* b, hh_ix** out);    /* AstPlusK / AstTimesK / AstR2K / AstI2K */
int hh_ix_compare(hh_ctx* ctx, int cmp, hh_ix* a, hh_ix* b, hh_ix** out);   /* AstLeqK */
int hh_ix_select(hh_ctx* ctx, hh_ix* c, hh_ix* a, hh_ix* b, hh_ix** out);   /* AstCondK -> kcond (ifH) */
int hh_ix_convert(hh_ctx* ctx, hh_ix* a, int dtype, int mode, hh_ix** out); /* AstFromIntegralK / AstCastK / AstFloorK */
/* AstIndexK (AstInterpret.hs:181-185): t `sindex0` [ix...], one index per dim of t. */
int hh_ix_index0(hh_ctx* ctx, hh_val* t, int n, hh_ix* const* ix, hh_ix** out);
/* AstArgMinK / AstArgMaxK of a partial index: kargMax (t !$ [ix...]); the
 * partial index must leave exactly the last dim of t. */
int hh_ix_argminmax(hh_ctx* ctx, hh_val* t, int n, hh_ix* const* ix, int want_max, hh_ix** out);
/* tkbuild / tsmap0N / tszipWith0N (Ops.hs:863-880, 929-941; Concrete runs them as one
 * vector map over the elements, OpsConcrete.hs:671-714, 1081-1087, 1748-1759).
 * hh_ix_from_val: the elements of an array (primal part) as a lane value over
 * the position space shm = the array's own shape, so the scalar closure of a
 * map runs once for all elements.  hh_ix_to_val: a lane value written out as
 * an array of shape shm (no dual part).  The closure's arithmetic in between
 * joins the deferred elementwise program like any other array arithmetic:
 *   tsmap0N f v       = to_val (f (from_val v))
 *   tszipWith0N f u v = to_val (f (from_val u) (from_val v))
 *   tkbuild @sh f     = to_val (f [hh_ix_var 0, .., hh_ix_var (n-1)]) */
int hh_ix_from_val(hh_ctx* ctx, hh_val* v, hh_ix** out);
int hh_ix_to_val(hh_ctx* ctx, hh_ix* x, hh_val** out);
/* The element type of a lane value (an hgpu dtype code). */
int hh_ix_dtype(hh_ix* x);
int hh_ix_free(hh_ix* x);
/* 1 when the value is an affine form of the position variables (diagnostic). */
int hh_ix_is_affine(hh_ix* x);
/* How many times this context has taken the named rewrite onto a fused entry
 * point of the provider (diagnostic; "contract_map", "contract_operands"). */
int64_t hh_counter(hh_ctx* ctx, const char* name);

/* tsgather (Ops.hs:701-705): out[m.., n..] = src[ix(m).., n..], zeros out of bounds. */
int hh_tsgather(hh_ctx* ctx, hh_val* src, int rank_m, const int64_t* shm, int n_ix, hh_ix* const* ix, hh_val** out);
/* tsscatter (Ops.hs:689-693): out[ix(m).., n..] += src[m.., n..]; shp has n_ix dims. */
int hh_tsscatter(hh_ctx* ctx, hh_val* src, int rank_m, int n_ix, const int64_t* shp, hh_ix* const* ix, hh_val** out);

#ifdef __cplusplus
}
#endif
#endif /* HORDEAD_HOST_H */

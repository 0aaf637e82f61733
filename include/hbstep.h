/*
 * hbstep.h - C ABI of libhbstep.so, the MI355X (gfx950) optimizer-step kernels.
 *
 * The reference (HomebrewML/HeavyBall 3.2.0) has no native code: its "kernels" are whatever torch.compile
 * generates from the list-of-tensor functions in heavyball/utils.py.  Each entry point below replaces one of
 * those fused regions; the comment on each names the reference function (file:line) it stands for.
 *
 * Conventions
 *   - every function returns 0 on success and a negative HB_E* code on failure; hb_last_error() gives the text.
 *     Nothing throws across the ABI.
 *   - all pointers are DEVICE pointers unless the name says "host"; the caller owns every buffer and keeps it
 *     alive until the stream has passed the call.  No entry point allocates, frees, synchronises or starts threads.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *   - scalars that the reference evaluates as fp32 0-d tensors (debiased betas, lr, ...) are computed by the caller
 *     and passed as floats, so the library never re-derives them in another precision.
 */
#ifndef HBSTEP_H
#define HBSTEP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HB_OK 0
#define HB_EINVAL (-1)  /* bad argument (null pointer, unknown enum, misaligned buffer, size over a limit) */
#define HB_ELAUNCH (-2) /* the HIP runtime refused the launch; hb_last_error() holds hipGetErrorString */
#define HB_EUNSUPPORTED (-3)

/* Raised whenever a struct layout, an enum value or a signature changes.  A binding records the value it was written
 * against and compares it with hb_abi_version() after loading the library. */
#define HB_ABI_VERSION 12

/* Elements per work chunk.  Every tensor starts at a slab offset that is a multiple of this, and a chunk never
 * spans two tensors. */
#ifndef HB_CHUNK
#define HB_CHUNK 4096
#endif

/* storage formats of a role (parameter, gradient, optimizer state) */
enum {
  HB_FMT_F32 = 0,
  HB_FMT_BF16 = 1,       /* plain bf16; fp32 values written to it are stochastically rounded (heavyball/utils.py:2341-2370) */
  HB_FMT_F16 = 2,        /* plain fp16, gradients only */
  HB_FMT_ECC_BF16_8 = 3, /* bf16 primary + int8 correction   (heavyball/chainable.py:226-231, "bf16+8")  */
  HB_FMT_ECC_BF16_16 = 4,
  HB_FMT_ECC_F16_8 = 5,
  HB_FMT_ECC_F16_16 = 6,
};

enum {
  HB_ALGO_ADAM = 0,     /* fused_adam_     heavyball/utils.py:1921-1965 */
  HB_ALGO_LAPROP = 1,   /* fused_laprop_   heavyball/utils.py:2247-2291 */
  HB_ALGO_ADOPT = 2,    /* fused_adopt_    heavyball/utils.py:2294-2315: update from the second moment of the steps before */
  HB_ALGO_ADEMAMIX = 3, /* fused_ademamix_ heavyball/utils.py:2086-2183: exp_avg is the fast momentum, exp_avg_slow the slow one */
  HB_ALGO_NADAM = 4,    /* fused_nadam_    heavyball/utils.py:2003-2083: per-tensor weights in tensor_scalars */
};

/* flags of HbStepDesc */
#define HB_FLAG_MARS 1u        /* MARS gradient correction, heavyball/chainable.py:642-647 */
#define HB_FLAG_CAUTION 2u     /* caution mask with per-tensor rescale, heavyball/utils.py:3652-3658 */
#define HB_FLAG_CAUTIOUS_WD 4u /* decay only where sign(p) == sign(update), heavyball/utils.py:2388 */
#define HB_FLAG_WRITE_GRAD 8u  /* MARS: write the corrected gradient back into the gradient buffer (chainable.py:646) */
/* The un-fused scale_by_adam / scale_by_laprop / scale_by_adopt / scale_by_ademamix / scale_by_nadam (heavyball/chainable.py:715-727,
 * :849-862, :1014-1023, :820-833, :754-769): the moments are updated and the transform's update is WRITTEN as fp32 to `update_out`
 * (an fp32 slab at the same offsets) while `param` is only read (NAdam's weight decay that is not decoupled); with `update_out`
 * NULL the update goes to `param`, which is then that fp32 slab (param_fmt HB_FMT_F32) and not the parameters.  With 16-bit
 * gradients the update is first rounded to their dtype, as the reference's update buffer holds it (bf16: stochastic, stream
 * HB_STREAM_UPDATE).  Weight decay, learning rate and caution do not apply (hb_update_param does them afterwards). */
#define HB_FLAG_UPDATE_ONLY 16u
/* HB_ALGO_ADOPT only, its warm-up step (heavyball/chainable.py:945-946 under WarmupGuard, :587-610): exp_avg_sq <- g*g through
 * the lerp with weights (a2, one_minus_a2) = (1, 0); exp_avg and the parameters are neither read nor written. */
#define HB_FLAG_ADOPT_WARMUP 32u
/* HB_ALGO_NADAM only, weight decay that is not decoupled (heavyball/utils.py:350-379): g <- fma(p, coupled_wd, g) before the
 * moments (also the gradient caution compares with), update <- update - p * coupled_wd afterwards. */
#define HB_FLAG_COUPLED_WD 64u

/* With HB_FLAG_MARS: only the MARS prologue runs.  mars_old_grad takes the raw gradient and the corrected gradient
 * (rounded to the gradient's dtype, heavyball/chainable.py:642-647) is WRITTEN as fp32 to `param`, which is then an fp32
 * slab (param_fmt HB_FMT_F32) and not the parameters; the moments and the parameters are neither read nor written.  For
 * chains that put a transform between MARS and the update (gradient clipping, heavyball/chainable.py:2694-2699). */
#define HB_FLAG_MARS_ONLY 128u

/* where the noise of stochastic rounding comes from */
enum {
  HB_RNG_HALF = 0,   /* uniform = 0.5, 16-bit noise = 0x8000: deterministic ("rounding disabled") */
  HB_RNG_PHILOX = 1, /* Philox4x32-10, counter (flat_index >> 2, step, stream >> 1), key = seed: one call serves 4 consecutive
                      * elements for the streams 2p and 2p + 1; element j of stream s takes the 16 bits at half-word j of the
                      * words (s & 1) * 2 and (s & 1) * 2 + 1 */
};

/* Philox stream ids: one per rounding site of the step (exp_avg and exp_avg_sq share their calls) */
enum {
  HB_STREAM_MARS_SR = 0,
  HB_STREAM_PARAM = 1, /* pairs with HB_STREAM_MARS_SR: a step with MARS and a narrow parameter makes one call for both */
  HB_STREAM_EXP_AVG = 2,
  HB_STREAM_EXP_AVG_SQ = 3,
  HB_STREAM_OLD_GRAD = 4,
  HB_STREAM_INIT_PARAM = 5,
  HB_STREAM_NS_INPUT = 6, /* the legacy Newton-Schulz variant also draws from 7 for its second rounding */
  HB_STREAM_CLIP = 8,     /* bf16 stochastic rounding of a clipped bf16 gradient */
  HB_STREAM_EXP_AVG_SLOW = 9, /* AdEMAMix's slow momentum */
  HB_STREAM_UPDATE = 10,      /* HB_FLAG_UPDATE_ONLY with bf16 gradients: the update is rounded to bf16 as the reference's update buffer is */
  HB_STREAM_SOAP_ROTATE = 11, /* SOAP: exp_avg written back to bf16 / ECC storage after its rotation into a refreshed basis */
  HB_STREAM_UPDATE_CLIP = 12, /* bf16 stochastic rounding of a clipped bf16 update (update_clipping with bf16 gradients); its own
                                 stream, so that a step with both clips draws independent noise for the two roundings */
  HB_STREAM_SOAP_GG = 16,     /* SOAP under 16-bit gradients: a factor kept in bf16, rewritten after its update; side li draws from 16 + 2 li */
  HB_STREAM_SOAP_Q = 17,      /* ... and a refreshed eigenbasis kept in bf16: 17 + 2 li */
};

/*
 * One optimizer step of AdamW, LaProp, ADOPT, AdEMAMix or NAdam over a whole slab of tensors.
 *
 * Layout: every role (param, exp_avg, exp_avg_sq, mars_old_grad and their ECC corrections) is one flat device
 * buffer; tensor t occupies elements [offsets[t], offsets[t] + numel[t]) of each of them, offsets[t] a multiple of
 * HB_CHUNK, and the buffers extend to a multiple of HB_CHUNK past the last tensor (the padding is owned by the
 * slab and may be read and written).  Gradients are either a slab with the same offsets (`grad`) or one pointer
 * per tensor (`grad_ptrs`, device array, each 16-byte aligned); exactly one of the two is non-null.
 * `chunks[c] = {tensor, chunk index inside the tensor}` lists the work; tensors without a gradient are left out.
 */
/* counters per tensor in HbStepDesc.caution_count */
#define HB_CAUTION_SLOTS 32

typedef struct HbStepDesc {
  void* param;
  void* param_corr; /* ECC formats only */
  const void* grad;
  const void* const* grad_ptrs;
  void* exp_avg;
  void* exp_avg_corr;
  void* exp_avg_sq;
  void* exp_avg_sq_corr;
  void* old_grad; /* HB_FLAG_MARS only */
  void* old_grad_corr;
  const int64_t* offsets;  /* [n_tensors]   */
  const int64_t* numel;    /* [n_tensors]   */
  const int32_t* chunks;   /* [n_chunks][2] */
  uint32_t* caution_count; /* [n_tensors][HB_CAUTION_SLOTS] scratch, HB_FLAG_CAUTION only; the call zeroes and fills it: the
                              masked elements of tensor t are the sum of its slots (workgroups add into the slot their work
                              unit's index picks, so that the additions of one tensor do not queue up on one address) */
  int64_t n_chunks;
  int32_t n_tensors;
  int32_t algo;
  uint32_t flags;
  int32_t param_fmt; /* F32, BF16 or an ECC format */
  int32_t grad_fmt;  /* F32, BF16 or F16 */
  int32_t state_fmt; /* F32, BF16 or an ECC format; shared by exp_avg, exp_avg_sq and mars_old_grad */
  /* fp32 scalars exactly as the reference's 0-d tensors hold them */
  float a1, one_minus_a1; /* a1 = 1 - beta1', one_minus_a1 = 1 - a1   (heavyball/utils.py:1847, :1048) */
  float a2, one_minus_a2;
  float mars_a, one_minus_mars_a; /* heavyball/utils.py:3624, :1048 */
  float neg_lr;                   /* -lr                              (heavyball/utils.py:2389) */
  float one_minus_decay_lr;       /* 1 - decay * lr                   (heavyball/utils.py:2389) */
  float eps;
  int32_t rng_mode;
  uint32_t step;
  uint64_t seed;
  /* HB_ALGO_ADEMAMIX: the slow momentum (same format as the other states), its lerp weights a3 = 1 - beta3 and 1 - a3, and
   * alpha in update = (fast + slow * alpha) / denom */
  void* exp_avg_slow;
  void* exp_avg_slow_corr;
  float a3, one_minus_a3, alpha;
  /* HB_ALGO_NADAM: tensor_scalars[2t], [2t+1] = the weights of g/denom and exp_avg/denom for tensor t
   * (heavyball/utils.py:407-409, device array of 2*n_tensors floats); coupled_wd with HB_FLAG_COUPLED_WD */
  float coupled_wd;
  const float* tensor_scalars;
  void* update_out; /* HB_FLAG_UPDATE_ONLY: where the update goes (fp32 slab); NULL = into `param` */
} HbStepDesc;

/* replaces fused_adam_ (heavyball/utils.py:1921-1965) / fused_laprop_ (:2247-2291) / fused_adopt_ (:2294-2315) /
 * fused_ademamix_ (:2086-2183) / fused_nadam_ (:2003-2083) together with the MARS prologue
 * (:3616-3627), the caution mask (:3652-3658), the parameter update (:2373-2390) and the ECC / stochastic-rounding
 * writes (:1288-1324, :2341-2370) */
int hb_fused_step(const HbStepDesc* desc, void* stream);

/* hb_fused_step for callers that cannot allocate device memory or hand over a scratch buffer: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same
 * descriptor and results as hb_fused_step, except that `caution_count` is ignored (it may be NULL): the per-tensor
 * caution counters live in a device array inside the library (4 * HB_CAUTION_SLOTS * HB_NOALLOC_MAX_TENSORS bytes = 1 MiB on
 * every GPU the library runs on, held until the process ends).  More than HB_NOALLOC_MAX_TENSORS tensors: HB_EINVAL.  The call
 * allocates and frees nothing and clears the counters it uses with a fill kernel.  Every call on one GPU shares that
 * GPU's array, so two calls with HB_FLAG_CAUTION that overlap on one GPU (different streams or threads) race. */
#define HB_NOALLOC_MAX_TENSORS 8192
int hb_fused_step_noalloc(const HbStepDesc* desc, void* stream);

/* chain()'s non-fused tail, update_param_ (heavyball/utils.py:2393-2406): p <- p*(1 - decay*lr) + u*(-lr) on a slab,
 * with `update` an fp32 slab at the same offsets.  Uses param/param_corr/param_fmt, offsets, numel, chunks, flags
 * (CAUTION needs grad/grad_fmt and caution_count), neg_lr, one_minus_decay_lr, rng_*, and reads the update from
 * `exp_avg`, an fp32 slab or (state_fmt == HB_FMT_BF16) a bf16 one. */
int hb_update_param(const HbStepDesc* desc, void* stream);

/* the codec on its own: the arithmetic of _ULPState.encode / decode (heavyball/utils.py:1296-1324) and
 * stochastic_round_ (:2341-2355) on n contiguous elements starting at flat index `flat_base` of stream `stream_id`.
 * Used by the tests of the codec, by param_ecc at construction and by SOAP's moments when they are stored narrow. */
int hb_ecc_encode(const float* src, void* primary, void* corr, int64_t n, int32_t fmt, int32_t rng_mode, uint64_t seed,
                  uint32_t step, uint32_t stream_id, int64_t flat_base, void* stream);
int hb_ecc_decode(const void* primary, const void* corr, float* dst, int64_t n, int32_t fmt, void* stream);
int hb_sr_bf16(const float* src, void* dst_bf16, int64_t n, int32_t rng_mode, uint64_t seed, uint32_t step,
               uint32_t stream_id, int64_t flat_base, void* stream);
/* raw Philox words of n calls with counters (q, step, stream_id), q = q0 .. q0 + n - 1: out[4*n] */
int hb_philox_words(uint32_t* out, int64_t n, uint64_t q0, uint64_t seed, uint32_t step, uint32_t stream_id, void* stream);

/* per-tensor sum of squares over a slab role, the reduction behind the clipping norms
 * (heavyball/utils.py:3235-3297): out[t] = sum x^2 as fp64.  `partial` is scratch of n_chunks doubles. */
int hb_sumsq(const void* x, int32_t fmt, const int64_t* offsets, const int64_t* numel, const int32_t* chunks,
             int64_t n_chunks, int32_t n_tensors, double* partial, double* out, void* stream);

/* x <- x * scale[t] (or one global scale when per_tensor == 0) on an fp32 slab: the second half of _clip
 * (heavyball/utils.py:3226-3232) */
int hb_scale(float* x, const float* scale, int32_t per_tensor, const int64_t* offsets, const int64_t* numel,
             const int32_t* chunks, int64_t n_chunks, void* stream);

/*
 * Muon.  hb_nesterov_ema replaces _compilable_nesterov_ema_ (heavyball/utils.py:766-769) on an fp32 slab:
 *   momentum <- momentum * one_minus_a + g * a ;  update <- g + momentum      (a = 1 - beta, no debias)
 * `update` is an fp32 slab at the same offsets; gradients as in HbStepDesc (slab or per-tensor pointers).
 */
int hb_nesterov_ema(float* momentum, float* update, const void* grad, const void* const* grad_ptrs, int32_t grad_fmt,
                    const int64_t* offsets, const int64_t* numel, const int32_t* chunks, int64_t n_chunks, float a,
                    float one_minus_a, void* stream);

/*
 * hb_momentum: the four momentum forms heavyball.Muon chooses between (heavyball/__init__.py:723-737), same layout as
 * hb_nesterov_ema (which is mode HB_MOM_NESTEROV_EMA):
 *   HB_MOM_EMA                 exp_avg (heavyball/chainable.py:652-653, utils.py:457-460): momentum <- lerp, update <- momentum;
 *                              a = 1 - beta_debias(beta, step)
 *   HB_MOM_HEAVYBALL           _compilable_heavyball_momentum_ (utils.py:737-741): momentum <- momentum * a + g, update <- momentum;
 *                              a = beta, one_minus_a unused
 *   HB_MOM_NESTEROV_HEAVYBALL  _compilable_nesterov_momentum_ (utils.py:745-749): momentum as above, update <- g + momentum * a
 * The momentum may be stored as float32, bfloat16 (storage_dtype) or an ECC pair (momentum_corr, HB_FMT_ECC_*): it is
 * written back through the rounding of copy_stochastic_ / _ULPState.encode (Philox stream HB_STREAM_EXP_AVG), while the
 * update is formed from the un-rounded value (heavyball/utils.py:1847-1849).  With 16-bit gradients the update itself
 * is rounded to their dtype, as the reference's update buffer is (bf16: stream HB_STREAM_MARS_SR); it is stored as fp32.
 */
enum { HB_MOM_NESTEROV_EMA = 0, HB_MOM_EMA = 1, HB_MOM_HEAVYBALL = 2, HB_MOM_NESTEROV_HEAVYBALL = 3 };
int hb_momentum(void* momentum, void* momentum_corr, int32_t momentum_fmt, float* update, const void* grad,
                const void* const* grad_ptrs, int32_t grad_fmt, const int64_t* offsets, const int64_t* numel,
                const int32_t* chunks, int64_t n_chunks, int32_t mode, float a, float one_minus_a, int32_t rng_mode,
                uint64_t seed, uint32_t step, void* stream);
/* hb_momentum that also leaves the sums of squares of the update it writes, for the norm that Newton-Schulz divides by
 * (heavyball/utils.py:555) without another pass over the update: sumsq_parts receives
 * hb_momentum_sumsq_parts_per_chunk() doubles per entry of `chunks`, in the order of `chunks` (zeros past a tensor's end); the
 * sum over a tensor's chunks is its sum of squares.  Plain stores, no atomics: the same bits in every run.  sumsq_parts
 * NULL: hb_momentum. */
int hb_momentum_sumsq_parts_per_chunk(void);
int hb_momentum_sumsq(void* momentum, void* momentum_corr, int32_t momentum_fmt, float* update, const void* grad,
                      const void* const* grad_ptrs, int32_t grad_fmt, const int64_t* offsets, const int64_t* numel,
                      const int32_t* chunks, int64_t n_chunks, int32_t mode, float a, float one_minus_a, int32_t rng_mode,
                      uint64_t seed, uint32_t step, double* sumsq_parts, void* stream);

/*
 * hb_ns5 replaces zeropower_via_newtonschulz5 (heavyball/utils.py:550-577; legacy != 0: legacy_zeropower_via_newtonschulz5,
 * :637-657) followed by the post-scale of _compilable_orthogonal_ (:808-809) for one fp32 matrix g[rows, cols]
 * (row-major, contiguous); `out` may alias `g`.  coeffs_host: 5 triples (a, b, c) in HOST memory.  The bf16 stochastic
 * round of the input draws from stream HB_STREAM_NS_INPUT at flat index flat_base + i*cols + j.
 * `workspace`: device scratch of hb_ns5_workspace_bytes(rows, cols) bytes, 256-byte aligned.
 * `legacy` is a set of flags: HB_NS_LEGACY selects the legacy variant; HB_NS_BF16_UPDATE says that the reference's update
 * buffer is bfloat16 (bf16 gradients): the norm, the normalised input and the scaled result are then bf16 values rounded to
 * nearest, as torch computes them on a bf16 tensor, and the input gets no stochastic round (heavyball/utils.py:555-556,
 * :2348-2349, :577, :808-809).  g and out stay fp32 buffers (holding bf16-representable values in that case).  Both flags
 * together: the legacy variant's first round is then the identity and its division, done in fp32 against the bf16-rounded
 * norm, keeps its stochastic round (stream HB_STREAM_NS_INPUT + 1; heavyball/utils.py:641-645, :1174-1179).
 * HB_NS_F16_UPDATE says that the update buffer is float16 (fp16 gradients): the norm, the clamp bound and the quotient are
 * fp16 values rounded to nearest, the quotient then takes the stochastic round to bf16 like an fp32 one, and the result is
 * cast to fp16 and scaled there (two roundings to nearest).  With HB_NS_LEGACY only the norm is an fp16 value (its division
 * runs in fp32).  The two update flags exclude each other.
 */
enum { HB_NS_LEGACY = 1, HB_NS_BF16_UPDATE = 2, HB_NS_F16_UPDATE = 4, HB_NS_APPLY_TO_PARAM = 8, HB_NS_CAUTIOUS_WD = 16 };
int hb_ns5_workspace_bytes(int64_t rows, int64_t cols, int64_t* bytes);
int hb_ns5(const float* g, float* out, int64_t rows, int64_t cols, const float* coeffs_host, int32_t legacy, float eps,
           float post_scale, int32_t rng_mode, uint64_t seed, uint32_t step, int64_t flat_base, void* workspace,
           int64_t workspace_bytes, void* stream);

/*
 * hb_ns5_batched: hb_ns5 for n_mats independent matrices at once; the counterpart in the reference is the loop over a
 * group's (same-shape-bucketed) matrices in orthogonalize_update (heavyball/chainable.py:1117-1126, :503-584).  Each of the
 * 15 products runs as one grouped launch over the tiles of every matrix, so small matrices and the half-empty grids of
 * the symmetric products (only the upper triangle of X X^T and of the polynomial in it is computed) fill the GPU
 * together.  g, out, rows, cols, post_scale, flat_base: HOST arrays of n_mats entries (g/out hold device pointers).
 * Results are bit-identical to n_mats calls of hb_ns5.  Workspace: hb_ns5_batched_workspace_bytes for the same shapes.
 */
int hb_ns5_batched_workspace_bytes(int32_t n_mats, const int64_t* rows, const int64_t* cols, int64_t* bytes);
int hb_ns5_batched(int32_t n_mats, const float* const* g, float* const* out, const int64_t* rows, const int64_t* cols,
                   const float* coeffs_host, int32_t legacy, float eps, const float* post_scale, int32_t rng_mode, uint64_t seed,
                   uint32_t step, const int64_t* flat_base, void* workspace, int64_t workspace_bytes, void* stream);
/* hb_ns5_batched with a coefficient table and a flag word per matrix (coeffs_host: n_mats x 15 floats, flags: n_mats
 * words, both in HOST memory): under zeroth_power_mode = "legacy_newtonschulz" the dispatcher gives square matrices the
 * legacy variant and the others the default one (heavyball/utils.py:790-795), and one call still covers the whole group.
 * HB_NS_BF16_UPDATE is per matrix as well (a bucket may hold gradients of both dtypes).  Bit-identical to separate calls per
 * matrix.  The descriptors of the launches are written into the workspace by the call itself, so the number of matrices is not
 * bounded by what a kernel argument holds. */
int hb_ns5_batched_mixed(int32_t n_mats, const float* const* g, float* const* out, const int64_t* rows, const int64_t* cols,
                         const float* coeffs_host, const int32_t* flags, float eps, const float* post_scale, int32_t rng_mode,
                         uint64_t seed, uint32_t step, const int64_t* flat_base, void* workspace, int64_t workspace_bytes,
                         void* stream);

/* hb_ns5_batched_mixed with a schedule of n_steps iterations instead of five (coeffs_host: n_mats x 3 n_steps floats):
 * replaces msign (heavyball/utils.py:605-631), the ten-step "Polar Express" schedule that square matrices take under
 * zeroth_power_mode = "thinky_polar_express" (:796-797), followed by the same post-scale; normalisation, input rounding and
 * the iteration are those of hb_ns5.  Same workspace as hb_ns5_batched for the same shapes; hb_ns5_batched_mixed is this call
 * with n_steps = 5 and param_step = NULL.
 * HB_NS_APPLY_TO_PARAM in a matrix' flag word fuses the chain's tail into the last product: out[i] is then the matrix' fp32
 * PARAMETER (not g[i]) and takes p <- p * param_step[0] + update * param_step[1], i.e. update_param_ without caution
 * (heavyball/utils.py:2373-2406) with param_step = {1 - decay * lr, -lr} in HOST memory, in the arithmetic of hb_update_param;
 * the update itself is not written anywhere.  HB_NS_CAUTIOUS_WD with it: the first factor is 1 where update and parameter
 * differ in sign (cautious weight decay).
 * sumsq_parts / n_sumsq_parts (HOST arrays of n_mats entries, or both NULL): where sumsq_parts[i] is not NULL it points to
 * n_sumsq_parts[i] doubles in DEVICE memory whose sum is the sum of squares of g[i] (hb_momentum_sumsq leaves them), and the
 * call does not read g[i] a first time to compute its norm. */
int hb_ns_batched_steps(int32_t n_mats, const float* const* g, float* const* out, const int64_t* rows, const int64_t* cols,
                        int32_t n_steps, const float* coeffs_host, const int32_t* flags, float eps, const float* post_scale,
                        const float* param_step, const double* const* sumsq_parts, const int32_t* n_sumsq_parts, int32_t rng_mode,
                        uint64_t seed, uint32_t step, const int64_t* flat_base, void* workspace, int64_t workspace_bytes,
                        void* stream);

/* The tile width (128 or 256) of the product kernel that a rows x cols matrix goes through.  The wide kernel runs one workgroup
 * per compute unit, with nothing to hide an epilogue behind: HB_NS_APPLY_TO_PARAM costs more there than the separate
 * hb_update_param it saves, so a caller asks first. */
int hb_ns_tile(int64_t rows, int64_t cols);

/* Test hook: ONE product of the Newton-Schulz iteration on bf16 operands (row-major, K contiguous: A [M, K], B [N, K]) through
 * the kernel of the given tile class (128 or 256), so that a test can put the same product through both kernels, whose
 * accumulation order is the same and whose results must agree bit for bit.  mode 0: C = bf16(A B^T), C2 = bf16(bf16(C * mul_c) +
 * diag on the diagonal) (heavyball/utils.py:568-570; A == B, M == N: upper triangle of tiles computed, mirrored); mode 1:
 * C = bf16(A B^T) with diag added on the diagonal (:571-572; M == N, upper triangle computed, mirrored); mode 2: C = bf16(A B^T)
 * [M, N] and C2 = its transpose [N, M] (:573).  M, N multiples of the tile, K of 64.  workspace: 4096 bytes, 256-byte aligned. */
int hb_ns_product(int32_t tile, int32_t mode, const void* A, const void* B, void* C, void* C2, int64_t M, int64_t N, int64_t K, float mul_c,
                  float diag, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * SOAP.  hb_gemm_f32: C[M,N] = op(A) op(B) in fp32 on the matrix cores; op(A) = A^T when trans_a (A given as [K,M]),
 * op(B) = B^T when trans_b (B given as [N,K]); row-major, arbitrary sizes and leading dimensions.  `accumulate` is a
 * set of HB_GEMM_* flags.  HB_GEMM_ACCUMULATE: C = C*beta_c + (op(A) op(B))*alpha_acc, the lerp of update_ggt.
 * HB_GEMM_SYMMETRIC: the caller states that the product is A A^T or A^T A of one matrix (A == B, lda == ldb, M == N,
 * exactly one of trans_a / trans_b; anything else is HB_EINVAL) and, when accumulating, that C is symmetric; the
 * library may then compute the upper triangle only and mirror it, with results bit-identical to the full product
 * (both triangles of the full product add the same terms in the same order).  Replaces the contractions of project
 * (heavyball/utils.py:1391-1411), update_ggt (:1205-1221) and get_orthogonal_matrix_QR (:829-900).
 * hb_adam_precond replaces _compilable_adam_ (heavyball/utils.py:1852-1868) on flat fp32 arrays:
 *   exp_avg <- exp_avg*one_minus_a1 + g*a1;  exp_avg_sq <- exp_avg_sq*one_minus_a2 + g*g*a2;
 *   out = exp_avg / max(sqrt(exp_avg_sq), eps)       (out may alias grad)
 */
#define HB_GEMM_ACCUMULATE 1
#define HB_GEMM_SYMMETRIC 2
int hb_gemm_f32(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                int64_t ldc, int32_t trans_a, int32_t trans_b, int32_t accumulate, float alpha_acc, float beta_c,
                void* stream);
/* n independent hb_gemm_f32 products of one orientation in as few launches as possible (HOST arrays of n entries; A, B, C
 * hold device pointers): the counterpart in the reference is the loop over a group's tensors around project / update_ggt
 * (heavyball/chainable.py:1257-1275).  A product that fills the GPU on its own runs as hb_gemm_f32 would run it; the others
 * share launches, every workgroup finding its product in a table, so that the mid-sized products of a model with many
 * matrices (108 tiles for a 768 x 2304 projection) fill the chip together.  Every product's result is bit-identical to its
 * own hb_gemm_f32 call.  The products must not depend on each other. */
int hb_gemm_f32_grouped(int32_t n, const float* const* A, const float* const* B, float* const* C, const int64_t* M,
                        const int64_t* N, const int64_t* K, const int64_t* lda, const int64_t* ldb, const int64_t* ldc,
                        int32_t trans_a, int32_t trans_b, const int32_t* accumulate, const float* alpha_acc,
                        const float* beta_c, void* stream);
int hb_adam_precond(float* exp_avg, float* exp_avg_sq, const float* grad, float* out, int64_t n, float a1,
                    float one_minus_a1, float a2, float one_minus_a2, float eps, void* stream);
/* hb_adam_precond for `count` tensors in as few launches as possible (HOST arrays of count entries holding device pointers and
 * element counts): the vectors of a model are a few hundred elements each, and one launch per tensor is all launch latency.
 * Elementwise, so every tensor's result is bit-identical to its own hb_adam_precond call. */
int hb_adam_precond_grouped(int32_t count, float* const* exp_avg, float* const* exp_avg_sq, const float* const* grad,
                            float* const* out, const int64_t* n, float a1, float one_minus_a1, float a2, float one_minus_a2,
                            float eps, void* stream);

/*
 * hb_orthonormalize_f32: Q[m, n] (row-major, leading dimension ld, n <= m) is replaced by the Q factor of its thin QR
 * decomposition with a positive diagonal of R, i.e. its columns orthonormalised in order.  Replaces the
 * torch.linalg.qr(...).Q of get_orthogonal_matrix_QR (heavyball/utils.py:887-892) in SOAP's basis refresh; the columns
 * agree with LAPACK's Householder Q up to sign, to which the SOAP step is invariant.  Method: block classical
 * Gram-Schmidt over panels of 128 columns with Cholesky QR inside the panel, every projection done twice, all of it on
 * hb_gemm_f32's kernel (split-K where the output is small).  *status (device int32) becomes non-zero when a panel was
 * numerically rank-deficient; the output is then finite but not trustworthy and the caller falls back to Householder QR.
 */
int hb_orthonormalize_workspace_bytes(int64_t m, int64_t n, int64_t* bytes);
int hb_orthonormalize_f32(float* Q, int64_t m, int64_t n, int64_t ld, void* workspace, int64_t workspace_bytes, int32_t* status,
                          void* stream);
#define HB_ORTHO_MAX_BATCH 64
/* hb_orthonormalize_f32 for n_mats (1..HB_ORTHO_MAX_BATCH) matrices of one shape, every launch covering all of them: the counterpart of
 * the reference's same-shape bucketing (heavyball/chainable.py:503-584) for the QR of get_orthogonal_matrix_QR.  A
 * factorisation is a chain of ~16 short dependent launches per panel, so n_mats matrices take about as long as one.
 * Q, workspace, status: HOST arrays of n_mats device pointers (each workspace of workspace_bytes >=
 * hb_orthonormalize_workspace_bytes(m, n), one status word per matrix; the matrices must agree in their address modulo
 * 16 bytes).  A matrix' result does not depend on the other matrices of its batch, but it may depend on their number: a
 * panel product is split along K when the whole batch has too few workgroups to fill the GPU, and the split changes the
 * order of the sum. */
int hb_orthonormalize_f32_batched(int32_t n_mats, float* const* Q, int64_t m, int64_t n, int64_t ld, void* const* workspace,
                                  int64_t workspace_bytes, int32_t* const* status, void* stream);

/* profiling yardstick with no counterpart in the reference: copies nbytes (a multiple of 16) with 128-bit accesses, so
 * that hardware byte counters can be scaled against a transfer of known size */
int hb_copy_probe(const void* src, void* dst, int64_t nbytes, void* stream);

const char* hb_last_error(void);
int hb_chunk_elems(void); /* == HB_CHUNK */
int hb_abi_version(void); /* == HB_ABI_VERSION of the header the library was built from */

#ifdef __cplusplus
}
#endif
#endif

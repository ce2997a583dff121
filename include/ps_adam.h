/*
 * ps_adam.h -- C ABI of the MI355X (gfx950) chunk-wise mixed-precision Adam step.
 *
 * This is the drop-in boundary for ONE path of PatrickStar: the native operator
 * `cpu_adam_op` {create_adam, adam_update, destroy_adam} (reference:
 * patrickstar/ops/csrc/adam/cpu_adam.cpp:751-756) together with the work the
 * reference does around it per optimizer step in Python: the whole-chunk
 * fp32->fp16 write-back (patrickstar/ops/chunk_io_buff.py:85-151), the fp16
 * gradient staging (chunk_io_buff.py:214-255), the inf/nan probe
 * (patrickstar/fp16/loss_scaler.py:133-155) and the loss-scale state machine
 * (loss_scaler.py:158-182).
 *
 * Conventions
 *   - plain C types only; every pointer named d_* (and every address inside a
 *     ps_chunk, unless stated otherwise) is a DEVICE address; arrays of
 *     ps_chunk descriptors themselves are ordinary HOST arrays that the call
 *     reads before it returns (descriptors reach the kernels as kernel
 *     arguments); the library never allocates, frees or keeps tensor memory.
 *   - every entry point that takes a stream only ENQUEUES work on it and
 *     returns; nothing here synchronises with the host except ps_state_read.
 *   - return value: 0 on success; a negative value on failure
 *     (-hipError_t for a HIP runtime error, PS_ERR_* otherwise);
 *     ps_last_error() gives the text.  Nothing throws across this boundary.
 *   - vector (16-byte) accesses are used when the four base addresses of a
 *     chunk / tensor are 16-byte aligned, and also when only momentum and
 *     variance sit at another element phase than the two parameter lists
 *     (their 16-byte accesses then go to 4-byte-aligned addresses); otherwise a
 *     slower element-wise path produces the same bits.
 */
#ifndef PS_ADAM_H
#define PS_ADAM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PS_ABI_VERSION 5

#define PS_ERR_BAD_ARG (-10001)     /* null pointer, negative count, unknown mode */
#define PS_ERR_UNKNOWN_ID (-10002)  /* optimizer id was never created (the reference dereferences null here) */
#define PS_ERR_NO_DEVICE (-10003)   /* no usable GPU */

typedef void* ps_stream_t; /* a hipStream_t; NULL is the null stream */

/*
 * One position of the four parallel chunk lists (reference: ChunkType in
 * patrickstar/core/const.py:76-81; optimizer-state chunks are mapped 1:1 to
 * the fp16 parameter chunk, patrickstar/core/client.py:282-309).  All four
 * payloads have `chunk_numel` elements and identical tensor offsets.
 * `param_fp16` holds the fp16 GRADIENTS when a step starts (backward writes each
 * gradient over its parameter's slot, patrickstar/core/hook.py:212-216) and the
 * refreshed fp16 PARAMETERS when it ends.
 */
typedef struct ps_chunk {
    float* param_fp32;    /* ChunkType.PARAM_FP32 payload */
    float* exp_avg;       /* ChunkType.MOMENTUM payload   */
    float* exp_avg_sq;    /* ChunkType.VARIANCE payload   */
    uint16_t* param_fp16; /* ChunkType.PARAM_FP16 payload (IEEE binary16 bit patterns) */
} ps_chunk;

/*
 * Device-resident state of the optimizer step: the DynamicLossScaler fields
 * (loss_scaler.py:107-125), the sticky overflow flag of FP16Adam
 * (fp16_cpu_adam.py:279-285) and the Adam step counter with its float
 * beta^t running products (cpu_adam.h:143-162).  It lives in device memory
 * so that "was there an overflow -> skip, restore, halve" needs no host
 * round trip.  256 bytes, 16-byte aligned.
 */
typedef struct ps_step_state {
    double cur_scale;           /* loss_scale; Python float semantics (binary64) */
    double scale_factor;
    double min_scale;
    int64_t cur_iter;           /* update_scale calls so far */
    int64_t last_overflow_iter; /* -1 initially */
    int64_t scale_window;
    int64_t adam_step;          /* completed (not skipped) optimizer steps == state[p]["step"] */
    int64_t skipped_steps;
    int32_t delayed_shift;
    int32_t cur_hysteresis;
    int32_t consecutive_hysteresis;
    int32_t scale_is_int;       /* Python type of cur_scale: int until the first true division */
    int32_t factor_is_int;
    int32_t min_is_int;
    uint32_t overflow;          /* sticky flag of the step being assembled (0/1) */
    uint32_t last_skipped;      /* what the latest ps_scaler_update decided */
    float beta1;                /* the betas of the NEXT step over whole chunk lists (the device-decided entry points */
    float beta2;                /* take none); ps_state_seed_step sets them */
    float beta1_t_next;         /* beta1^t that the FIRST operator call of step t = adam_step + 1 uses */
    float beta2_t_next;
    uint32_t reserved[4];
    /* torch-formula arithmetic (PS_ARITH_TORCH): the Python floats behind the betas and the
     * binary64 bias corrections 1 - beta ** t for t = adam_step + 1 (fp16_cpu_adam.py:412-413) */
    double beta1_f64;
    double beta2_f64;
    double bias_correction1_next;
    double bias_correction2_next;
    /* The native operator object as Adam_Optimizer::IncrementStep (cpu_adam.h:143-162) leaves it.  The
     * reference calls the operator once per tensor with the same step number; only the first call of a
     * step can continue the running float product (`_step + 1 == step`), every later call of the step
     * evaluates pow. */
    int64_t operator_step;      /* its _step: the step number of its latest call (0: never called) */
    float beta1_t_cur;          /* its _betta1_t / _betta2_t after that call */
    float beta2_t_cur;
    float beta1_t_rest;         /* (float)pow((double)beta, adam_step + 1): what every operator call */
    float beta2_t_rest;         /* of step adam_step + 1 after the first one uses */
    uint32_t reserved2[2];
    float operator_beta1;       /* its _betta1 / _betta2: the betas of its latest call (create_adam's before any) */
    float operator_beta2;
    /* What the operator object holds after the last call of a step queued by ps_adam_step_tensors_each (every
     * tensor its own step number and betas).  ps_scaler_update adopts it if the step turns out clean and drops
     * it if the step is skipped.  pending_operator_step == 0: nothing is pending. */
    int64_t pending_operator_step;
    float pending_beta1_t;
    float pending_beta2_t;
    float pending_beta1;
    float pending_beta2;
    uint32_t reserved3[8];
} ps_step_state;

/*
 * How the reference would have cut one step over a chunk list into operator calls.  FP16Adam calls
 * adam_update once per trainable tensor, in param_groups order, all with the same step number
 * (patrickstar/ops/fp16_cpu_adam.py:336-428), and Adam_Optimizer::IncrementStep (cpu_adam.h:143-162)
 * gives the first of those calls the running float product beta^t and every later one
 * (float)pow(beta, t).  The two differ in the last bits (1 / sqrt(1 - beta2^t) by up to 1e-5
 * relative at small t), so a fused pass over whole chunks has to know which elements the first call
 * covered.  Only the operator's arithmetic looks at this; the torch formula has no such state.
 *
 * One step may be spread over several calls of the step entry points (say ps_adam_step_tensors for
 * chunks that hold frozen parameters and ps_adam_step_hybrid for the rest): every call is given the
 * n_calls of the WHOLE step; the call whose list holds the first operator call's tensor is made first and
 * names it; every other call passes first_numel = 0.  ps_scaler_update follows the last of them, once.
 */
typedef struct ps_call_pattern {
    int64_t n_calls;       /* operator calls of the step over this list = its trainable tensors (>= 1) */
    int64_t first_chunk;   /* index of the chunk that holds the first call's tensor (ps_adam_step_hybrid:
                              chunks[] counted first, host_chunks[] after them) */
    uint64_t first_offset; /* element offset of that tensor inside its chunk */
    uint64_t first_numel;  /* its length in elements */
} ps_call_pattern;

/* One entry of the optional per-iteration log written by ps_scaler_update. */
typedef struct ps_scale_record {
    double scale_after;   /* loss_scale after the call */
    uint32_t overflow;    /* the flag the call consumed */
    uint32_t scale_is_int;
} ps_scale_record;

/* ---- library ---------------------------------------------------------- */

int ps_abi_version(void);
const char* ps_last_error(void); /* text of the calling thread's latest failure */

/* ---- native operator (replaces pybind module cpu_adam_op) --------------- */

/* create_adam (cpu_adam.cpp:379-417).  Holds the host-side scalar state of
 * one optimizer (alpha, betas, eps, weight decay, beta^t, step); ids are
 * chosen by the caller (FP16Adam.optimizer_id, fp16_cpu_adam.py:62,175-176).
 * Re-creating an id replaces it.  should_log prints one line like the reference. */
int ps_adam_create(int optimizer_id, float alpha, float beta1, float beta2, float eps,
                   float weight_decay, int adamw_mode, int should_log);

/* FP16Adam's element-wise "gradient clipping" (patrickstar/ops/fp16_cpu_adam.py:364-379, the
 * GPU branch): fp16 gradients are clamped to +-min(65504, gradient_clipping * loss_scale),
 * the bound narrowed double -> float -> half as Tensor.clamp_ does.  Applied inside the
 * chunk-list kernels (ps_adam_step_chunks, _gated, _hybrid) at no extra memory traffic; the
 * device-gated form uses the device-resident scale.  ps_adam_update does not clamp (the
 * reference clamps in Python before it calls the operator).  <= 0 switches it off (default). */
int ps_adam_set_grad_clamp(int optimizer_id, double gradient_clipping);

#define PS_ARITH_OPERATOR 0
#define PS_ARITH_TORCH 1
/* Which of the reference's two arithmetics the chunk-list entry points (ps_adam_step_chunks,
 * _gated, _hybrid) apply to chunks that are updated in place in HBM.  FP16Adam picks by where a
 * chunk's optimizer state lives (patrickstar/ops/fp16_cpu_adam.py:415-443):
 *   PS_ARITH_OPERATOR (default)  the native operator's order of operations (cpu_adam.cpp:91-141)
 *                                with its float step scalars (cpu_adam.h:143-175): what the
 *                                reference runs for state held in host memory;
 *   PS_ARITH_TORCH               FP16Adam.torch_adam_update (fp16_cpu_adam.py:245-277): what the
 *                                reference runs for state held in GPU memory.  Each torch
 *                                element-wise kernel it calls is restated with the rounding that
 *                                torch's GPU kernels have: Python-double scalars narrowed to float
 *                                at the kernel, `x / python_scalar` = x * (float)(1.0 / s),
 *                                add(alpha) / addcmul / addcdiv as one fused multiply-add around
 *                                the separately rounded product or quotient, bias corrections
 *                                1 - beta ** t in binary64.
 * Host-resident chunks streamed by ps_adam_step_hybrid always take the operator's arithmetic, as
 * the reference updates those with the operator.  ps_adam_update is the operator itself. */
int ps_adam_set_arithmetic(int optimizer_id, int arithmetic);

/* destroy_adam (cpu_adam.cpp:744-749).  Unknown ids are ignored, as there. */
int ps_adam_destroy(int optimizer_id);

/* adam_update (cpu_adam.cpp:700-742) on ONE flat tensor in device memory:
 * advances the host scalar state exactly like Adam_Optimizer::IncrementStep /
 * update_state (cpu_adam.h:143-175) and applies the update of
 * Adam_Optimizer::Step (cpu_adam.cpp:91-141) to every element.
 *   d_grads          fp16 (grads_are_half != 0) or fp32; never written
 *   loss_scale <= 0  no unscale (cpu_adam.cpp:101)
 *   d_param_fp16_out optional: receives RNE(fp32 param) per element (the
 *                    write-back of chunk_io_buff.py:116-126); may alias d_grads
 *                    when the gradients are fp16; NULL to skip. */
int ps_adam_update(int optimizer_id, size_t step, float lr, float beta1, float beta2, float epsilon,
                   float weight_decay, int bias_correction, float* d_params, const void* d_grads,
                   int grads_are_half, float* d_exp_avg, float* d_exp_avg_sq, size_t numel,
                   float loss_scale, uint16_t* d_param_fp16_out, ps_stream_t stream);

/* ---- chunk-list step (what FP16Adam.step does per step, fp16_cpu_adam.py:312-470,609) */

/* One fused pass over a whole chunk list: for every element of every chunk
 * read fp16 grad, fp32 param, m, v once; write fp32 param, m, v and the fp16
 * param (over the grad) once: 28 bytes per element.  chunks is a host array of
 * n_chunks descriptors.
 *   calls       how the reference would have cut the step into operator calls (ps_call_pattern).
 *               NULL: the whole list is one flat tensor for the operator and its host scalar state
 *               (cpu_adam.h:143-162) advances once; with n_calls >= 2 it is taken through the first
 *               call and one further call, from which on the object no longer moves.
 *   used_numel  NULL: every chunk is updated over all chunk_numel elements.  Else a host array of
 *               n_chunks lengths: chunk i holds tensors in its first used_numel[i] elements only and
 *               ZEROS behind them in all four payloads (the reference allocates payloads with
 *               torch.zeros and only ever writes tensor spans, patrickstar/core/chunk_data.py:148-154).
 *               Zeros are a fixed point of the update (g = m = v = p = 0 gives m = v = 0 and
 *               p = 0 under L2 and decoupled decay alike, fp16 0), so the pass leaves the tail alone:
 *               same bits, fewer bytes.  The one case where the reference's arithmetic does not keep
 *               the zeros (a denominator of 0: eps == 0, or a non-finite step size: it writes NaNs into
 *               the padding) is detected and the tail is then computed like everything else.
 * Hyper-parameters and loss_scale are the Python numbers (binary64).  The operator's
 * arithmetic narrows them to float first, as the pybind signature of adam_update does
 * (cpu_adam.cpp:700-712); the torch arithmetic uses them as torch does.
 * loss_scale <= 0: no unscale (no loss scaler). */
int ps_adam_step_chunks(int optimizer_id, size_t step, double lr, double beta1, double beta2,
                        double epsilon, double weight_decay, int bias_correction,
                        const ps_chunk* chunks, int n_chunks, size_t chunk_numel,
                        const size_t* used_numel, const ps_call_pattern* calls, double loss_scale,
                        ps_stream_t stream);

/* Same pass, decided on the device: if d_state->overflow is set, every chunk's
 * fp16 payload is restored from the fp32 master copy (fp16_cpu_adam.py:298-309)
 * and nothing else changes; otherwise the Adam update runs with
 * loss_scale = d_state->cur_scale and t = d_state->adam_step + 1 (beta^t of the first and of the
 * later operator calls, or the binary64 bias corrections of the torch arithmetic, from d_state; the
 * betas are d_state's: ps_state_seed_step changes them).  used_numel as for ps_adam_step_chunks.
 * Follow with ps_scaler_update(..., PS_FLAG_FROM_DEVICE, ..., calls ? calls->n_calls : 1). */
int ps_adam_step_chunks_gated(int optimizer_id, double lr, double epsilon, double weight_decay,
                              int bias_correction, const ps_chunk* chunks, int n_chunks,
                              size_t chunk_numel, const size_t* used_numel,
                              const ps_call_pattern* calls, const ps_step_state* d_state,
                              ps_stream_t stream);

/* The per-tensor loop of FP16Adam.fp16_chunk_adam_ops (fp16_cpu_adam.py:336-468) as ONE call, for chunk layouts
 * in which a parameter's exp_avg / exp_avg_sq do not sit at the parameter's own offset inside their chunks (the
 * reference packs optimizer-state tensors first-fit in parameters() order, patrickstar/core/client.py:282-309,
 * which can permute them inside a chunk), so that the whole-chunk pass of ps_adam_step_chunks does not apply.
 *   tensors[i]  the four DEVICE addresses of parameter i: fp32 param, exp_avg, exp_avg_sq and its fp16 slot
 *               (gradient in, fp16 parameter out), numels[i] elements each; both are host arrays
 *   d_state     NULL: host-decided step with loss_scale; else device-gated like ps_adam_step_chunks_gated
 *               (step, betas and loss_scale ignored; a flagged step restores the fp16 slots from fp32)
 *   calls       NULL: the list is the whole step, n_tensors operator calls, tensors[0] the first.  Else
 *               n_calls = the operator calls of the whole step (some of them may be made through other
 *               entry points, see ps_call_pattern) and first_chunk = the index in tensors[] of the
 *               step's first call, with first_offset = 0 and first_numel = numels[first_chunk]
 *               (a tensor is one call); first_numel = 0: the first call is not in this list
 * Same arithmetic, clamp and 28 B/element as the chunk-list form.  Every tensor is one operator call of the
 * reference's loop (zero-length tensors included: the reference calls the operator for them too); follow a
 * device-gated call with ps_scaler_update(..., the step's number of calls).
 * Tensors of (nearly) equal length share a launch, up to 64 of them; the order of the list decides nothing
 * but, without a pattern, which tensor is the first call. */
int ps_adam_step_tensors(int optimizer_id, size_t step, double lr, double beta1, double beta2,
                         double epsilon, double weight_decay, int bias_correction,
                         const ps_chunk* tensors, const size_t* numels, int n_tensors,
                         const ps_call_pattern* calls, double loss_scale, const ps_step_state* d_state,
                         ps_stream_t stream);

/* One adam_update call of the reference's per-tensor loop with the numbers of ITS tensor: FP16Adam.step counts
 * state[p]["step"] per parameter and reads lr / betas / eps / weight_decay from state[p] per parameter
 * (patrickstar/ops/fp16_cpu_adam.py:571-606), and fp16_chunk_adam_ops hands each call its own (:403-428).  They
 * differ between tensors when a parameter was frozen for some steps (its count stays behind) or when somebody
 * wrote state[p]["lr"] for some parameters only. */
typedef struct ps_tensor_call {
    double lr, beta1, beta2, eps, weight_decay;
    int64_t step;       /* host-decided step: this tensor's step number (state[p]["step"] after its increment, >= 1);
                           device-decided step: its distance d from the device's counter, the tensor's step number
                           then being d_state->adam_step + 1 + d (which must come out >= 1) */
    int32_t arithmetic; /* PS_ARITH_OPERATOR, PS_ARITH_TORCH, or -1 for the optimizer's own (ps_adam_set_arithmetic) */
    int32_t flags;      /* 0, or PS_TENSOR_GRAD_F32 */
} ps_tensor_call;

/* ps_tensor_call::flags.  PS_TENSOR_GRAD_F32: a parameter that PyTorch manages itself in binary32 (the reference's
 * TORCH_BASED parameters, i.e. embedding weights under "use_cpu_embedding": fp16_cpu_adam.py:345-353 takes their
 * binary32 .grad and updates the parameter itself, and :459-460 writes no fp16 copy).  The tensor's descriptor then
 * holds the address of its binary32 GRADIENT in the param_fp16 field; the gradient is only read, and a flagged
 * device-decided step leaves the tensor alone (the reference restores nothing for it, :301-302).  The gradient clamp
 * is applied with its binary32 bound, (float)min(65504, clipping * loss_scale). */
#define PS_TENSOR_GRAD_F32 1

/* Device memory ps_adam_step_tensors_each needs for a device-decided step over n_tensors tensors (the step
 * constants of every distinct call, formed on the device): 64 bytes per tensor at most. */
size_t ps_tensors_each_workspace_bytes(int n_tensors);

/* ps_adam_step_tensors with per-tensor step numbers and hyper-parameters: tensors[i] is updated with each[i].
 * The list is the WHOLE step, in the reference's call order (param_groups order): the native operator object is
 * taken through every call that uses the operator's arithmetic, in that order, exactly as
 * Adam_Optimizer::IncrementStep (cpu_adam.h:143-162) moves: a call continues the running float product beta^t
 * only if its step number is the previous call's plus one and its betas are the previous call's, and evaluates
 * (float)pow((double)beta, step) otherwise.  Calls with the torch arithmetic form 1 - beta ** step in binary64
 * from their own numbers and leave the object alone.  Launches are cut by the tensors' lengths as in
 * ps_adam_step_tensors and take tensors of any step number and any lr / betas / eps (every tensor finds its
 * call's constants through an index), so a list in which every tensor has numbers of its own runs like a
 * uniform one; only the arithmetic and the weight-decay form (none, L2, decoupled) separate launches.
 *   d_state == NULL  host-decided: each[i].step is the step number; loss_scale as for ps_adam_step_chunks;
 *                    d_workspace is not used
 *   d_state != NULL  device-decided: a flagged step restores the fp16 slots from fp32; else every call's
 *                    constants are formed ON THE DEVICE from d_state (adam_step, cur_scale, the operator
 *                    object's state) by a small kernel in front of the update kernels, into d_workspace (at
 *                    least ps_tensors_each_workspace_bytes(n_tensors) bytes of device memory, 16-byte aligned,
 *                    owned by the caller and left alone by it until the step has run).  loss_scale is ignored.
 *                    The object's state after the step's last call is left in d_state's pending_* fields: follow
 *                    with ps_scaler_update (operator_calls = the number of operator-arithmetic calls), which
 *                    adopts it on a clean step and drops it on a skipped one.
 * Addresses may be pinned host memory (host-resident optimizer state is then read and written over the link in
 * place).  The clamp of ps_adam_set_grad_clamp applies.  Tensors flagged PS_TENSOR_GRAD_F32 (above) take part in
 * the call sequence like any other. */
int ps_adam_step_tensors_each(int optimizer_id, int bias_correction, const ps_chunk* tensors,
                              const size_t* numels, const ps_tensor_call* each, int n_tensors,
                              double loss_scale, ps_step_state* d_state, void* d_workspace,
                              size_t workspace_bytes, ps_stream_t stream);

/* Unconditional restore p16 = RNE(p32) of a chunk list (FP16ChunkWriteBuffer,
 * chunk_io_buff.py:85-151), or only when d_state->overflow is set if d_state != NULL. */
int ps_restore_fp16_chunks(const ps_chunk* chunks, int n_chunks, size_t chunk_numel,
                           const ps_step_state* d_state, ps_stream_t stream);

/* ---- chunks that live in pinned host memory (hybrid placement) ------------
 *
 * The reference updates host-resident chunks with the CPU operator after
 * staging their fp16 gradients (chunk_io_buff.py:214-255) and casts the result
 * back through a GPU buffer (chunk_io_buff.py:85-151).  Here such chunks are
 * streamed through HBM instead: for chunk k, slot k % n_slots of `staging`
 * receives fp16 grad + fp32 param/m/v by hipMemcpyAsync on a side stream
 * (14 B/element), the fused kernel runs on it, and fp32 param/m/v + fp16 param
 * go back on another side stream (14 B/element); events order the three, so
 * with n_slots >= 2 the copies of neighbouring chunks overlap the kernel.
 *   chunks       host array of descriptors of HBM-resident chunks (may be empty): updated
 *                by the same kernels on `stream`, concurrently with the first copies
 *   host_chunks  host array of descriptors whose fp32 param / m / v addresses are PINNED HOST
 *                memory.  param_fp16 is either pinned host memory too (streamed with the rest) or
 *                a DEVICE address (the fp16 payload stays in HBM, where forward and backward use
 *                it, as in the reference; it is then read and written in place and 12 instead of
 *                14 B/element cross the link each way); the library asks the HIP runtime which
 *   staging      host array of n_slots (1..8) descriptors of DEVICE buffers of
 *                chunk_numel elements each, owned by the caller; param_fp16 may be NULL when
 *                every host chunk keeps its fp16 payload in HBM
 *   used_numel   as for ps_adam_step_chunks, over chunks[] followed by host_chunks[] (NULL: all full);
 *                only the used part of a host chunk crosses the link
 *   calls        as for ps_adam_step_chunks, over chunks[] followed by host_chunks[]; with
 *                PS_ARITH_TORCH only host_chunks[] reach the operator and the pattern describes those
 *                (first_chunk >= n_chunks).  NULL: one operator call for everything
 *   d_state      NULL: host-decided step with loss_scale; else device-gated exactly like
 *                ps_adam_step_chunks_gated (step, betas and loss_scale ignored)
 * Work queued on `stream` before the call is waited for; work queued on it
 * afterwards waits for the last write-back.  The call itself never blocks.
 * Calls on one device (from several host threads, on several streams) take turns: a per-device
 * lock is held while a call queues its work, and the streamed part of a later call is ordered
 * behind everything an earlier call left on the side streams, so concurrent callers get correct
 * results but their copies do not overlap one another's.  The same holds between this entry
 * point and ps_overflow_scan_host_chunks. */
int ps_adam_step_hybrid(int optimizer_id, size_t step, double lr, double beta1, double beta2,
                        double epsilon, double weight_decay, int bias_correction,
                        const ps_chunk* chunks, int n_chunks, const ps_chunk* host_chunks,
                        int n_host_chunks, size_t chunk_numel, const size_t* used_numel,
                        const ps_chunk* staging, int n_slots, const ps_call_pattern* calls,
                        double loss_scale, const ps_step_state* d_state, ps_stream_t stream);

/* The inf/nan probe for host-resident chunks: only the fp16 payloads are
 * streamed (2 B/element) through staging[i].param_fp16; fp16 payloads that
 * live in HBM are probed in place.  used_numel (NULL: all full): only the first used_numel[i] elements
 * of chunk i can hold anything but zeros and only they are looked at. */
int ps_overflow_scan_host_chunks(const ps_chunk* host_chunks, int n_chunks, size_t chunk_numel,
                                 const size_t* used_numel, const ps_chunk* staging, int n_slots,
                                 ps_step_state* d_state, ps_stream_t stream);

/* Whole-buffer RNE cast (payload_fp16.copy_(payload_fp32), chunk_io_buff.py:116-126). */
int ps_cast_fp32_to_fp16(const float* d_src, uint16_t* d_dst, size_t numel, ps_stream_t stream);

/* ---- overflow probe and device-resident loss scaler --------------------- */

/* Initialise *d_state (DynamicLossScaler.__init__, loss_scaler.py:107-125, plus
 * adam_step = 0, beta^t_next = beta).  *_is_int carry the Python types of the
 * three numbers so that loss_scale reads back as int or float like the reference.
 * The betas are the Python floats; the operator's fields hold them narrowed. */
int ps_state_init(ps_step_state* d_state, double init_scale, int init_is_int, double scale_factor,
                  int factor_is_int, int64_t scale_window, double min_scale, int min_is_int,
                  int delayed_shift, int consecutive_hysteresis, double beta1, double beta2,
                  ps_stream_t stream);

/* Set the Adam step counter (load_state_dict, fp16_cpu_adam.py:660-694) and the betas of the next step (the
 * reference hands state[p]["betas"] to the operator with every call, fp16_cpu_adam.py:404-407: betas that
 * differ from the object's restart beta^t from pow, cpu_adam.h:145-150).
 *   fresh_operator != 0  a new operator object stands behind them (step 0, beta^t = 1, as create_adam leaves
 *                        it): its first call, for step adam_step + 1, multiplies only if adam_step is 0 and
 *                        otherwise evaluates pow((float)beta, adam_step + 1) in double and narrows, i.e. the
 *                        reference's cold branch;
 *   fresh_operator == 0  the operator object is the one that has been running (the reference's
 *                        load_state_dict does not touch it): the first call of step adam_step + 1
 *                        continues its running product only if its own step is adam_step and the betas are
 *                        unchanged, as IncrementStep decides (cpu_adam.h:143-162).
 * The torch arithmetic's bias corrections become 1 - pow(beta, adam_step + 1). */
int ps_state_seed_step(ps_step_state* d_state, int64_t adam_step, double beta1, double beta2,
                       int fresh_operator, ps_stream_t stream);

/* Overwrite the loss-scaler fields only (restoring a checkpointed scaler). */
int ps_state_set_scaler(ps_step_state* d_state, double cur_scale, int scale_is_int,
                        int64_t cur_iter, int64_t last_overflow_iter, int cur_hysteresis,
                        ps_stream_t stream);

/* _has_inf_or_nan (loss_scaler.py:133-155) over fp16 data, OR-ed into
 * d_state->overflow.  Wave shuffle + LDS reduction, one atomic per block
 * that saw a hit.  2 bytes per element. */
int ps_overflow_scan(const uint16_t* d_grads_fp16, size_t numel, ps_step_state* d_state,
                     ps_stream_t stream);
int ps_overflow_scan_f32(const float* d_grads_fp32, size_t numel, ps_step_state* d_state,
                         ps_stream_t stream);
/* ... over the fp16 payloads of a chunk list; used_numel as for ps_adam_step_chunks (the zeros behind a
 * chunk's last tensor are finite: they are not read). */
int ps_overflow_scan_chunks(const ps_chunk* chunks, int n_chunks, size_t chunk_numel,
                            const size_t* used_numel, ps_step_state* d_state, ps_stream_t stream);

/* ps_overflow_scan_chunks for callers that cannot allocate device memory.  It has no counterpart in the
 * reference: it exists for code running under HIP graph capture, tight serving loops and harnesses that
 * forbid hipMalloc, which have no ps_step_state to hand over.  The flag is an ordinary word of the
 * caller's (device-accessible, 4-byte aligned), set to 1 if any fp16 payload holds an inf / nan and
 * left alone otherwise (sticky, like ps_step_state::overflow).  The probe runs without atomics: every
 * workgroup leaves its partial result in a word of a file-scope device array inside the library
 * (4 MiB per GPU, resolved with hipGetSymbolAddress at the first call on a device: make that call
 * outside a stream capture), and a second kernel reduces those words.  The call allocates and frees
 * nothing and records kernel launches only (no memset), so it can be captured into a HIP graph.
 *   limit   n_chunks * ceil(chunk_numel / 8192) <= 1,048,576 scratch words, i.e. at most 8 Gi elements
 *           per call; more is rejected with PS_ERR_BAD_ARG before anything is queued
 *   sharing every call on one GPU uses that GPU's one scratch array: calls that overlap in time on
 *           one GPU (different streams or host threads) race.  Nothing in it needs clearing: each call
 *           overwrites every word it later reads. */
int ps_overflow_scan_chunks_noalloc(const ps_chunk* chunks, int n_chunks, size_t chunk_numel,
                                    uint32_t* d_flag, ps_stream_t stream);

/* Backward-side producer (patrickstar/core/hook.py:200-230): copy one parameter's
 * gradient (fp16, or fp32 rounded RNE) into its slot of the fp16 chunk and, in
 * the same pass, OR "holds inf/nan" into d_state->overflow (skipped when
 * d_state is NULL).  Replaces tmp_tensor.copy_(param.grad) plus
 * optimizer.check_overflow(param) and its host sync. */
int ps_grad_to_chunk(const void* d_grad, int grad_is_half, uint16_t* d_slot_fp16, size_t numel,
                     ps_step_state* d_state, ps_stream_t stream);

#define PS_FLAG_FALSE 0
#define PS_FLAG_TRUE 1
#define PS_FLAG_FROM_DEVICE 2
/* DynamicLossScaler.update_scale (loss_scaler.py:158-182) on the device.
 * flag_mode chooses the `overflow` argument: a host-given bool or the sticky
 * device flag.  A clean step also advances adam_step, the operator's beta^t
 * state (cpu_adam.h:143-162) and the binary64 bias corrections of
 * the torch arithmetic.  operator_calls says how often the step that was just
 * queued called the operator in the reference's terms: the n_calls of its
 * ps_call_pattern (1 without one, the tensor count of ps_adam_step_tensors, 0 if
 * every chunk took the torch formula); a pending record left by ps_adam_step_tensors_each takes its place.
 * Clears the sticky flag and the pending record.  If d_log
 * is not NULL, entry [cur_iter % log_capacity] (cur_iter before the
 * increment) records the decision. */
int ps_scaler_update(ps_step_state* d_state, int flag_mode, ps_scale_record* d_log,
                     int64_t log_capacity, int64_t operator_calls, ps_stream_t stream);

/* Copy *d_state to host memory and wait for it: the only synchronising call. */
int ps_state_read(const ps_step_state* d_state, ps_step_state* host_out, ps_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PS_ADAM_H */

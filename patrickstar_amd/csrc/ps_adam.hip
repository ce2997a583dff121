// Chunk-wise mixed-precision Adam step for MI355X (gfx950, wave64).
//
// Everything here is HBM-bandwidth bound: 28 bytes move per element per step
// (read fp16 grad + fp32 param/m/v, write fp32 param/m/v + fp16 param) for
// ~20 flops.  No matrix cores are involved.  What the kernels are organised
// around, all of it measured on MI355X:
//   * one pass over the data, in place; per lane one 16-byte access to each
//     fp32 array and one 8-byte access to the fp16 array, so that every wave
//     instruction covers a contiguous span of whole cache lines;
//   * one small tile (256 elements) per single-wave workgroup and a CAP on
//     resident workgroups (9 per CU, enforced by requesting 17 KiB of unused
//     dynamic LDS): the pass touches four arrays for reading and the same four
//     for writing, and HBM efficiency drops when the set of in-flight cache
//     lines gets wide; a narrow, steadily advancing window per array gave
//     6.3 TB/s where the fully occupied machine gave 5.3 TB/s (a plain
//     1-read-1-write copy peaks at 6.3-6.4 TB/s on the same GPU);
//   * chunk descriptors travel in the kernel-argument segment (64 per launch),
//     so a wave's first data load depends on one scalar load, not two;
//   * plain (temporal) loads/stores: non-temporal loads cost 6 % at this
//     operating point (20-25 % with fully occupied CUs), non-temporal stores
//     change nothing.
//
// Arithmetic contract (ps_arith.h).  Operator arithmetic: bit-exact with the
// explicit-intrinsic body of the reference operator
// (patrickstar/ops/csrc/adam/cpu_adam.cpp:91-141): every a*b+c the reference
// writes as SIMD_FMA is one __builtin_fmaf; every other operation is an
// individually rounded IEEE binary32 op.  Torch arithmetic: one rounding step
// per torch kernel of FP16Adam.torch_adam_update
// (patrickstar/ops/fp16_cpu_adam.py:259-277), as torch's GPU kernels round.
// Everything must be compiled with -ffp-contract=off and with correctly rounded
// fp32 divide and sqrt (hipcc's default), denormals preserved.
//
// Layout of the sources: ps_config.h (tuning knobs), ps_arith.h (step constants
// and per-element arithmetic), ps_tile.h (vector accesses, one tile per wave),
// ps_kernels.h (the kernels), this file (host state, launches, streaming of
// host-resident chunks, the C ABI).
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <exception>
#include <memory>
#include <mutex>
#include <new>
#include <string>
#include <unordered_map>
#include <vector>

#include "ps_adam.h"

#include "ps_config.h"
#include "ps_arith.h"
#include "ps_tile.h"
#include "ps_kernels.h"

namespace {

// ------------------------------------------------------------------ errors

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char* what)
{
    return fail(-(int)e, "%s: %s", what, hipGetErrorString(e));
}

#define PS_HIP(call)                                      \
    do {                                                  \
        hipError_t e_ = (call);                           \
        if (e_ != hipSuccess) return hip_fail(e_, #call); \
    } while (0)

// ------------------------------------------------------- host scalar state
//
// One object per optimizer id: the float scalars the reference keeps in
// Adam_Optimizer (cpu_adam.h:177-197) and their update rules.

struct HostAdam {
    float alpha, beta1, beta2, eps, weight_decay;
    float beta1_t = 1.0f, beta2_t = 1.0f;
    size_t step = 0;
    bool adamw;
    double grad_clamp = -1.0;  // FP16Adam.gradient_clipping; <= 0: off
    int arith = PS_ARITH_OPERATOR;  // arithmetic for chunks updated in place in HBM

    // cpu_adam.h:143-162
    void advance(size_t s, float b1, float b2)
    {
        if (b1 != beta1 || b2 != beta2) {
            step = s;
            beta1 = b1;
            beta2 = b2;
            beta1_t = (float)std::pow((double)b1, (double)s);
            beta2_t = (float)std::pow((double)b2, (double)s);
            return;
        }
        step += 1;
        if (step != s) {
            beta1_t = (float)std::pow((double)beta1, (double)s);
            beta2_t = (float)std::pow((double)beta2, (double)s);
            step = s;
        } else {
            beta1_t = beta1_t * beta1;
            beta2_t = beta2_t * beta2;
        }
    }
    // cpu_adam.h:163-170 (the bias-correction scalars follow in finish_consts)
    void set(float lr, float epsilon, float wd)
    {
        alpha = lr;
        eps = epsilon;
        weight_decay = wd;
    }
};

std::mutex g_registry_mutex;
std::unordered_map<int, std::shared_ptr<HostAdam>> g_registry;

std::shared_ptr<HostAdam> find_opt(int id)
{
    std::lock_guard<std::mutex> lock(g_registry_mutex);
    auto it = g_registry.find(id);
    return it == g_registry.end() ? nullptr : it->second;
}

// ------------------------------------------------------------ launch helpers

// The runtime refuses a launch whose grid times block size reaches 2^32 threads in a dimension.  Kernels that take one
// tile per single-wave workgroup are checked against kMaxGridX before anything is queued (2^26 - 1 tiles: chunks and
// tensors of up to 17 G elements); kernels that loop over their tiles are simply capped (grid_1d).
constexpr size_t kMaxGridX = 0xFFFFFFFFull / 64;
static_assert(kBlock == 64 && kScanBlock == 64, "kMaxGridX is for 64-thread workgroups");

unsigned grid_1d(size_t n_blocks, size_t block_threads)
{
    const size_t most = 0xFFFFFFFFull / block_threads;
    size_t g = n_blocks < most ? n_blocks : most;
    return (unsigned)(g ? g : 1);
}

// Validated view of a host array of chunk descriptors.
struct ChunkList {
    const ps_chunk* chunks;
    int n_chunks;
    size_t chunk_numel;
    const size_t* used;  // per chunk: elements in front of the zero padding; nullptr: every chunk is full
    size_t tile;         // elements per workgroup of the kernel that will run over the list

    size_t numel_of(int i) const { return used ? used[i] : chunk_numel; }
};

// All descriptors are checked here, before anything is enqueued or any host state advances.
int make_chunk_list(ChunkList& a, const ps_chunk* chunks, int n_chunks, size_t chunk_numel, const size_t* used_numel,
                    size_t tile, bool fp16_only = false, const char* what = "chunk")
{
    if (n_chunks < 0) return fail(PS_ERR_BAD_ARG, "n_chunks = %d is negative", n_chunks);
    if (chunks == nullptr && n_chunks > 0) return fail(PS_ERR_BAD_ARG, "chunks is NULL");
    for (int i = 0; i < n_chunks; ++i) {
        const ps_chunk& c = chunks[i];
        if (!c.param_fp16 || (!fp16_only && (!c.param_fp32 || !c.exp_avg || !c.exp_avg_sq)))
            return fail(PS_ERR_BAD_ARG, "%s %d has a NULL payload address", what, i);
        if (used_numel && used_numel[i] > chunk_numel)
            return fail(PS_ERR_BAD_ARG, "%s %d: used_numel = %zu is beyond chunk_numel = %zu", what, i, used_numel[i],
                        chunk_numel);
    }
    a.chunks = chunks;
    a.n_chunks = n_chunks;
    a.chunk_numel = chunk_numel;
    a.used = used_numel;
    a.tile = tile;
    if ((chunk_numel + tile - 1) / tile > kMaxGridX)
        return fail(PS_ERR_BAD_ARG, "chunk_numel = %zu is beyond the launch grid", chunk_numel);
    return 0;
}

// Calls launch(batch, grid, index of the batch's first chunk) for every group of up to kBatch chunks.  The grid is
// as wide as the longest chunk of the batch; workgroups beyond a shorter chunk's end leave at once.
template <typename F>
int for_each_batch(const ChunkList& a, F launch)
{
    for (int first = 0; first < a.n_chunks; first += kBatch) {
        int n = a.n_chunks - first < kBatch ? a.n_chunks - first : kBatch;
        ChunkBatch b;
        memset(&b, 0, sizeof(b));
        size_t tiles = 0;
        for (int i = 0; i < n; ++i) {
            b.c[i] = a.chunks[first + i];
            b.n[i] = a.numel_of(first + i);
            tiles = std::max(tiles, (b.n[i] + a.tile - 1) / a.tile);
        }
        if (tiles == 0) continue;
        launch(b, dim3((unsigned)tiles, (unsigned)n), first);
        PS_HIP(hipGetLastError());
    }
    return 0;
}

// Validated copy of a ps_call_pattern: how many operator calls the reference makes in the step and
// which elements its first call covers, as a chunk index over the call's whole list.
struct Calls {
    int64_t n_calls = 1;
    int64_t first_chunk = -1;  // -1: the first call's span is not needed (one call, or no elements)
    uint64_t lo = 0, hi = 0;

    // The span as the launch of chunks [batch_first, batch_first + n) sees it.
    FirstCall in_batch(int64_t batch_first, int n) const
    {
        FirstCall fc{-1, 0, 0};
        if (first_chunk >= batch_first && first_chunk < batch_first + n) {
            fc.chunk = (int)(first_chunk - batch_first);
            fc.lo = lo;
            fc.hi = hi;
        }
        return fc;
    }
};

int make_calls(Calls& out, const ps_call_pattern* calls, int64_t n_chunks_total, size_t chunk_numel)
{
    out = Calls();
    if (calls == nullptr) return 0;
    if (calls->n_calls < 1) return fail(PS_ERR_BAD_ARG, "calls->n_calls = %lld must be at least 1", (long long)calls->n_calls);
    out.n_calls = calls->n_calls;
    if (calls->n_calls == 1 || calls->first_numel == 0) return 0;  // one call, or a first call without elements
    if (calls->first_chunk < 0 || calls->first_chunk >= n_chunks_total)
        return fail(PS_ERR_BAD_ARG, "calls->first_chunk = %lld is outside the list of %lld chunks",
                    (long long)calls->first_chunk, (long long)n_chunks_total);
    if (calls->first_offset > chunk_numel || calls->first_numel > chunk_numel - calls->first_offset)
        return fail(PS_ERR_BAD_ARG, "the first call's tensor (offset %llu, %llu elements) does not fit a chunk of %zu",
                    (unsigned long long)calls->first_offset, (unsigned long long)calls->first_numel, chunk_numel);
    out.first_chunk = calls->first_chunk;
    out.lo = calls->first_offset;
    out.hi = calls->first_offset + calls->first_numel;
    return 0;
}

template <int ARITH, int WD>
void launch_adam_batch_wd(const ChunkBatch& b, dim3 grid, const StepConsts& c, const FirstCall& fc, hipStream_t s)
{
    dim3 block(kBlock);
    if (c.unscale == UNSCALE_MUL)
        hipLaunchKernelGGL((adam_chunks_kernel<ARITH, WD, UNSCALE_MUL>), grid, block, kLdsBytes, s, b, c, fc);
    else if (ARITH == PS_ARITH_OPERATOR && c.unscale == UNSCALE_DIV)  // the torch formula never divides
        hipLaunchKernelGGL((adam_chunks_kernel<ARITH, WD, UNSCALE_DIV>), grid, block, kLdsBytes, s, b, c, fc);
    else
        hipLaunchKernelGGL((adam_chunks_kernel<ARITH, WD, UNSCALE_NONE>), grid, block, kLdsBytes, s, b, c, fc);
}

template <int ARITH>
void launch_adam_batch_arith(const ChunkBatch& b, dim3 grid, const StepConsts& c, const FirstCall& fc, hipStream_t s)
{
    if (c.wd_mode == WD_DECOUPLED)
        launch_adam_batch_wd<ARITH, WD_DECOUPLED>(b, grid, c, fc, s);
    else if (c.wd_mode == WD_L2)
        launch_adam_batch_wd<ARITH, WD_L2>(b, grid, c, fc, s);
    else
        launch_adam_batch_wd<ARITH, WD_NONE>(b, grid, c, fc, s);
}

// `c` must have been built for `arith` (finish_consts / torch_consts).  `fc`: which elements of the
// batch the step's first operator call covers; the torch formula has no such distinction.
void launch_adam_batch(int arith, const ChunkBatch& b, dim3 grid, const StepConsts& c, const FirstCall& fc,
                       hipStream_t s)
{
    if (arith == PS_ARITH_TORCH)
        launch_adam_batch_arith<PS_ARITH_TORCH>(b, grid, c, FirstCall{-1, 0, 0}, s);
    else
        launch_adam_batch_arith<PS_ARITH_OPERATOR>(b, grid, c, fc, s);
}

template <int ARITH>
void launch_gated_batch_arith(const ChunkBatch& b, dim3 grid, size_t chunk_numel,
                              const GatedArgs& ga, const FirstCall& fc, const ps_step_state* d_state,
                              hipStream_t s)
{
    dim3 block(kBlock);
    // the operator tests its float weight decay "> 0" (cpu_adam.cpp:42), the torch formula "!= 0"
    const bool decay = ARITH == PS_ARITH_OPERATOR ? (float)ga.wd > 0.0f : ga.wd != 0.0;
    if (decay && ga.adamw)
        hipLaunchKernelGGL((adam_chunks_gated_kernel<ARITH, WD_DECOUPLED>), grid, block, kLdsBytes, s, b, chunk_numel, ga, fc, d_state);
    else if (decay)
        hipLaunchKernelGGL((adam_chunks_gated_kernel<ARITH, WD_L2>), grid, block, kLdsBytes, s, b, chunk_numel, ga, fc, d_state);
    else
        hipLaunchKernelGGL((adam_chunks_gated_kernel<ARITH, WD_NONE>), grid, block, kLdsBytes, s, b, chunk_numel, ga, fc, d_state);
}

void launch_gated_batch(int arith, const ChunkBatch& b, dim3 grid, size_t chunk_numel,
                        const GatedArgs& ga, const FirstCall& fc, const ps_step_state* d_state,
                        hipStream_t s)
{
    if (arith == PS_ARITH_TORCH)
        launch_gated_batch_arith<PS_ARITH_TORCH>(b, grid, chunk_numel, ga, FirstCall{-1, 0, 0}, d_state, s);
    else
        launch_gated_batch_arith<PS_ARITH_OPERATOR>(b, grid, chunk_numel, ga, fc, d_state, s);
}

template <int ARITH, int WD>
void launch_tensors_wd(const TensorBatch& b, dim3 grid, const StepConsts& c, hipStream_t s)
{
    dim3 block(kBlock);
    if (c.unscale == UNSCALE_MUL)
        hipLaunchKernelGGL((adam_tensors_kernel<ARITH, WD, UNSCALE_MUL>), grid, block, kLdsBytes, s, b, c);
    else if (ARITH == PS_ARITH_OPERATOR && c.unscale == UNSCALE_DIV)
        hipLaunchKernelGGL((adam_tensors_kernel<ARITH, WD, UNSCALE_DIV>), grid, block, kLdsBytes, s, b, c);
    else
        hipLaunchKernelGGL((adam_tensors_kernel<ARITH, WD, UNSCALE_NONE>), grid, block, kLdsBytes, s, b, c);
}

template <int ARITH>
void launch_tensors_arith(const TensorBatch& b, dim3 grid, const StepConsts& c, hipStream_t s)
{
    if (c.wd_mode == WD_DECOUPLED)
        launch_tensors_wd<ARITH, WD_DECOUPLED>(b, grid, c, s);
    else if (c.wd_mode == WD_L2)
        launch_tensors_wd<ARITH, WD_L2>(b, grid, c, s);
    else
        launch_tensors_wd<ARITH, WD_NONE>(b, grid, c, s);
}

template <int ARITH>
void launch_tensors_gated_arith(const TensorBatch& b, dim3 grid, const GatedArgs& ga,
                                const ps_step_state* d_state, hipStream_t s)
{
    dim3 block(kBlock);
    const bool decay = ARITH == PS_ARITH_OPERATOR ? (float)ga.wd > 0.0f : ga.wd != 0.0;
    if (decay && ga.adamw)
        hipLaunchKernelGGL((adam_tensors_gated_kernel<ARITH, WD_DECOUPLED>), grid, block, kLdsBytes, s, b, ga, d_state);
    else if (decay)
        hipLaunchKernelGGL((adam_tensors_gated_kernel<ARITH, WD_L2>), grid, block, kLdsBytes, s, b, ga, d_state);
    else
        hipLaunchKernelGGL((adam_tensors_gated_kernel<ARITH, WD_NONE>), grid, block, kLdsBytes, s, b, ga, d_state);
}

// The Python numbers of one step as they cross the boundary.
struct HyperParams {
    double lr, beta1, beta2, eps, wd;
    double loss_scale;  // <= 0: no loss scaler
    bool bias_correction;
    bool grad_f32 = false;  // the call's gradient tensor is binary32 (the clamp bound then narrows to float only)
};

// Host-decided step, operator arithmetic: narrow like the pybind signature of adam_update
// (float arguments, cpu_adam.cpp:700-712) and take the operator object through the n_calls
// adam_update calls of the reference's per-tensor loop, all with this step number: the first call's
// beta^t, then (from the second call on the object no longer moves) every later call's.
StepConsts operator_step_consts(HostAdam& o, size_t step, const HyperParams& hp, int64_t n_calls)
{
    o.advance(step, (float)hp.beta1, (float)hp.beta2);
    const float first_b1t = o.beta1_t, first_b2t = o.beta2_t;
    if (n_calls >= 2) o.advance(step, (float)hp.beta1, (float)hp.beta2);
    o.set((float)hp.lr, (float)hp.eps, (float)hp.wd);
    StepConsts c;
    finish_consts(c, o.alpha, o.beta1, o.beta2, o.eps, o.weight_decay, o.adamw, o.beta1_t,
                  o.beta2_t, hp.bias_correction, (float)hp.loss_scale, clamp_bound(o.grad_clamp, hp.loss_scale, hp.grad_f32));
    bias_scalars(o.alpha, first_b1t, first_b2t, hp.bias_correction, &c.first_step_size, &c.first_bc2inv);
    return c;
}

// Host-decided step, torch arithmetic (fp16_cpu_adam.py:412-413: Python's float ** int is the C
// library's pow).  The operator object is not touched: the reference does not call it here.
StepConsts torch_step_consts(const HostAdam& o, size_t step, const HyperParams& hp)
{
    double bc1 = 1.0, bc2 = 1.0;
    if (hp.bias_correction) {
        bc1 = 1.0 - std::pow(hp.beta1, (double)step);
        bc2 = 1.0 - std::pow(hp.beta2, (double)step);
    }
    StepConsts c;
    torch_consts(c, hp.lr, hp.beta1, hp.beta2, hp.eps, hp.wd, o.adamw, bc1, bc2, hp.loss_scale,
                 clamp_bound(o.grad_clamp, hp.loss_scale, hp.grad_f32));
    return c;
}

GatedArgs gated_args(const HostAdam& o, double lr, double eps, double wd, int bias_correction,
                     int64_t n_calls)
{
    GatedArgs ga;
    ga.lr = lr;
    ga.eps = eps;
    ga.wd = wd;
    ga.grad_clamp = o.grad_clamp;
    ga.n_calls = n_calls;
    ga.adamw = o.adamw ? 1 : 0;
    ga.bias_correction = bias_correction;
    return ga;
}

// ------------------------------------------- host-resident chunks: streaming
//
// Chunks that live in pinned host memory are streamed through caller-owned
// staging buffers in HBM: H2D copies on one side stream, the fused kernel on a
// compute side stream, D2H copies on another side stream, tied together with
// events, so that with two or more staging slots the copy of chunk k+1 and the
// write-back of chunk k-1 overlap the kernel on chunk k.  Nothing blocks the
// host.  The streams and events are created once per device and kept.

constexpr int kMaxSlots = 8;

struct Pipeline {
    bool ready = false;
    std::mutex in_use;  // held by a call while it queues work on the side streams: calls on one device take turns
    hipStream_t h2d = nullptr, compute = nullptr, d2h = nullptr;
    hipEvent_t entry = nullptr;
    hipEvent_t joined[3] = {};  // one per side stream: "everything queued there so far"
    hipEvent_t h2d_done[kMaxSlots] = {}, compute_done[kMaxSlots] = {}, d2h_done[kMaxSlots] = {};
    bool slot_used[kMaxSlots] = {};

    int create()
    {
        // default priority on purpose
        PS_HIP(hipStreamCreateWithFlags(&h2d, hipStreamNonBlocking));
        PS_HIP(hipStreamCreateWithFlags(&compute, hipStreamNonBlocking));
        PS_HIP(hipStreamCreateWithFlags(&d2h, hipStreamNonBlocking));
        PS_HIP(hipEventCreateWithFlags(&entry, hipEventDisableTiming));
        for (hipEvent_t& e : joined) PS_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
        for (int i = 0; i < kMaxSlots; ++i) {
            PS_HIP(hipEventCreateWithFlags(&h2d_done[i], hipEventDisableTiming));
            PS_HIP(hipEventCreateWithFlags(&compute_done[i], hipEventDisableTiming));
            PS_HIP(hipEventCreateWithFlags(&d2h_done[i], hipEventDisableTiming));
        }
        return 0;
    }

    // give back whatever a failed create() got as far as making
    void destroy()
    {
        for (hipStream_t* st : {&h2d, &compute, &d2h})
            if (*st) (void)hipStreamDestroy(*st), *st = nullptr;
        auto drop = [](hipEvent_t& e) {
            if (e) (void)hipEventDestroy(e), e = nullptr;
        };
        drop(entry);
        for (hipEvent_t& e : joined) drop(e);
        for (int i = 0; i < kMaxSlots; ++i) drop(h2d_done[i]), drop(compute_done[i]), drop(d2h_done[i]);
    }

    // A call begins: the copies and kernels it is about to queue on the side streams come after everything `caller`
    // has queued so far (gradients written, the device flag set) and after whatever an EARLIER call, possibly of
    // another host thread on another stream, left on any side stream (its staging slots may be the same memory).  For
    // one caller the second part is implied by the first (every call ends with join()).
    int begin(hipStream_t caller)
    {
        hipStream_t side[3] = {h2d, compute, d2h};
        for (int i = 0; i < 3; ++i) PS_HIP(hipEventRecord(joined[i], side[i]));
        PS_HIP(hipEventRecord(entry, caller));
        for (hipStream_t st : {h2d, compute}) {
            PS_HIP(hipStreamWaitEvent(st, entry, 0));
            for (int i = 0; i < 3; ++i)
                if (side[i] != st) PS_HIP(hipStreamWaitEvent(st, joined[i], 0));
        }
        for (int i = 0; i < kMaxSlots; ++i) slot_used[i] = false;
        return 0;
    }

    // Later work on `caller` comes after everything queued on the side streams so far.  Also used on
    // an error path, so that a half-queued step cannot race with whatever the caller does next.
    int join(hipStream_t caller)
    {
        hipStream_t side[3] = {h2d, compute, d2h};
        for (int i = 0; i < 3; ++i) {
            PS_HIP(hipEventRecord(joined[i], side[i]));
            PS_HIP(hipStreamWaitEvent(caller, joined[i], 0));
        }
        return 0;
    }
};

std::mutex g_pipeline_mutex;
std::unordered_map<int, Pipeline> g_pipelines;

int get_pipeline(Pipeline** out)
{
    int dev = 0;
    PS_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_pipeline_mutex);
    Pipeline* p = nullptr;
    try {
        p = &g_pipelines[dev];
    } catch (const std::exception&) {  // nothing may throw across the boundary
        return fail(PS_ERR_BAD_ARG, "no host memory for the streaming state of device %d", dev);
    }
    if (!p->ready) {
        if (int rc = p->create()) {
            p->destroy();
            return rc;
        }
        p->ready = true;
    }
    *out = p;
    return 0;
}

int check_slots(const ps_chunk* staging, int n_slots, bool need_state, bool need_fp16)
{
    if (n_slots < 1 || n_slots > kMaxSlots)
        return fail(PS_ERR_BAD_ARG, "n_slots = %d must be in 1..%d", n_slots, kMaxSlots);
    if (!staging) return fail(PS_ERR_BAD_ARG, "staging is NULL");
    for (int i = 0; i < n_slots; ++i) {
        if ((need_fp16 && !staging[i].param_fp16) ||
            (need_state && (!staging[i].param_fp32 || !staging[i].exp_avg || !staging[i].exp_avg_sq)))
            return fail(PS_ERR_BAD_ARG, "staging slot %d has a NULL buffer", i);
    }
    return 0;
}

// A host-resident chunk position may keep its fp16 payload in HBM (only the optimizer state lives in
// host memory): say for every position whether its fp16 address is device memory.
int fp16_payloads_in_hbm(const ps_chunk* host_chunks, int n, bool* in_hbm, bool* any_on_host)
{
    *any_on_host = false;
    for (int i = 0; i < n; ++i) {
        hipPointerAttribute_t attr;
        hipError_t e = hipPointerGetAttributes(&attr, host_chunks[i].param_fp16);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return fail(PS_ERR_BAD_ARG, "host chunk %d: the fp16 address is neither device nor pinned host memory (%s)",
                        i, hipGetErrorString(e));
        }
        in_hbm[i] = attr.type == hipMemoryTypeDevice;
        if (!in_hbm[i]) *any_on_host = true;
    }
    return 0;
}

}  // namespace

// ------------------------------------------- library-owned device scratch
//
// Partial results of ps_overflow_scan_chunks_noalloc: one word per workgroup of its first kernel.  A
// file-scope device array, so the entry point needs no allocation; every GPU the library runs on
// holds its own copy (4 MiB) at its own address until the process ends.  In host code the array's
// name is only a handle: the device address comes from hipGetSymbolAddress, once per device.
constexpr size_t kScratchWords = (size_t)1 << 20;
static __device__ __align__(256) uint32_t g_scan_scratch[kScratchWords];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
uint32_t* g_scratch_ptr[kMaxDevices] = {};

// The current device's copy of g_scan_scratch.
int scratch_address(uint32_t** out)
{
    int dev = 0;
    PS_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(PS_ERR_BAD_ARG, "device ordinal %d is beyond %d", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        PS_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(g_scan_scratch)));
        if (p == nullptr) return fail(PS_ERR_NO_DEVICE, "hipGetSymbolAddress gave no address for the scratch array");
        g_scratch_ptr[dev] = static_cast<uint32_t*>(p);
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

}  // namespace

// ====================================================================== ABI

extern "C" {

int ps_abi_version(void) { return PS_ABI_VERSION; }

const char* ps_last_error(void) { return g_err; }

int ps_adam_create(int optimizer_id, float alpha, float beta1, float beta2, float eps,
                   float weight_decay, int adamw_mode, int should_log)
{
    try {
        auto o = std::make_shared<HostAdam>();
        o->alpha = alpha;
        o->beta1 = beta1;
        o->beta2 = beta2;
        o->eps = eps;
        o->weight_decay = weight_decay;
        o->adamw = adamw_mode != 0;
        std::lock_guard<std::mutex> lock(g_registry_mutex);
        g_registry[optimizer_id] = o;
    } catch (const std::exception&) {  // nothing may throw across the boundary
        return fail(PS_ERR_BAD_ARG, "no host memory for optimizer %d", optimizer_id);
    }
    if (should_log) {
        printf("Adam Optimizer #%d is created with gfx950 HIP arithmetic capability.\n",
               optimizer_id);
        printf("Config: alpha=%f, betas=(%f, %f), weight_decay=%f, adam_w=%d\n", alpha, beta1,
               beta2, weight_decay, (int)(adamw_mode != 0));
    }
    return 0;
}

int ps_adam_set_grad_clamp(int optimizer_id, double gradient_clipping)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    o->grad_clamp = gradient_clipping;
    return 0;
}

int ps_adam_set_arithmetic(int optimizer_id, int arithmetic)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    if (arithmetic != PS_ARITH_OPERATOR && arithmetic != PS_ARITH_TORCH)
        return fail(PS_ERR_BAD_ARG, "arithmetic = %d is neither PS_ARITH_OPERATOR nor PS_ARITH_TORCH", arithmetic);
    o->arith = arithmetic;
    return 0;
}

int ps_adam_destroy(int optimizer_id)
{
    std::lock_guard<std::mutex> lock(g_registry_mutex);
    g_registry.erase(optimizer_id);
    return 0;
}

int ps_adam_update(int optimizer_id, size_t step, float lr, float beta1, float beta2, float epsilon,
                   float weight_decay, int bias_correction, float* d_params, const void* d_grads,
                   int grads_are_half, float* d_exp_avg, float* d_exp_avg_sq, size_t numel,
                   float loss_scale, uint16_t* d_param_fp16_out, ps_stream_t stream)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    if (numel > 0 && (!d_params || !d_grads || !d_exp_avg || !d_exp_avg_sq))
        return fail(PS_ERR_BAD_ARG, "ps_adam_update: NULL tensor pointer");
    o->advance(step, beta1, beta2);
    o->set(lr, epsilon, weight_decay);
    if (numel == 0) return 0;
    StepConsts c;
    // the reference clamps gradients in Python before it calls the operator: not here
    finish_consts(c, o->alpha, o->beta1, o->beta2, o->eps, o->weight_decay, o->adamw, o->beta1_t,
                  o->beta2_t, bias_correction != 0, loss_scale, 0.0f);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t gsz = grads_are_half ? 2 : 4;
    const char* gbytes = static_cast<const char*>(d_grads);

    // element-wise pass over [lo, hi)
    auto scalar_span = [&](size_t lo, size_t hi) {
        if (hi <= lo) return;
        const size_t n = hi - lo;
        dim3 grid(grid_1d((n + kAuxBlock - 1) / kAuxBlock, kAuxBlock)), block(kAuxBlock);
        uint16_t* out = d_param_fp16_out ? d_param_fp16_out + lo : nullptr;
#define PS_FLAT(WD, HALF)                                                                      \
    hipLaunchKernelGGL((adam_flat_kernel<WD, HALF>), grid, block, 0, s, c, d_params + lo,      \
                       static_cast<const void*>(gbytes + lo * gsz), d_exp_avg + lo,            \
                       d_exp_avg_sq + lo, out, n)
        if (grads_are_half) {
            if (c.wd_mode == WD_DECOUPLED) PS_FLAT(WD_DECOUPLED, true);
            else if (c.wd_mode == WD_L2) PS_FLAT(WD_L2, true);
            else PS_FLAT(WD_NONE, true);
        } else {
            if (c.wd_mode == WD_DECOUPLED) PS_FLAT(WD_DECOUPLED, false);
            else if (c.wd_mode == WD_L2) PS_FLAT(WD_L2, false);
            else PS_FLAT(WD_NONE, false);
        }
#undef PS_FLAT
    };

    // Tensors handed to the operator are views at one element offset into the four chunk payloads, so their
    // addresses normally share a phase relative to 16-byte (4-element) boundaries: whole 256-element tiles with
    // vector accesses from the fp32 parameter's first 1 KiB boundary on (every wave access then covers one aligned
    // KiB); the up to 255 elements before it and the remainder behind the last whole tile go element-wise, in the
    // same launch.
    auto elem_phase = [](const void* a, size_t elem_size) -> int {
        uintptr_t u = reinterpret_cast<uintptr_t>(a);
        if (u % elem_size) return -1;
        return (int)((u / elem_size) & 3u);
    };
    // (momentum and variance may sit at any other element phase: the reference packs them in another order than the
    // parameters; their 16-byte accesses then go to 4-byte-aligned addresses)
    const int ph = elem_phase(d_params, 4);
    const bool vec_ok = ph >= 0 && numel >= 4096 && elem_phase(d_exp_avg, 4) >= 0 && elem_phase(d_exp_avg_sq, 4) >= 0 &&
                        elem_phase(d_grads, gsz) == ph &&
                        (d_param_fp16_out == nullptr || elem_phase(d_param_fp16_out, 2) == ph);
    const bool state_aligned = elem_phase(d_exp_avg, 4) == ph && elem_phase(d_exp_avg_sq, 4) == ph;
    if (!vec_ok) {
        scalar_span(0, numel);
        PS_HIP(hipGetLastError());
        return 0;
    }
    const size_t head = (size_t)((kTile - (reinterpret_cast<uintptr_t>(d_params) / sizeof(float)) % kTile) % kTile);
    // one tile per workgroup: a tensor beyond the launch grid (2^39 elements) goes in several launches
    const size_t max_tiles = kMaxGridX - 1;
    size_t done = 0;  // elements behind the head that earlier launches of this call have covered
    const size_t body = numel - head;
    do {
        const size_t left = body - done;
        const bool last = left / kTile <= max_tiles;
        const size_t n_tiles = last ? left / kTile : max_tiles;
        const int tail = last ? (int)(left - n_tiles * kTile) : 0;
        const int this_head = done == 0 ? (int)head : 0;
        const size_t at = head + done;
        dim3 grid((unsigned)(n_tiles + 1)), block(kBlock);  // + 1: the workgroup that does head and tail
        uint16_t* out = d_param_fp16_out ? d_param_fp16_out + at : nullptr;
#define PS_FLAT_VEC_5(WD, UNS, HALF, OUT, DWORD)                                                              \
    hipLaunchKernelGGL((adam_flat_vec_kernel<WD, UNS, HALF, OUT, DWORD>), grid, block, kLdsBytes, s, c,       \
                       d_params + at, static_cast<const void*>(gbytes + at * gsz), d_exp_avg + at,            \
                       d_exp_avg_sq + at, out, n_tiles, this_head, tail)
#define PS_FLAT_VEC_4(WD, UNS, HALF, OUT)                  \
    do {                                                   \
        if (state_aligned)                                 \
            PS_FLAT_VEC_5(WD, UNS, HALF, OUT, false);      \
        else                                               \
            PS_FLAT_VEC_5(WD, UNS, HALF, OUT, true);       \
    } while (0)
#define PS_FLAT_VEC_3(WD, UNS, HALF)                       \
    do {                                                   \
        if (out != nullptr)                                \
            PS_FLAT_VEC_4(WD, UNS, HALF, true);            \
        else                                               \
            PS_FLAT_VEC_4(WD, UNS, HALF, false);           \
    } while (0)
#define PS_FLAT_VEC_2(WD, UNS)                             \
    do {                                                   \
        if (grads_are_half)                                \
            PS_FLAT_VEC_3(WD, UNS, true);                  \
        else                                               \
            PS_FLAT_VEC_3(WD, UNS, false);                 \
    } while (0)
#define PS_FLAT_VEC_1(WD)                                  \
    do {                                                   \
        if (c.unscale == UNSCALE_MUL)                      \
            PS_FLAT_VEC_2(WD, UNSCALE_MUL);                \
        else if (c.unscale == UNSCALE_DIV)                 \
            PS_FLAT_VEC_2(WD, UNSCALE_DIV);                \
        else                                               \
            PS_FLAT_VEC_2(WD, UNSCALE_NONE);               \
    } while (0)
        if (c.wd_mode == WD_DECOUPLED) PS_FLAT_VEC_1(WD_DECOUPLED);
        else if (c.wd_mode == WD_L2) PS_FLAT_VEC_1(WD_L2);
        else PS_FLAT_VEC_1(WD_NONE);
#undef PS_FLAT_VEC_1
#undef PS_FLAT_VEC_2
#undef PS_FLAT_VEC_3
#undef PS_FLAT_VEC_4
#undef PS_FLAT_VEC_5
        PS_HIP(hipGetLastError());
        done += n_tiles * kTile + tail;
    } while (done < body);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_adam_step_chunks(int optimizer_id, size_t step, double lr, double beta1, double beta2,
                        double epsilon, double weight_decay, int bias_correction,
                        const ps_chunk* chunks, int n_chunks, size_t chunk_numel,
                        const size_t* used_numel, const ps_call_pattern* calls, double loss_scale,
                        ps_stream_t stream)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    ChunkList a;
    if (int rc = make_chunk_list(a, chunks, n_chunks, chunk_numel, used_numel, kTile)) return rc;
    Calls k;
    if (int rc = make_calls(k, calls, n_chunks, chunk_numel)) return rc;
    const HyperParams hp{lr, beta1, beta2, epsilon, weight_decay, loss_scale, bias_correction != 0};
    StepConsts c;
    if (o->arith == PS_ARITH_TORCH)
        c = torch_step_consts(*o, step, hp);
    else
        c = operator_step_consts(*o, step, hp, k.n_calls);
    if (!zeros_are_a_fixed_point(c)) a.used = nullptr;  // the padding is computed like everything else
    const int arith = o->arith;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return for_each_batch(a, [&](const ChunkBatch& b, dim3 grid, int first) {
        launch_adam_batch(arith, b, grid, c, k.in_batch(first, (int)grid.y), s);
    });
}

int ps_adam_step_chunks_gated(int optimizer_id, double lr, double epsilon, double weight_decay,
                              int bias_correction, const ps_chunk* chunks, int n_chunks,
                              size_t chunk_numel, const size_t* used_numel,
                              const ps_call_pattern* calls, const ps_step_state* d_state,
                              ps_stream_t stream)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    ChunkList a;
    if (int rc = make_chunk_list(a, chunks, n_chunks, chunk_numel, used_numel, kTile)) return rc;
    Calls k;
    if (int rc = make_calls(k, calls, n_chunks, chunk_numel)) return rc;
    const GatedArgs ga = gated_args(*o, lr, epsilon, weight_decay, bias_correction, k.n_calls);
    const int arith = o->arith;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // (whether the padding may be left alone depends on the device-resident scalars: the kernel decides)
    return for_each_batch(a, [&](const ChunkBatch& b, dim3 grid, int first) {
        launch_gated_batch(arith, b, grid, chunk_numel, ga, k.in_batch(first, (int)grid.y), d_state, s);
    });
}

}  // extern "C"

namespace {

// ---------------------------------------------------------- tensor lists
//
// Where a tensor's tile grid starts (the fp32 parameter's first 1 KiB boundary; what lies in front of it is a tile of
// its own) and how many tiles it has.  Addresses that are not even element-aligned keep the plain numbering.
struct TensorItem {
    int index;  // in the caller's list
    uint32_t head;
    size_t body, tiles;
    int cls;  // the class of calls it belongs to (steps whose tensors carry their own numbers; 0 otherwise)
};
static_assert(kTile <= 256, "TensorBatch::numel_head keeps the head length (up to kTile - 1 elements) in 8 bits");

int check_tensor_list(const ps_chunk* tensors, const size_t* numels, int n_tensors)
{
    if (n_tensors < 0) return fail(PS_ERR_BAD_ARG, "n_tensors = %d is negative", n_tensors);
    if (n_tensors > 0 && (!tensors || !numels)) return fail(PS_ERR_BAD_ARG, "tensors or numels is NULL");
    for (int i = 0; i < n_tensors; ++i) {
        const ps_chunk& t = tensors[i];
        if (numels[i] > 0 && (!t.param_fp32 || !t.exp_avg || !t.exp_avg_sq || !t.param_fp16))
            return fail(PS_ERR_BAD_ARG, "tensor %d has a NULL address", i);
        if ((numels[i] + kTile - 1) / kTile >= kMaxGridX || numels[i] > kNumelMask)
            return fail(PS_ERR_BAD_ARG, "tensor %d: numel = %zu is beyond the launch grid", i, numels[i]);
    }
    return 0;
}

TensorItem tensor_item(const ps_chunk* tensors, const size_t* numels, int i, bool from_first_element = false)
{
    const uintptr_t p_addr = reinterpret_cast<uintptr_t>(tensors[i].param_fp32);
    size_t head = p_addr % sizeof(float) || from_first_element ? 0 : (kTile - (p_addr / sizeof(float)) % kTile) % kTile;
    if (head > numels[i]) head = numels[i];
    const size_t body = numels[i] - head;
    return TensorItem{i, (uint32_t)head, body, (head ? 1 : 0) + (body + kTile - 1) / kTile, 0};
}

// Calls launch(batch, grid, classes) for groups of the given tensors (all of them non-empty): longest first; one launch
// takes tensors of nearly the same length (its grid is as wide as the longest of them: at most a tenth of a
// launch's workgroups find nothing to do), short tensors all together.  `first_tensor`: the index (in the caller's
// list) of the tensor that is the step's first operator call, marked in its batch; -1: none.
//
// `classes`: which class each tensor of the batch belongs to.  max_classes == 0: the items' own class numbers.
// max_classes > 0: a launch takes at most that many distinct classes; classes.k[] then numbers them 0, 1, ... in the
// order of their first tensor in the batch and classes.of[] says which of the items' classes each one is.
struct BatchClasses {
    ClassIndex k;
    int of[kTensorBatch];
    int n;
};

template <typename F>
int for_each_tensor_batch(std::vector<TensorItem>& items, const ps_chunk* tensors, int first_tensor, int max_classes,
                          F launch)
{
    std::stable_sort(items.begin(), items.end(), [](const TensorItem& a, const TensorItem& b) { return a.tiles > b.tiles; });
    constexpr size_t kShortTensorTiles = 256;
    TensorBatch b;
    BatchClasses bc;
    size_t next = 0;
    while (next < items.size()) {
        memset(&b, 0, sizeof(b));
        memset(&bc, 0, sizeof(bc));
        b.first_call = -1;
        const size_t widest = items[next].tiles;
        int in_batch = 0;
        while (next < items.size() && in_batch < kTensorBatch &&
               (items[next].tiles * 10 >= widest * 9 || widest <= kShortTensorTiles)) {
            const TensorItem& it = items[next];
            if (max_classes > 0) {
                int j = 0;
                while (j < bc.n && bc.of[j] != it.cls) ++j;
                if (j == bc.n) {
                    if (bc.n == max_classes) break;  // the next launch starts with this tensor
                    bc.of[bc.n++] = it.cls;
                }
                bc.k.k[in_batch] = (uint16_t)j;
            } else {
                bc.k.k[in_batch] = (uint16_t)it.cls;
            }
            ps_chunk t = tensors[it.index];
            t.param_fp32 += it.head;
            t.exp_avg += it.head;
            t.exp_avg_sq += it.head;
            t.param_fp16 += it.head;
            b.t[in_batch] = t;
            b.numel_head[in_batch] = (uint64_t)it.body | ((uint64_t)it.head << 56);
            if (it.index == first_tensor) b.first_call = in_batch;
            in_batch += 1;
            next += 1;
        }
        launch(b, dim3((unsigned)widest, (unsigned)in_batch), bc);
        PS_HIP(hipGetLastError());
    }
    return 0;
}

// Weight-decay form of a call, as the two arithmetics decide it: the operator tests its float weight decay "> 0"
// (cpu_adam.cpp:42), the torch formula the Python number "!= 0".
int wd_mode_of(int arith, double wd, bool adamw)
{
    const bool decay = arith == PS_ARITH_OPERATOR ? (float)wd > 0.0f : wd != 0.0;
    return decay ? (adamw ? WD_DECOUPLED : WD_L2) : WD_NONE;
}

template <int ARITH, int WD>
void launch_tensors_planned_wd(const TensorBatch& b, dim3 grid, const ClassIndex& ci, bool grad_f32,
                               const PlannedConsts* d_consts, const ps_step_state* d_state, hipStream_t s)
{
    dim3 block(kBlock);
    if (grad_f32)
        hipLaunchKernelGGL((adam_tensors_planned_f32grad_kernel<ARITH, WD>), grid, block, kLdsBytes, s, b, ci, d_consts, d_state);
    else
        hipLaunchKernelGGL((adam_tensors_planned_kernel<ARITH, WD>), grid, block, kLdsBytes, s, b, ci, d_consts, d_state);
}

template <int ARITH>
void launch_tensors_planned_arith(const TensorBatch& b, dim3 grid, const ClassIndex& ci, int wd_mode, bool grad_f32,
                                  const PlannedConsts* d_consts, const ps_step_state* d_state, hipStream_t s)
{
    if (wd_mode == WD_DECOUPLED)
        launch_tensors_planned_wd<ARITH, WD_DECOUPLED>(b, grid, ci, grad_f32, d_consts, d_state, s);
    else if (wd_mode == WD_L2)
        launch_tensors_planned_wd<ARITH, WD_L2>(b, grid, ci, grad_f32, d_consts, d_state, s);
    else
        launch_tensors_planned_wd<ARITH, WD_NONE>(b, grid, ci, grad_f32, d_consts, d_state, s);
}

// Numbers the distinct records (classes of calls) of a step by their bytes; records are zero-filled before they are
// set, so equal records have equal bytes.  Consecutive tensors mostly repeat the previous record.
template <typename T>
struct ClassTable {
    std::vector<T> records;
    std::vector<int> arith;
    std::unordered_map<std::string, int> by_bytes;
    int last = -1;

    int intern(const T& r, int a)
    {
        if (last >= 0 && arith[last] == a && memcmp(&records[last], &r, sizeof(T)) == 0) return last;
        std::string key(reinterpret_cast<const char*>(&r), sizeof(T));
        key.push_back((char)a);
        auto found = by_bytes.find(key);
        if (found == by_bytes.end()) {
            found = by_bytes.emplace(std::move(key), (int)records.size()).first;
            records.push_back(r);
            arith.push_back(a);
        }
        return last = found->second;
    }
    int size() const { return (int)records.size(); }
};

// What a launch of the per-tensor-numbers step is compiled for; classes that agree in it share launches.
struct Flavour {
    int arith, wd_mode, unscale;
    bool grad_f32;  // PS_TENSOR_GRAD_F32 tensors: binary32 gradients, no fp16 copy
    bool operator==(const Flavour& o) const
    {
        return arith == o.arith && wd_mode == o.wd_mode && unscale == o.unscale && grad_f32 == o.grad_f32;
    }
};

// What ClassTable keeps beside a record: the arithmetic, and whether the tensors' gradients are binary32.
int class_key(int arith, bool grad_f32) { return arith | (grad_f32 ? 2 : 0); }
int key_arith(int key) { return key & 1; }
bool key_grad_f32(int key) { return (key & 2) != 0; }
static_assert(PS_ARITH_OPERATOR == 0 && PS_ARITH_TORCH == 1, "class_key keeps the arithmetic in one bit");

template <int ARITH, int WD, int UNS>
void launch_tensors_each_uns(const TensorBatch& b, dim3 grid, const ClassIndex& ci, const ConstsBatch& cb, bool grad_f32,
                             hipStream_t s)
{
    dim3 block(kBlock);
    if (grad_f32)
        hipLaunchKernelGGL((adam_tensors_each_f32grad_kernel<ARITH, WD, UNS>), grid, block, kLdsBytes, s, b, ci, cb);
    else
        hipLaunchKernelGGL((adam_tensors_each_kernel<ARITH, WD, UNS>), grid, block, kLdsBytes, s, b, ci, cb);
}

template <int ARITH, int WD>
void launch_tensors_each_wd(const TensorBatch& b, dim3 grid, const ClassIndex& ci, const ConstsBatch& cb,
                            const Flavour& f, hipStream_t s)
{
    if (f.unscale == UNSCALE_MUL)
        launch_tensors_each_uns<ARITH, WD, UNSCALE_MUL>(b, grid, ci, cb, f.grad_f32, s);
    else if (ARITH == PS_ARITH_OPERATOR && f.unscale == UNSCALE_DIV)  // the torch formula never divides
        launch_tensors_each_uns<ARITH, WD, UNSCALE_DIV>(b, grid, ci, cb, f.grad_f32, s);
    else
        launch_tensors_each_uns<ARITH, WD, UNSCALE_NONE>(b, grid, ci, cb, f.grad_f32, s);
}

template <int ARITH>
void launch_tensors_each_arith(const TensorBatch& b, dim3 grid, const ClassIndex& ci, const ConstsBatch& cb,
                               const Flavour& f, hipStream_t s)
{
    if (f.wd_mode == WD_DECOUPLED)
        launch_tensors_each_wd<ARITH, WD_DECOUPLED>(b, grid, ci, cb, f, s);
    else if (f.wd_mode == WD_L2)
        launch_tensors_each_wd<ARITH, WD_L2>(b, grid, ci, cb, f, s);
    else
        launch_tensors_each_wd<ARITH, WD_NONE>(b, grid, ci, cb, f, s);
}

}  // namespace

extern "C" {

int ps_adam_step_tensors(int optimizer_id, size_t step, double lr, double beta1, double beta2,
                         double epsilon, double weight_decay, int bias_correction,
                         const ps_chunk* tensors, const size_t* numels, int n_tensors,
                         const ps_call_pattern* calls, double loss_scale, const ps_step_state* d_state,
                         ps_stream_t stream)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    if (int rc = check_tensor_list(tensors, numels, n_tensors)) return rc;
    const int arith = o->arith;
    // One operator call per tensor.  Without a pattern the list is the whole step and tensors[0] its first call;
    // a pattern says how many calls the step has in all and which tensor of THIS list, if any, is the first.
    int64_t n_calls = n_tensors;
    int first_tensor = 0;
    if (calls != nullptr) {
        if (calls->n_calls < 1)
            return fail(PS_ERR_BAD_ARG, "calls->n_calls = %lld must be at least 1", (long long)calls->n_calls);
        n_calls = calls->n_calls;
        first_tensor = -1;
        if (calls->first_numel != 0) {
            if (calls->first_chunk < 0 || calls->first_chunk >= n_tensors)
                return fail(PS_ERR_BAD_ARG, "calls->first_chunk = %lld is outside the list of %d tensors",
                            (long long)calls->first_chunk, n_tensors);
            if (calls->first_offset != 0 || calls->first_numel != numels[calls->first_chunk])
                return fail(PS_ERR_BAD_ARG, "the first call is a whole tensor: calls->first_offset must be 0 and "
                            "calls->first_numel the length of tensor %lld", (long long)calls->first_chunk);
            first_tensor = (int)calls->first_chunk;
        }
    }
    if (arith != PS_ARITH_OPERATOR) first_tensor = -1;  // the torch formula has no first call
    StepConsts c;
    GatedArgs ga = gated_args(*o, lr, epsilon, weight_decay, bias_correction, n_calls);
    if (d_state == nullptr && n_tensors > 0) {
        const HyperParams hp{lr, beta1, beta2, epsilon, weight_decay, loss_scale, bias_correction != 0};
        c = arith == PS_ARITH_TORCH ? torch_step_consts(*o, step, hp) : operator_step_consts(*o, step, hp, n_calls);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::vector<TensorItem> items;
    try {
        items.reserve((size_t)n_tensors);
    } catch (const std::exception&) {  // nothing may throw across the boundary
        return fail(PS_ERR_BAD_ARG, "no host memory for a list of %d tensors", n_tensors);
    }
    for (int i = 0; i < n_tensors; ++i)
        if (numels[i] != 0) items.push_back(tensor_item(tensors, numels, i));
    return for_each_tensor_batch(items, tensors, first_tensor, 0, [&](const TensorBatch& b, dim3 grid, const BatchClasses&) {
        if (d_state == nullptr) {
            if (arith == PS_ARITH_TORCH)
                launch_tensors_arith<PS_ARITH_TORCH>(b, grid, c, s);
            else
                launch_tensors_arith<PS_ARITH_OPERATOR>(b, grid, c, s);
        } else {
            if (arith == PS_ARITH_TORCH)
                launch_tensors_gated_arith<PS_ARITH_TORCH>(b, grid, ga, d_state, s);
            else
                launch_tensors_gated_arith<PS_ARITH_OPERATOR>(b, grid, ga, d_state, s);
        }
    });
}

size_t ps_tensors_each_workspace_bytes(int n_tensors)
{
    return n_tensors > 0 ? (size_t)n_tensors * sizeof(PlannedConsts) : 0;
}

int ps_adam_step_tensors_each(int optimizer_id, int bias_correction, const ps_chunk* tensors,
                              const size_t* numels, const ps_tensor_call* each, int n_tensors,
                              double loss_scale, ps_step_state* d_state, void* d_workspace,
                              size_t workspace_bytes, ps_stream_t stream)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    if (int rc = check_tensor_list(tensors, numels, n_tensors)) return rc;
    if (n_tensors > 0 && !each) return fail(PS_ERR_BAD_ARG, "each is NULL");
    for (int i = 0; i < n_tensors; ++i) {
        const int a = each[i].arithmetic;
        if (a != -1 && a != PS_ARITH_OPERATOR && a != PS_ARITH_TORCH)
            return fail(PS_ERR_BAD_ARG, "each[%d].arithmetic = %d", i, a);
        if (d_state == nullptr && each[i].step < 1)
            return fail(PS_ERR_BAD_ARG, "each[%d].step = %lld: a host-decided step number is at least 1", i,
                        (long long)each[i].step);
        if (each[i].flags & ~PS_TENSOR_GRAD_F32) return fail(PS_ERR_BAD_ARG, "each[%d].flags = %d", i, each[i].flags);
    }
    if (d_state != nullptr && n_tensors > 0) {
        if (!d_workspace || workspace_bytes < ps_tensors_each_workspace_bytes(n_tensors))
            return fail(PS_ERR_BAD_ARG, "d_workspace holds %zu bytes; a device-decided step over %d tensors needs %zu",
                        d_workspace ? workspace_bytes : (size_t)0, n_tensors, ps_tensors_each_workspace_bytes(n_tensors));
        if (reinterpret_cast<uintptr_t>(d_workspace) % 16)
            return fail(PS_ERR_BAD_ARG, "d_workspace must be 16-byte aligned");
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool bias = bias_correction != 0;
    auto arith_of = [&](int i) { return each[i].arithmetic < 0 ? o->arith : each[i].arithmetic; };
    auto grad_f32_of = [&](int i) { return (each[i].flags & PS_TENSOR_GRAD_F32) != 0; };
    try {
        // Calls that come out with the same constants form a class; class_of[i] says which one tensor i belongs to.
        std::vector<int> class_of((size_t)n_tensors, -1);
        if (d_state == nullptr) {
            // ---- host-decided: the operator object goes through the calls, in order
            ClassTable<StepConsts> classes;
            for (int i = 0; i < n_tensors; ++i) {
                const ps_tensor_call& e = each[i];
                const int arith = arith_of(i);
                const HyperParams hp{e.lr, e.beta1, e.beta2, e.eps, e.weight_decay, loss_scale, bias, grad_f32_of(i)};
                StepConsts c;
                memset(&c, 0, sizeof(c));
                if (arith == PS_ARITH_TORCH)
                    c = torch_step_consts(*o, (size_t)e.step, hp);
                else
                    c = operator_step_consts(*o, (size_t)e.step, hp, 1);
                class_of[i] = classes.intern(c, class_key(arith, grad_f32_of(i)));
            }
            const std::vector<StepConsts>& consts = classes.records;
            // one pass of launches per flavour (what the kernels are compiled for); inside it, tensors of any class
            std::vector<Flavour> flavours;
            std::vector<int> flavour_of(consts.size());
            for (size_t k = 0; k < consts.size(); ++k) {
                const Flavour f{key_arith(classes.arith[k]), consts[k].wd_mode, consts[k].unscale, key_grad_f32(classes.arith[k])};
                size_t j = 0;
                while (j < flavours.size() && !(flavours[j] == f)) ++j;
                if (j == flavours.size()) flavours.push_back(f);
                flavour_of[k] = (int)j;
            }
            std::vector<TensorItem> items;
            for (size_t j = 0; j < flavours.size(); ++j) {
                items.clear();
                for (int i = 0; i < n_tensors; ++i)
                    if (numels[i] != 0 && flavour_of[class_of[i]] == (int)j) {
                        items.push_back(tensor_item(tensors, numels, i, flavours[j].grad_f32));
                        items.back().cls = class_of[i];
                    }
                const Flavour& f = flavours[j];
                int rc = for_each_tensor_batch(items, tensors, -1, kLaunchClasses,
                                               [&](const TensorBatch& b, dim3 grid, const BatchClasses& bc) {
                    ConstsBatch cb;
                    memset(&cb, 0, sizeof(cb));
                    for (int q = 0; q < bc.n; ++q) cb.c[q] = consts[bc.of[q]];
                    if (f.arith == PS_ARITH_TORCH)
                        launch_tensors_each_arith<PS_ARITH_TORCH>(b, grid, bc.k, cb, f, s);
                    else
                        launch_tensors_each_arith<PS_ARITH_OPERATOR>(b, grid, bc.k, cb, f, s);
                });
                if (rc) return rc;
            }
            return 0;
        }

        // ---- device-decided: the step numbers (adam_step + 1 + d), the loss scale and the operator object live on
        // the device.  The host knows how the calls relate to one another (IncrementStep, cpu_adam.h:143-162, looks
        // only at differences between consecutive calls), which leaves three kinds of operator call and one
        // torch call; the device turns each distinct one into constants.
        ClassTable<PlanClass> table_of_classes;
        const std::vector<PlanClass>& classes = table_of_classes.records;
        const std::vector<int>& class_keys = table_of_classes.arith;  // class_key(arithmetic, binary32 gradients)
        std::vector<int> class_wd;
        int prev_class = -1;  // of the previous operator call
        int last_operator = -1;
        for (int i = 0; i < n_tensors; ++i) {
            const ps_tensor_call& e = each[i];
            const int arith = arith_of(i);
            PlanClass k;
            memset(&k, 0, sizeof(k));
            k.lr = e.lr, k.beta1 = e.beta1, k.beta2 = e.beta2, k.eps = e.eps, k.wd = e.weight_decay;
            k.d = e.step;
            k.prev = -1;
            if (arith == PS_ARITH_TORCH) {
                k.mode = PLAN_TORCH;
            } else if (prev_class < 0) {
                k.mode = PLAN_FIRST;  // continues the product only if the object, as the last clean step left it, allows
            } else {
                const PlanClass& q = classes[prev_class];
                const bool same_betas = (float)q.beta1 == (float)e.beta1 && (float)q.beta2 == (float)e.beta2;
                if (same_betas && e.step == q.d + 1) {
                    k.mode = PLAN_MUL;
                    k.prev = prev_class;
                } else {
                    k.mode = PLAN_POW;
                }
            }
            if (grad_f32_of(i)) k.mode |= PLAN_GRAD_F32;
            const int c = table_of_classes.intern(k, class_key(arith, grad_f32_of(i)));
            if (c == (int)class_wd.size()) class_wd.push_back(wd_mode_of(arith, e.weight_decay, o->adamw));
            class_of[i] = c;
            if (arith != PS_ARITH_TORCH) prev_class = last_operator = c;
        }
        PlannedConsts* table = static_cast<PlannedConsts*>(d_workspace);
        const int n_classes = (int)classes.size();
        for (int first = 0; first < n_classes || first == 0; first += kPlanBatch) {
            PlanBatch pb;
            memset(&pb, 0, sizeof(pb));
            PlanArgs pa;
            memset(&pa, 0, sizeof(pa));
            pa.n = std::min(kPlanBatch, n_classes - first);
            for (int j = 0; j < pa.n; ++j) pb.k[j] = classes[first + j];
            pa.grad_clamp = o->grad_clamp;
            pa.adamw = o->adamw ? 1 : 0;
            pa.bias_correction = bias ? 1 : 0;
            pa.first_class = first;
            pa.is_last_launch = first + kPlanBatch >= n_classes;
            pa.last_operator_class = last_operator;
            if (last_operator >= 0) {
                pa.last_d = classes[last_operator].d;
                pa.last_beta1 = (float)classes[last_operator].beta1;
                pa.last_beta2 = (float)classes[last_operator].beta2;
            }
            hipLaunchKernelGGL(plan_consts_kernel, dim3(1), dim3(64), 0, s, pb, pa, d_state, table);
            PS_HIP(hipGetLastError());
            if (n_classes == 0) break;
        }
        // One pass of launches per (arithmetic, weight-decay form); inside it, tensors of any class.  A launch names
        // its tensors' classes in 16 bits, relative to the window of 65536 records it is handed.
        constexpr int kWindow = 1 << 16;
        std::vector<TensorItem> items;
        for (int window = 0; window < n_classes; window += kWindow) {
            for (int key : {class_key(PS_ARITH_OPERATOR, false), class_key(PS_ARITH_TORCH, false),
                            class_key(PS_ARITH_OPERATOR, true), class_key(PS_ARITH_TORCH, true)}) {
                const bool grad_f32 = key_grad_f32(key);
                for (int wd_mode : {WD_NONE, WD_L2, WD_DECOUPLED}) {
                    items.clear();
                    for (int i = 0; i < n_tensors; ++i) {
                        const int k = class_of[i];
                        if (numels[i] == 0 || k < window || k >= window + kWindow) continue;
                        if (class_keys[k] != key || class_wd[k] != wd_mode) continue;
                        items.push_back(tensor_item(tensors, numels, i, grad_f32));
                        items.back().cls = k - window;
                    }
                    if (items.empty()) continue;
                    int rc = for_each_tensor_batch(items, tensors, -1, 0,
                                                   [&](const TensorBatch& b, dim3 grid, const BatchClasses& bc) {
                        if (key_arith(key) == PS_ARITH_TORCH)
                            launch_tensors_planned_arith<PS_ARITH_TORCH>(b, grid, bc.k, wd_mode, grad_f32, table + window, d_state, s);
                        else
                            launch_tensors_planned_arith<PS_ARITH_OPERATOR>(b, grid, bc.k, wd_mode, grad_f32, table + window, d_state, s);
                    });
                    if (rc) return rc;
                }
            }
        }
        return 0;
    } catch (const std::exception&) {  // nothing may throw across the boundary
        return fail(PS_ERR_BAD_ARG, "no host memory for a list of %d tensors", n_tensors);
    }
}

int ps_restore_fp16_chunks(const ps_chunk* chunks, int n_chunks, size_t chunk_numel,
                           const ps_step_state* d_state, ps_stream_t stream)
{
    ChunkList a;
    if (int rc = make_chunk_list(a, chunks, n_chunks, chunk_numel, nullptr, kTile)) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return for_each_batch(a, [&](const ChunkBatch& b, dim3 grid, int) {
        hipLaunchKernelGGL(restore_chunks_kernel, grid, dim3(kBlock), 0, s, b, d_state);
    });
}

int ps_cast_fp32_to_fp16(const float* d_src, uint16_t* d_dst, size_t numel, ps_stream_t stream)
{
    if (numel == 0) return 0;
    if (!d_src || !d_dst) return fail(PS_ERR_BAD_ARG, "ps_cast_fp32_to_fp16: NULL pointer");
    size_t n_tiles = (numel + kTile - 1) / kTile;
    hipLaunchKernelGGL(cast_kernel, dim3(grid_1d(n_tiles, kBlock)), dim3(kBlock), 0,
                       static_cast<hipStream_t>(stream), d_src, d_dst, numel, n_tiles);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_adam_step_hybrid(int optimizer_id, size_t step, double lr, double beta1, double beta2,
                        double epsilon, double weight_decay, int bias_correction,
                        const ps_chunk* chunks, int n_chunks, const ps_chunk* host_chunks,
                        int n_host_chunks, size_t chunk_numel, const size_t* used_numel,
                        const ps_chunk* staging, int n_slots, const ps_call_pattern* calls,
                        double loss_scale, const ps_step_state* d_state, ps_stream_t stream)
{
    auto o = find_opt(optimizer_id);
    if (!o) return fail(PS_ERR_UNKNOWN_ID, "optimizer id %d was never created", optimizer_id);
    if (n_chunks < 0) return fail(PS_ERR_BAD_ARG, "n_chunks = %d is negative", n_chunks);
    ChunkList resident, host;
    if (int rc = make_chunk_list(resident, chunks, n_chunks, chunk_numel, used_numel, kTile)) return rc;
    if (int rc = make_chunk_list(host, host_chunks, n_host_chunks, chunk_numel, used_numel ? used_numel + n_chunks : nullptr,
                                 kTile, false, "host chunk"))
        return rc;
    std::unique_ptr<bool[]> fp16_in_hbm(new (std::nothrow) bool[n_host_chunks > 0 ? n_host_chunks : 1]);
    if (!fp16_in_hbm) return fail(PS_ERR_BAD_ARG, "no host memory for a list of %d host chunks", n_host_chunks);
    if (n_host_chunks > 0) {
        if (int rc = check_slots(staging, n_slots, true, false)) return rc;
        bool any_on_host = false;
        if (int rc = fp16_payloads_in_hbm(host_chunks, n_host_chunks, fp16_in_hbm.get(), &any_on_host)) return rc;
        if (any_on_host)
            if (int rc = check_slots(staging, n_slots, true, true)) return rc;
    }
    // Resident chunks take the optimizer's arithmetic, streamed host chunks the operator's (the
    // reference updates those with the operator).  The operator object goes through the calls of
    // the pattern (over both lists), and only if the operator's arithmetic is used at all.
    const int arith = o->arith;
    Calls k;
    if (int rc = make_calls(k, calls, (int64_t)n_chunks + n_host_chunks, chunk_numel)) return rc;
    if (arith == PS_ARITH_TORCH && k.first_chunk >= 0 && k.first_chunk < n_chunks)
        return fail(PS_ERR_BAD_ARG, "calls->first_chunk = %lld names a resident chunk, which the torch arithmetic "
                    "never hands to the operator", (long long)k.first_chunk);
    StepConsts c_resident, c_host;
    const GatedArgs ga = gated_args(*o, lr, epsilon, weight_decay, bias_correction, k.n_calls);
    if (d_state == nullptr) {
        const HyperParams hp{lr, beta1, beta2, epsilon, weight_decay, loss_scale, bias_correction != 0};
        if (arith == PS_ARITH_OPERATOR || n_host_chunks > 0) c_host = operator_step_consts(*o, step, hp, k.n_calls);
        c_resident = arith == PS_ARITH_TORCH ? torch_step_consts(*o, step, hp) : c_host;
        if (!zeros_are_a_fixed_point(c_resident)) resident.used = nullptr;
        if (n_host_chunks > 0 && !zeros_are_a_fixed_point(c_host)) host.used = nullptr;
    } else {
        // Streamed chunks move only their used part over the link, so whether their padding may be left alone has
        // to be known here, from the host's numbers (the kernel's own check, on the device-resident scalars, stays
        // in force for the resident chunks): a positive eps and finite scalars, betas below one as floats.
        const bool plain = (float)epsilon > 0.0f && std::isfinite((float)lr) && std::isfinite((float)weight_decay) &&
                           std::isfinite((float)epsilon) && (float)beta1 < 1.0f && (float)beta2 < 1.0f;
        if (!plain) host.used = nullptr;
    }
    hipStream_t caller = static_cast<hipStream_t>(stream);
    bool stream_host = false;
    for (int i = 0; i < n_host_chunks; ++i) stream_host = stream_host || host.numel_of(i) > 0;
    Pipeline* p = nullptr;
    std::unique_lock<std::mutex> turn;
    if (stream_host) {
        if (int rc = get_pipeline(&p)) return rc;
        turn = std::unique_lock<std::mutex>(p->in_use);
        // the resident chunks' kernels, queued next on the caller's stream, do NOT hold the copies back
        if (int rc = p->begin(caller)) return rc;
    }
    int rc = for_each_batch(resident, [&](const ChunkBatch& b, dim3 grid, int first) {
        const FirstCall fc = k.in_batch(first, (int)grid.y);
        if (d_state == nullptr)
            launch_adam_batch(arith, b, grid, c_resident, fc, caller);
        else
            launch_gated_batch(arith, b, grid, chunk_numel, ga, fc, d_state, caller);
    });
    if (!stream_host) return rc;

    auto stream_chunk = [&](int k_host) -> int {
        const size_t numel = host.numel_of(k_host);
        if (numel == 0) return 0;
        const size_t b32 = numel * sizeof(float), b16 = numel * sizeof(uint16_t);
        const int s = k_host % n_slots;
        const ps_chunk& h = host_chunks[k_host];
        ps_chunk d = staging[s];
        // a fp16 payload that already lives in HBM is read and written in place: 12 instead of
        // 14 bytes per element cross the link in each direction
        const bool stage_fp16 = !fp16_in_hbm[k_host];
        if (!stage_fp16) d.param_fp16 = h.param_fp16;
        // the slot is free once its previous occupant has been written back
        if (p->slot_used[s]) PS_HIP(hipStreamWaitEvent(p->h2d, p->d2h_done[s], 0));
        if (stage_fp16)
            PS_HIP(hipMemcpyAsync(d.param_fp16, h.param_fp16, b16, hipMemcpyHostToDevice, p->h2d));
        PS_HIP(hipMemcpyAsync(d.param_fp32, h.param_fp32, b32, hipMemcpyHostToDevice, p->h2d));
        PS_HIP(hipMemcpyAsync(d.exp_avg, h.exp_avg, b32, hipMemcpyHostToDevice, p->h2d));
        PS_HIP(hipMemcpyAsync(d.exp_avg_sq, h.exp_avg_sq, b32, hipMemcpyHostToDevice, p->h2d));
        PS_HIP(hipEventRecord(p->h2d_done[s], p->h2d));

        PS_HIP(hipStreamWaitEvent(p->compute, p->h2d_done[s], 0));
        ChunkBatch b;
        memset(&b, 0, sizeof(b));
        b.c[0] = d;
        b.n[0] = numel;
        dim3 grid((unsigned)((numel + kTile - 1) / kTile), 1);
        const FirstCall fc = k.in_batch((int64_t)n_chunks + k_host, 1);
        if (d_state == nullptr)
            launch_adam_batch(PS_ARITH_OPERATOR, b, grid, c_host, fc, p->compute);
        else  // the staged copy ends at `numel`: nothing behind it for the kernel to decide about
            launch_gated_batch(PS_ARITH_OPERATOR, b, grid, numel, ga, fc, d_state, p->compute);
        PS_HIP(hipGetLastError());
        PS_HIP(hipEventRecord(p->compute_done[s], p->compute));

        PS_HIP(hipStreamWaitEvent(p->d2h, p->compute_done[s], 0));
        // (on a device-skipped step fp32 param / m / v come back unchanged; copying them anyway
        // keeps the host free of any knowledge of the flag)
        if (stage_fp16)
            PS_HIP(hipMemcpyAsync(h.param_fp16, d.param_fp16, b16, hipMemcpyDeviceToHost, p->d2h));
        PS_HIP(hipMemcpyAsync(h.param_fp32, d.param_fp32, b32, hipMemcpyDeviceToHost, p->d2h));
        PS_HIP(hipMemcpyAsync(h.exp_avg, d.exp_avg, b32, hipMemcpyDeviceToHost, p->d2h));
        PS_HIP(hipMemcpyAsync(h.exp_avg_sq, d.exp_avg_sq, b32, hipMemcpyDeviceToHost, p->d2h));
        PS_HIP(hipEventRecord(p->d2h_done[s], p->d2h));
        p->slot_used[s] = true;
        return 0;
    };
    for (int i = 0; i < n_host_chunks && rc == 0; ++i) rc = stream_chunk(i);
    // later work on the caller's stream sees every chunk written back (also if queuing stopped half way, or never
    // started because a resident launch failed: the side streams already wait on the caller, the caller must wait
    // on them)
    const int joined = p->join(caller);
    return rc ? rc : joined;
}

int ps_overflow_scan_host_chunks(const ps_chunk* host_chunks, int n_chunks, size_t chunk_numel,
                                 const size_t* used_numel, const ps_chunk* staging, int n_slots,
                                 ps_step_state* d_state, ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    ChunkList a;
    if (int rc = make_chunk_list(a, host_chunks, n_chunks, chunk_numel, used_numel, kScanTile, true, "host chunk")) return rc;
    if (n_chunks == 0 || chunk_numel == 0) return 0;
    std::unique_ptr<bool[]> fp16_in_hbm(new (std::nothrow) bool[n_chunks]);
    if (!fp16_in_hbm) return fail(PS_ERR_BAD_ARG, "no host memory for a list of %d host chunks", n_chunks);
    bool any_on_host = false;
    if (int rc = fp16_payloads_in_hbm(host_chunks, n_chunks, fp16_in_hbm.get(), &any_on_host)) return rc;
    hipStream_t caller = static_cast<hipStream_t>(stream);
    auto tiles_of = [&](int k) { return (a.numel_of(k) + kScanTile - 1) / kScanTile; };
    // fp16 payloads that live in HBM are probed in place on the caller's stream
    for (int k = 0; k < n_chunks; ++k) {
        if (!fp16_in_hbm[k] || a.numel_of(k) == 0) continue;
        hipLaunchKernelGGL(scan_f16_kernel, dim3(grid_1d(tiles_of(k), kScanBlock)), dim3(kScanBlock), kScanLdsBytes, caller,
                           host_chunks[k].param_fp16, a.numel_of(k), tiles_of(k), d_state);
        PS_HIP(hipGetLastError());
    }
    any_on_host = false;
    for (int k = 0; k < n_chunks; ++k) any_on_host = any_on_host || (!fp16_in_hbm[k] && a.numel_of(k) > 0);
    if (!any_on_host) return 0;
    if (int rc = check_slots(staging, n_slots, false, true)) return rc;
    Pipeline* p = nullptr;
    if (int rc = get_pipeline(&p)) return rc;
    std::lock_guard<std::mutex> turn(p->in_use);
    if (int rc = p->begin(caller)) return rc;
    int streamed = 0;
    auto stream_chunk = [&](int k) -> int {
        const int s = streamed++ % n_slots;
        if (p->slot_used[s]) PS_HIP(hipStreamWaitEvent(p->h2d, p->compute_done[s], 0));
        PS_HIP(hipMemcpyAsync(staging[s].param_fp16, host_chunks[k].param_fp16, a.numel_of(k) * sizeof(uint16_t),
                              hipMemcpyHostToDevice, p->h2d));
        PS_HIP(hipEventRecord(p->h2d_done[s], p->h2d));
        PS_HIP(hipStreamWaitEvent(p->compute, p->h2d_done[s], 0));
        hipLaunchKernelGGL(scan_f16_kernel, dim3(grid_1d(tiles_of(k), kScanBlock)), dim3(kScanBlock), kScanLdsBytes, p->compute,
                           staging[s].param_fp16, a.numel_of(k), tiles_of(k), d_state);
        PS_HIP(hipGetLastError());
        PS_HIP(hipEventRecord(p->compute_done[s], p->compute));
        p->slot_used[s] = true;
        return 0;
    };
    int rc = 0;
    for (int k = 0; k < n_chunks && rc == 0; ++k)
        if (!fp16_in_hbm[k] && a.numel_of(k) > 0) rc = stream_chunk(k);
    const int joined = p->join(caller);
    return rc ? rc : joined;
}

int ps_state_init(ps_step_state* d_state, double init_scale, int init_is_int, double scale_factor,
                  int factor_is_int, int64_t scale_window, double min_scale, int min_is_int,
                  int delayed_shift, int consecutive_hysteresis, double beta1, double beta2,
                  ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    if (scale_window <= 0)
        return fail(PS_ERR_BAD_ARG, "scale_window = %lld must be positive", (long long)scale_window);
    ps_step_state s;
    memset(&s, 0, sizeof(s));
    s.cur_scale = init_scale;
    s.scale_is_int = init_is_int != 0;
    s.scale_factor = scale_factor;
    s.factor_is_int = factor_is_int != 0;
    s.min_scale = min_scale;
    s.min_is_int = min_is_int != 0;
    s.cur_iter = 0;
    s.last_overflow_iter = -1;
    s.scale_window = scale_window;
    s.delayed_shift = delayed_shift;
    s.cur_hysteresis = delayed_shift;
    s.consecutive_hysteresis = consecutive_hysteresis != 0;
    s.beta1 = (float)beta1;
    s.beta2 = (float)beta2;
    // Adam_Optimizer starts with beta^t = 1 and step 0; the first update multiplies once.
    s.operator_step = 0;
    s.operator_beta1 = s.beta1;
    s.operator_beta2 = s.beta2;
    s.beta1_t_cur = 1.0f;
    s.beta2_t_cur = 1.0f;
    s.beta1_t_next = 1.0f * s.beta1;
    s.beta2_t_next = 1.0f * s.beta2;
    // a second call of step 1 finds _step + 1 = 2 != 1 and evaluates pow(beta, 1)
    s.beta1_t_rest = (float)std::pow((double)s.beta1, 1.0);
    s.beta2_t_rest = (float)std::pow((double)s.beta2, 1.0);
    s.beta1_f64 = beta1;
    s.beta2_f64 = beta2;
    s.bias_correction1_next = 1.0 - std::pow(beta1, 1.0);
    s.bias_correction2_next = 1.0 - std::pow(beta2, 1.0);
    hipLaunchKernelGGL(state_init_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                       d_state, s);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_state_seed_step(ps_step_state* d_state, int64_t adam_step, double beta1, double beta2,
                       int fresh_operator, ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    if (adam_step < 0) return fail(PS_ERR_BAD_ARG, "adam_step is negative");
    SeedArgs a;
    a.adam_step = adam_step;
    a.beta1 = (float)beta1;
    a.beta2 = (float)beta2;
    // what a call for step adam_step + 1 gets when it cannot continue a running product; whether the
    // first call of that step can is decided on the device, where the operator object's state lives
    a.b1t_rest = (float)std::pow((double)a.beta1, (double)(adam_step + 1));
    a.b2t_rest = (float)std::pow((double)a.beta2, (double)(adam_step + 1));
    a.fresh_operator = fresh_operator != 0;
    a.beta1_f64 = beta1;
    a.beta2_f64 = beta2;
    a.bc1_next = 1.0 - std::pow(beta1, (double)(adam_step + 1));
    a.bc2_next = 1.0 - std::pow(beta2, (double)(adam_step + 1));
    hipLaunchKernelGGL(state_seed_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                       d_state, a);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_state_set_scaler(ps_step_state* d_state, double cur_scale, int scale_is_int,
                        int64_t cur_iter, int64_t last_overflow_iter, int cur_hysteresis,
                        ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    hipLaunchKernelGGL(state_set_scaler_kernel, dim3(1), dim3(64), 0,
                       static_cast<hipStream_t>(stream), d_state, cur_scale, scale_is_int, cur_iter,
                       last_overflow_iter, cur_hysteresis);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_overflow_scan(const uint16_t* d_grads_fp16, size_t numel, ps_step_state* d_state,
                     ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    if (numel == 0) return 0;
    if (!d_grads_fp16) return fail(PS_ERR_BAD_ARG, "d_grads_fp16 is NULL");
    size_t n_tiles = (numel + kScanTile - 1) / kScanTile;
    hipLaunchKernelGGL(scan_f16_kernel, dim3(grid_1d(n_tiles, kScanBlock)), dim3(kScanBlock), kScanLdsBytes,
                       static_cast<hipStream_t>(stream), d_grads_fp16, numel, n_tiles, d_state);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_overflow_scan_f32(const float* d_grads_fp32, size_t numel, ps_step_state* d_state,
                         ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    if (numel == 0) return 0;
    if (!d_grads_fp32) return fail(PS_ERR_BAD_ARG, "d_grads_fp32 is NULL");
    size_t n_tiles = (numel + kScanTileF32 - 1) / kScanTileF32;
    hipLaunchKernelGGL(scan_f32_kernel, dim3(grid_1d(n_tiles, kScanBlock)), dim3(kScanBlock), kScanLdsBytes,
                       static_cast<hipStream_t>(stream), d_grads_fp32, numel, n_tiles, d_state);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_overflow_scan_chunks(const ps_chunk* chunks, int n_chunks, size_t chunk_numel,
                            const size_t* used_numel, ps_step_state* d_state, ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    ChunkList a;
    if (int rc = make_chunk_list(a, chunks, n_chunks, chunk_numel, used_numel, kScanTile, true)) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return for_each_batch(a, [&](const ChunkBatch& b, dim3 grid, int) {
        hipLaunchKernelGGL(scan_chunks_kernel, grid, dim3(kScanBlock), kScanLdsBytes, s, b, d_state);
    });
}

int ps_overflow_scan_chunks_noalloc(const ps_chunk* chunks, int n_chunks, size_t chunk_numel,
                                    uint32_t* d_flag, ps_stream_t stream)
{
    if (!d_flag) return fail(PS_ERR_BAD_ARG, "d_flag is NULL");
    ChunkList a;
    if (int rc = make_chunk_list(a, chunks, n_chunks, chunk_numel, nullptr, kPartialTile)) return rc;
    const size_t tiles_per_chunk = (chunk_numel + kPartialTile - 1) / kPartialTile;
    if (n_chunks == 0 || tiles_per_chunk == 0) return 0;
    // one scratch word per workgroup of the first kernel
    const size_t max_chunks = kScratchWords / tiles_per_chunk;  // 0 when one chunk alone is too long
    if ((size_t)n_chunks > max_chunks)
        return fail(PS_ERR_BAD_ARG,
                    "%d chunks of %zu elements need %zu scratch words; this entry point holds %zu (at most %zu "
                    "elements per call): split the list or use ps_overflow_scan_chunks",
                    n_chunks, chunk_numel, (size_t)n_chunks * tiles_per_chunk, kScratchWords,
                    kScratchWords * (size_t)kPartialTile);
    uint32_t* scratch = nullptr;
    if (int rc = scratch_address(&scratch)) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    int rc = for_each_batch(a, [&](const ChunkBatch& b, dim3 grid, int first) {
        hipLaunchKernelGGL(scan_chunks_partial_kernel, grid, dim3(kPartialBlock), kScanLdsBytes, s, b,
                           scratch + (size_t)first * tiles_per_chunk);
    });
    if (rc) return rc;
    // a workgroup per 8192 words (a single one took 33 us over the 196,608 words of 24 x 64 Mi elements)
    const size_t n_words = (size_t)n_chunks * tiles_per_chunk;
    const unsigned reducers = (unsigned)std::min<size_t>((n_words + 8191) / 8192, 128);
    hipLaunchKernelGGL(scan_reduce_kernel, dim3(reducers), dim3(kReduceBlock), 0, s, scratch, n_words, d_flag);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_grad_to_chunk(const void* d_grad, int grad_is_half, uint16_t* d_slot_fp16, size_t numel,
                     ps_step_state* d_state, ps_stream_t stream)
{
    if (numel == 0) return 0;
    if (!d_grad || !d_slot_fp16) return fail(PS_ERR_BAD_ARG, "ps_grad_to_chunk: NULL pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t esz = grad_is_half ? 2 : 4;
    const char* gbytes = static_cast<const char*>(d_grad);

    auto scalar_span = [&](size_t lo, size_t hi) {
        if (hi <= lo) return;
        const size_t n = hi - lo;
        size_t blocks = (n + (size_t)kAuxBlock * 4 - 1) / ((size_t)kAuxBlock * 4);
        dim3 grid(grid_1d(blocks, kAuxBlock)), block(kAuxBlock);
        const void* src = gbytes + lo * esz;
        if (grad_is_half)
            hipLaunchKernelGGL(grad_to_chunk_kernel<true>, grid, block, 0, s, src, d_slot_fp16 + lo, n, d_state);
        else
            hipLaunchKernelGGL(grad_to_chunk_kernel<false>, grid, block, 0, s, src, d_slot_fp16 + lo, n, d_state);
    };

    const uintptr_t dst = reinterpret_cast<uintptr_t>(d_slot_fp16);
    const uintptr_t src = reinterpret_cast<uintptr_t>(d_grad);
    const bool addressable = (dst % 2 == 0) && (src % esz == 0);
    if (!addressable || numel < 4096) {
        scalar_span(0, numel);
    } else {
        // elements before the slot's first 16-byte boundary, whole 8-element vectors, remainder: one launch, whose
        // last workgroup does the at most 14 elements in front of and behind the vectors
        const size_t head = (size_t)(((16 - dst % 16) % 16) / 2);
        const size_t n_vec = (numel - head) / 8;
        const size_t body_end = head + n_vec * 8;
        const CopyEdges edges{d_grad, d_slot_fp16, head, body_end, numel};
        size_t blocks = (n_vec + kCopyBlock - 1) / kCopyBlock;
        unsigned body_blocks = grid_1d(blocks, kCopyBlock);
        if (((size_t)body_blocks + 1) * kCopyBlock > 0xFFFFFFFFull) body_blocks -= 1;  // room for the edge workgroup
        dim3 grid(body_blocks + 1), block(kCopyBlock);
        uint16_t* dst_al = d_slot_fp16 + head;
        if (grad_is_half) {
            const uintptr_t first = src + head * 2;
            const int shift = (int)((first % 16) / 2);
            const uint16_t* src_al = reinterpret_cast<const uint16_t*>(first - (uintptr_t)shift * 2);
            hipLaunchKernelGGL(grad_to_chunk_f16_vec_kernel, grid, block, kCopyLdsBytes, s, src_al, shift, dst_al, n_vec, edges, d_state);
        } else {
            hipLaunchKernelGGL(grad_to_chunk_f32_vec_kernel, grid, block, kCopyLdsBytes, s,
                               static_cast<const float*>(d_grad) + head, dst_al, n_vec, edges, d_state);
        }
    }
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_scaler_update(ps_step_state* d_state, int flag_mode, ps_scale_record* d_log,
                     int64_t log_capacity, int64_t operator_calls, ps_stream_t stream)
{
    if (!d_state) return fail(PS_ERR_BAD_ARG, "d_state is NULL");
    if (flag_mode < 0 || flag_mode > 2) return fail(PS_ERR_BAD_ARG, "flag_mode = %d", flag_mode);
    if (d_log != nullptr && log_capacity <= 0)
        return fail(PS_ERR_BAD_ARG, "log_capacity must be positive when d_log is given");
    if (operator_calls < 0) return fail(PS_ERR_BAD_ARG, "operator_calls = %lld is negative", (long long)operator_calls);
    hipLaunchKernelGGL(scaler_update_kernel, dim3(1), dim3(64), 0,
                       static_cast<hipStream_t>(stream), d_state, flag_mode, d_log, log_capacity,
                       operator_calls);
    PS_HIP(hipGetLastError());
    return 0;
}

int ps_state_read(const ps_step_state* d_state, ps_step_state* host_out, ps_stream_t stream)
{
    if (!d_state || !host_out) return fail(PS_ERR_BAD_ARG, "ps_state_read: NULL pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    PS_HIP(hipMemcpyAsync(host_out, d_state, sizeof(ps_step_state), hipMemcpyDeviceToHost, s));
    PS_HIP(hipStreamSynchronize(s));
    return 0;
}

}  // extern "C"

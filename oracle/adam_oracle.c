/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * CPU restatement of the reference's native Adam operator, used only as the
 * parity checker in tests/, by __graft_entry__.smoke() and as the timed CPU
 * baseline leg of bench.py.  Nothing under patrickstar_amd/ may call it.
 *
 * What it follows (paths relative to the reference tree):
 *   patrickstar/ops/csrc/includes/cpu_adam.h:143-162   host step / beta^t state
 *   patrickstar/ops/csrc/includes/cpu_adam.h:163-175   bias-correction scalars
 *   patrickstar/ops/csrc/adam/cpu_adam.cpp:42-46       step_size / w_decay scalars
 *   patrickstar/ops/csrc/adam/cpu_adam.cpp:91-141      per-element op order (SIMD body)
 *   patrickstar/ops/chunk_io_buff.py:116-126,143-146   fp32 -> fp16 write-back (RNE cast)
 *   patrickstar/ops/fp16_cpu_adam.py:245-277,430       the torch-formula (GPU) branch
 *
 * The per-element order is that of the reference's explicit-intrinsic body:
 * every product-sum the reference writes as SIMD_FMA is ONE fused rounding,
 * everything else (mul, div, sqrt) is a separately rounded IEEE-754 binary32
 * operation.  The reference's scalar remainder loop (cpu_adam.cpp:146-184,
 * the last n mod SIMD_WIDTH elements of a call) is compiler-contracted code
 * whose rounding depends on the compiler; it is deliberately NOT restated:
 * this oracle applies the SIMD-body order to every element.
 *
 * Pinning status (see tests/test_oracle_adam.py):
 *   oracle_adam_span        pinned: torch.optim.Adam/AdamW library step, fp64
 *                           textbook Adam, step-1 closed forms, zero-padding and
 *                           power-of-two-scale invariants, three code paths
 *                           (scalar / AVX2 / AVX-512) bit-identical.
 *   oracle_adam_advance/set pinned: float32 running-product and pow() closed forms.
 *   oracle_f32_to_f16       pinned: numpy RNE cast over every binade incl. all
 *                           65536 fp16 values and their fp32 neighbours.
 *   oracle_torch_adam_span  the reference's GPU branch delegates its arithmetic to PyTorch's
 *                           element-wise kernels (third-party; torch is unpinned in the
 *                           reference's requirements.txt:1); this restates each kernel of the call
 *                           sequence at fp16_cpu_adam.py:259-277 as one rounding step.  Pinned:
 *                           against that literal call sequence executed by torch itself, on CPU
 *                           tensors in tests/test_oracle_torch_formula.py and bit for bit against
 *                           torch's GPU kernels in tests/test_gpu_torch_arithmetic.py and, on the CPU,
 *                           against vectors those kernels wrote (tests/golden/torch_branch_vectors.npz); against
 *                           torch.optim.Adam/AdamW; against the textbook recurrences in float64.
 *   The reference ships no golden vectors for this path, and its C++ cannot be
 *   compiled in this image without CUDA headers, so no oracle/_ref build exists.
 *
 * Build: see oracle/Makefile (needs -ffp-contract=off; fused ops are explicit).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#include <immintrin.h>

typedef struct oracle_adam {
    float lr, beta1, beta2, eps, weight_decay;
    float beta1_t, beta2_t;
    uint64_t step;
    float bc1, bc2inv;
    int adamw;
} oracle_adam;

/* ---- host scalar state ------------------------------------------------- */

/* cpu_adam.h:68-86 constructor defaults: beta^t = 1, step = 0. */
void oracle_adam_init(oracle_adam* o, float lr, float beta1, float beta2, float eps,
                      float weight_decay, int adamw)
{
    o->lr = lr;
    o->beta1 = beta1;
    o->beta2 = beta2;
    o->eps = eps;
    o->weight_decay = weight_decay;
    o->beta1_t = 1.0f;
    o->beta2_t = 1.0f;
    o->step = 0;
    o->bc1 = 1.0f;
    o->bc2inv = 1.0f;
    o->adamw = adamw;
}

/* cpu_adam.h:143-162.  beta^t is a float: either the running float product
 * (step follows the previous one, betas unchanged) or pow() evaluated in
 * double (the float and size_t arguments promote) and narrowed to float. */
void oracle_adam_advance(oracle_adam* o, uint64_t step, float beta1, float beta2)
{
    if (beta1 != o->beta1 || beta2 != o->beta2) {
        o->step = step;
        o->beta1 = beta1;
        o->beta2 = beta2;
        o->beta1_t = (float)pow((double)beta1, (double)step);
        o->beta2_t = (float)pow((double)beta2, (double)step);
        return;
    }
    o->step += 1;
    if (o->step != step) {
        o->beta1_t = (float)pow((double)o->beta1, (double)step);
        o->beta2_t = (float)pow((double)o->beta2, (double)step);
        o->step = step;
    } else {
        o->beta1_t = o->beta1_t * o->beta1;
        o->beta2_t = o->beta2_t * o->beta2;
    }
}

/* cpu_adam.h:163-175. */
void oracle_adam_set(oracle_adam* o, float lr, float eps, float weight_decay, int bias_correction)
{
    o->lr = lr;
    o->eps = eps;
    o->weight_decay = weight_decay;
    o->bc1 = 1.0f;
    o->bc2inv = 1.0f;
    if (bias_correction) {
        o->bc1 = 1.0f - o->beta1_t;
        o->bc2inv = 1.0f / sqrtf(1.0f - o->beta2_t);
    }
}

/* The per-call constants of cpu_adam.cpp:39-46. */
typedef struct span_consts {
    float beta1, beta2, b1m, b2m, bc2inv, eps, step_size, wd_term, loss_scale;
    int l2, decoupled, unscale;
} span_consts;

static span_consts make_consts(const oracle_adam* o, float loss_scale)
{
    span_consts c;
    c.beta1 = o->beta1;
    c.beta2 = o->beta2;
    c.b1m = 1.0f - o->beta1;
    c.b2m = 1.0f - o->beta2;
    c.bc2inv = o->bc2inv;
    c.eps = o->eps;
    c.step_size = (-1.0f * o->lr) / o->bc1;
    c.l2 = (o->weight_decay > 0.0f) && !o->adamw;
    c.decoupled = (o->weight_decay > 0.0f) && o->adamw;
    c.wd_term = o->adamw ? (-1.0f * o->lr) * o->weight_decay : o->weight_decay;
    c.loss_scale = loss_scale;
    c.unscale = loss_scale > 0.0f;
    return c;
}

void oracle_adam_consts(const oracle_adam* o, float loss_scale, float out[6])
{
    span_consts c = make_consts(o, loss_scale);
    out[0] = c.b1m;
    out[1] = c.b2m;
    out[2] = c.bc2inv;
    out[3] = c.step_size;
    out[4] = c.wd_term;
    out[5] = o->bc1;
}

/* ---- fp16 <-> fp32, bit-level (no hardware dependence) ------------------- */

float oracle_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t expo = (h >> 10) & 0x1Fu;
    uint32_t mant = h & 0x3FFu;
    uint32_t bits;
    if (expo == 0) {
        if (mant == 0) {
            bits = sign;
        } else {
            /* subnormal half: renormalise */
            int shift = 0;
            while (!(mant & 0x400u)) {
                mant <<= 1;
                ++shift;
            }
            mant &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (mant << 13);
        }
    } else if (expo == 31) {
        bits = sign | 0x7F800000u | (mant << 13);
    } else {
        bits = sign | ((expo + (127 - 15)) << 23) | (mant << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* Round-to-nearest-even binary32 -> binary16; overflow goes to +-inf, NaN stays
 * NaN (quiet).  This is what Tensor.copy_ from fp32 to fp16 does in the
 * reference's whole-chunk write-back. */
uint16_t oracle_f32_to_f16(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) { /* inf / nan */
        if (ax == 0x7F800000u) return sign | 0x7C00u;
        return sign | 0x7E00u | (uint16_t)((ax >> 13) & 0x3FFu);
    }
    if (ax >= 0x477FF000u) return sign | 0x7C00u; /* >= 65520 rounds to inf */
    if (ax < 0x33000001u) return sign;            /* <= 2^-25 rounds to zero */
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t m = (ax & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
    int shift;                                  /* bits to drop */
    uint32_t base;
    if (e < -14) { /* result subnormal: value = m * 2^(e-23), ulp = 2^-24 */
        shift = -e - 1;                         /* e=-15 -> 14, e=-25 -> 24 */
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        m &= 0x7FFFFFu;
    }
    uint32_t kept = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    uint32_t r = base + kept;
    if (rem > half || (rem == half && (r & 1u))) r += 1; /* carries propagate into the exponent */
    return sign | (uint16_t)r;
}

void oracle_cast_f32_to_f16(const float* src, uint16_t* dst, size_t n)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) dst[i] = oracle_f32_to_f16(src[i]);
}

/* loss_scaler.py:133-155 reduces to "some element is not finite". */
int oracle_any_nonfinite_f16(const uint16_t* g, size_t n)
{
    int hit = 0;
#pragma omp parallel for schedule(static) reduction(| : hit)
    for (size_t i = 0; i < n; ++i) hit |= ((g[i] & 0x7C00u) == 0x7C00u);
    return hit;
}

/* ---- per-element update: three code paths, one arithmetic --------------- */

static inline void update_one(const span_consts* c, float* p, float g, float* m, float* v)
{
    float pp = *p, mm = *m, vv = *v;
    if (c->unscale) g = g / c->loss_scale;
    if (c->l2) g = fmaf(pp, c->wd_term, g);
    mm = mm * c->beta1;
    mm = fmaf(g, c->b1m, mm);
    vv = vv * c->beta2;
    float gg = g * g;
    vv = fmaf(gg, c->b2m, vv);
    float d = sqrtf(vv);
    d = fmaf(d, c->bc2inv, c->eps);
    float u = mm / d;
    if (c->decoupled) pp = fmaf(pp, c->wd_term, pp);
    pp = fmaf(u, c->step_size, pp);
    *p = pp;
    *m = mm;
    *v = vv;
}

static void span_scalar(const span_consts* c, float* p, const void* g, int g_half, float* m,
                        float* v, size_t lo, size_t hi)
{
    const uint16_t* gh = (const uint16_t*)g;
    const float* gf = (const float*)g;
    for (size_t i = lo; i < hi; ++i) {
        float gi = g_half ? oracle_f16_to_f32(gh[i]) : gf[i];
        update_one(c, p + i, gi, m + i, v + i);
    }
}

__attribute__((target("avx2,fma,f16c"))) static void span_avx2(const span_consts* c, float* p,
                                                               const void* g, int g_half, float* m,
                                                               float* v, size_t lo, size_t hi)
{
    const __m256 k_b1 = _mm256_set1_ps(c->beta1), k_b2 = _mm256_set1_ps(c->beta2);
    const __m256 k_b1m = _mm256_set1_ps(c->b1m), k_b2m = _mm256_set1_ps(c->b2m);
    const __m256 k_bc2 = _mm256_set1_ps(c->bc2inv), k_eps = _mm256_set1_ps(c->eps);
    const __m256 k_ss = _mm256_set1_ps(c->step_size), k_wd = _mm256_set1_ps(c->wd_term);
    const __m256 k_ls = _mm256_set1_ps(c->loss_scale);
    const uint16_t* gh = (const uint16_t*)g;
    const float* gf = (const float*)g;
    size_t i = lo;
    for (; i + 8 <= hi; i += 8) {
        __m256 gr = g_half ? _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(gh + i)))
                           : _mm256_loadu_ps(gf + i);
        __m256 pp = _mm256_loadu_ps(p + i);
        __m256 mm = _mm256_loadu_ps(m + i);
        __m256 vv = _mm256_loadu_ps(v + i);
        if (c->unscale) gr = _mm256_div_ps(gr, k_ls);
        if (c->l2) gr = _mm256_fmadd_ps(pp, k_wd, gr);
        mm = _mm256_fmadd_ps(gr, k_b1m, _mm256_mul_ps(mm, k_b1));
        vv = _mm256_fmadd_ps(_mm256_mul_ps(gr, gr), k_b2m, _mm256_mul_ps(vv, k_b2));
        __m256 d = _mm256_fmadd_ps(_mm256_sqrt_ps(vv), k_bc2, k_eps);
        __m256 u = _mm256_div_ps(mm, d);
        if (c->decoupled) pp = _mm256_fmadd_ps(pp, k_wd, pp);
        pp = _mm256_fmadd_ps(u, k_ss, pp);
        _mm256_storeu_ps(p + i, pp);
        _mm256_storeu_ps(m + i, mm);
        _mm256_storeu_ps(v + i, vv);
    }
    if (i < hi) span_scalar(c, p, g, g_half, m, v, i, hi);
}

__attribute__((target("avx512f,fma,f16c"))) static void span_avx512(const span_consts* c, float* p,
                                                                    const void* g, int g_half,
                                                                    float* m, float* v, size_t lo,
                                                                    size_t hi)
{
    const __m512 k_b1 = _mm512_set1_ps(c->beta1), k_b2 = _mm512_set1_ps(c->beta2);
    const __m512 k_b1m = _mm512_set1_ps(c->b1m), k_b2m = _mm512_set1_ps(c->b2m);
    const __m512 k_bc2 = _mm512_set1_ps(c->bc2inv), k_eps = _mm512_set1_ps(c->eps);
    const __m512 k_ss = _mm512_set1_ps(c->step_size), k_wd = _mm512_set1_ps(c->wd_term);
    const __m512 k_ls = _mm512_set1_ps(c->loss_scale);
    const uint16_t* gh = (const uint16_t*)g;
    const float* gf = (const float*)g;
    size_t i = lo;
    for (; i + 16 <= hi; i += 16) {
        __m512 gr = g_half ? _mm512_cvtph_ps(_mm256_loadu_si256((const __m256i*)(gh + i)))
                           : _mm512_loadu_ps(gf + i);
        __m512 pp = _mm512_loadu_ps(p + i);
        __m512 mm = _mm512_loadu_ps(m + i);
        __m512 vv = _mm512_loadu_ps(v + i);
        if (c->unscale) gr = _mm512_div_ps(gr, k_ls);
        if (c->l2) gr = _mm512_fmadd_ps(pp, k_wd, gr);
        mm = _mm512_fmadd_ps(gr, k_b1m, _mm512_mul_ps(mm, k_b1));
        vv = _mm512_fmadd_ps(_mm512_mul_ps(gr, gr), k_b2m, _mm512_mul_ps(vv, k_b2));
        __m512 d = _mm512_fmadd_ps(_mm512_sqrt_ps(vv), k_bc2, k_eps);
        __m512 u = _mm512_div_ps(mm, d);
        if (c->decoupled) pp = _mm512_fmadd_ps(pp, k_wd, pp);
        pp = _mm512_fmadd_ps(u, k_ss, pp);
        _mm512_storeu_ps(p + i, pp);
        _mm512_storeu_ps(m + i, mm);
        _mm512_storeu_ps(v + i, vv);
    }
    if (i < hi) span_scalar(c, p, g, g_half, m, v, i, hi);
}

/* isa: 0 = best the CPU offers, 1 = scalar, 2 = AVX2, 3 = AVX-512.
 * Returns the path actually taken (1/2/3), or -1 if the requested one is
 * not supported by this CPU. */
int oracle_adam_span(const oracle_adam* o, float* p, const void* g, int g_half, float* m, float* v,
                     size_t n, float loss_scale, int isa)
{
    __builtin_cpu_init();
    int have512 = __builtin_cpu_supports("avx512f");
    int have2 = __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma") &&
                __builtin_cpu_supports("f16c");
    if (isa == 0) isa = have512 ? 3 : (have2 ? 2 : 1);
    if ((isa == 3 && !have512) || (isa == 2 && !have2) || isa < 1 || isa > 3) return -1;
    span_consts c = make_consts(o, loss_scale);
    const size_t block = 1u << 14; /* elements per work item; a multiple of every vector width */
    size_t n_blocks = (n + block - 1) / block;
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < n_blocks; ++b) {
        size_t lo = b * block;
        size_t hi = lo + block < n ? lo + block : n;
        if (isa == 3)
            span_avx512(&c, p, g, g_half, m, v, lo, hi);
        else if (isa == 2)
            span_avx2(&c, p, g, g_half, m, v, lo, hi);
        else
            span_scalar(&c, p, g, g_half, m, v, lo, hi);
    }
    return isa;
}

/* One call of the reference operator's adam_update on a flat tensor
 * (cpu_adam.cpp:700-742): advance, set, update every element. */
int oracle_adam_update(oracle_adam* o, uint64_t step, float lr, float beta1, float beta2, float eps,
                       float weight_decay, int bias_correction, float* p, const void* g, int g_half,
                       float* m, float* v, size_t n, float loss_scale, int isa)
{
    oracle_adam_advance(o, step, beta1, beta2);
    oracle_adam_set(o, lr, eps, weight_decay, bias_correction);
    return oracle_adam_span(o, p, g, g_half, m, v, n, loss_scale, isa);
}

int oracle_sizeof_state(void) { return (int)sizeof(oracle_adam); }

/* ---- the torch-formula branch (FP16Adam.torch_adam_update) ------------------
 *
 * fp16_cpu_adam.py:430 and :259-277, one statement per torch kernel, each kernel one rounding
 * step per element the way torch's GPU kernels compute it:
 *   x.mul_(s), x.add_(s)                 separately rounded, the Python scalar narrowed to float
 *   x.div_(s), x / s   (Python scalar)   x * (float)(1.0 / s): the reciprocal is formed in double
 *   a.add_(b, alpha=s), a.add(b, alpha)  fmaf(b, s, a)
 *   a.addcmul_(b, c, value=s)            fmaf(s, b * c, a)
 *   a.addcdiv_(b, c, value=s)            fmaf(s, b / c, a)
 *   sqrt                                 correctly rounded
 * The caller (oracle/__init__.py: TorchFormulaOracle) forms the scalars in Python arithmetic
 * exactly as the reference's Python does and narrows them:
 *   k[0] (float)(1.0 / loss_scale)       grad.div_(loss_scale)             (if has_scale)
 *   k[1] (float)(1 - lr * wd) | (float)wd  data.mul_(..) | grad.add(data, alpha=wd)
 *   k[2] (float)beta1   k[3] (float)(1 - beta1)   k[4] (float)beta2   k[5] (float)(1 - beta2)
 *   k[6] (float)(1.0 / math.sqrt(bias_correction2))   k[7] (float)eps
 *   k[8] (float)(-(lr / bias_correction1))
 *   k[9] clamp bound of the fp16 gradients (fp16_cpu_adam.py:375-379), 0 = off
 * wd_mode: 0 none, 1 L2 (grad.add), 2 decoupled (data.mul_). */
void oracle_torch_adam_span(const float k[10], int wd_mode, int has_scale, float* p,
                            const uint16_t* g16, float* m, float* v, size_t n)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        float g = oracle_f16_to_f32(g16[i]); /* fp16_grad_tensor.float() */
        if (k[9] > 0.0f) g = g < -k[9] ? -k[9] : (g > k[9] ? k[9] : g); /* clamp_ on the fp16 tensor */
        float pp = p[i], mm = m[i], vv = v[i];
        if (has_scale) g = g * k[0];
        if (wd_mode == 2) pp = pp * k[1];
        if (wd_mode == 1) g = fmaf(pp, k[1], g);
        mm = mm * k[2];
        mm = fmaf(g, k[3], mm);
        vv = vv * k[4];
        float gg = g * g;
        vv = fmaf(k[5], gg, vv);
        float d = sqrtf(vv);
        d = d * k[6];
        d = d + k[7];
        float q = mm / d;
        pp = fmaf(k[8], q, pp);
        p[i] = pp;
        m[i] = mm;
        v[i] = vv;
    }
}

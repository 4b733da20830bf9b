/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the fused multi-tensor Adam step.
 *
 * A plain-C, one-element-at-a-time restatement of the reference update
 * equations in IEEE float32 (no FMA contraction, correctly rounded / and
 * sqrt, round-to-nearest-even float->half at every fp16 store).  It exists so
 * that tests, the smoke check and the benchmark's CPU-baseline leg have
 * something to compare the HIP kernels with; the product never links, loads
 * or calls it.
 *
 * Reference lines followed (paths relative to the fairscale checkout):
 *   fairscale/clib/fused_adam_cuda/fused_adam_cuda_kernel.cu:94-114   scaled (fp16 state) branch
 *   fairscale/clib/fused_adam_cuda/fused_adam_cuda_kernel.cu:115-130  unscaled (fp32 state) branch
 *   fairscale/clib/fused_adam_cuda/fused_adam_cuda_kernel.cu:153-162  step_size
 *   fairscale/clib/fused_adam_cuda/fused_adam_cuda_kernel.cu:169      use_optim_scaling = (state dtype is half)
 *   fairscale/clib/fused_adam_cuda/fused_adam_cuda_kernel.cu:172-256  the four dtype combinations
 *
 * What pins each function (the checks live in tests/test_oracle.py):
 *   oracle_half_to_float / oracle_float_to_half : exhaustive (all 65536 halves) and 2^24 sampled
 *       floats incl. every rounding boundary, against numpy's float16 conversions.
 *   fsadam_oracle_step_size : closed form in float64, bias_correction=0 => lr, rounding order
 *       against an independent numpy float32/float64 evaluation.
 *   fsadam_oracle_step, unscaled branch : torch.optim.Adam (float64, CPU) with eps re-expressed per
 *       step (eps outside sqrt), torch.optim.AdamW with weight decay re-expressed per step, closed
 *       forms for eps inside sqrt / constant gradient / zero gradient, power-of-two grad_scale
 *       equivariance, p_copy == half(p) bitwise.
 *   fsadam_oracle_step, scaled branch : torch.optim.Adam (float64) with the state rounded through
 *       fp16 between steps, power-of-two optim_scale invariance, flag <=> stored state non-finite.
 *
 * The reference itself is CUDA built with nvcc --use_fast_math (setup.py:50: approximate division
 * and square root, flush-to-zero, FMA contraction).  Those last-ulp choices cannot be pinned from
 * source; the stated tolerances (1e-6 relative on fp32 state, 1 fp16 ulp on fp16 outputs) absorb them.
 *
 * Build: see oracle/Makefile  (gcc -O2 -ffp-contract=off, no -ffast-math, no -march).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* Precision-mode codes shared with include/fsadam.h (kept numerically equal by a test). */
enum {
    ORACLE_FULL_PRECISION = 0,                   /* p f32, g f32, m/v f32            kernel.cu:197-216 */
    ORACLE_MIXED_PRECISION = 1,                  /* p f32, g f16, m/v f32, p_copy f16 kernel.cu:172-193 */
    ORACLE_MEMORY_EFFICIENT_MIXED_PRECISION = 2, /* p f16, g f16, m/v f32            kernel.cu:217-237 */
    ORACLE_PURE_FP16 = 3,                        /* p f16, g f16, m/v f16            kernel.cu:238-256 */
    /* extension, no dispatch case in the reference: the fp32 step with the DEPTH==5 copy-out of
     * kernel.cu:114,129 (p_copy = half(stored p)) applied to fp32 gradients */
    ORACLE_FULL_PRECISION_FP16_COPY = 4
};

/* ---- IEEE binary16 <-> binary32, software, independent of the host's F16C support ---- */

float oracle_half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal half: value = man * 2^-24, normalise */
            int shift = 0;
            while (!(man & 0x400u)) {
                man <<= 1;
                ++shift;
            }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + (127 - 15)) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t oracle_float_to_half(float f) { /* round to nearest, ties to even */
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        if (ax == 0x7f800000u) return (uint16_t)(sign | 0x7c00u);
        /* quiet NaN, keep the top mantissa bits so that the payload is not silently lost */
        return (uint16_t)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu));
    }
    if (ax >= 0x477ff000u) { /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax < 0x33000001u) { /* <= 2^-25 rounds to zero (tie goes to even = 0) */
        return sign;
    }
    int32_t e = (int32_t)(ax >> 23) - 127; /* unbiased exponent */
    uint32_t man = (ax & 0x7fffffu) | 0x800000u; /* 24-bit significand with the hidden one */
    int shift; /* how many low bits of the 24-bit significand are dropped */
    uint32_t base;
    if (e < -14) { /* result is a subnormal half: unit in the last place is 2^-24 */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7fffffu; /* hidden one is carried by the exponent field */
    }
    uint32_t kept = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half_ulp = 1u << (shift - 1);
    if (rem > half_ulp || (rem == half_ulp && (kept & 1u))) ++kept; /* may carry into the exponent: still right */
    return (uint16_t)(sign | (base + kept));
}

void oracle_float_to_half_array(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = oracle_float_to_half(in[i]);
}

void oracle_half_to_float_array(const uint16_t* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = oracle_half_to_float(in[i]);
}

/* ---- step size, fused_adam_cuda_kernel.cu:153-162 ----
 * std::pow(float, int) promotes to double; "1 - pow" is a double subtraction that is then narrowed
 * to float; sqrt, multiply and divide are float operations evaluated left to right. */
float fsadam_oracle_step_size(float lr, float beta1, float beta2, int step, int bias_correction) {
    if (bias_correction == 1) {
        const float bias_correction1 = (float)(1.0 - pow((double)beta1, (double)step));
        const float bias_correction2 = (float)(1.0 - pow((double)beta2, (double)step));
        const float root = sqrtf(bias_correction2);
        const float num = lr * root;
        return num / bias_correction1;
    }
    return lr;
}

static inline float load_elem(const void* base, int64_t i, int is_half) {
    if (is_half) return oracle_half_to_float(((const uint16_t*)base)[i]);
    return ((const float*)base)[i];
}

/*
 * One Adam step over one tensor of n elements, in place.
 * Returns 0, or -1 for an unknown mode / missing p_copy.
 * found_inf is only ever set to 1.0f, never cleared (kernel.cu:103-105; the caller zero-fills it,
 * fairscale/optim/adam.py:256).
 */
int fsadam_oracle_step(int mode, void* p, void* m, void* v, const void* g, void* p_copy, int64_t n,
                       float lr, float b1, float b2, float eps, float grad_scale, float optim_scale,
                       float decay, int step, int eps_mode, int bias_correction, float* found_inf) {
    int p_half, g_half, s_half;
    switch (mode) {
        case ORACLE_FULL_PRECISION: p_half = 0; g_half = 0; s_half = 0; break;
        case ORACLE_MIXED_PRECISION: p_half = 0; g_half = 1; s_half = 0; break;
        case ORACLE_MEMORY_EFFICIENT_MIXED_PRECISION: p_half = 1; g_half = 1; s_half = 0; break;
        case ORACLE_PURE_FP16: p_half = 1; g_half = 1; s_half = 1; break;
        case ORACLE_FULL_PRECISION_FP16_COPY: p_half = 0; g_half = 0; s_half = 0; break;
        default: return -1;
    }
    const int depth5 = (mode == ORACLE_MIXED_PRECISION || mode == ORACLE_FULL_PRECISION_FP16_COPY);
    if (depth5 && p_copy == 0) return -1;
    const float step_size = fsadam_oracle_step_size(lr, b1, b2, step, bias_correction);
    const float one_minus_b1 = 1 - b1; /* float subtraction, kernel.cu:97,118 */
    const float one_minus_b2 = 1 - b2; /* kernel.cu:98,119 */
    int any_nonfinite = 0;

#ifdef _OPENMP
#pragma omp parallel for schedule(static) reduction(| : any_nonfinite)
#endif
    for (int64_t j = 0; j < n; ++j) {
        const float in_p = load_elem(p, j, p_half);
        const float in_m = load_elem(m, j, s_half);
        const float in_v = load_elem(v, j, s_half);
        const float in_g = load_elem(g, j, g_half);
        float momentum, velocity;
        const float scaled_grad = in_g / grad_scale; /* kernel.cu:96,117: a true division */
        if (s_half) { /* use_optim_scaling, kernel.cu:94-105 */
            const float m_un = in_m / optim_scale;
            const float v_un = in_v / optim_scale;
            const float a1 = b1 * m_un;
            const float a2 = one_minus_b1 * scaled_grad;
            momentum = a1 + a2;
            const float c1 = b2 * v_un;
            const float c2 = one_minus_b2 * scaled_grad; /* ((1-b2)*g)*g, left to right */
            const float c3 = c2 * scaled_grad;
            velocity = c1 + c3;
            const float ms = momentum * optim_scale;
            const float vs = velocity * optim_scale;
            const uint16_t mh = oracle_float_to_half(ms);
            const uint16_t vh = oracle_float_to_half(vs);
            ((uint16_t*)m)[j] = mh;
            ((uint16_t*)v)[j] = vh;
            /* isfinite() of the STORED halves, kernel.cu:103 */
            if ((mh & 0x7c00u) == 0x7c00u || (vh & 0x7c00u) == 0x7c00u) any_nonfinite |= 1;
        } else { /* kernel.cu:115-121 */
            const float a1 = b1 * in_m;
            const float a2 = one_minus_b1 * scaled_grad;
            momentum = a1 + a2;
            const float c1 = b2 * in_v;
            const float c2 = one_minus_b2 * scaled_grad;
            const float c3 = c2 * scaled_grad;
            velocity = c1 + c3;
            ((float*)m)[j] = momentum;
            ((float*)v)[j] = velocity;
        }
        float denom;
        if (eps_mode == 0) { /* eps under the square root, kernel.cu:108-109,123-124 */
            const float t = velocity + eps;
            denom = sqrtf(t);
        } else { /* kernel.cu:110-111,125-126 */
            const float r = sqrtf(velocity);
            denom = r + eps;
        }
        const float q = momentum / denom;
        const float wd = decay * in_p;
        const float update = q + wd; /* kernel.cu:112,127 */
        const float su = step_size * update;
        const float new_p = in_p - su; /* kernel.cu:113,128 */
        if (p_half) {
            ((uint16_t*)p)[j] = oracle_float_to_half(new_p);
        } else {
            ((float*)p)[j] = new_p;
            /* p_copy is converted from the stored p (kernel.cu:114,129): one rounding of the fp32 result */
            if (depth5) ((uint16_t*)p_copy)[j] = oracle_float_to_half(new_p);
        }
    }
    if (any_nonfinite && found_inf) *found_inf = 1.0f;
    return 0;
}

int fsadam_oracle_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

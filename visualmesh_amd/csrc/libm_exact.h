/*
 * libm_exact.h - acosf, sinf and tanf with the exact results of the host C library (glibc 2.35, x86-64
 * with FMA), written with IEEE-754 operations only so that host and device compute the same bits.
 *
 * Why: the engine contract is parity with the CPU engine on noise images, where a pixel coordinate that
 * differs in its last bit changes the bilinear sample by up to 1e-4. The CPU engine's pixel coordinates
 * come from acosf / sinf / tanf of the host C library (reference utility/projection.hpp:26-60,166-167),
 * so the device must return the same bits for them.
 *
 * How it is pinned: this header compiles for the host as well (VM_HD is empty without hipcc), and
 * tests/test_libm_exact.py compares each function against the host's libm over every float of its input
 * range (acosf: all of [-1, 1]; sinf: [0, pi]; tanf: [0, pi/2]). The algorithms are the classic ones:
 *   acosf  rational approximation on |x| < 0.5, half-angle reduction with a split square root above
 *   sinf   double-precision odd/even polynomials after reduction by pi/2; the fused multiply-adds are
 *          the ones an FMA build of the library performs
 *   tanf   13-term odd polynomial on |x| < 0.6744, pi/4 - x reflection above, reduction by pi/2 in double
 *          precision with a float head and tail
 * Every operation is a single IEEE operation: compile with -ffp-contract=off, correctly rounded
 * division and square root, denormals kept.
 */
#ifndef VMHIP_LIBM_EXACT_H
#define VMHIP_LIBM_EXACT_H

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#pragma clang fp contract(off)
#define VM_HD __host__ __device__ __forceinline__
#else
#include <cmath>
#define VM_HD inline
#endif

VM_HD uint32_t vm_float_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
VM_HD float vm_bits_float(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}
/* Correctly rounded square root. The device's square root instruction alone is only accurate to an ulp; what the
 * compiler makes of sqrtf() in device code (HIP's default: correctly rounded division and square root) is that
 * instruction followed by a choice among the result and its two neighbours by the sign of their exact residuals
 * x - s * s', which is the correctly rounded root, denormals included. The GPU test of this header compares it with
 * the host's over every float from zero to four. */
VM_HD float vm_sqrtf(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_sqrtf(x);
#else
    return sqrtf(x);
#endif
}
VM_HD double vm_fma(double a, double b, double c) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __fma_rn(a, b, c);
#else
    return fma(a, b, c);
#endif
}

VM_HD float vm_acosf(float x) {
    const float one = 1.0000000000e+00f, pi = 3.1415925026e+00f, pio2_hi = 1.5707962513e+00f, pio2_lo = 7.5497894159e-08f;
    const float pS0 = 1.6666667163e-01f, pS1 = -3.2556581497e-01f, pS2 = 2.0121252537e-01f, pS3 = -4.0055535734e-02f,
                pS4 = 7.9153501429e-04f, pS5 = 3.4793309169e-05f;
    const float qS1 = -2.4033949375e+00f, qS2 = 2.0209457874e+00f, qS3 = -6.8828397989e-01f, qS4 = 7.7038154006e-02f;
    const int32_t hx = (int32_t) vm_float_bits(x);
    const int32_t ix = hx & 0x7fffffff;
    if (ix == 0x3f800000) { return hx > 0 ? 0.0f : pi + 2.0f * pio2_lo; }
    if (ix > 0x3f800000) { return (x - x) / (x - x); }
    if (ix < 0x3f000000) { /* |x| < 0.5 */
        if (ix <= 0x23000000) return pio2_hi + pio2_lo;
        const float z = x * x;
        const float p = z * (pS0 + z * (pS1 + z * (pS2 + z * (pS3 + z * (pS4 + z * pS5)))));
        const float q = one + z * (qS1 + z * (qS2 + z * (qS3 + z * qS4)));
        const float r = p / q;
        return pio2_hi - (x - (pio2_lo - x * r));
    }
    if (hx < 0) { /* x < -0.5 */
        const float z = (one + x) * 0.5f;
        const float p = z * (pS0 + z * (pS1 + z * (pS2 + z * (pS3 + z * (pS4 + z * pS5)))));
        const float q = one + z * (qS1 + z * (qS2 + z * (qS3 + z * qS4)));
        const float s = vm_sqrtf(z);
        const float r = p / q;
        const float w = r * s - pio2_lo;
        return pi - 2.0f * (s + w);
    }
    { /* x > 0.5 */
        const float z = (one - x) * 0.5f;
        const float s = vm_sqrtf(z);
        const float df = vm_bits_float(vm_float_bits(s) & 0xfffff000u);
        const float c = (z - df * df) / (s + df);
        const float p = z * (pS0 + z * (pS1 + z * (pS2 + z * (pS3 + z * (pS4 + z * pS5)))));
        const float q = one + z * (qS1 + z * (qS2 + z * (qS3 + z * qS4)));
        const float r = p / q;
        const float w = r * s + c;
        return 2.0f * (df + w);
    }
}

/* sinf for |y| < 120 (the lens maths only needs [0, pi/2]); larger arguments are not supported. */
VM_HD float vm_sinf(float y) {
    const double hpi_inv = 0x1.45F306DC9C883p+23; /* 2/pi * 2^24 */
    const double hpi = 0x1.921FB54442D18p0;
    const double c0 = 0x1p0, c1 = -0x1.ffffffd0c621cp-2, c2 = 0x1.55553e1068f19p-5, c3 = -0x1.6c087e89a359dp-10,
                 c4 = 0x1.99343027bf8c3p-16;
    const double s1 = -0x1.555545995a603p-3, s2 = 0x1.1107605230bc4p-7, s3 = -0x1.994eb3774cf24p-13;
    const uint32_t top = (vm_float_bits(y) >> 20) & 0x7ff;
    double x = (double) y;
    double xs = x;
    int n = 0;
    if (top < 0x3f4u) {                 /* |y| < pi/4 judged by sign-less top 12 bits */
        if (top < 0x398u) return y;     /* |y| < 2^-12 */
    }
    else {
        const double r = x * hpi_inv;
        n = ((int32_t) r + 0x800000) >> 24;
        x = vm_fma(-(double) n, hpi, x);
        xs = ((n & 3) == 1 || (n & 3) == 2) ? x * -1.0 : x * 1.0;
    }
    const double x2 = x * x;
    if ((n & 1) == 0) {
        const double x3 = xs * x2;
        const double t = vm_fma(x2, s3, s2);
        const double x7 = x3 * x2;
        const double s = vm_fma(x3, s1, xs);
        return (float) vm_fma(x7, t, s);
    }
    const double f = (n & 2) ? -1.0 : 1.0; /* the cosine coefficients of the second half turn are negated */
    const double x4 = x2 * x2;
    const double t2 = vm_fma(x2, f * c4, f * c3);
    const double t1 = vm_fma(x2, f * c1, f * c0);
    const double x6 = x4 * x2;
    const double c = vm_fma(x4, f * c2, t1);
    return (float) vm_fma(x6, t2, c);
}

/* Kernel tangent on [-pi/4, pi/4] of x + y (y the tail of x); iy = 1 returns tan, iy = -1 returns -1/tan. */
VM_HD float vm_kernel_tanf(float x, float y, int iy) {
    const float one = 1.0000000000e+00f, pio4 = 7.8539812565e-01f, pio4lo = 3.7748947079e-08f;
    const float T0 = 3.3333334327e-01f, T1 = 1.3333334029e-01f, T2 = 5.3968254477e-02f, T3 = 2.1869488060e-02f,
                T4 = 8.8632395491e-03f, T5 = 3.5920790397e-03f, T6 = 1.4562094584e-03f, T7 = 5.8804126456e-04f,
                T8 = 2.4646313977e-04f, T9 = 7.8179444245e-05f, T10 = 7.1407252108e-05f, T11 = -1.8558637748e-05f,
                T12 = 2.5907305826e-05f;
    const int32_t hx = (int32_t) vm_float_bits(x);
    const int32_t ix = hx & 0x7fffffff;
    float z, r, v, w, s;
    if (ix < 0x39000000) { /* |x| < 2^-13 */
        if ((int) x == 0) {
            if ((ix | (iy + 1)) == 0) return one / (x < 0 ? -x : x);
            if (iy == 1) return x;
            return -one / x;
        }
    }
    if (ix >= 0x3f2ca140) { /* |x| >= 0.6744 */
        if (hx < 0) {
            x = -x;
            y = -y;
        }
        z = pio4 - x;
        w = pio4lo - y;
        x = z + w;
        y = 0.0f;
        if ((x < 0 ? -x : x) < 0x1p-13f) return (float) (1 - ((hx >> 30) & 2)) * (float) iy * (1.0f - (float) (2 * iy) * x);
    }
    z = x * x;
    w = z * z;
    r = T1 + w * (T3 + w * (T5 + w * (T7 + w * (T9 + w * T11))));
    v = z * (T2 + w * (T4 + w * (T6 + w * (T8 + w * (T10 + w * T12)))));
    s = z * x;
    r = y + z * (s * (r + v) + y);
    r += T0 * s;
    w = x + r;
    if (ix >= 0x3f2ca140) {
        v = (float) iy;
        return (float) (1 - ((hx >> 30) & 2)) * (v - 2.0f * (x - (w * w / (w + v) - r)));
    }
    if (iy == 1) return w;
    { /* -1 / (x + r) with a split quotient */
        z = vm_bits_float(vm_float_bits(w) & 0xfffff000u);
        v = r - (z - x);
        const float a = -1.0f / w;
        const float t = vm_bits_float(vm_float_bits(a) & 0xfffff000u);
        s = 1.0f + t * z;
        return t + a * (s + t * v);
    }
}

/* tanf for |x| < 3 pi / 4 (the lens maths only needs [0, pi/2]); larger arguments are not supported.
 * Above pi/4 the argument is reduced by pi/2 in double precision and handed to the kernel as a float head
 * and tail; tan(x) = -1 / tan(x - pi/2). */
VM_HD float vm_tanf(float x) {
    const uint32_t hx = vm_float_bits(x);
    const uint32_t ix = hx & 0x7fffffffu;
    if (ix <= 0x3f490fdau) return vm_kernel_tanf(x, 0.0f, 1);
    const float sign = (hx >> 31) ? -1.0f : 1.0f;
    const double reduced = (double) (sign * x) - 0x1.921fb54442d18p0;
    const float head = (float) reduced;
    const float tail = (float) (reduced - (double) head);
    return sign * vm_kernel_tanf(head, tail, -1);
}

#endif

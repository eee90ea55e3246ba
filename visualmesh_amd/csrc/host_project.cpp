/*
 * Host-side lens projection in the reference's exact arithmetic, for Scalar = T = float or double.
 *
 * The device decides "is this node on screen" from acosf/sinf/tanf results whose last bit may differ
 * from the host C library's. The few candidates that project within a small band of a screen edge are
 * re-decided here, with the same operation order and operand types as the reference
 * (utility/projection.hpp:162-187, :79-120 for the distortion polynomial; the strict comparison is
 * engine/cpu/engine.hpp:116-117), so the visible set is the one the CPU engine produces.
 *
 * Compile with -ffp-contract=off and without -ffast-math: every operation in T must be a single
 * IEEE-754 operation of that type.
 */
#include <algorithm>
#include <cmath>

#include "host_project.h"

/* utility/projection.hpp:79-87 */
template <typename T>
static void inverse_coefficients(const T* k, T* ik) {
    ik[0] = -k[0];
    ik[1] = T(3.0) * (k[0] * k[0]) - k[1];
    ik[2] = -T(12.0) * (k[0] * k[0]) * k[0] + T(8.0) * k[0] * k[1];
    ik[3] = T(55.0) * (k[0] * k[0]) * (k[0] * k[0]) - T(55.0) * (k[0] * k[0]) * k[1] + T(5.0) * (k[1] * k[1]);
}

template <typename T>
static int on_screen(const T* Rco, const T* ray, int projection, T focal, const T* centre,
                      const T* ik, int width, int height, T* px_out) {
    /* cam = Rco * ray with dot(a, b) = a2*b2 + (a1*b1 + a0*b0): utility/math.hpp:145-164, :254-257 */
    T cam[3];
    for (int i = 0; i < 3; ++i) cam[i] = Rco[i * 3 + 2] * ray[2] + (Rco[i * 3 + 1] * ray[1] + Rco[i * 3 + 0] * ray[0]);

    const T theta = std::acos(cam[0]);
    const T rsin_theta = T(1.0) / std::sqrt(T(1.0) - cam[0] * cam[0]);
    T r_u;
    switch (projection) {
        case 0: r_u = focal * std::tan(std::min(std::max(theta, T(0.0)), T(M_PI_2))); break;
        case 1: r_u = T(2.0) * focal * std::sin(theta * T(0.5)); break;
        default: r_u = focal * theta; break;
    }
    /* the bracket is a double sum of T terms because of the reference's literal 1.0 */
    const T r2 = r_u * r_u;
    const double s = 1.0 + double(ik[0] * r2) + double(ik[1] * (r2 * r2)) + double(ik[2] * (r2 * r2) * r2)
                     + double(ik[3] * (r2 * r2) * (r2 * r2));
    const T r_d = T(double(r_u) * s);

    T sx = T(0.0), sy = T(0.0);
    if (!(cam[0] >= 1)) {
        sx = r_d * cam[1] * rsin_theta;
        sy = r_d * cam[2] * rsin_theta;
    }
    const T px = (T(width) * T(0.5) - sx) - centre[0];
    const T py = (T(height) * T(0.5) - sy) - centre[1];
    if (px_out) {
        px_out[0] = px;
        px_out[1] = py;
    }
    return (0 <= px && px + 1 < width && 0 <= py && py + 1 < height) ? 1 : 0;
}

void vm_host_inverse_coefficients(const float* k, float* ik) { inverse_coefficients<float>(k, ik); }
int vm_host_on_screen(const float* Rco, const float* ray, int projection, float focal, const float* centre,
                      const float* ik, int width, int height, float* px_out) {
    return on_screen<float>(Rco, ray, projection, focal, centre, ik, width, height, px_out);
}
void vm_host_inverse_coefficients_f64(const double* k, double* ik) { inverse_coefficients<double>(k, ik); }
int vm_host_on_screen_f64(const double* Rco, const double* ray, int projection, double focal, const double* centre,
                          const double* ik, int width, int height, double* px_out) {
    return on_screen<double>(Rco, ray, projection, focal, centre, ik, width, height, px_out);
}

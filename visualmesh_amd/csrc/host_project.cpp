/*
 * Host-side lens projection in the reference's exact fp32 arithmetic.
 *
 * The device decides "is this node on screen" from acosf/sinf/tanf results whose last bit may differ
 * from the host C library's. The few candidates that project within a small band of a screen edge are
 * re-decided here, with the same operation order and operand types as the reference
 * (utility/projection.hpp:162-187, :79-120 for the distortion polynomial; the strict comparison is
 * engine/cpu/engine.hpp:116-117), so the visible set is the one the CPU engine produces.
 *
 * Compile with -ffp-contract=off and without -ffast-math: every float operation must be a single
 * IEEE-754 binary32 operation.
 */
#include <algorithm>
#include <cmath>

#include "host_project.h"

/* utility/projection.hpp:79-87 */
void vm_host_inverse_coefficients(const float* k, float* ik) {
    ik[0] = -k[0];
    ik[1] = 3.0f * (k[0] * k[0]) - k[1];
    ik[2] = -12.0f * (k[0] * k[0]) * k[0] + 8.0f * k[0] * k[1];
    ik[3] = 55.0f * (k[0] * k[0]) * (k[0] * k[0]) - 55.0f * (k[0] * k[0]) * k[1] + 5.0f * (k[1] * k[1]);
}

int vm_host_on_screen(const float* Rco, const float* ray, int projection, float focal, const float* centre,
                      const float* ik, int width, int height, float* px_out) {
    /* cam = Rco * ray with dot(a, b) = a2*b2 + (a1*b1 + a0*b0): utility/math.hpp:145-164, :254-257 */
    float cam[3];
    for (int i = 0; i < 3; ++i) cam[i] = Rco[i * 3 + 2] * ray[2] + (Rco[i * 3 + 1] * ray[1] + Rco[i * 3 + 0] * ray[0]);

    const float theta = std::acos(cam[0]);
    const float rsin_theta = 1.0f / std::sqrt(1.0f - cam[0] * cam[0]);
    float r_u;
    switch (projection) {
        case 0: r_u = focal * std::tan(std::min(std::max(theta, 0.0f), float(M_PI_2))); break;
        case 1: r_u = 2.0f * focal * std::sin(theta * 0.5f); break;
        default: r_u = focal * theta; break;
    }
    /* the bracket is a double sum of float terms because of the reference's literal 1.0 */
    const float r2 = r_u * r_u;
    const double s = 1.0 + double(ik[0] * r2) + double(ik[1] * (r2 * r2)) + double(ik[2] * (r2 * r2) * r2)
                     + double(ik[3] * (r2 * r2) * (r2 * r2));
    const float r_d = float(double(r_u) * s);

    float sx = 0.0f, sy = 0.0f;
    if (!(cam[0] >= 1)) {
        sx = r_d * cam[1] * rsin_theta;
        sy = r_d * cam[2] * rsin_theta;
    }
    const float px = (float(width) * 0.5f - sx) - centre[0];
    const float py = (float(height) * 0.5f - sy) - centre[1];
    if (px_out) {
        px_out[0] = px;
        px_out[1] = py;
    }
    return (0 <= px && px + 1 < width && 0 <= py && py + 1 < height) ? 1 : 0;
}

/* Host-side lens projection in the reference's arithmetic for Scalar = float and, with the _f64 names, double
 * (host_project.cpp). Plain C++, no HIP. */
#ifndef VMHIP_HOST_PROJECT_H
#define VMHIP_HOST_PROJECT_H

/* Host re-decision of an on-screen test with the CPU arithmetic (glibc libm, one IEEE operation per
 * step). ray is the node's unit vector in observation-plane space. Returns 1 if the node is kept. */
int vm_host_on_screen(const float* Rco, const float* ray, int projection, float focal, const float* centre,
                      const float* ik, int width, int height, float* px_out);
void vm_host_inverse_coefficients(const float* k, float* ik);
int vm_host_on_screen_f64(const double* Rco, const double* ray, int projection, double focal, const double* centre,
                          const double* ik, int width, int height, double* px_out);
void vm_host_inverse_coefficients_f64(const double* k, double* ik);

#endif

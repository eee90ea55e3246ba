/* Host-side lens projection in the reference's fp32 arithmetic (host_project.cpp). Plain C++, no HIP. */
#ifndef VMHIP_HOST_PROJECT_H
#define VMHIP_HOST_PROJECT_H

/* Host re-decision of an on-screen test with the CPU arithmetic (glibc libm, one IEEE operation per
 * step). ray is the node's unit vector in observation-plane space. Returns 1 if the node is kept. */
int vm_host_on_screen(const float* Rco, const float* ray, int projection, float focal, const float* centre,
                      const float* ik, int width, int height, float* px_out);
void vm_host_inverse_coefficients(const float* k, float* ik);

#endif

// TEST INFRASTRUCTURE ONLY -- never linked into, or called by, the product library.
//
// C-linkage doorway onto the reference's own CPU kernels, compiled in place from
// /root/reference/gpu_featurizer/kernel_cpu.cpp (see oracle/Makefile, target _ref).
// The reference's TensorFlow functor (functor_op_cpu.cpp:13-43, 46-83, 86-121) is only
// "zero the outputs, then call the kernel"; that contract is restated here in a few lines so
// that the compiled reference can be driven without TensorFlow.  No reference source text is
// copied: the templates are declared by including the reference's own header through -I.
#include <cstring>
#include "kernel_cpu.h"   // resolved with -I/root/reference/gpu_featurizer at build time

namespace {

template <typename T>
void fwd(const T *x, const T *y, const T *z, const int *a, const int *mos, const int *macs,
         int n_mols, const int *sis, T *h, T *c, T *n, T *o, const int *acs) {
    // functor_op_cpu.cpp:31-34 -- outputs are zero-filled per bucket before accumulation
    T *out[4] = {h, c, n, o};
    for (int t = 0; t < 4; ++t)
        if (acs[t] > 0) std::memset(out[t], 0, sizeof(T) * (size_t)acs[t] * TOTAL_FEATURE_SIZE);
    featurize_cpu<T>(x, y, z, a, mos, macs, n_mols, sis, h, c, n, o);
}

template <typename T>
void bwd(const T *x, const T *y, const T *z, const int *a, const int *mos, const int *macs,
         int n_mols, const int *sis, const T *gh, const T *gc, const T *gn, const T *go,
         T *gx, T *gy, T *gz, const int *acs) {
    // functor_op_cpu.cpp:68-72 -- coordinate gradients of sum(acs) atoms are zeroed first
    const size_t n_atoms = (size_t)acs[0] + acs[1] + acs[2] + acs[3];
    std::memset(gx, 0, sizeof(T) * n_atoms);
    std::memset(gy, 0, sizeof(T) * n_atoms);
    std::memset(gz, 0, sizeof(T) * n_atoms);
    featurize_grad_cpu<T>(x, y, z, a, mos, macs, n_mols, sis, gh, gc, gn, go, gx, gy, gz);
}

template <typename T>
void bwd_inv(const T *x, const T *y, const T *z, const int *a, const int *mos, const int *macs,
             int n_mols, const int *sis, const T *gx, const T *gy, const T *gz,
             T *h, T *c, T *n, T *o, const int *acs) {
    // functor_op_cpu.cpp:106-109
    T *out[4] = {h, c, n, o};
    for (int t = 0; t < 4; ++t)
        if (acs[t] > 0) std::memset(out[t], 0, sizeof(T) * (size_t)acs[t] * TOTAL_FEATURE_SIZE);
    featurize_grad_inverse<T>(x, y, z, a, mos, macs, n_mols, sis, gx, gy, gz, h, c, n, o);
}

}  // namespace

extern "C" {

void ref_featurize_f32(const float *x, const float *y, const float *z, const int *a,
                       const int *mos, const int *macs, int n_mols, const int *sis,
                       float *h, float *c, float *n, float *o, const int *acs) {
    fwd<float>(x, y, z, a, mos, macs, n_mols, sis, h, c, n, o, acs);
}
void ref_featurize_f64(const double *x, const double *y, const double *z, const int *a,
                       const int *mos, const int *macs, int n_mols, const int *sis,
                       double *h, double *c, double *n, double *o, const int *acs) {
    fwd<double>(x, y, z, a, mos, macs, n_mols, sis, h, c, n, o, acs);
}
void ref_featurize_grad_f32(const float *x, const float *y, const float *z, const int *a,
                            const int *mos, const int *macs, int n_mols, const int *sis,
                            const float *gh, const float *gc, const float *gn, const float *go,
                            float *gx, float *gy, float *gz, const int *acs) {
    bwd<float>(x, y, z, a, mos, macs, n_mols, sis, gh, gc, gn, go, gx, gy, gz, acs);
}
void ref_featurize_grad_f64(const double *x, const double *y, const double *z, const int *a,
                            const int *mos, const int *macs, int n_mols, const int *sis,
                            const double *gh, const double *gc, const double *gn,
                            const double *go, double *gx, double *gy, double *gz,
                            const int *acs) {
    bwd<double>(x, y, z, a, mos, macs, n_mols, sis, gh, gc, gn, go, gx, gy, gz, acs);
}
void ref_featurize_grad_inverse_f32(const float *x, const float *y, const float *z, const int *a,
                                    const int *mos, const int *macs, int n_mols, const int *sis,
                                    const float *gx, const float *gy, const float *gz,
                                    float *h, float *c, float *n, float *o, const int *acs) {
    bwd_inv<float>(x, y, z, a, mos, macs, n_mols, sis, gx, gy, gz, h, c, n, o, acs);
}
void ref_featurize_grad_inverse_f64(const double *x, const double *y, const double *z,
                                    const int *a, const int *mos, const int *macs, int n_mols,
                                    const int *sis, const double *gx, const double *gy,
                                    const double *gz, double *h, double *c, double *n, double *o,
                                    const int *acs) {
    bwd_inv<double>(x, y, z, a, mos, macs, n_mols, sis, gx, gy, gz, h, c, n, o, acs);
}

}  // extern "C"

// ANI-1 featurization parameters as device-side constants.
//
// Every parameter of the reference is a `const float` (gpu_featurizer/parameters.h:10,61-114), and
// its double-precision path widens those rounded floats.  The double tables below are therefore the
// float literals widened, not the "exact" decimals; cos/sin of the float-rounded theta_t values were
// evaluated once in double.  M_PI is the only true double constant (kernel_cpu.cpp:31).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace khan {

// Measurement builds only (khan_amd/build.py: build_stage_variants): KHAN_PROFILE_SKIP compiles a stage of the AEV
// kernels out, so that the time of the rest can be measured.  Bit 0: the angular part, bit 1: the radial part, bit 2: the
// forward kernels' stores of feature rows (the values are still computed), bit 3: every atom reads the upstream row of
// the first atom of its type (the small backward kernel: its loads then hit the caches).
// Such a library gives wrong results by design and is never the one the package loads by default.
#ifndef KHAN_PROFILE_SKIP
#define KHAN_PROFILE_SKIP 0
#endif
constexpr bool kSkipAngular = (KHAN_PROFILE_SKIP & 1) != 0;
constexpr bool kSkipRadial = (KHAN_PROFILE_SKIP & 2) != 0;
constexpr bool kSkipStores = (KHAN_PROFILE_SKIP & 4) != 0;
constexpr bool kOneUpstreamRow = (KHAN_PROFILE_SKIP & 8) != 0;

constexpr int kNumTypes = 4;
constexpr int kNumRRs = 16;
constexpr int kNumAThetas = 8;
constexpr int kNumARs = 4;
constexpr int kRadial = kNumTypes * kNumRRs;                          // 64
constexpr int kAngBlock = kNumAThetas * kNumARs;                      // 32
constexpr int kNumPairBlocks = kNumTypes * (kNumTypes + 1) / 2;       // 10
constexpr int kAngular = kAngBlock * kNumPairBlocks;                  // 320
constexpr int kFeats = kRadial + kAngular;                            // 384

constexpr float kR_eta_f = 16.0f;
constexpr float kR_Rc_f = 4.6f;
constexpr float kA_Rc_f = 3.1f;
constexpr float kA_eta_f = 6.0f;
constexpr float kChargeK_f = 0.529176917f;
constexpr double kPi = 3.14159265358979323846;

__device__ static const float kR_Rs_f[kNumRRs] = {
    5.0000000e-01f, 7.5625000e-01f, 1.0125000e+00f, 1.2687500e+00f, 1.5250000e+00f, 1.7812500e+00f,
    2.0375000e+00f, 2.2937500e+00f, 2.5500000e+00f, 2.8062500e+00f, 3.0625000e+00f, 3.3187500e+00f,
    3.5750000e+00f, 3.8312500e+00f, 4.0875000e+00f, 4.3437500e+00f};
__device__ static const float kA_Rs_f[kNumARs] = {5.0000000e-01f, 1.1500000e+00f, 1.8000000e+00f,
                                                  2.4500000e+00f};
// cos / sin of (double)A_thetas[t], A_thetas = {0, 0.78539816f, 1.5707963f, 2.3561945f, 3.1415927f,
// 3.9269908f, 4.7123890f, 5.4977871f} (parameters.h:97-106)
__device__ static const double kCosTheta[kNumAThetas] = {
    1.0, 0.7071067657322372, 7.549789954891874e-08, -0.7071067854026294,
    -0.9999999999999962, -0.7071068303555407, 1.1924880454806035e-08, 0.7071066786324686};
__device__ static const double kSinTheta[kNumAThetas] = {
    0.0, 0.7071067966408575, 0.9999999999999971, 0.7071067769704656,
    -8.742278000372475e-08, -0.707106732017551, -0.9999999999999999, -0.7071068837406116};

// index of the 32-wide angular block of an unordered type pair: HH0 HC1 HN2 HO3 CC4 CN5 CO6 NN7 NO8 OO9
// (kernel_cpu.cpp:9-23 with the theta/Rs indices taken out)
__device__ __forceinline__ int pair_block(int a, int b)
{
    const int lo = a < b ? a : b, hi = a < b ? b : a;
    return 6 - ((4 - lo) * (3 - lo)) / 2 + hi;
}

// kernel_cpu.cpp:439-447: any type other than 0,1,2 is treated as O.  The reference indexes feature
// columns with the raw type (undefined for types outside 0..3); here such types are folded into 3.
__device__ __forceinline__ int fold_type(int t) { return (static_cast<unsigned>(t) > 3u) ? 3 : t; }

template <typename T> struct Real;
template <> struct Real<float> {
    __device__ static __forceinline__ float exp_(float x) { return expf(x); }
    __device__ static __forceinline__ float sqrt_(float x) { return sqrtf(x); }
    __device__ static __forceinline__ float cos_(float x) { return cosf(x); }
    __device__ static __forceinline__ float sin_(float x) { return sinf(x); }
    static constexpr float kCotEps = 1e-12f;
};
template <> struct Real<double> {
    __device__ static __forceinline__ double exp_(double x) { return exp(x); }
    __device__ static __forceinline__ double sqrt_(double x) { return sqrt(x); }
    __device__ static __forceinline__ double cos_(double x) { return cos(x); }
    __device__ static __forceinline__ double sin_(double x) { return sin(x); }
    static constexpr double kCotEps = 1e-24;
};

// cot(theta) = c/s from c = cos(theta) and s = sin(theta) >= 0, regularised on the line theta = 0, pi where
// the angle has a cusp: c s / (s^2 + eps) differs from c/s by eps/s^2 relative and goes to zero with s.
template <typename T>
__device__ __forceinline__ T cot_reg(T c, T s)
{
    return c * s / (s * s + Real<T>::kCotEps);
}

// f_C(r, rc) = 0.5 cos(pi r / rc) + 0.5 for r <= rc (kernel_cpu.cpp:29-35); callers only evaluate it
// inside the strict cutoff, so the r > rc branch is not needed here.
template <typename T>
__device__ __forceinline__ T cutoff_fn(T r, T pi_over_rc)
{
    return T(0.5) * Real<T>::cos_(pi_over_rc * r) + T(0.5);
}
// d f_C / d r = -(pi / (2 rc)) sin(pi r / rc)
template <typename T>
__device__ __forceinline__ T cutoff_dfn(T r, T pi_over_rc)
{
    return T(-0.5) * pi_over_rc * Real<T>::sin_(pi_over_rc * r);
}

}  // namespace khan

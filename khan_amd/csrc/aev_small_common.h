// Building blocks shared by the small-molecule (one wavefront per molecule) AEV kernels.
#pragma once
#include "aev_generic_center.h"

namespace khan {

// One wavefront per workgroup: molecules differ a lot in cost, and a workgroup's LDS is only released when
// its slowest wavefront ends, so wider workgroups leave wave slots idle.
constexpr int kWavesPerBlock = 1;
constexpr int kFB = 6;         // centres per batch of the one-wavefront forward kernels
constexpr int kB = 6;          // centres per batch: 6 x 10 type pairs = 60 segment lanes
constexpr int kCapA = 32;      // angular neighbours kept per centre
// words of slot bits for a batch of n centres: at most 496 triples and 10 padding slots each, one bit per slot, and
// one word beyond the last step's (96 for six centres)
constexpr int bit_words(int n) { return (n * 506 + 31) / 32 + 1; }

// One (centre, type pair) segment of a batch's triples, laid out so that a lane decodes its triple with few
// instructions: fields sit on byte / half-word boundaries (the operand selects of the vector instructions read them
// in place) and the list offsets are byte offsets, ready to be added to.
struct __align__(16) SegDesc {
    unsigned start_cnt;  // first triple slot of the segment inside the batch (even, low 16 bits) | triples << 16
    unsigned aj;         // byte offset, inside the batch's neighbour lists, of the centre's first entry of type a
    unsigned ak;         // the same for type b
    unsigned div;        // floor(2^15 / n_a) + 1 (low 16 bits: q / n_a = q * that >> 15 for q < 1024) | n_a << 16 | (a == b) << 24
};


__device__ __forceinline__ float lane_read(float v, int src_lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src_lane));
}
__device__ __forceinline__ int lane_read(int v, int src_lane) { return __builtin_amdgcn_readlane(v, src_lane); }
__device__ __forceinline__ float lane_push(int dest_lane, float v)   // the value lands in lane dest_lane
{
    return __int_as_float(__builtin_amdgcn_ds_permute(dest_lane << 2, __float_as_int(v)));
}
__device__ __forceinline__ int lane_push(int dest_lane, int v) { return __builtin_amdgcn_ds_permute(dest_lane << 2, v); }
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
// 64-bit values travel as two 32-bit halves
__device__ __forceinline__ double lane_read(double v, int src_lane)
{
    const long long b = __double_as_longlong(v);
    const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(b), src_lane));
    const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(b >> 32), src_lane));
    return __longlong_as_double(static_cast<long long>((static_cast<unsigned long long>(hi) << 32) | lo));
}
__device__ __forceinline__ double lane_push(int dest_lane, double v)
{
    const long long b = __double_as_longlong(v);
    const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_ds_permute(dest_lane << 2, static_cast<int>(b)));
    const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_ds_permute(dest_lane << 2, static_cast<int>(b >> 32)));
    return __longlong_as_double(static_cast<long long>((static_cast<unsigned long long>(hi) << 32) | lo));
}

// Row pointers are rebuilt from two 32-bit lane reads; storing through an explicit global-address-space
// pointer keeps the stores on the global (not the flat) path.
typedef float __attribute__((address_space(1))) global_float;
__device__ __forceinline__ void store_global(float* p, float v)
{
    if constexpr (kSkipStores) asm volatile("" ::"v"(v), "v"(p));      // measurement build: the value is formed, not stored
    else *((global_float*)(p)) = v;
}
typedef double __attribute__((address_space(1))) global_double;
__device__ __forceinline__ void store_global(double* p, double v)
{
    if constexpr (kSkipStores) asm volatile("" ::"v"(v), "v"(p));
    else *((global_double*)(p)) = v;
}
// acc + a' * g, where a' is the value of `a` held by lane k of this lane's quad (k is a constant after unrolling).
// The lane exchange is a modifier of the multiply-add, not an instruction of its own.  It reads `a` early: two
// wait states have to lie between a vector instruction that writes `a` and this one, and the compiler does not
// see inside the asm.  `a` comes from an LDS read here, never from a vector instruction; the build checks the
// generated code for that (khan_amd/build.py: check_dpp_operands) instead of paying two idle cycles per use.
__device__ __forceinline__ float fma_quad(float a, int k, float g, float acc)
{
    if (k == 0) asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(a), "v"(g));
    else if (k == 1) asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(a), "v"(g));
    else if (k == 2) asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(a), "v"(g));
    else asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(a), "v"(g));
    return acc;
}
__device__ __forceinline__ double fma_quad(double a, int, double g, double acc) { return fma(a, g, acc); }   // float only
// 16 bytes of zeros to a 16-byte aligned global address
typedef float __attribute__((ext_vector_type(4))) zero_v4f;
typedef zero_v4f __attribute__((address_space(1))) global_v4f_store;
__device__ __forceinline__ void store_global16(void* p)
{
    if constexpr (kSkipStores) asm volatile("" ::"v"(p));
    else *((global_v4f_store*)(p)) = zero_v4f{0.f, 0.f, 0.f, 0.f};
}
// sum of the two half-waves, in every lane: swap the upper half of one copy with the lower half of
// the other (one cross-lane VALU move, no LDS round trip), then add
__device__ __forceinline__ float half_wave_sum(float v)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_int(v), __float_as_int(v), false, false);
    return __int_as_float(r[0]) + __int_as_float(r[1]);
}

__device__ __forceinline__ double half_wave_sum(double v)
{
    const long long b = __double_as_longlong(v);
    const int lo = static_cast<int>(b), hi = static_cast<int>(b >> 32);
    const auto rl = __builtin_amdgcn_permlane32_swap(lo, lo, false, false);
    const auto rh = __builtin_amdgcn_permlane32_swap(hi, hi, false, false);
    const double a0 = __longlong_as_double(static_cast<long long>((static_cast<unsigned long long>(static_cast<unsigned>(rh[0])) << 32) | static_cast<unsigned>(rl[0])));
    const double a1 = __longlong_as_double(static_cast<long long>((static_cast<unsigned long long>(static_cast<unsigned>(rh[1])) << 32) | static_cast<unsigned>(rl[1])));
    return a0 + a1;
}

// Inclusive add-scan across the 64 lanes with data-parallel-primitive moves: four shifts inside each
// row of 16 lanes, then lane 15 of rows 0,2 is carried into rows 1,3 and lane 31 into rows 2,3.
// Lanes without a source take the identity 0.
template <int kCtrl, int kRowMask>
__device__ __forceinline__ int dpp_take(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, kCtrl, kRowMask, 0xf, false);
}
__device__ __forceinline__ int scan_add(int v)
{
    v += dpp_take<0x111, 0xf>(v);   // row_shr:1
    v += dpp_take<0x112, 0xf>(v);   // row_shr:2
    v += dpp_take<0x114, 0xf>(v);   // row_shr:4
    v += dpp_take<0x118, 0xf>(v);   // row_shr:8
    v += dpp_take<0x142, 0xa>(v);   // row_bcast:15 into rows 1 and 3
    v += dpp_take<0x143, 0xc>(v);   // row_bcast:31 into rows 2 and 3
    return v;
}

__device__ __forceinline__ int wave_max(int v)       // all inputs >= 0; result is wave-uniform
{
    v = max(v, dpp_take<0x111, 0xf>(v));
    v = max(v, dpp_take<0x112, 0xf>(v));
    v = max(v, dpp_take<0x114, 0xf>(v));
    v = max(v, dpp_take<0x118, 0xf>(v));
    v = max(v, dpp_take<0x142, 0xa>(v));
    v = max(v, dpp_take<0x143, 0xc>(v));
    return __builtin_amdgcn_readlane(v, 63);
}

// Float add-scan with the same data-parallel-primitive moves.  After `rows` steps the last lane of
// each group of 16 (rows = 4), 32 (rows = 5) or 64 (rows = 6) lanes holds that group's sum.
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_take_f(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, kRowMask, 0xf, false));
}
template <int kCtrl, int kRowMask>
__device__ __forceinline__ double dpp_take_f(double v)
{
    const long long b = __double_as_longlong(v);
    const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(b), kCtrl, kRowMask, 0xf, false));
    const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(b >> 32), kCtrl, kRowMask, 0xf, false));
    return __longlong_as_double(static_cast<long long>((static_cast<unsigned long long>(hi) << 32) | lo));
}
// the value lane (byte_index / 4) holds (per-lane source; every lane takes part)
__device__ __forceinline__ float lane_fetch(float v, int byte_index)
{
    return __int_as_float(__builtin_amdgcn_ds_bpermute(byte_index, __float_as_int(v)));
}
__device__ __forceinline__ double lane_fetch(double v, int byte_index)
{
    const long long b = __double_as_longlong(v);
    const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(byte_index, static_cast<int>(b)));
    const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(byte_index, static_cast<int>(b >> 32)));
    return __longlong_as_double(static_cast<long long>((static_cast<unsigned long long>(hi) << 32) | lo));
}
__device__ __forceinline__ double group_sum_to_last_lane(double v, int log_group)
{
    v += dpp_take_f<0x111, 0xf>(v);
    v += dpp_take_f<0x112, 0xf>(v);
    v += dpp_take_f<0x114, 0xf>(v);
    v += dpp_take_f<0x118, 0xf>(v);
    if (log_group >= 5) v += dpp_take_f<0x142, 0xa>(v);
    if (log_group >= 6) v += dpp_take_f<0x143, 0xc>(v);
    return v;
}
__device__ __forceinline__ float group_sum_to_last_lane(float v, int log_group)
{
    v += dpp_take_f<0x111, 0xf>(v);
    v += dpp_take_f<0x112, 0xf>(v);
    v += dpp_take_f<0x114, 0xf>(v);
    v += dpp_take_f<0x118, 0xf>(v);
    if (log_group >= 5) v += dpp_take_f<0x142, 0xa>(v);
    if (log_group >= 6) v += dpp_take_f<0x143, 0xc>(v);
    return v;
}

// 1 + cos(theta - theta_t) for the eight theta_t = t pi/4, from c = cos(theta) and s = sin(theta) >= 0.
// double: each from the table's cos/sin of the float-rounded theta_t, as the 1e-12 tolerance needs.
// float: theta_0 = 0 is exact; theta_2, theta_4 and theta_6 are within 9e-8 of pi/2, pi and 3 pi/2, so their values are
// 1 + s, 1 - c and 1 - s to 9e-8; theta_1 and theta_5 are within 7e-8 of pi/4 and 5 pi/4 and share
// p = (c + s)/sqrt(2): 12 instructions instead of 16, the values within 1e-7 of the table's (a few percent of
// the tolerance after the eighth power).  theta_3 and theta_7 (the latter 1.5e-7 off) keep their table entries.
template <typename T>
__device__ __forceinline__ void theta_bases(T c, T s, T (&b)[8])
{
    if constexpr (sizeof(T) == 4) {
        const T p = T(0.70710678118654752) * (c + s);
        b[0] = T(1) + c;
        b[4] = T(1) - c;
        b[2] = T(1) + s;
        b[6] = T(1) - s;
        b[1] = T(1) + p;
        b[5] = T(1) - p;
        b[3] = fma(s, static_cast<T>(kSinTheta[3]), fma(c, static_cast<T>(kCosTheta[3]), T(1)));
        b[7] = fma(s, static_cast<T>(kSinTheta[7]), fma(c, static_cast<T>(kCosTheta[7]), T(1)));
    } else {
#pragma unroll
        for (int t = 0; t < 8; ++t)
            b[t] = fma(s, static_cast<T>(kSinTheta[t]), fma(c, static_cast<T>(kCosTheta[t]), T(1)));
    }
}

template <typename T>
__device__ __forceinline__ T pow8(T b)
{
    const T b2 = b * b, b4 = b2 * b2;
    return b4 * b4;
}
__device__ __forceinline__ int sel4(int a, int v0, int v1, int v2, int v3)
{
    return a == 0 ? v0 : a == 1 ? v1 : a == 2 ? v2 : v3;
}
__device__ __forceinline__ int popc64(unsigned long long m) { return __popcll(m); }
__device__ __forceinline__ unsigned long long low_bits(int w)   // w ones, 1 <= w <= 64
{
    return w >= 64 ? ~0ull : ((1ull << w) - 1ull);
}

// f_C(r, rc) = 0.5 cos(pi u) + 0.5 = cos^2(pi u / 2), u = r / rc in [0, 1).
// With w = min(u, 1-u) and s = sin(pi w / 2) (odd minimax polynomial on [0, 0.5], |err| < 1.1e-7):
// f_C = 1 - s^2 for u <= 0.5 and s^2 above, which keeps full relative accuracy where f_C -> 0.
__device__ __forceinline__ float cutoff_poly(float u)
{
    const float w = fminf(u, 1.0f - u);
    const float w2 = w * w;
    float p = fmaf(w2, -0.00459228908981766f, 0.07967590297660462f);
    p = fmaf(w2, p, -0.645962938168251f);
    p = fmaf(w2, p, 1.5707963050854938f);
    const float s = p * w;
    const float q = s * s;
    return (u <= 0.5f) ? 1.0f - q : q;
}


// f_C and d f_C / d r for the backward pass.  With w = min(u, 1-u), s = sin(pi w/2), c = cos(pi w/2)
// (minimax polynomials on [0, 0.5]):  f_C = cos^2(pi u/2) is c^2 below u = 0.5 and s^2 above;
// d f_C / d u = -(pi/2) sin(pi u) = -pi s c on both sides.
__device__ __forceinline__ void cutoff_poly_grad(float u, float inv_rc, float& fc, float& dfc_dr)
{
    const float w = fminf(u, 1.0f - u);
    const float w2 = w * w;
    float ps = fmaf(w2, -0.00459228908981766f, 0.07967590297660462f);
    ps = fmaf(w2, ps, -0.645962938168251f);
    ps = fmaf(w2, ps, 1.5707963050854938f);
    const float sn = ps * w;
    float pc = fmaf(w2, 0.0009036319656957207f, -0.02086007146631888f);
    pc = fmaf(w2, pc, 0.2536692039669182f);
    pc = fmaf(w2, pc, -1.2337005406492898f);
    const float cs = fmaf(w2, pc, 0.9999999999526366f);
    fc = (u <= 0.5f) ? cs * cs : sn * sn;
    dfc_dr = -3.14159265358979323846f * inv_rc * sn * cs;
}

// Arithmetic of the one-wavefront kernels per precision.  float: hardware approximations (v_exp_f32,
// v_rcp_f32, v_sqrt_f32, minimax cutoff), good to a few 1e-7 relative; double: correctly rounded library
// routines, as the 1e-12 tolerance of the double-precision path needs.
template <typename T> struct Fast;
template <> struct Fast<float> {
    typedef float4 vec4;
    typedef float2 vec2;
    static __device__ __forceinline__ float4 make4(float a, float b, float c, float d) { return make_float4(a, b, c, d); }
    static __device__ __forceinline__ float2 make2(float a, float b) { return make_float2(a, b); }
    static __device__ __forceinline__ float sqrt_(float x) { return __builtin_amdgcn_sqrtf(x); }
    // Square root to half an ulp (the distances: their rounding is what limits the float results) without the
    // library routine's scaling for denormals and its two trial roundings: the hardware's reciprocal square root
    // (1 ulp) and one Newton step, whose fused residual x - s^2 is exact.  The reciprocal is capped so that
    // x = 0 gives 0 and not 0 * inf.  6 instructions instead of 14.
    static __device__ __forceinline__ float sqrt_rn(float x)
    {
        const float y = fminf(__builtin_amdgcn_rsqf(x), 1.0e18f);
        const float s = x * y;
        const float e = fmaf(-s, s, x);
        return fmaf(e, 0.5f * y, s);
    }
    static __device__ __forceinline__ float rcp(float x) { return __builtin_amdgcn_rcpf(x); }
    // exp(-eta d^2)
    static __device__ __forceinline__ float gauss(float eta, float d) { return __builtin_amdgcn_exp2f((-eta * 1.44269504088896340736f) * d * d); }
    static __device__ __forceinline__ float cutoff(float r, float rc) { return cutoff_poly(r * (1.0f / rc)); }
    static __device__ __forceinline__ void cutoff_grad(float r, float rc, float& fc, float& dfc)
    {
        cutoff_poly_grad(r * (1.0f / rc), 1.0f / rc, fc, dfc);
    }
};
// double-precision building blocks without library calls: the library's sqrt, division, cos and sin spend most of their
// instructions on range reduction and special cases that cannot occur for distances of the order of an angstrom.
// r = sqrt(x) and 1/r for x > 0: v_rsq_f64 is good to 5e-8; one coupled Goldschmidt step (g -> sqrt, h -> 1/(2 sqrt))
// squares that, the fused residual x - g^2 is exact and brings g to half an ulp, and one Newton step on the reciprocal
// of that g gives 1/r to an ulp (measured against long double on 2^20 arguments: 1.1e-16 and 2.1e-16).  x = 0 -> 0, 0.
__device__ __forceinline__ void sqrt_and_rcp(double x0, double& r, double& inv)
{
    const double x = fmax(x0, 1e-300);
    const double y = __builtin_amdgcn_rsq(x);
    double g = x * y, h = 0.5 * y;
    const double e = fma(-h, g, 0.5);
    g = fma(g, e, g);
    h = fma(h, e, h);
    g = fma(fma(-g, g, x), h, g);
    double v = h + h;
    v = fma(v, fma(-g, v, 1.0), v);
    r = x0 > 0.0 ? g : 0.0;
    inv = x0 > 0.0 ? v : 0.0;
}
// 1/x for x of ordinary size: v_rcp_f64 and two Newton steps (no scaling, no fix-up of special cases)
__device__ __forceinline__ double rcp_newton(double x)
{
    double v = __builtin_amdgcn_rcp(x);
    v = fma(v, fma(-x, v, 1.0), v);
    v = fma(v, fma(-x, v, 1.0), v);
    return v;
}
// sin(y) and cos(y) for y in [0, pi/2] (for other y: finite values without meaning): y is folded onto [0, pi/4], where
// the Taylor polynomials to w^15 and w^16 are exact to 5e-17 and 2e-18
__device__ __forceinline__ void sincos_quarter(double y, double& sn, double& cs)
{
    const bool fold = y > 0.25 * kPi;
    const double w = fold ? 0.5 * kPi - y : y;
    const double w2 = w * w;
    double ps = -1.0 / 1307674368000.0;
    ps = fma(ps, w2, 1.0 / 6227020800.0);
    ps = fma(ps, w2, -1.0 / 39916800.0);
    ps = fma(ps, w2, 1.0 / 362880.0);
    ps = fma(ps, w2, -1.0 / 5040.0);
    ps = fma(ps, w2, 1.0 / 120.0);
    ps = fma(ps, w2, -1.0 / 6.0);
    const double sw = fma(ps * w2, w, w);
    double pc = 1.0 / 20922789888000.0;
    pc = fma(pc, w2, -1.0 / 87178291200.0);
    pc = fma(pc, w2, 1.0 / 479001600.0);
    pc = fma(pc, w2, -1.0 / 3628800.0);
    pc = fma(pc, w2, 1.0 / 40320.0);
    pc = fma(pc, w2, -1.0 / 720.0);
    pc = fma(pc, w2, 1.0 / 24.0);
    pc = fma(pc, w2, -0.5);
    const double cw = fma(pc, w2, 1.0);
    sn = fold ? cw : sw;
    cs = fold ? sw : cw;
}

template <> struct Fast<double> {
    typedef double4 vec4;
    typedef double2 vec2;
    static __device__ __forceinline__ double4 make4(double a, double b, double c, double d) { return make_double4(a, b, c, d); }
    static __device__ __forceinline__ double2 make2(double a, double b) { return make_double2(a, b); }
    static __device__ __forceinline__ double sqrt_(double x)
    {
        double r, inv;
        sqrt_and_rcp(x, r, inv);
        return r;
    }
    static __device__ __forceinline__ double rcp(double x) { return rcp_newton(x); }
    static __device__ __forceinline__ double sqrt_rn(double x) { return sqrt_(x); }
    static __device__ __forceinline__ double gauss(double eta, double d) { return exp(-eta * d * d); }
    // f_C = 0.5 cos(pi r / rc) + 0.5 = cos^2(y), f_C' = -(pi / rc) sin(y) cos(y), y = pi r / (2 rc) in [0, pi/2] for r <= rc
    // the same from the library's cos and sin: three times the instructions, but no table of fifteen double constants
    // kept in registers across the kernel (a kernel at its register limit takes this one)
    static __device__ __forceinline__ void cutoff_grad_library(double r, double rc, double& fc, double& dfc)
    {
        const double w = kPi / rc;
        fc = 0.5 * cos(w * r) + 0.5;
        dfc = -0.5 * w * sin(w * r);
    }
    static __device__ __forceinline__ double cutoff(double r, double rc)
    {
        double sn, cs;
        sincos_quarter((kPi / (2.0 * rc)) * r, sn, cs);
        return cs * cs;
    }
    static __device__ __forceinline__ void cutoff_grad(double r, double rc, double& fc, double& dfc)
    {
        double sn, cs;
        sincos_quarter((kPi / (2.0 * rc)) * r, sn, cs);
        fc = cs * cs;
        dfc = (-kPi / rc) * sn * cs;
    }
};
// f_C and f_C' in the form a kernel asks for: `kLibrary` (double only) takes Fast<double>::cutoff_grad_library
template <typename T, bool kLibrary> __device__ __forceinline__ void cutoff_grad_as(T r, T rc, T& fc, T& dfc)
{
    if constexpr (kLibrary && sizeof(T) == 8) Fast<T>::cutoff_grad_library(r, rc, fc, dfc);
    else Fast<T>::cutoff_grad(r, rc, fc, dfc);
}

}  // namespace khan

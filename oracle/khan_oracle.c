/* TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement of the ANI-1 featurization path of proteneer/khan, used solely as the checker
 * for the HIP library (tests/, the smoke check, and the cpu_baseline leg of bench.py).  Nothing in
 * the product library links, loads or calls this file.
 *
 * What follows which reference lines:
 *   parameters              gpu_featurizer/parameters.h:10,61-114  (all `const float`, widened on use)
 *   pair_block / linearize  gpu_featurizer/kernel_cpu.cpp:9-23
 *   dist_diff, f_C          gpu_featurizer/kernel_cpu.cpp:25-35
 *   khan_oracle_featurize_* gpu_featurizer/kernel_cpu.cpp:406-537 + functor_op_cpu.cpp:31-38
 *   khan_oracle_featurize_grad_*  gpu_featurizer/kernel_cpu.cpp:217-366 + functor_op_cpu.cpp:68-78
 *                                 (reduced-form derivative, see aev_real.inc)
 *   khan_oracle_featurize_grad_inverse_*  the contraction meant by gpu_featurizer/kernel_cpu.cpp:37-179
 *                                 (indexed by atom; the reference indexes by atomic number, see aev_real.inc)
 *   khan_oracle_ani_sort    gpu_featurizer/ani_sort.cpp:71-115
 *   khan_oracle_mol_offsets khan/training/trainer_multi_tower.py:302-303 (segment_sum + exclusive cumsum)
 *   khan_oracle_ani_charge* gpu_featurizer/ani_charges.cpp:58-71, 138-160
 *
 * Pinning status (each check lives under tests/):
 *   ani_sort          reference KATs (test_kernel.py:310-312, test_nn.py:95), brute-force rank count
 *   mol_offsets       reference fixture (test_kernel.py:300-301 on mol_idxs of the 11-atom case), numpy
 *   featurize f32/f64 bit-compared with the compiled reference (oracle/_ref) where that is built;
 *                     committed golden vectors written from it; brute-force closed form
 *   featurize_grad    f64 compared with the compiled reference; central differences; invariants
 *   featurize_grad_inverse  adjoint identity <u, Jv> = <J^T u, v> against featurize_grad, central
 *                     differences of the forward, the reference's zero result for a uniform vector
 *   ani_charge, ani_charge_grad   closed form / brute force in long double, Euler identity, FD in q.
 *                     The reference holds no value KAT for charges (test_charges.py has no asserts).
 *   ani_charge_grad_xyz  no reference counterpart: pinned by finite differences only.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define KHAN_NUM_R_RS 16
#define KHAN_NUM_A_THETAS 8
#define KHAN_NUM_A_RS 4
#define KHAN_RADIAL 64
#define KHAN_FEATS 384

/* parameters.h:10,61-114 -- float-typed on purpose: the double path widens these rounded values */
static const float CHARGE_CONSTANT = 0.529176917f;
static const float R_eta = 16.0f;
static const float R_Rc = 4.6f;
static const float A_Rc = 3.1f;
static const float A_eta = 6.0f;
static const float A_zeta = 8.0f;
static const float R_Rs[KHAN_NUM_R_RS] = {
    5.0000000e-01f, 7.5625000e-01f, 1.0125000e+00f, 1.2687500e+00f, 1.5250000e+00f, 1.7812500e+00f,
    2.0375000e+00f, 2.2937500e+00f, 2.5500000e+00f, 2.8062500e+00f, 3.0625000e+00f, 3.3187500e+00f,
    3.5750000e+00f, 3.8312500e+00f, 4.0875000e+00f, 4.3437500e+00f};
static const float A_thetas[KHAN_NUM_A_THETAS] = {
    0.0000000e+00f, 7.8539816e-01f, 1.5707963e+00f, 2.3561945e+00f,
    3.1415927e+00f, 3.9269908e+00f, 4.7123890e+00f, 5.4977871e+00f};
static const float A_Rs[KHAN_NUM_A_RS] = {5.0000000e-01f, 1.1500000e+00f, 1.8000000e+00f, 2.4500000e+00f};

/* kernel_cpu.cpp:439-447 -- any type other than 0,1,2 lands in the O bucket */
static inline int bucket_of(int32_t t) { return (t == 0) ? 0 : (t == 1) ? 1 : (t == 2) ? 2 : 3; }

/* kernel_cpu.cpp:9-23 with k=l=0 and the K*L=32 factor taken out: HH0 HC1 HN2 HO3 CC4 CN5 CO6 NN7 NO8 OO9 */
static inline int pair_block(int a, int b)
{
    if (b < a) { int t = a; a = b; b = t; }
    return 4 * 3 / 2 - (4 - a) * (4 - a - 1) / 2 + b;
}

static inline double dist_diff(double dx, double dy, double dz) { return sqrt(dx * dx + dy * dy + dz * dz); }

static inline double f_C(double r, double rc) { return (r <= rc) ? 0.5 * cos((M_PI * r) / rc) + 0.5 : 0.0; }

int khan_oracle_pair_block(int a, int b) { return pair_block(a, b); }

/* ---- ani_sort.cpp:71-115 -------------------------------------------------------------------
 * atom_counts[t] = #{A==t}; scatter_idxs[g] = rank of g among atoms of its own type (:95-100);
 * gather_idxs[g] = position of g under a stable sort by type (:102-113)
 *                = sum_{t<A[g]} atom_counts[t] + scatter_idxs[g].
 * Types must be 0..3 (the reference indexes atom_counts[type] unchecked). Returns -1 otherwise. */
int khan_oracle_ani_sort(const int32_t *A, int64_t n, int32_t *scatter, int32_t *gather, int32_t *counts)
{
    counts[0] = counts[1] = counts[2] = counts[3] = 0;
    for (int64_t g = 0; g < n; ++g) {
        if (A[g] < 0 || A[g] > 3) return -1;
        scatter[g] = counts[A[g]]++;
    }
    int32_t base[4] = {0, counts[0], counts[0] + counts[1], counts[0] + counts[1] + counts[2]};
    for (int64_t g = 0; g < n; ++g) gather[g] = base[A[g]] + scatter[g];
    return 0;
}

/* trainer_multi_tower.py:302-303: mol_atom_counts = segment_sum(ones_like(m), m);
 * mol_offsets = cumsum(mol_atom_counts, exclusive=True).  mol_idxs must be sorted ascending. */
int khan_oracle_mol_offsets(const int32_t *mol_idxs, int64_t n, int32_t n_mols, int32_t *MACs, int32_t *MOs)
{
    for (int32_t m = 0; m < n_mols; ++m) MACs[m] = 0;
    for (int64_t g = 0; g < n; ++g) {
        if (mol_idxs[g] < 0 || mol_idxs[g] >= n_mols) return -1;
        if (g > 0 && mol_idxs[g] < mol_idxs[g - 1]) return -2;
        MACs[mol_idxs[g]] += 1;
    }
    int32_t run = 0;
    for (int32_t m = 0; m < n_mols; ++m) { MOs[m] = run; run += MACs[m]; }
    return 0;
}

/* parameter tables for tests that restate the closed form independently */
void khan_oracle_params(float *r_rs16, float *a_thetas8, float *a_rs4, float *scalars6)
{
    memcpy(r_rs16, R_Rs, sizeof R_Rs);
    memcpy(a_thetas8, A_thetas, sizeof A_thetas);
    memcpy(a_rs4, A_Rs, sizeof A_Rs);
    scalars6[0] = R_eta; scalars6[1] = R_Rc; scalars6[2] = A_Rc;
    scalars6[3] = A_eta; scalars6[4] = A_zeta; scalars6[5] = CHARGE_CONSTANT;
}

#define REAL float
#define FN(name) name##_f32
#define TRIG_ACOS acosf
#define TRIG_COS cosf
#define POW_ZETA powf
#include "aev_real.inc"
#undef REAL
#undef FN
#undef TRIG_ACOS
#undef TRIG_COS
#undef POW_ZETA

#define REAL double
#define FN(name) name##_f64
#define TRIG_ACOS acos
#define TRIG_COS cos
#define POW_ZETA pow
#include "aev_real.inc"

/* khan_aev.h -- C ABI of libkhan_aev.so: the ANI-1 featurization path of proteneer/khan on one
 * AMD MI355X (gfx950).
 *
 * Each entry point replaces one TensorFlow custom op of the reference's ani.so.  Arguments keep the
 * reference's order, meaning and layout: every tensor is a flat, contiguous, rank-1 array; float
 * tensors are float32 (_f32) or float64 (_f64); every index tensor is int32.  All pointers are
 * DEVICE pointers unless the name ends in _host.  Work is enqueued on `stream` (a hipStream_t passed
 * as void*; NULL is the default stream) and the call returns without synchronising.  The library
 * keeps no state between calls, never frees or retains caller memory, and writes every element of
 * every output (outputs need not be zeroed by the caller), provided that the molecules cover every
 * atom: sum(macs) = number of atoms.  Rows and gradients of atoms that belong to no molecule are left
 * untouched, except in a batch with atoms and no molecule at all (n_mols = 0), whose outputs are
 * zeros, as in the reference (functor_op_cpu.cpp:31-38, 68-72).
 *
 * Device memory: ordinary (coarse-grained) allocations from hipMalloc / a framework's allocator.  By default the
 * gradient kernels for molecules of more than 32 atoms (float32; 64 in float64) add to x/y/z_grads
 * with hardware floating-point atomics, which fine-grained or host-coherent memory does not support
 * (the adds would be lost), and whose order varies: those gradients differ from run to run in the
 * last bits.  Everything else is bit-reproducible, and after khan_set_reproducible_gradients(1) so are the
 * gradients of every molecule of up to 256 atoms.
 *
 * Return value: KHAN_OK, or a KHAN_ERR_* code; khan_status_string() describes it.  Nothing here
 * calls exit().  An empty batch (0 atoms, 0 molecules) is a successful no-op: the reference trainer
 * feeds such batches (khan/training/trainer_multi_tower.py:795-817).
 *
 * Atom types are 0=H 1=C 2=N 3=O.  As in the reference (kernel_cpu.cpp:439-447) any other value is
 * treated as O.
 */
#ifndef KHAN_AEV_H_
#define KHAN_AEV_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KHAN_OK 0
#define KHAN_ERR_INVALID_ARG 1   /* null pointer with non-empty input, negative size */
#define KHAN_ERR_HIP 2           /* a HIP runtime call or kernel launch failed */
#define KHAN_ERR_TOO_LARGE 3     /* size exceeds what int32 indices can address */

typedef void *khan_stream_t;     /* hipStream_t */

/* Width of one atomic-environment vector: 64 radial + 320 angular = 384.
 * Replaces the `feature_size` attr of the Featurize op (gpu_featurizer/ani_op.cpp:108). */
int32_t khan_feature_size(void);

const char *khan_status_string(int status);

/* Text of the last HIP error seen by the calling thread inside this library ("" if none). */
const char *khan_last_hip_error(void);

/* Reproducible gradients (process-wide setting, default 0; returns the previous value; no reference counterpart:
 * the reference's gradient runs on the CPU in a fixed order, kernel_cpu.cpp:217-366).  With 1, khan_featurize_grad_*
 * sums the forces of molecules of 33..256 atoms (float32; 65..256 in float64) in on-chip memory in a fixed order and
 * stores every gradient once: the same bits on every run, no atomics, and no requirement on the kind of memory the
 * gradient arrays live in.  Costs 11 % of that kernel's speed in float32 (it runs three workgroups per CU instead
 * of four) and more in float64 (one instead of two).  Not covered: molecules of more than 256 atoms, centres with more than 64
 * partners inside the angular cutoff, and upstream buckets that are not 16-byte aligned (the general kernels, atomics). */
int khan_set_reproducible_gradients(int on);

/* Featurization parameters for introspection (gpu_featurizer/parameters.h:61-114), host arrays:
 * r_rs[16], a_thetas[8], a_rs[4], scalars[6] = {R_eta, R_Rc, A_Rc, A_eta, A_zeta, CHARGE_CONSTANT}. */
void khan_get_parameters(float *r_rs_host, float *a_thetas_host, float *a_rs_host, float *scalars_host);

/* mol_atom_counts = segment_sum(ones_like(mol_idxs), mol_idxs); mol_offsets = cumsum(exclusive).
 * Replaces the two TensorFlow ops the reference trainer runs before AniSort
 * (khan/training/trainer_multi_tower.py:302-303; gpu_featurizer/test_kernel.py:300-301).
 * mol_idxs[n_atoms] must be sorted ascending with values in [0, n_mols). Outputs: macs[n_mols], mos[n_mols]. */
int khan_mol_offsets(const int32_t *mol_idxs, int64_t n_atoms, int32_t n_mols, int32_t *macs,
                     int32_t *mos, khan_stream_t stream);

/* AniSort (gpu_featurizer/ani_sort.cpp:27-31 registration, 71-115 Compute).
 * in : atomic_numbers[n_atoms]
 * out: scatter_idxs[n_atoms]  rank of each atom among atoms of its own type
 *      gather_idxs[n_atoms]   position of each atom under a stable sort by type
 *      atom_counts[4]         atoms per type (DEVICE memory here; the reference op is host-only)
 * Bit-identical to the reference's host algorithm. Allocates a small stream-ordered workspace. */
int khan_ani_sort(const int32_t *atomic_numbers, int64_t n_atoms, int32_t *scatter_idxs,
                  int32_t *gather_idxs, int32_t *atom_counts, khan_stream_t stream);

/* Featurize (op: gpu_featurizer/ani_op.cpp:95-117; functor: functor_op.h:8-25, functor_op_gpu.cu:57-88;
 * kernel: kernel_cpu.cpp:406-537 / kernel.cu:72-268).
 * in : xs, ys, zs [n_atoms]; as [n_atoms]; mos, macs [n_mols]; sis = scatter_idxs [n_atoms];
 *      acs_host[4] = atom_counts in HOST memory (the reference declares it HostMemory, ani_op.cpp:333)
 * out: h_feat[acs[0]*384], c_feat[acs[1]*384], n_feat[acs[2]*384], o_feat[acs[3]*384], row-major;
 *      the row of atom g is bucket[as[g]] + sis[g]*384.
 * Scratch, from the stream-ordered allocator on every call: the molecule indices in order of decreasing size, and,
 * for molecules of more than 256 atoms, a sorted copy of the atoms (about 25 bytes per atom and 48 per molecule of the batch in float32, 41 per atom in
 * float64).  While the stream is being captured into a graph neither is taken: molecules then run in the order given,
 * and those of more than 256 atoms in slower kernels that need no scratch.
 * Precondition for batches with molecules of more than 256 atoms: mos increases with the molecule index and the
 * molecules do not overlap (mos[m+1] >= mos[m] + macs[m], as the exclusive prefix sum of macs gives).  The sorted copy
 * keeps a molecule's boxes at a place derived from its offset and its index; with permuted offsets two such molecules
 * could share box entries and their features would be wrong (every access stays in bounds).  Molecules of up to 256
 * atoms accept any offsets, as the reference's kernels do. */
int khan_featurize_f32(const float *xs, const float *ys, const float *zs, const int32_t *as,
                       const int32_t *mos, const int32_t *macs, int32_t n_mols, const int32_t *sis,
                       float *h_feat, float *c_feat, float *n_feat, float *o_feat,
                       const int32_t *acs_host, khan_stream_t stream);
int khan_featurize_f64(const double *xs, const double *ys, const double *zs, const int32_t *as,
                       const int32_t *mos, const int32_t *macs, int32_t n_mols, const int32_t *sis,
                       double *h_feat, double *c_feat, double *n_feat, double *o_feat,
                       const int32_t *acs_host, khan_stream_t stream);

/* khan_featurize_f32 for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments,
 * same results.  khan_featurize_f32 takes its scratch buffer (the molecule indices in order of decreasing
 * size, one int per molecule + 520) from the stream-ordered allocator on every call; this one keeps it in a
 * fixed array inside the library's code object (4.2 MB per GPU, held until the process ends) and calls no
 * hipMalloc, hipFree or other allocating routine.  More than KHAN_FEATURIZE_NOALLOC_MAX_MOLS molecules:
 * KHAN_ERR_TOO_LARGE, nothing launched.  Every call on a GPU uses that GPU's one array: calls that overlap
 * on one GPU (two streams, two threads) race; calls on one stream are ordered and safe.  The first call on
 * a device looks the array's address up (hipGetSymbolAddress); make that call outside graph capture.
 * Molecules of more than 256 atoms run in the kernels that need no scratch (slower than khan_featurize_f32's). */
#define KHAN_FEATURIZE_NOALLOC_MAX_MOLS (1 << 20)
int khan_featurize_f32_noalloc(const float *xs, const float *ys, const float *zs, const int32_t *as,
                               const int32_t *mos, const int32_t *macs, int32_t n_mols,
                               const int32_t *sis, float *h_feat, float *c_feat, float *n_feat,
                               float *o_feat, const int32_t *acs_host, khan_stream_t stream);

/* FeaturizeGrad (op: gpu_featurizer/ani_op.cpp:200-221; functor: functor_op.h:27-47,
 * functor_op_cpu.cpp:46-83; kernel: kernel_cpu.cpp:217-366 -- CPU-only in the reference).
 * in : the Featurize inputs, then the upstream gradients h_grads..o_grads laid out like its outputs
 * out: x_grads, y_grads, z_grads [sum(acs_host)] in original atom order. */
int khan_featurize_grad_f32(const float *xs, const float *ys, const float *zs, const int32_t *as,
                            const int32_t *mos, const int32_t *macs, int32_t n_mols,
                            const int32_t *sis, const float *h_grads, const float *c_grads,
                            const float *n_grads, const float *o_grads, float *x_grads,
                            float *y_grads, float *z_grads, const int32_t *acs_host,
                            khan_stream_t stream);
int khan_featurize_grad_f64(const double *xs, const double *ys, const double *zs, const int32_t *as,
                            const int32_t *mos, const int32_t *macs, int32_t n_mols,
                            const int32_t *sis, const double *h_grads, const double *c_grads,
                            const double *n_grads, const double *o_grads, double *x_grads,
                            double *y_grads, double *z_grads, const int32_t *acs_host,
                            khan_stream_t stream);

/* FeaturizeGradInverse (op: gpu_featurizer/ani_op.cpp:309-343; functor: functor_op.h:50-69,
 * functor_op_cpu.cpp:86-121; kernel: kernel_cpu.cpp:37-179 -- CPU-only in the reference; it is the
 * gradient of FeaturizeGrad with respect to its upstream gradients, trainer_multi_tower.py:64-91).
 * in : the Featurize inputs, then x_grads, y_grads, z_grads [sum(acs_host)]: one vector per atom
 * out: h..o laid out like the Featurize outputs: row_i[f] = sum_a dAEV_i[f]/dxyz_a . (x,y,z)_grads[a].
 * The reference routine reads the incoming vectors by the centre's atomic number instead of by atom
 * (kernel_cpu.cpp:111, 118, 155, 162, 169), which makes its result zero for every input; this entry
 * point computes the contraction that the gradient wiring means, indexed by atom. */
int khan_featurize_grad_inverse_f32(const float *xs, const float *ys, const float *zs,
                                    const int32_t *as, const int32_t *mos, const int32_t *macs,
                                    int32_t n_mols, const int32_t *sis, const float *x_grads,
                                    const float *y_grads, const float *z_grads, float *h_grads,
                                    float *c_grads, float *n_grads, float *o_grads,
                                    const int32_t *acs_host, khan_stream_t stream);
int khan_featurize_grad_inverse_f64(const double *xs, const double *ys, const double *zs,
                                    const int32_t *as, const int32_t *mos, const int32_t *macs,
                                    int32_t n_mols, const int32_t *sis, const double *x_grads,
                                    const double *y_grads, const double *z_grads, double *h_grads,
                                    double *c_grads, double *n_grads, double *o_grads,
                                    const int32_t *acs_host, khan_stream_t stream);

/* Size order of a batch, computed once and shared by the passes.  No reference counterpart (the reference's
 * CUDA grid takes the molecules as they come, functor_op_gpu.cu:82-85).  The AEV kernels start the largest
 * molecules first; every khan_featurize* / khan_featurize_grad* call above works this order out for itself in a
 * stream-ordered scratch allocation (and goes without it while its stream is being captured into a graph).
 * khan_size_order writes it into caller memory instead -- order[n_mols + KHAN_SIZE_ORDER_EXTRA] int32, device:
 * the molecule indices by decreasing atom count, then per-size counts, and in its last four elements the number
 * of molecules of up to 32 atoms, of 33..64, of 65..256 and of more -- and the *_ordered entry points take it as
 * an argument: the same results bit for bit, one order per batch instead of one per call, no allocation (but for
 * the stream-ordered scratch of molecules of more than 256 atoms, see below), and usable under graph capture.  `order` may be NULL (molecules are then taken in batch order).
 * size_classes_host (HOST memory, may be NULL) is a copy of those last four elements: a caller that brings them
 * to the host anyway -- as it does the four atom counts of khan_ani_sort -- spares every pass the launches of
 * the kernels whose size class is empty in this batch (with NULL every kernel is launched and leaves by itself). */
#define KHAN_SIZE_ORDER_EXTRA 520
int khan_size_order(const int32_t *macs, int32_t n_mols, int32_t *order, khan_stream_t stream);
int khan_featurize_ordered_f32(const float *xs, const float *ys, const float *zs, const int32_t *as,
                               const int32_t *mos, const int32_t *macs, int32_t n_mols,
                               const int32_t *sis, float *h_feat, float *c_feat, float *n_feat,
                               float *o_feat, const int32_t *acs_host, const int32_t *order,
                               const int32_t *size_classes_host, khan_stream_t stream);
int khan_featurize_ordered_f64(const double *xs, const double *ys, const double *zs, const int32_t *as,
                               const int32_t *mos, const int32_t *macs, int32_t n_mols,
                               const int32_t *sis, double *h_feat, double *c_feat, double *n_feat,
                               double *o_feat, const int32_t *acs_host, const int32_t *order,
                               const int32_t *size_classes_host, khan_stream_t stream);
int khan_featurize_grad_ordered_f32(const float *xs, const float *ys, const float *zs,
                                    const int32_t *as, const int32_t *mos, const int32_t *macs,
                                    int32_t n_mols, const int32_t *sis, const float *h_grads,
                                    const float *c_grads, const float *n_grads, const float *o_grads,
                                    float *x_grads, float *y_grads, float *z_grads,
                                    const int32_t *acs_host, const int32_t *order,
                                    const int32_t *size_classes_host, khan_stream_t stream);
int khan_featurize_grad_ordered_f64(const double *xs, const double *ys, const double *zs,
                                    const int32_t *as, const int32_t *mos, const int32_t *macs,
                                    int32_t n_mols, const int32_t *sis, const double *h_grads,
                                    const double *c_grads, const double *n_grads, const double *o_grads,
                                    double *x_grads, double *y_grads, double *z_grads,
                                    const int32_t *acs_host, const int32_t *order,
                                    const int32_t *size_classes_host, khan_stream_t stream);
int khan_featurize_grad_inverse_ordered_f32(const float *xs, const float *ys, const float *zs,
                                            const int32_t *as, const int32_t *mos, const int32_t *macs,
                                            int32_t n_mols, const int32_t *sis, const float *x_grads,
                                            const float *y_grads, const float *z_grads, float *h_grads,
                                            float *c_grads, float *n_grads, float *o_grads,
                                            const int32_t *acs_host, const int32_t *order,
                                            const int32_t *size_classes_host, khan_stream_t stream);
int khan_featurize_grad_inverse_ordered_f64(const double *xs, const double *ys, const double *zs,
                                            const int32_t *as, const int32_t *mos, const int32_t *macs,
                                            int32_t n_mols, const int32_t *sis, const double *x_grads,
                                            const double *y_grads, const double *z_grads,
                                            double *h_grads, double *c_grads, double *n_grads,
                                            double *o_grads, const int32_t *acs_host,
                                            const int32_t *order, const int32_t *size_classes_host,
                                            khan_stream_t stream);

/* AniCharge (gpu_featurizer/ani_charges.cpp:45-52 registration, 58-71 charge_energy, 81-119 Compute;
 * CUDA twin ani_charges_gpu.cu:70-128).
 * in : xs, ys, zs, qs [n_atoms]; mos, macs [n_mols]      out: charge_energies[n_mols] */
int khan_ani_charge_f32(const float *xs, const float *ys, const float *zs, const float *qs,
                        const int32_t *mos, const int32_t *macs, int32_t n_mols,
                        float *charge_energies, khan_stream_t stream);
int khan_ani_charge_f64(const double *xs, const double *ys, const double *zs, const double *qs,
                        const int32_t *mos, const int32_t *macs, int32_t n_mols,
                        double *charge_energies, khan_stream_t stream);

/* AniChargeGrad (gpu_featurizer/ani_charges.cpp:123-131 registration, 138-160 charge_grads,
 * 170-217 Compute; CUDA twin ani_charges_gpu.cu:197-260).
 * in : the AniCharge inputs, then grads[n_mols] (upstream gradient per molecule)
 * out: q_grads[n_atoms].  Atoms not covered by any molecule are left untouched. */
int khan_ani_charge_grad_f32(const float *xs, const float *ys, const float *zs, const float *qs,
                             const int32_t *mos, const int32_t *macs, int32_t n_mols,
                             const float *grads, float *q_grads, khan_stream_t stream);
int khan_ani_charge_grad_f64(const double *xs, const double *ys, const double *zs, const double *qs,
                             const int32_t *mos, const int32_t *macs, int32_t n_mols,
                             const double *grads, double *q_grads, khan_stream_t stream);

/* Coordinate gradient of the charge energy.  No reference counterpart: the reference's registered
 * gradient returns None for xs, ys, zs (khan/training/trainer_multi_tower.py:112-119).  Same inputs
 * as AniChargeGrad; out: x_grads, y_grads, z_grads [n_atoms]; q_grads may be NULL to skip it. */
int khan_ani_charge_grad_xyz_f32(const float *xs, const float *ys, const float *zs, const float *qs,
                                 const int32_t *mos, const int32_t *macs, int32_t n_mols,
                                 const float *grads, float *q_grads, float *x_grads, float *y_grads,
                                 float *z_grads, khan_stream_t stream);
int khan_ani_charge_grad_xyz_f64(const double *xs, const double *ys, const double *zs,
                                 const double *qs, const int32_t *mos, const int32_t *macs,
                                 int32_t n_mols, const double *grads, double *q_grads,
                                 double *x_grads, double *y_grads, double *z_grads,
                                 khan_stream_t stream);

/* AniCharge and both gradients in one pass over the pairs: charge_energies[n_mols] as khan_ani_charge_* gives them
 * (not multiplied by grads) and q_grads, x_grads, y_grads, z_grads [n_atoms] as khan_ani_charge_grad_xyz_* gives them
 * (q_grads may be NULL).  No reference counterpart as one op: the reference runs AniCharge forward and AniChargeGrad on
 * the way back, each a pass of its own over the pairs (ani_charges.cpp:81-119, 170-217); a caller that knows it will
 * need the gradients (training, force evaluation) gets the energy from the same pair terms at no extra cost. */
int khan_ani_charge_all_f32(const float *xs, const float *ys, const float *zs, const float *qs,
                            const int32_t *mos, const int32_t *macs, int32_t n_mols, const float *grads,
                            float *charge_energies, float *q_grads, float *x_grads, float *y_grads,
                            float *z_grads, khan_stream_t stream);
int khan_ani_charge_all_f64(const double *xs, const double *ys, const double *zs, const double *qs,
                            const int32_t *mos, const int32_t *macs, int32_t n_mols, const double *grads,
                            double *charge_energies, double *q_grads, double *x_grads, double *y_grads,
                            double *z_grads, khan_stream_t stream);

/* First dense layer of the per-type atomic networks, right behind the featurizer (khan/model/nn.py:38-68: matmul +
 * bias + activation per atom type; activation CELU, khan/model/activations.py:63-65, or none):
 *     out_t[r, :] = act(rows_t[r, :] . W_t + b_t),  t = H, C, N, O,  one launch for the four types.
 * Every *_host4 argument is a HOST array of four DEVICE pointers: rows_t [acs[t], 384] (the featurizer's buckets,
 * 16-byte aligned), wt_t [128, 384] = the layer's [384, 128] weights TRANSPOSED (16-byte aligned), bias_t [128],
 * out_t [acs[t], 128].  float32 in, float32 accumulation on the matrix cores.  The layer width is fixed at 128
 * (the reference's default network, energy_server.py:121); khan_dense_f32 takes other widths.
 * All khan_dense_* entry points compute the float32 product to float32 accuracy.  By default the partial products
 * are formed on the bfloat16 matrix instructions, every float32 operand split exactly into three bfloat16 parts and
 * the six largest of the nine partial products accumulated in float32 (what is dropped is below 2^-23 of a product);
 * KHAN_DENSE_MATRIX=f32 in the environment (read once per process) selects the float32 matrix instructions.  With the
 * split products a non-finite input gives NaN where a float32 product would give +-inf. */
#define KHAN_ACT_NONE 0
#define KHAN_ACT_CELU 1
int khan_dense_first_f32(const float *const *rows_host4, const int32_t *acs_host,
                         const float *const *wt_host4, const float *const *bias_host4,
                         int32_t activation, float alpha, float *const *out_host4,
                         khan_stream_t stream);

/* Any dense layer of the per-type networks, forward or on the way back (khan/model/nn.py:38-68 and its gradient
 * with respect to the layer's input, which the reference leaves to TensorFlow's matmul gradient), one launch for
 * the four types:
 *     out_t[r, :] = act(in_t'[r, :] . W_t + b_t),   in_t' = in_t, or in_t .* CELU'(z) with CELU(z) = deriv_of_t.
 * in_t [n_t, k], wt_t [n_out, k] (the summed index contiguous), bias_t [n_out] or bias_host4 = NULL, deriv_of_t
 * [n_t, k] or deriv_of_host4 = NULL, out_t [n_t, n_out]; k a multiple of 32, n_out a multiple of 64; in, deriv_of and
 * wt 16-byte aligned.  Forward of a layer with weights W [k, n_out]: wt = W transposed, bias, activation.  Data
 * gradient of a layer with weights W [k_l, n_l] and CELU outputs h: in = d/dh [n_t, n_l], deriv_of = h, wt = W
 * as it is (k = n_l, n_out = k_l), no bias, no activation.  float32 in, float32 accumulation on the matrix cores. */
int khan_dense_f32(const float *const *rows_host4, const int32_t *n_host4, int32_t k, int32_t n_out,
                   const float *const *wt_host4, const float *const *bias_host4, int32_t activation,
                   float alpha, const float *const *deriv_of_host4, float *const *out_host4,
                   khan_stream_t stream);

/* The last hidden layer of the per-type networks together with the output layer behind it (khan/model/nn.py:38-68
 * with layer sizes (..., 64, 1): the output layer is a matmul to one column plus bias, no activation), one launch
 * for the four types:
 *     out_t[r, :] = act(in_t[r, :] . W_t + b_t),    head_out_t[r] = out_t[r, :] . head_w_t + head_b_t[0].
 * Arguments as khan_dense_f32, with n_out = 64; head_w_t [64], head_b_t [1] or head_b_host4 = NULL, head_out_t [n_t].
 * out_t is still written: the way back needs the activations. */
int khan_dense_head_f32(const float *const *rows_host4, const int32_t *n_host4, int32_t k, int32_t n_out,
                        const float *const *wt_host4, const float *const *bias_host4, int32_t activation,
                        float alpha, const float *const *head_w_host4, const float *const *head_b_host4,
                        float *const *out_host4, float *const *head_out_host4, khan_stream_t stream);

/* The way back through the output layer and the last hidden layer (the gradient TensorFlow derives for
 * nn.py:38-68), one launch for the four types: given scale_t[r] = d/d head_out_t[r],
 *     out_t[r, :] = (scale_t[r] head_w_t[:] .* CELU'(z)) . W_t^T,   CELU(z) = deriv_of_t (the layer's activations),
 * the gradient with respect to the last hidden layer's input.  scale_t [n_t], head_w_t [k] (16-byte aligned),
 * deriv_of_t [n_t, k], wt_t [n_out, k] = the layer's weights as stored (k = the layer's width, n_out = its input
 * width: the convention of khan_dense_f32's data gradient), out_t [n_t, n_out].  The outer product is formed in
 * registers; no [n_t, k] gradient matrix is written or read. */
int khan_dense_head_grad_f32(const float *const *scale_host4, const float *const *head_w_host4,
                             const int32_t *n_host4, int32_t k, int32_t n_out, const float *const *wt_host4,
                             float alpha, const float *const *deriv_of_host4, float *const *out_host4,
                             khan_stream_t stream);

/* The whole atomic network of the reference's default size -- 384-128-128-64-1, CELU after all layers but the last
 * (khan/model/nn.py:38-68; sizes khan/inference/energy_server.py:121) -- for the four atom types in ONE launch, and on
 * request the gradient back to the feature rows in the same launch:
 *     value_t[r] = (celu(celu(celu(rows_t[r] W1 + b1) W2 + b2) W3 + b3)) w4 + b4
 *     grad_t[r, :] = scale_t[r] * d value_t[r] / d rows_t[r, :]            (grad_host4 non-NULL)
 * A feature row is read once and its gradient written once; no activation of a hidden layer is written to memory
 * (layer by layer, khan_dense_f32 and khan_dense_head_f32 write every activation and read it twice).  It is the pass of
 * energy-and-force inference (energy_server.py:141-187): the values summed by molecule are the energies, and grad with
 * scale = 1 is what khan_featurize_grad_f32 takes as its upstream rows.
 * The products are float32 products to float32 accuracy, formed on the half-precision matrix instructions: every float32
 * operand x is split into h = half(x) and l = half(2^11 (x - h)) (x - h - 2^-11 l is at most 2^-24 |x|), and three of
 * the four partial products are accumulated in float32 (the fourth is below 2^-24 of the product).  OPERAND RANGE: a
 * feature, activation or weight of 65,504 or more in size (half precision's largest number) makes that row's value and
 * gradient NaN -- never a wrong finite number, and no other row's; an operand below 6e-5 in size keeps an absolute
 * accuracy of 2^-36 instead of a relative one (it then no longer counts beside the row's other terms).  The gradient
 * is carried through the layers for scale = 1 and multiplied by scale_t[r] when it is stored, so its accuracy does not
 * depend on the size of scale.
 *   rows_host4[t]          [n_t, 384] feature rows (the featurizer's buckets), 16-byte aligned
 *   weights_t_host12[4l+t] layer l = 0, 1, 2 of type t TRANSPOSED: [128, 384], [128, 128], [64, 128]
 *   weights_host12[4l+t]   the same layers as stored: [384, 128], [128, 128], [128, 64] (read for the gradient only;
 *                          NULL when grad_host4 is NULL)
 *   packed                 DEVICE buffer written by khan_atomic_networks_pack_f32 from the same 24 matrices, or NULL.
 *                          With it neither weights array is read (both may be NULL) and the kernel loads the weights'
 *                          two half-precision parts as they are instead of splitting the float32 weights again in every
 *                          wavefront: the same bits out, less time.  Pack once per set of weights
 *                          (khan_atomic_networks_packed_bytes() bytes, 16-byte aligned); pack again after the weights change.
 *   biases_host12[4l+t]    [128], [128], [64]
 *   head_w_host4[t] [64], head_b_host4[t] one float (head_b_host4 or an entry may be NULL: no bias)
 *   scale_host4[t]         [n_t] gradient with respect to each row's value, or NULL (the array or an entry): ones
 *   value_host4[t] [n_t];  grad_host4[t] [n_t, 384], or grad_host4 = NULL: values only
 * All are HOST arrays of DEVICE pointers; an empty type's pointers may be NULL. */
int64_t khan_atomic_networks_packed_bytes(void);
int khan_atomic_networks_pack_f32(const float *const *weights_t_host12, const float *const *weights_host12,
                                  void *packed, khan_stream_t stream);
int khan_atomic_networks_f32(const float *const *rows_host4, const int32_t *n_host4,
                             const float *const *weights_t_host12, const float *const *weights_host12,
                             const void *packed, const float *const *biases_host12, const float *const *head_w_host4,
                             const float *const *head_b_host4, const float *const *scale_host4, float alpha,
                             float *const *value_host4, float *const *grad_host4, khan_stream_t stream);

/* Per-molecule sums of the atomic networks' outputs: e[m] = sum over the atoms g of molecule m of
 * out_{as[g]}[sis[g]] -- the gather to the batch's atom order and the segment sum by molecule of the reference
 * (khan/model/nn.py:165-177; trainer_multi_tower.py:350) in one launch, without the gathered copy, each molecule's
 * sum formed in a fixed order (the same bits on every run).  out_host4: a HOST array of four DEVICE pointers, the
 * per-type vectors [acs[t]] (an empty type's pointer may be NULL); as, sis [n_atoms]; mos, macs, e [n_mols]. */
int khan_mol_energy_f32(const float *const *out_host4, const int32_t *as, const int32_t *sis, const int32_t *mos,
                        const int32_t *macs, int32_t n_mols, float *e, khan_stream_t stream);
int khan_mol_energy_f64(const double *const *out_host4, const int32_t *as, const int32_t *sis, const int32_t *mos,
                        const int32_t *macs, int32_t n_mols, double *e, khan_stream_t stream);
/* The way back: grad_t[sis[g]] = e_grads[m] for every atom g of molecule m (every element of the four vectors that
 * belongs to an atom of a molecule is written). */
int khan_mol_energy_grad_f32(const float *e_grads, const int32_t *as, const int32_t *sis, const int32_t *mos,
                             const int32_t *macs, int32_t n_mols, float *const *grad_host4, khan_stream_t stream);
int khan_mol_energy_grad_f64(const double *e_grads, const int32_t *as, const int32_t *sis, const int32_t *mos,
                             const int32_t *macs, int32_t n_mols, double *const *grad_host4, khan_stream_t stream);

/* Plain Coulomb sums, E_m = k sum_{i<j in m} q_i q_j / r_ij, and their gradients: the charge kernels with
 * the damping (1 - f_C) switched off and the constant chosen by the caller (k = 1 for charges in e and
 * distances in the unit the energy is wanted in).  No reference counterpart: khan's own op is the damped,
 * K-scaled form above (ani_charges.cpp:58-71); this is the bare sum for callers who want it.
 * khan_coulomb_grad: grads[n_mols] upstream; out q_grads[n_atoms] (may be NULL) and x/y/z_grads[n_atoms]. */
int khan_coulomb_f32(const float *xs, const float *ys, const float *zs, const float *qs,
                     const int32_t *mos, const int32_t *macs, int32_t n_mols, float k,
                     float *energies, khan_stream_t stream);
int khan_coulomb_f64(const double *xs, const double *ys, const double *zs, const double *qs,
                     const int32_t *mos, const int32_t *macs, int32_t n_mols, double k,
                     double *energies, khan_stream_t stream);
int khan_coulomb_grad_f32(const float *xs, const float *ys, const float *zs, const float *qs,
                          const int32_t *mos, const int32_t *macs, int32_t n_mols,
                          const float *grads, float k, float *q_grads, float *x_grads,
                          float *y_grads, float *z_grads, khan_stream_t stream);
int khan_coulomb_grad_f64(const double *xs, const double *ys, const double *zs, const double *qs,
                          const int32_t *mos, const int32_t *macs, int32_t n_mols,
                          const double *grads, double k, double *q_grads, double *x_grads,
                          double *y_grads, double *z_grads, khan_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* KHAN_AEV_H_ */

/* Host-side batch assembly for the featurizer: gathers the molecules of one batch out of a data set that is
 * packed once into flat arrays (all atoms end to end, plus molecule offsets) straight into the flat arrays the
 * ops take -- xs, ys, zs, atom types and the per-atom molecule index -- which may be pinned staging buffers.
 *
 * What it replaces: khan/data/dataset.py:118-183 builds each batch with np.concatenate over the batch's molecule
 * arrays and khan/training/trainer_multi_tower.py:769-779 splits the columns again; that costs a Python-level
 * operation per molecule.  Here one pass computes the batch's atom offsets and the copies run over the molecules
 * in parallel.  Plain C, no GPU code.
 */
#include <stdint.h>
#include <string.h>

#define KHAN_EXPORT __attribute__((visibility("default")))

/* out_off[k] = first atom of batch molecule k inside the batch, k = 0..n_sel (out_off[n_sel] = atoms in the batch).
 * Returns that total, or -1 if a selected index is out of range. */
KHAN_EXPORT int64_t khan_host_batch_offsets(const int64_t* mol_offsets, int64_t n_mols_total, const int64_t* sel,
                                            int64_t n_sel, int64_t* out_off)
{
    int64_t run = 0;
    for (int64_t k = 0; k < n_sel; ++k) {
        const int64_t m = sel[k];
        if (m < 0 || m >= n_mols_total) return -1;
        out_off[k] = run;
        run += mol_offsets[m + 1] - mol_offsets[m];
    }
    out_off[n_sel] = run;
    return run;
}

#define DEFINE_GATHER(NAME, T)                                                                                       \
    KHAN_EXPORT void NAME(const int64_t* mol_offsets, const int32_t* types, const T* x, const T* y, const T* z,      \
                          const int64_t* sel, int64_t n_sel, const int64_t* out_off, T* xs, T* ys, T* zs,            \
                          int32_t* as, int32_t* mol_ids, int n_threads)                                              \
    {                                                                                                                \
        _Pragma("omp parallel for schedule(static) num_threads(n_threads) if (n_sel > 256)")                        \
        for (int64_t k = 0; k < n_sel; ++k) {                                                                        \
            const int64_t src = mol_offsets[sel[k]];                                                                 \
            const int64_t cnt = mol_offsets[sel[k] + 1] - src;                                                       \
            const int64_t dst = out_off[k];                                                                          \
            memcpy(xs + dst, x + src, (size_t)cnt * sizeof(T));                                                      \
            memcpy(ys + dst, y + src, (size_t)cnt * sizeof(T));                                                      \
            memcpy(zs + dst, z + src, (size_t)cnt * sizeof(T));                                                      \
            memcpy(as + dst, types + src, (size_t)cnt * sizeof(int32_t));                                            \
            for (int64_t a = 0; a < cnt; ++a) mol_ids[dst + a] = (int32_t)k;                                         \
        }                                                                                                            \
    }

DEFINE_GATHER(khan_host_gather_f32, float)
DEFINE_GATHER(khan_host_gather_f64, double)

/* per-atom rows of width 3 (reference gradients / forces), gathered the same way */
KHAN_EXPORT void khan_host_gather_rows3_f64(const int64_t* mol_offsets, const double* rows, const int64_t* sel,
                                            int64_t n_sel, const int64_t* out_off, double* out, int n_threads)
{
#pragma omp parallel for schedule(static) num_threads(n_threads) if (n_sel > 256)
    for (int64_t k = 0; k < n_sel; ++k) {
        const int64_t src = mol_offsets[sel[k]];
        const int64_t cnt = mol_offsets[sel[k] + 1] - src;
        memcpy(out + 3 * out_off[k], rows + 3 * src, (size_t)cnt * 3 * sizeof(double));
    }
}

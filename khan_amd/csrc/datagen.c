/* Seeded synthetic batches for the featurization benchmarks and parity tests (host code, plain C).
 *
 * The reference has no generator of its own: its random tests draw unit-cube noise
 * (khan/model/test_symmetrizer.py:226-231).  The batches here follow the workload definitions
 * this package is measured on:
 *
 *  organic  1..8 heavy atoms, each C/N/O with p = 0.6/0.2/0.2, bonded as a random tree (a new heavy
 *           atom bonds to a uniformly chosen earlier heavy atom that still has free valence, C4 N3 O2)
 *           with bond length U(1.2,1.55) A in a uniform random direction; hydrogens fill the remaining
 *           valence at U(0.95,1.10) A in random directions; N(0,0.05^2) A noise on every coordinate;
 *           minimum pair distance 0.8 A enforced by rejection (a placement that lands within 0.8 A of
 *           an existing atom is redrawn; after the noise the whole molecule is redrawn if any pair is
 *           closer than 0.8 A).  Atom order: each heavy atom followed by its hydrogens, so types
 *           interleave.  3..26 atoms per molecule.  Types H0 C1 N2 O3.
 *  boxes    n ~ U{64..256} atoms in a cube of side (n/0.1)^(1/3) A (number density 0.1 / A^3), placed by
 *           dart throwing with minimum distance 0.9 A, open boundaries, types H/C/N/O with
 *           p = 0.5/0.3/0.1/0.1.  One box is one "molecule".
 *  bigboxes the same with n ~ U{1024..4096} atoms (systems of more than 256 atoms).
 *
 * Every molecule has its own random stream keyed by (seed, stream tag, molecule index), so a batch of
 * M molecules is a prefix of any larger batch made with the same seed.  Coordinates are drawn in
 * double and rounded to float; double-precision runs widen those floats, so both precisions see the
 * same geometry.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* ---- counter-keyed xoshiro256** ------------------------------------------------------------ */
typedef struct { uint64_t s[4]; int has_spare; double spare; } rng_t;

static inline uint64_t splitmix64(uint64_t *x)
{
    uint64_t z = (*x += 0x9E3779B97F4A7C15ULL);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

static void rng_seed(rng_t *g, uint64_t seed, uint64_t tag, uint64_t index)
{
    uint64_t x = seed ^ (tag * 0xD1342543DE82EF95ULL) ^ (index * 0xA0761D6478BD642FULL + 0x2545F4914F6CDD1DULL);
    for (int i = 0; i < 4; ++i) g->s[i] = splitmix64(&x);
    g->has_spare = 0;
    g->spare = 0.0;
}

static inline uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

static inline uint64_t rng_next(rng_t *g)
{
    uint64_t *s = g->s;
    const uint64_t result = rotl64(s[1] * 5, 7) * 9;
    const uint64_t t = s[1] << 17;
    s[2] ^= s[0]; s[3] ^= s[1]; s[1] ^= s[2]; s[0] ^= s[3];
    s[2] ^= t;
    s[3] = rotl64(s[3], 45);
    return result;
}

static inline double rng_uniform(rng_t *g) { return (double)(rng_next(g) >> 11) * (1.0 / 9007199254740992.0); }

static inline double rng_range(rng_t *g, double lo, double hi) { return lo + (hi - lo) * rng_uniform(g); }

static inline int rng_below(rng_t *g, int n) { return (int)(rng_uniform(g) * n); }

static double rng_normal(rng_t *g)   /* Box-Muller, both variates used */
{
    if (g->has_spare) { g->has_spare = 0; return g->spare; }
    double u1;
    do { u1 = rng_uniform(g); } while (u1 <= 0.0);
    const double u2 = rng_uniform(g);
    const double rad = sqrt(-2.0 * log(u1)), ang = 6.283185307179586476925 * u2;
    g->spare = rad * sin(ang);
    g->has_spare = 1;
    return rad * cos(ang);
}

static void rng_direction(rng_t *g, double *u)   /* uniform on the unit sphere */
{
    const double z = rng_range(g, -1.0, 1.0), phi = 6.283185307179586476925 * rng_uniform(g);
    const double s = sqrt(fmax(0.0, 1.0 - z * z));
    u[0] = s * cos(phi); u[1] = s * sin(phi); u[2] = z;
}

#define MAX_ORGANIC_ATOMS 26
#define TAG_ORGANIC 1ULL
#define TAG_BOX 2ULL
#define TAG_BIGBOX 3ULL
#define MAX_MOL_ATOMS 4096

static int too_close(const double (*p)[3], int n, const double *q, double dmin)
{
    for (int a = 0; a < n; ++a) {
        const double dx = p[a][0] - q[0], dy = p[a][1] - q[1], dz = p[a][2] - q[2];
        if (dx * dx + dy * dy + dz * dz < dmin * dmin) return 1;
    }
    return 0;
}

/* one organic molecule; returns its atom count and fills type[], pos[][3] (atom order as documented) */
static int organic_molecule(rng_t *g, int32_t *type, double (*pos)[3])
{
    static const int valence[4] = {1, 4, 3, 2};
    for (;;) {
        const int h = 1 + rng_below(g, 8);
        int htype[8], hdeg[8], parent[8];
        double hpos[8][3], placed[MAX_ORGANIC_ATOMS][3];
        int n_placed = 0, ok = 1;
        for (int a = 0; a < h; ++a) {
            const double u = rng_uniform(g);
            htype[a] = (u < 0.6) ? 1 : (u < 0.8) ? 2 : 3;
            hdeg[a] = 0;
            parent[a] = -1;
        }
        hpos[0][0] = hpos[0][1] = hpos[0][2] = 0.0;
        memcpy(placed[n_placed++], hpos[0], sizeof hpos[0]);
        for (int a = 1; a < h && ok; ++a) {
            int cand[8], nc = 0;
            for (int b = 0; b < a; ++b)
                if (hdeg[b] < valence[htype[b]]) cand[nc++] = b;
            const int p = cand[rng_below(g, nc)];
            parent[a] = p;
            hdeg[p]++; hdeg[a]++;
            int tries = 0;
            do {
                double u[3];
                const double L = rng_range(g, 1.2, 1.55);
                rng_direction(g, u);
                for (int c = 0; c < 3; ++c) hpos[a][c] = hpos[p][c] + L * u[c];
            } while (too_close((const double(*)[3])placed, n_placed, hpos[a], 0.8) && ++tries < 64);
            if (tries >= 64) ok = 0;
            memcpy(placed[n_placed++], hpos[a], sizeof hpos[a]);
        }
        if (!ok) continue;
        (void)parent;
        /* hydrogens, remembered per heavy atom so the output order can interleave them */
        double hyd[8][4][3];
        int nhyd[8];
        for (int a = 0; a < h && ok; ++a) {
            nhyd[a] = valence[htype[a]] - hdeg[a];
            for (int b = 0; b < nhyd[a] && ok; ++b) {
                int tries = 0;
                do {
                    double u[3];
                    const double L = rng_range(g, 0.95, 1.10);
                    rng_direction(g, u);
                    for (int c = 0; c < 3; ++c) hyd[a][b][c] = hpos[a][c] + L * u[c];
                } while (too_close((const double(*)[3])placed, n_placed, hyd[a][b], 0.8) && ++tries < 64);
                if (tries >= 64) ok = 0;
                memcpy(placed[n_placed++], hyd[a][b], sizeof hyd[a][b]);
            }
        }
        if (!ok) continue;
        int n = 0;
        for (int a = 0; a < h; ++a) {
            type[n] = htype[a];
            memcpy(pos[n++], hpos[a], sizeof hpos[a]);
            for (int b = 0; b < nhyd[a]; ++b) {
                type[n] = 0;
                memcpy(pos[n++], hyd[a][b], sizeof hyd[a][b]);
            }
        }
        for (int a = 0; a < n; ++a)
            for (int c = 0; c < 3; ++c) pos[a][c] += 0.05 * rng_normal(g);
        for (int a = 1; a < n && ok; ++a)
            if (too_close((const double(*)[3])pos, a, pos[a], 0.8)) ok = 0;
        if (ok) return n;
    }
}

static int box_molecule(rng_t *g, int32_t *type, double (*pos)[3], int n_min, int n_span)
{
    const int n = n_min + rng_below(g, n_span);
    const double side = cbrt((double)n / 0.1);
    int placed = 0;
    while (placed < n) {
        double q[3] = {side * rng_uniform(g), side * rng_uniform(g), side * rng_uniform(g)};
        if (too_close((const double(*)[3])pos, placed, q, 0.9)) continue;
        memcpy(pos[placed], q, sizeof q);
        const double u = rng_uniform(g);
        type[placed] = (u < 0.5) ? 0 : (u < 0.8) ? 1 : (u < 0.9) ? 2 : 3;
        ++placed;
    }
    return n;
}

/* Generates molecules [first_mol, first_mol+n_mols) of the batch `kind` (0 organic, 1 boxes, 2 bigboxes).
 * mol_atom_counts[n_mols] is always written.  If X is non-NULL, coordinates/types/mol_idxs of up to
 * `capacity` atoms are written too (mol_idxs counts from 0 at first_mol).  Returns the total atom
 * count, or -1 if capacity was too small, -2 for an unknown kind. */
int64_t khan_gen_batch(int32_t kind, uint64_t seed, int64_t first_mol, int64_t n_mols,
                       int32_t *mol_atom_counts, float *X, float *Y, float *Z, int32_t *A,
                       int32_t *mol_idxs, int64_t capacity)
{
    if (kind < 0 || kind > 2) return -2;
    int64_t total = 0;
    static _Thread_local int32_t type[MAX_MOL_ATOMS];
    static _Thread_local double pos[MAX_MOL_ATOMS][3];
    for (int64_t m = 0; m < n_mols; ++m) {
        rng_t g;
        rng_seed(&g, seed, kind == 0 ? TAG_ORGANIC : kind == 1 ? TAG_BOX : TAG_BIGBOX, (uint64_t)(first_mol + m));
        const int n = (kind == 0)   ? organic_molecule(&g, type, pos)
                      : (kind == 1) ? box_molecule(&g, type, pos, 64, 193)
                                    : box_molecule(&g, type, pos, 1024, 3073);
        mol_atom_counts[m] = n;
        if (X) {
            if (total + n > capacity) return -1;
            for (int a = 0; a < n; ++a) {
                X[total + a] = (float)pos[a][0];
                Y[total + a] = (float)pos[a][1];
                Z[total + a] = (float)pos[a][2];
                A[total + a] = type[a];
                mol_idxs[total + a] = (int32_t)m;
            }
        }
        total += n;
    }
    return total;
}

/* i.i.d. normal variates N(0, sigma^2), element e drawn from the stream (seed, tag, e / 1024) so that
 * any sub-range is reproducible.  Used for per-atom charges and upstream feature gradients. */
void khan_gen_normal(uint64_t seed, uint64_t tag, int64_t first, int64_t count, double sigma, float *out)
{
    const int64_t BLOCK = 1024;
    int64_t e = first;
    while (e < first + count) {
        const int64_t blk = e / BLOCK, lo = blk * BLOCK;
        rng_t g;
        rng_seed(&g, seed, 0x100ULL + tag, (uint64_t)blk);
        for (int64_t q = lo; q < lo + BLOCK && q < first + count; ++q) {
            const double v = sigma * rng_normal(&g);
            if (q >= first) out[q - first] = (float)v;
        }
        e = lo + BLOCK;
    }
}

/* Exact integer work counts of a batch, with distances evaluated the way the float32 op does
 * (float differences, r rounded to float, strict < against the float cutoffs):
 *   out[0] D   = sum_m n_m (n_m - 1)            ordered intramolecular pairs
 *   out[1] P_R = ordered pairs with r < 4.6
 *   out[2] P_A = ordered pairs with r < 3.1
 *   out[3] T   = triples (i; j<k) with r_ij, r_ik < 3.1
 *   out[4] C   = sum_m n_m (n_m - 1) / 2        unordered pairs */
void khan_gen_work_counts(const float *X, const float *Y, const float *Z, const int32_t *MOs,
                          const int32_t *MACs, int64_t n_mols, int64_t *out)
{
    const float R_Rc = 4.6f, A_Rc = 3.1f;
    int64_t D = 0, PR = 0, PA = 0, T = 0, C = 0;
    for (int64_t m = 0; m < n_mols; ++m) {
        const int64_t n = MACs[m], off = MOs[m];
        D += n * (n - 1);
        C += n * (n - 1) / 2;
        for (int64_t i = 0; i < n; ++i) {
            int64_t na = 0;
            for (int64_t j = 0; j < n; ++j) {
                if (j == i) continue;
                const float dx = X[off + i] - X[off + j], dy = Y[off + i] - Y[off + j],
                            dz = Z[off + i] - Z[off + j];
                const float r = (float)sqrt((double)dx * dx + (double)dy * dy + (double)dz * dz);
                if (r < R_Rc) ++PR;
                if (r < A_Rc) { ++PA; ++na; }
            }
            T += na * (na - 1) / 2;
        }
    }
    out[0] = D; out[1] = PR; out[2] = PA; out[3] = T; out[4] = C;
}

/*
 * CPU oracle for the permutohedral-lattice filter -- TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C restatement, for T = float and T = double, of what the reference CPU path computes
 * (src/PermutohedralLatticeCPU.h and the op-level shape logic of
 * src/LatticeFilterKernel.cpp in the reference tree).  Only tests, the smoke check and the
 * benchmark's CPU-baseline leg may use it; the HIP library never does.
 *
 * Build with:  gcc -O2 -ffp-contract=off  (no -ffast-math, no FMA contraction): the integer
 * results (rem0, rank, keys, vertex count) depend on every float operation being a single
 * correctly rounded IEEE operation, and on the three places where the reference computes in
 * double and rounds back to float (marked DOUBLE below).
 *
 * What pins each function (see tests/test_oracle.py, tests/golden/):
 *   plo_scale_factor        golden bit patterns from the reference header for pd = 1..8;
 *                           closed form (pd+1)*sqrt(2/3)/sqrt((i+1)(i+2)).
 *   plo_embed               golden elevated vectors (bit-exact); sum of coordinates ~ 0;
 *                           equality with the dense matrix product E*(pos*scale) in double.
 *   plo_simplex             golden rem0/rank (bit-exact); rem0 multiples of pd+1 summing to 0,
 *                           rank a permutation, differences ordered by rank.
 *   plo_barycentric         golden weights (bit-exact); weights >= 0 summing to 1; weighted
 *                           vertex sum reconstructs the elevated point.
 *   plo_vertex_key          golden keys (bit-exact); full key sums to 0, all coordinates
 *                           congruent to the remainder mod pd+1.
 *   hash table / M          golden vertex count and first-touch key list (bit-exact, with the
 *                           reference's growth quirk switched on, see vertex_find);
 *                           quirk off: M == number of distinct per-pixel keys by sort+unique.
 *   plo_splat/blur/slice    golden outputs forward and reverse (bit-exact with the reference
 *                           header built by oracle/Makefile); the reference's own BMP fixtures
 *                           (input.bmp -> bilateral_out_1.bmp, gray_original.bmp ->
 *                           filtered_grey.bmp) within one grey level; brute-force dense
 *                           W*B*W^T on tiny inputs; constant-in/constant-out; adjointness.
 *   plo_compute_positions   golden positions (bit-exact); closed form coord/std.
 *   plo_lattice_filter_op   the BMP fixtures above (they were produced through the op).
 */
#include "pl_oracle.h"

#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

static double now_seconds(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

#define PLO_INITIAL_CELLS ((size_t)1 << 15)
#define PLO_CAT_(a, b) a##b
#define PLO_CAT(a, b) PLO_CAT_(a, b)

/* T = float: plo_<name>, struct plo_lattice */
#define PLO_T float
#define PLO_FN(name) plo_##name
#define PLO_STATIC(name) name##_f32
#define PLO_LATTICE plo_lattice
#include "pl_oracle_impl.h"
#undef PLO_T
#undef PLO_FN
#undef PLO_STATIC
#undef PLO_LATTICE

/* T = double: plo_<name>_f64, struct plo_lattice_f64 */
#define PLO_T double
#define PLO_FN(name) plo_##name##_f64
#define PLO_STATIC(name) name##_f64
#define PLO_LATTICE plo_lattice_f64
#include "pl_oracle_impl.h"

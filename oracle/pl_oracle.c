/*
 * CPU oracle for the permutohedral-lattice filter -- TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C restatement, for T = float, of what the reference CPU path computes
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

/* ------------------------------------------------------------------------------------------
 * Per-point arithmetic
 * ---------------------------------------------------------------------------------------- */

void plo_scale_factor(int pd, float *scale) {
    /* DOUBLE: (pd+1)*sqrt(2/3) is formed in double and stored as float; each entry is
     * 1/sqrt((i+1)(i+2)) in double times that float, rounded once. */
    const float inv_std_dev = (float)((double)(pd + 1) * sqrt(2.0 / 3.0));
    for (int i = 0; i < pd; ++i) {
        const double diag = 1.0 / sqrt((double)((i + 1) * (i + 2)));
        scale[i] = (float)(diag * (double)inv_std_dev);
    }
}

void plo_embed(int pd, const float *scale, const float *position, float *elevated) {
    /* Running-sum form of the rotation onto the hyperplane x.1 = 0.  All float, unfused. */
    float running = 0.0f;
    for (int i = pd; i >= 1; --i) {
        const float c = position[i - 1] * scale[i - 1];
        const float ic = (float)i * c;
        elevated[i] = running - ic;
        running = running + c;
    }
    elevated[0] = running;
}

void plo_simplex(int pd, const float *elevated, float *rem0, short *rank) {
    const int d1 = pd + 1;
    const double inv_d1 = 1.0 / (double)d1;
    short coord_sum = 0;

    for (int i = 0; i < d1; ++i) {
        /* DOUBLE: the division by pd+1 is a double multiply by the double reciprocal. */
        const float v = (float)((double)elevated[i] * inv_d1);
        const float above = (float)(ceil((double)v) * (double)d1);
        const float below = (float)(floor((double)v) * (double)d1);
        /* strictly closer to `above` wins; a tie goes down */
        if (above - elevated[i] < elevated[i] - below)
            rem0[i] = (float)(short)above;
        else
            rem0[i] = (float)(short)below;
        coord_sum = (short)((float)coord_sum + rem0[i]);
    }
    coord_sum = (short)(coord_sum / d1);

    /* rank[i] = how many coordinates have a larger residual; ties are broken by the
     * comparison order (i < j, strict <, the later index loses the tie). */
    for (int i = 0; i < d1; ++i) rank[i] = 0;
    for (int i = 0; i < pd; ++i) {
        const float di = elevated[i] - rem0[i];
        for (int j = i + 1; j < d1; ++j) {
            const float dj = elevated[j] - rem0[j];
            if (di < dj) rank[i]++;
            else rank[j]++;
        }
    }

    /* the rounded point may be off the plane by coord_sum steps: shift ranks, wrap */
    for (int i = 0; i < d1; ++i) {
        rank[i] = (short)(rank[i] + coord_sum);
        if (rank[i] < 0) {
            rank[i] = (short)(rank[i] + d1);
            rem0[i] += (float)d1;
        } else if (rank[i] > pd) {
            rank[i] = (short)(rank[i] - d1);
            rem0[i] -= (float)d1;
        }
    }
}

void plo_barycentric(int pd, const float *elevated, const float *rem0, const short *rank,
                     float *barycentric) {
    const int d1 = pd + 1;
    const double inv_d1 = 1.0 / (double)d1;
    for (int k = 0; k < pd + 2; ++k) barycentric[k] = 0.0f;
    for (int i = 0; i < d1; ++i) {
        /* DOUBLE: float residual times the double reciprocal, rounded to float */
        const float delta = (float)((double)(elevated[i] - rem0[i]) * inv_d1);
        barycentric[pd - rank[i]] += delta;
        barycentric[pd - rank[i] + 1] -= delta;
    }
    /* DOUBLE: wrap-around term is added in double */
    barycentric[0] = (float)((double)barycentric[0] + (1.0 + (double)barycentric[pd + 1]));
}

void plo_vertex_key(int pd, const float *rem0, const short *rank, int remainder, short *key) {
    for (int i = 0; i < pd; ++i) {
        short k = (short)(rem0[i] + (float)remainder);
        if (rank[i] > pd - remainder) k = (short)(k - (pd + 1));
        key[i] = k;
    }
}

void plo_dump_simplex(int pd, int N, const float *positions, short *rem0_out, short *rank_out,
                      short *keys_out, float *bary_out, float *elevated_out) {
    const int d1 = pd + 1;
    float *scale = (float *)malloc(sizeof(float) * (size_t)pd);
    float *elevated = (float *)malloc(sizeof(float) * (size_t)d1);
    float *rem0 = (float *)malloc(sizeof(float) * (size_t)d1);
    short *rank = (short *)malloc(sizeof(short) * (size_t)d1);
    float *bary = (float *)malloc(sizeof(float) * (size_t)(pd + 2));
    plo_scale_factor(pd, scale);
    for (int n = 0; n < N; ++n) {
        plo_embed(pd, scale, positions + (size_t)n * pd, elevated);
        plo_simplex(pd, elevated, rem0, rank);
        plo_barycentric(pd, elevated, rem0, rank, bary);
        for (int i = 0; i < d1; ++i) {
            if (elevated_out) elevated_out[(size_t)n * d1 + i] = elevated[i];
            if (rem0_out) rem0_out[(size_t)n * d1 + i] = (short)rem0[i];
            if (rank_out) rank_out[(size_t)n * d1 + i] = rank[i];
            if (bary_out) bary_out[(size_t)n * d1 + i] = bary[i];
            if (keys_out) plo_vertex_key(pd, rem0, rank, i, keys_out + ((size_t)n * d1 + i) * pd);
        }
    }
    free(scale); free(elevated); free(rem0); free(rank); free(bary);
}

void plo_compute_positions(const float *reference, float *positions, int num_super_pixels,
                           int reference_channels, int n_sdims, const int *sdims,
                           float spatial_std, float feature_std) {
    const int pd = n_sdims + reference_channels;
    for (int n = 0; n < num_super_pixels; ++n) {
        float *row = positions + (size_t)n * pd;
        /* linear index -> coordinates, last spatial dimension fastest */
        int stride = 1;
        for (int s = n_sdims - 1; s >= 0; --s) {
            const int coord = (n / stride) % sdims[s];
            row[s] = (float)coord / spatial_std;
            stride *= sdims[s];
        }
        for (int c = 0; c < reference_channels; ++c)
            row[n_sdims + c] = reference[(size_t)n * reference_channels + c] / feature_std;
    }
}

/* ------------------------------------------------------------------------------------------
 * Sparse lattice: vertices are numbered in first-touch order, as the reference numbers them
 * (src/PermutohedralLatticeCPU.h:59-91).
 * ---------------------------------------------------------------------------------------- */

struct plo_lattice {
    int pd, vd, N;
    float *scale;
    /* open-addressed index: cell -> vertex id or -1 */
    int *cells;
    size_t n_cells;          /* power of two */
    short *keys;             /* vertex id -> pd shorts */
    float *values;           /* vertex id -> vd floats */
    float *scratch_values;
    size_t vertex_capacity;
    int M;
    int n_growths;
    int stale_cell_after_growth;
    int *replay_vertex;      /* N*(pd+1) */
    float *replay_weight;    /* N*(pd+1) */
    double t_splat, t_blur, t_slice;
};

#define PLO_INITIAL_CELLS ((size_t)1 << 15)

/* src/PermutohedralLatticeCPU.h:44-51 -- positional hash, base 2531011, 64-bit wrap-around.
 * The hash decides nothing about vertex numbering (first touch does) except at the moment the
 * index grows, see vertex_find below; it is restated here so that moment can be reproduced. */
static size_t key_hash(const short *key, int pd) {
    size_t h = 0;
    for (int i = 0; i < pd; ++i) {
        h += (size_t)(long long)key[i];
        h *= (size_t)2531011;
    }
    return h;
}

static void index_reset(plo_lattice *l) {
    if (l->n_cells != PLO_INITIAL_CELLS) {
        free(l->cells);
        l->n_cells = PLO_INITIAL_CELLS;
        l->cells = (int *)malloc(sizeof(int) * l->n_cells);
    }
    memset(l->cells, 0xff, sizeof(int) * l->n_cells);
    l->M = 0;
    l->n_growths = 0;
}

/* src/PermutohedralLatticeCPU.h:94-128 -- double the index; vertices are re-entered in the
 * order of the OLD cells, which fixes where colliding keys land in the new one. */
static void index_grow(plo_lattice *l) {
    const size_t old_n = l->n_cells, new_n = old_n * 2;
    int *grown = (int *)malloc(sizeof(int) * new_n);
    memset(grown, 0xff, sizeof(int) * new_n);
    for (size_t c = 0; c < old_n; ++c) {
        const int v = l->cells[c];
        if (v < 0) continue;
        size_t at = key_hash(l->keys + (size_t)v * l->pd, l->pd) % new_n;
        while (grown[at] >= 0) at = (at + 1 == new_n) ? 0 : at + 1;
        grown[at] = v;
    }
    free(l->cells);
    l->cells = grown;
    l->n_cells = new_n;
    l->n_growths++;
}

static void vertices_reserve(plo_lattice *l, size_t want) {
    if (want <= l->vertex_capacity) return;
    size_t cap = l->vertex_capacity ? l->vertex_capacity : 1024;
    while (cap < want) cap *= 2;
    l->keys = (short *)realloc(l->keys, sizeof(short) * cap * (size_t)l->pd);
    l->values = (float *)realloc(l->values, sizeof(float) * cap * (size_t)l->vd);
    l->scratch_values = (float *)realloc(l->scratch_values, sizeof(float) * cap * (size_t)l->vd);
    l->vertex_capacity = cap;
}

/* src/PermutohedralLatticeCPU.h:59-91,163-170 -- vertex id of `key`, or -1; with create != 0 a
 * missing key becomes vertex M (values zeroed).  The index doubles when it is half full, and
 * the check runs before every lookup, creating or not.
 *
 * Quirk of the reference, reproduced only when stale_cell_after_growth is set: the start cell
 * is computed BEFORE the growth check (`hash % capacity` with the old capacity), so the one
 * lookup that triggers a doubling probes from a stale cell, can miss a key that is present,
 * and then enters it a second time as a new vertex.  With the flag clear the start cell is
 * recomputed and every distinct key is exactly one vertex. */
static int vertex_find(plo_lattice *l, const short *key, int create) {
    const int pd = l->pd;
    size_t c = key_hash(key, pd) % l->n_cells;
    if ((size_t)l->M >= l->n_cells / 2 - 1) {
        index_grow(l);
        if (!l->stale_cell_after_growth) c = key_hash(key, pd) % l->n_cells;
    }
    for (;;) {
        const int v = l->cells[c];
        if (v < 0) break;
        if (memcmp(l->keys + (size_t)v * pd, key, sizeof(short) * (size_t)pd) == 0) return v;
        c = (c + 1 == l->n_cells) ? 0 : c + 1;
    }
    if (!create) return -1;
    const int v = l->M;
    vertices_reserve(l, (size_t)v + 1);
    memcpy(l->keys + (size_t)v * pd, key, sizeof(short) * (size_t)pd);
    memset(l->values + (size_t)v * l->vd, 0, sizeof(float) * (size_t)l->vd);
    l->cells[c] = v;
    l->M = v + 1;
    return v;
}

void plo_set_reference_growth_quirk(plo_lattice *l, int on) { l->stale_cell_after_growth = on; }
int plo_num_growths(const plo_lattice *l) { return l->n_growths; }

plo_lattice *plo_create(int pd, int vd, int N) {
    if (pd < 1 || vd < 2 || N < 0) return NULL;
    plo_lattice *l = (plo_lattice *)calloc(1, sizeof(plo_lattice));
    l->pd = pd; l->vd = vd; l->N = N;
    l->scale = (float *)malloc(sizeof(float) * (size_t)pd);
    plo_scale_factor(pd, l->scale);
    l->n_cells = PLO_INITIAL_CELLS;
    l->cells = (int *)malloc(sizeof(int) * l->n_cells);
    index_reset(l);
    vertices_reserve(l, 1024);
    const size_t rows = (size_t)N * (size_t)(pd + 1);
    l->replay_vertex = (int *)malloc(sizeof(int) * (rows ? rows : 1));
    l->replay_weight = (float *)malloc(sizeof(float) * (rows ? rows : 1));
    return l;
}

void plo_destroy(plo_lattice *l) {
    if (!l) return;
    free(l->scale); free(l->cells); free(l->keys); free(l->values); free(l->scratch_values);
    free(l->replay_vertex); free(l->replay_weight); free(l);
}

/* splat with values carrying `in_channels` channels; the last lattice channel receives the
 * bare weight when in_channels == vd-1 (homogeneous coordinate), else all vd are given */
static void splat_impl(plo_lattice *l, const float *positions, const float *values,
                       int in_channels) {
    const int pd = l->pd, vd = l->vd, d1 = pd + 1;
    float elevated[32], rem0[32], bary[34];
    short rank[32], key[32];
    const double t0 = now_seconds();
    index_reset(l);
    for (int n = 0; n < l->N; ++n) {
        const float *value = values + (size_t)n * in_channels;
        plo_embed(pd, l->scale, positions + (size_t)n * pd, elevated);
        plo_simplex(pd, elevated, rem0, rank);
        plo_barycentric(pd, elevated, rem0, rank, bary);
        for (int r = 0; r < d1; ++r) {
            plo_vertex_key(pd, rem0, rank, r, key);
            const int v = vertex_find(l, key, 1);
            float *acc = l->values + (size_t)v * vd;
            const float w = bary[r];
            for (int j = 0; j < in_channels; ++j) acc[j] += w * value[j];
            if (in_channels == vd - 1) acc[vd - 1] += w;
            l->replay_vertex[(size_t)n * d1 + r] = v;
            l->replay_weight[(size_t)n * d1 + r] = w;
        }
    }
    l->t_splat = now_seconds() - t0;
}

void plo_splat(plo_lattice *l, const float *positions, const float *values) {
    splat_impl(l, positions, values, l->vd - 1);
}

void plo_blur(plo_lattice *l, int reverse) {
    const int pd = l->pd, vd = l->vd, M = l->M;
    short plus[32], minus[32];
    const double t0 = now_seconds();
    for (int step = 0; step <= pd; ++step) {
        const int axis = reverse ? pd - step : step;
        for (int v = 0; v < M; ++v) {
            const short *key = l->keys + (size_t)v * pd;
            /* neighbours along `axis`: +-(1,...,1) with -+(pd+1) on that coordinate; the
             * (pd)th coordinate is implicit, so axis == pd only shifts every stored one */
            for (int k = 0; k < pd; ++k) {
                plus[k] = (short)(key[k] + 1);
                minus[k] = (short)(key[k] - 1);
            }
            if (axis < pd) {
                plus[axis] = (short)(key[axis] - pd);
                minus[axis] = (short)(key[axis] + pd);
            }
            const int vp = vertex_find(l, plus, 0);
            const int vm = vertex_find(l, minus, 0);
            const float *self = l->values + (size_t)v * vd;
            float *dst = l->scratch_values + (size_t)v * vd;
            for (int k = 0; k < vd; ++k) {
                /* DOUBLE: the three-tap mix is evaluated in double, rounded once */
                const double a = vp >= 0 ? (double)l->values[(size_t)vp * vd + k] : 0.0;
                const double b = vm >= 0 ? (double)l->values[(size_t)vm * vd + k] : 0.0;
                dst[k] = (float)(0.25 * a + 0.5 * (double)self[k] + 0.25 * b);
            }
        }
        float *t = l->values; l->values = l->scratch_values; l->scratch_values = t;
    }
    l->t_blur = now_seconds() - t0;
}

void plo_slice(plo_lattice *l, float *out, int normalize) {
    const int pd = l->pd, vd = l->vd, d1 = pd + 1;
    float acc[256];
    float *big = NULL, *a = acc;
    if (vd > 256) a = big = (float *)malloc(sizeof(float) * (size_t)vd);
    const double t0 = now_seconds();
    for (int n = 0; n < l->N; ++n) {
        for (int j = 0; j < vd; ++j) a[j] = 0.0f;
        for (int r = 0; r < d1; ++r) {
            const float w = l->replay_weight[(size_t)n * d1 + r];
            const float *src = l->values + (size_t)l->replay_vertex[(size_t)n * d1 + r] * vd;
            for (int j = 0; j < vd; ++j) a[j] += w * src[j];
        }
        if (normalize) {
            /* DOUBLE: reciprocal of the homogeneous channel in double, rounded to float */
            const float s = (float)(1.0 / (double)a[vd - 1]);
            for (int j = 0; j < vd - 1; ++j) out[(size_t)n * (vd - 1) + j] = a[j] * s;
        } else {
            for (int j = 0; j < vd; ++j) out[(size_t)n * vd + j] = a[j];
        }
    }
    l->t_slice = now_seconds() - t0;
    free(big);
}

void plo_filter(plo_lattice *l, float *output, const float *input, const float *positions,
                int reverse) {
    plo_splat(l, positions, input);
    plo_blur(l, reverse);
    plo_slice(l, output, 1);
}

void plo_filter_raw(plo_lattice *l, float *output, const float *input_vd,
                    const float *positions, int reverse) {
    splat_impl(l, positions, input_vd, l->vd);
    plo_blur(l, reverse);
    plo_slice(l, output, 0);
}

int plo_num_vertices(const plo_lattice *l) { return l->M; }
const short *plo_keys(const plo_lattice *l) { return l->keys; }
const float *plo_values(const plo_lattice *l) { return l->values; }
const int *plo_replay_vertex(const plo_lattice *l) { return l->replay_vertex; }
const float *plo_replay_weight(const plo_lattice *l) { return l->replay_weight; }
void plo_stage_seconds(const plo_lattice *l, double *splat, double *blur, double *slice) {
    if (splat) *splat = l->t_splat;
    if (blur) *blur = l->t_blur;
    if (slice) *slice = l->t_slice;
}

/* ------------------------------------------------------------------------------------------
 * Op level
 * ---------------------------------------------------------------------------------------- */

int plo_lattice_filter_op(const float *input, const float *reference, float *output, int batch,
                          int n_spatial_dims, const int *spatial_dims, int n_input_channels,
                          int n_reference_channels, int bilateral, float theta_alpha,
                          float theta_beta, float theta_gamma, int reverse) {
    if (batch < 0 || n_spatial_dims < 1 || n_input_channels < 1) return -1;
    long long n = 1;
    for (int i = 0; i < n_spatial_dims; ++i) {
        if (spatial_dims[i] < 1) return -1;
        n *= spatial_dims[i];
    }
    if (n * (long long)batch * n_input_channels > 2147483647LL) return -1;
    const int N = (int)n;
    const int vd = n_input_channels + 1;
    /* bilateral: features = (coords / theta_alpha, reference / theta_beta);
     * otherwise: features = coords / theta_gamma and the reference image is ignored */
    const int ref_ch = bilateral ? n_reference_channels : 0;
    const int pd = n_spatial_dims + ref_ch;
    const float spatial_std = bilateral ? theta_alpha : theta_gamma;
    const float feature_std = bilateral ? theta_beta : -1.0f;
    if (bilateral && (n_reference_channels < 1 || reference == NULL)) return -1;

    float *positions = (float *)malloc(sizeof(float) * (size_t)N * (size_t)pd);
    for (int b = 0; b < batch; ++b) {
        const float *ref_b = ref_ch ? reference + (size_t)b * N * ref_ch : NULL;
        plo_compute_positions(ref_b, positions, N, ref_ch, n_spatial_dims, spatial_dims,
                              spatial_std, feature_std);
        plo_lattice *l = plo_create(pd, vd, N);
        plo_filter(l, output + (size_t)b * N * n_input_channels,
                   input + (size_t)b * N * n_input_channels, positions, reverse);
        plo_destroy(l);
    }
    free(positions);
    return 0;
}

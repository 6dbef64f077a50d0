/*
 * Body of the CPU oracle, written once for the value type PLO_T and compiled for float and for
 * double by pl_oracle.c (TEST INFRASTRUCTURE ONLY, see there).  The reference is a template over
 * T (src/PermutohedralLatticeCPU.h:173); every cast below that reads (PLO_T)((double)...) is a
 * place where its expression is evaluated in double whatever T is and stored to T: for float one
 * rounding, for double none.
 */
/* ------------------------------------------------------------------------------------------
 * Per-point arithmetic
 * ---------------------------------------------------------------------------------------- */

void PLO_FN(scale_factor)(int pd, PLO_T *scale) {
    /* DOUBLE: (pd+1)*sqrt(2/3) is formed in double and stored as PLO_T; each entry is
     * 1/sqrt((i+1)(i+2)) in double times that PLO_T, rounded once. */
    const PLO_T inv_std_dev = (PLO_T)((double)(pd + 1) * sqrt(2.0 / 3.0));
    for (int i = 0; i < pd; ++i) {
        const double diag = 1.0 / sqrt((double)((i + 1) * (i + 2)));
        scale[i] = (PLO_T)(diag * (double)inv_std_dev);
    }
}

void PLO_FN(embed)(int pd, const PLO_T *scale, const PLO_T *position, PLO_T *elevated) {
    /* Running-sum form of the rotation onto the hyperplane x.1 = 0, unfused.  The scaled
     * coordinate is a float whatever T is (`float cf`, src/PermutohedralLatticeCPU.h:226), and so
     * is its product with the index; sums and differences are in T. */
    PLO_T running = (PLO_T)0;
    for (int i = pd; i >= 1; --i) {
        const float c = (float)(position[i - 1] * scale[i - 1]);
        const float ic = (float)i * c;
        elevated[i] = running - (PLO_T)ic;
        running = running + (PLO_T)c;
    }
    elevated[0] = running;
}

void PLO_FN(simplex)(int pd, const PLO_T *elevated, PLO_T *rem0, short *rank) {
    const int d1 = pd + 1;
    const double inv_d1 = 1.0 / (double)d1;
    short coord_sum = 0;

    for (int i = 0; i < d1; ++i) {
        /* DOUBLE: the division by pd+1 is a double multiply by the double reciprocal. */
        const PLO_T v = (PLO_T)((double)elevated[i] * inv_d1);
        const PLO_T above = (PLO_T)(ceil((double)v) * (double)d1);
        const PLO_T below = (PLO_T)(floor((double)v) * (double)d1);
        /* strictly closer to `above` wins; a tie goes down */
        if (above - elevated[i] < elevated[i] - below)
            rem0[i] = (PLO_T)(short)above;
        else
            rem0[i] = (PLO_T)(short)below;
        coord_sum = (short)((PLO_T)coord_sum + rem0[i]);
    }
    coord_sum = (short)(coord_sum / d1);

    /* rank[i] = how many coordinates have a larger residual; ties are broken by the
     * comparison order (i < j, strict <, the later index loses the tie). */
    for (int i = 0; i < d1; ++i) rank[i] = 0;
    for (int i = 0; i < pd; ++i) {
        const PLO_T di = elevated[i] - rem0[i];
        for (int j = i + 1; j < d1; ++j) {
            const PLO_T dj = elevated[j] - rem0[j];
            if (di < dj) rank[i]++;
            else rank[j]++;
        }
    }

    /* the rounded point may be off the plane by coord_sum steps: shift ranks, wrap */
    for (int i = 0; i < d1; ++i) {
        rank[i] = (short)(rank[i] + coord_sum);
        if (rank[i] < 0) {
            rank[i] = (short)(rank[i] + d1);
            rem0[i] += (PLO_T)d1;
        } else if (rank[i] > pd) {
            rank[i] = (short)(rank[i] - d1);
            rem0[i] -= (PLO_T)d1;
        }
    }
}

void PLO_FN(barycentric)(int pd, const PLO_T *elevated, const PLO_T *rem0, const short *rank,
                     PLO_T *barycentric) {
    const int d1 = pd + 1;
    const double inv_d1 = 1.0 / (double)d1;
    for (int k = 0; k < pd + 2; ++k) barycentric[k] = (PLO_T)0;
    for (int i = 0; i < d1; ++i) {
        /* DOUBLE: PLO_T residual times the double reciprocal, rounded to PLO_T */
        const PLO_T delta = (PLO_T)((double)(elevated[i] - rem0[i]) * inv_d1);
        barycentric[pd - rank[i]] += delta;
        barycentric[pd - rank[i] + 1] -= delta;
    }
    /* DOUBLE: wrap-around term is added in double */
    barycentric[0] = (PLO_T)((double)barycentric[0] + (1.0 + (double)barycentric[pd + 1]));
}

void PLO_FN(vertex_key)(int pd, const PLO_T *rem0, const short *rank, int remainder, short *key) {
    for (int i = 0; i < pd; ++i) {
        short k = (short)(rem0[i] + (PLO_T)remainder);
        if (rank[i] > pd - remainder) k = (short)(k - (pd + 1));
        key[i] = k;
    }
}

void PLO_FN(dump_simplex)(int pd, int N, const PLO_T *positions, short *rem0_out, short *rank_out,
                      short *keys_out, PLO_T *bary_out, PLO_T *elevated_out) {
    const int d1 = pd + 1;
    PLO_T *scale = (PLO_T *)malloc(sizeof(PLO_T) * (size_t)pd);
    PLO_T *elevated = (PLO_T *)malloc(sizeof(PLO_T) * (size_t)d1);
    PLO_T *rem0 = (PLO_T *)malloc(sizeof(PLO_T) * (size_t)d1);
    short *rank = (short *)malloc(sizeof(short) * (size_t)d1);
    PLO_T *bary = (PLO_T *)malloc(sizeof(PLO_T) * (size_t)(pd + 2));
    PLO_FN(scale_factor)(pd, scale);
    for (int n = 0; n < N; ++n) {
        PLO_FN(embed)(pd, scale, positions + (size_t)n * pd, elevated);
        PLO_FN(simplex)(pd, elevated, rem0, rank);
        PLO_FN(barycentric)(pd, elevated, rem0, rank, bary);
        for (int i = 0; i < d1; ++i) {
            if (elevated_out) elevated_out[(size_t)n * d1 + i] = elevated[i];
            if (rem0_out) rem0_out[(size_t)n * d1 + i] = (short)rem0[i];
            if (rank_out) rank_out[(size_t)n * d1 + i] = rank[i];
            if (bary_out) bary_out[(size_t)n * d1 + i] = bary[i];
            if (keys_out) PLO_FN(vertex_key)(pd, rem0, rank, i, keys_out + ((size_t)n * d1 + i) * pd);
        }
    }
    free(scale); free(elevated); free(rem0); free(rank); free(bary);
}

void PLO_FN(compute_positions)(const PLO_T *reference, PLO_T *positions, int num_super_pixels,
                           int reference_channels, int n_sdims, const int *sdims,
                           PLO_T spatial_std, PLO_T feature_std) {
    const int pd = n_sdims + reference_channels;
    for (int n = 0; n < num_super_pixels; ++n) {
        PLO_T *row = positions + (size_t)n * pd;
        /* linear index -> coordinates, last spatial dimension fastest */
        int stride = 1;
        for (int s = n_sdims - 1; s >= 0; --s) {
            const int coord = (n / stride) % sdims[s];
            row[s] = (PLO_T)coord / spatial_std;
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

struct PLO_LATTICE {
    int pd, vd, N;
    PLO_T *scale;
    /* open-addressed index: cell -> vertex id or -1 */
    int *cells;
    size_t n_cells;          /* power of two */
    short *keys;             /* vertex id -> pd shorts */
    PLO_T *values;           /* vertex id -> vd floats */
    PLO_T *scratch_values;
    size_t vertex_capacity;
    int M;
    int n_growths;
    int stale_cell_after_growth;
    /* the key that was being looked up when the index doubled, per doubling (pd shorts each,
     * the first PLO_MAX_GROWTHS of them): with the quirk on, the lookups that probed from a
     * stale cell */
    short growth_keys[PLO_MAX_GROWTHS * 32];
    int *replay_vertex;      /* N*(pd+1) */
    PLO_T *replay_weight;    /* N*(pd+1) */
    double t_splat, t_blur, t_slice;
};


/* src/PermutohedralLatticeCPU.h:44-51 -- positional hash, base 2531011, 64-bit wrap-around.
 * The hash decides nothing about vertex numbering (first touch does) except at the moment the
 * index grows, see PLO_STATIC(vertex_find) below; it is restated here so that moment can be reproduced. */
static size_t PLO_STATIC(key_hash)(const short *key, int pd) {
    size_t h = 0;
    for (int i = 0; i < pd; ++i) {
        h += (size_t)(long long)key[i];
        h *= (size_t)2531011;
    }
    return h;
}

static void PLO_STATIC(index_reset)(PLO_LATTICE *l) {
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
static void PLO_STATIC(index_grow)(PLO_LATTICE *l) {
    const size_t old_n = l->n_cells, new_n = old_n * 2;
    int *grown = (int *)malloc(sizeof(int) * new_n);
    memset(grown, 0xff, sizeof(int) * new_n);
    for (size_t c = 0; c < old_n; ++c) {
        const int v = l->cells[c];
        if (v < 0) continue;
        size_t at = PLO_STATIC(key_hash)(l->keys + (size_t)v * l->pd, l->pd) % new_n;
        while (grown[at] >= 0) at = (at + 1 == new_n) ? 0 : at + 1;
        grown[at] = v;
    }
    free(l->cells);
    l->cells = grown;
    l->n_cells = new_n;
    l->n_growths++;
}

static void PLO_STATIC(vertices_reserve)(PLO_LATTICE *l, size_t want) {
    if (want <= l->vertex_capacity) return;
    size_t cap = l->vertex_capacity ? l->vertex_capacity : 1024;
    while (cap < want) cap *= 2;
    l->keys = (short *)realloc(l->keys, sizeof(short) * cap * (size_t)l->pd);
    l->values = (PLO_T *)realloc(l->values, sizeof(PLO_T) * cap * (size_t)l->vd);
    l->scratch_values = (PLO_T *)realloc(l->scratch_values, sizeof(PLO_T) * cap * (size_t)l->vd);
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
static int PLO_STATIC(vertex_find)(PLO_LATTICE *l, const short *key, int create) {
    const int pd = l->pd;
    size_t c = PLO_STATIC(key_hash)(key, pd) % l->n_cells;
    if ((size_t)l->M >= l->n_cells / 2 - 1) {
        if (l->n_growths < PLO_MAX_GROWTHS)
            memcpy(l->growth_keys + (size_t)l->n_growths * 32, key, sizeof(short) * (size_t)pd);
        PLO_STATIC(index_grow)(l);
        if (!l->stale_cell_after_growth) c = PLO_STATIC(key_hash)(key, pd) % l->n_cells;
    }
    for (;;) {
        const int v = l->cells[c];
        if (v < 0) break;
        if (memcmp(l->keys + (size_t)v * pd, key, sizeof(short) * (size_t)pd) == 0) return v;
        c = (c + 1 == l->n_cells) ? 0 : c + 1;
    }
    if (!create) return -1;
    const int v = l->M;
    PLO_STATIC(vertices_reserve)(l, (size_t)v + 1);
    memcpy(l->keys + (size_t)v * pd, key, sizeof(short) * (size_t)pd);
    memset(l->values + (size_t)v * l->vd, 0, sizeof(PLO_T) * (size_t)l->vd);
    l->cells[c] = v;
    l->M = v + 1;
    return v;
}

void PLO_FN(set_reference_growth_quirk)(PLO_LATTICE *l, int on) { l->stale_cell_after_growth = on; }
int PLO_FN(num_growths)(const PLO_LATTICE *l) { return l->n_growths; }
int PLO_FN(growth_keys)(const PLO_LATTICE *l, short *out) {
    const int n = l->n_growths < PLO_MAX_GROWTHS ? l->n_growths : PLO_MAX_GROWTHS;
    for (int g = 0; g < n; ++g)
        memcpy(out + (size_t)g * l->pd, l->growth_keys + (size_t)g * 32, sizeof(short) * (size_t)l->pd);
    return n;
}

PLO_LATTICE *PLO_FN(create)(int pd, int vd, int N) {
    if (pd < 1 || vd < 2 || N < 0) return NULL;
    PLO_LATTICE *l = (PLO_LATTICE *)calloc(1, sizeof(PLO_LATTICE));
    l->pd = pd; l->vd = vd; l->N = N;
    l->scale = (PLO_T *)malloc(sizeof(PLO_T) * (size_t)pd);
    PLO_FN(scale_factor)(pd, l->scale);
    l->n_cells = PLO_INITIAL_CELLS;
    l->cells = (int *)malloc(sizeof(int) * l->n_cells);
    PLO_STATIC(index_reset)(l);
    PLO_STATIC(vertices_reserve)(l, 1024);
    const size_t rows = (size_t)N * (size_t)(pd + 1);
    l->replay_vertex = (int *)malloc(sizeof(int) * (rows ? rows : 1));
    l->replay_weight = (PLO_T *)malloc(sizeof(PLO_T) * (rows ? rows : 1));
    return l;
}

void PLO_FN(destroy)(PLO_LATTICE *l) {
    if (!l) return;
    free(l->scale); free(l->cells); free(l->keys); free(l->values); free(l->scratch_values);
    free(l->replay_vertex); free(l->replay_weight); free(l);
}

/* splat with values carrying `in_channels` channels; the last lattice channel receives the
 * bare weight when in_channels == vd-1 (homogeneous coordinate), else all vd are given */
static void PLO_STATIC(splat_impl)(PLO_LATTICE *l, const PLO_T *positions, const PLO_T *values,
                       int in_channels) {
    const int pd = l->pd, vd = l->vd, d1 = pd + 1;
    PLO_T elevated[32], rem0[32], bary[34];
    short rank[32], key[32];
    const double t0 = now_seconds();
    PLO_STATIC(index_reset)(l);
    for (int n = 0; n < l->N; ++n) {
        const PLO_T *value = values + (size_t)n * in_channels;
        PLO_FN(embed)(pd, l->scale, positions + (size_t)n * pd, elevated);
        PLO_FN(simplex)(pd, elevated, rem0, rank);
        PLO_FN(barycentric)(pd, elevated, rem0, rank, bary);
        for (int r = 0; r < d1; ++r) {
            PLO_FN(vertex_key)(pd, rem0, rank, r, key);
            const int v = PLO_STATIC(vertex_find)(l, key, 1);
            PLO_T *acc = l->values + (size_t)v * vd;
            const PLO_T w = bary[r];
            for (int j = 0; j < in_channels; ++j) acc[j] += w * value[j];
            if (in_channels == vd - 1) acc[vd - 1] += w;
            l->replay_vertex[(size_t)n * d1 + r] = v;
            l->replay_weight[(size_t)n * d1 + r] = w;
        }
    }
    l->t_splat = now_seconds() - t0;
}

void PLO_FN(splat)(PLO_LATTICE *l, const PLO_T *positions, const PLO_T *values) {
    PLO_STATIC(splat_impl)(l, positions, values, l->vd - 1);
}

void PLO_FN(blur)(PLO_LATTICE *l, int reverse) {
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
            const int vp = PLO_STATIC(vertex_find)(l, plus, 0);
            const int vm = PLO_STATIC(vertex_find)(l, minus, 0);
            const PLO_T *self = l->values + (size_t)v * vd;
            PLO_T *dst = l->scratch_values + (size_t)v * vd;
            for (int k = 0; k < vd; ++k) {
                /* DOUBLE: the three-tap mix is evaluated in double, rounded once */
                const double a = vp >= 0 ? (double)l->values[(size_t)vp * vd + k] : 0.0;
                const double b = vm >= 0 ? (double)l->values[(size_t)vm * vd + k] : 0.0;
                dst[k] = (PLO_T)(0.25 * a + 0.5 * (double)self[k] + 0.25 * b);
            }
        }
        PLO_T *t = l->values; l->values = l->scratch_values; l->scratch_values = t;
    }
    l->t_blur = now_seconds() - t0;
}

void PLO_FN(slice)(PLO_LATTICE *l, PLO_T *out, int normalize) {
    const int pd = l->pd, vd = l->vd, d1 = pd + 1;
    PLO_T acc[256];
    PLO_T *big = NULL, *a = acc;
    if (vd > 256) a = big = (PLO_T *)malloc(sizeof(PLO_T) * (size_t)vd);
    const double t0 = now_seconds();
    for (int n = 0; n < l->N; ++n) {
        for (int j = 0; j < vd; ++j) a[j] = (PLO_T)0;
        for (int r = 0; r < d1; ++r) {
            const PLO_T w = l->replay_weight[(size_t)n * d1 + r];
            const PLO_T *src = l->values + (size_t)l->replay_vertex[(size_t)n * d1 + r] * vd;
            for (int j = 0; j < vd; ++j) a[j] += w * src[j];
        }
        if (normalize) {
            /* DOUBLE: reciprocal of the homogeneous channel in double, rounded to PLO_T */
            const PLO_T s = (PLO_T)(1.0 / (double)a[vd - 1]);
            for (int j = 0; j < vd - 1; ++j) out[(size_t)n * (vd - 1) + j] = a[j] * s;
        } else {
            for (int j = 0; j < vd; ++j) out[(size_t)n * vd + j] = a[j];
        }
    }
    l->t_slice = now_seconds() - t0;
    free(big);
}

void PLO_FN(filter)(PLO_LATTICE *l, PLO_T *output, const PLO_T *input, const PLO_T *positions,
                int reverse) {
    PLO_FN(splat)(l, positions, input);
    PLO_FN(blur)(l, reverse);
    PLO_FN(slice)(l, output, 1);
}

void PLO_FN(filter_raw)(PLO_LATTICE *l, PLO_T *output, const PLO_T *input_vd,
                    const PLO_T *positions, int reverse) {
    PLO_STATIC(splat_impl)(l, positions, input_vd, l->vd);
    PLO_FN(blur)(l, reverse);
    PLO_FN(slice)(l, output, 0);
}

int PLO_FN(num_vertices)(const PLO_LATTICE *l) { return l->M; }
const short *PLO_FN(keys)(const PLO_LATTICE *l) { return l->keys; }
const PLO_T *PLO_FN(values)(const PLO_LATTICE *l) { return l->values; }
const int *PLO_FN(replay_vertex)(const PLO_LATTICE *l) { return l->replay_vertex; }
const PLO_T *PLO_FN(replay_weight)(const PLO_LATTICE *l) { return l->replay_weight; }
void PLO_FN(stage_seconds)(const PLO_LATTICE *l, double *splat, double *blur, double *slice) {
    if (splat) *splat = l->t_splat;
    if (blur) *blur = l->t_blur;
    if (slice) *slice = l->t_slice;
}

/* ------------------------------------------------------------------------------------------
 * Op level
 * ---------------------------------------------------------------------------------------- */

int PLO_FN(lattice_filter_op)(const PLO_T *input, const PLO_T *reference, PLO_T *output, int batch,
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
    /* the attributes are floats whatever T is (src/LatticeFilterKernel.cpp:36-38) */
    const PLO_T spatial_std = (PLO_T)(bilateral ? theta_alpha : theta_gamma);
    const PLO_T feature_std = bilateral ? (PLO_T)theta_beta : (PLO_T)-1;
    if (bilateral && (n_reference_channels < 1 || reference == NULL)) return -1;

    PLO_T *positions = (PLO_T *)malloc(sizeof(PLO_T) * (size_t)N * (size_t)pd);
    for (int b = 0; b < batch; ++b) {
        const PLO_T *ref_b = ref_ch ? reference + (size_t)b * N * ref_ch : NULL;
        PLO_FN(compute_positions)(ref_b, positions, N, ref_ch, n_spatial_dims, spatial_dims,
                              spatial_std, feature_std);
        PLO_LATTICE *l = PLO_FN(create)(pd, vd, N);
        PLO_FN(filter)(l, output + (size_t)b * N * n_input_channels,
                   input + (size_t)b * N * n_input_channels, positions, reverse);
        PLO_FN(destroy)(l);
    }
    free(positions);
    return 0;
}

/*
 * CPU oracle for the permutohedral-lattice filter.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the arithmetic of the
 * reference CPU path (src/PermutohedralLatticeCPU.h in the reference tree) for T = float and,
 * with the suffix _f64, for T = double.
 * It exists to check the HIP library; nothing in the shipped library links, loads or
 * calls it, and it is never the thing whose speed is reported as the product's.
 *
 * Every function names the reference lines whose results it reproduces.  What pins each
 * of them (golden vectors produced by the real reference header, BMP fixtures held by
 * the reference's tests, closed forms and invariants) is listed at the top of
 * pl_oracle.c.
 */
#ifndef PL_ORACLE_H
#define PL_ORACLE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct plo_lattice plo_lattice;

/* src/PermutohedralLatticeCPU.h:194-217 -- per-axis scale of the elevation. */
void plo_scale_factor(int pd, float *scale);

/* src/PermutohedralLatticeCPU.h:220-231 -- position (pd) -> point on the hyperplane (pd+1). */
void plo_embed(int pd, const float *scale, const float *position, float *elevated);

/* src/PermutohedralLatticeCPU.h:233-273 -- nearest remainder-0 point and rank permutation. */
void plo_simplex(int pd, const float *elevated, float *rem0, short *rank);

/* src/PermutohedralLatticeCPU.h:275-286 -- barycentric[pd+2]; [0..pd] are the vertex weights. */
void plo_barycentric(int pd, const float *elevated, const float *rem0, const short *rank,
                     float *barycentric);

/* src/PermutohedralLatticeCPU.h:297-304 -- first pd coordinates of simplex vertex `remainder`. */
void plo_vertex_key(int pd, const float *rem0, const short *rank, int remainder, short *key);

/* Per-pixel dump of the integer results (any output pointer may be NULL):
 * rem0[N*(pd+1)], rank[N*(pd+1)], keys[N*(pd+1)*pd] (vertex-major inside a pixel),
 * barycentric[N*(pd+1)], elevated[N*(pd+1)]. */
void plo_dump_simplex(int pd, int N, const float *positions, short *rem0, short *rank,
                      short *keys, float *barycentric, float *elevated);

/* src/PermutohedralLatticeCPU.h:452-474 -- feature vectors of one batch item. */
void plo_compute_positions(const float *reference, float *positions, int num_super_pixels,
                           int reference_channels, int n_sdims, const int *sdims,
                           float spatial_std, float feature_std);

/* src/PermutohedralLatticeCPU.h:419-440 -- lattice for (pd, vd, N); vd counts the homogeneous channel. */
plo_lattice *plo_create(int pd, int vd, int N);
void plo_destroy(plo_lattice *l);

/* src/PermutohedralLatticeCPU.h:288-326 -- splat all N points (resets the lattice first). */
void plo_splat(plo_lattice *l, const float *positions, const float *values);
/* src/PermutohedralLatticeCPU.h:362-415 -- blur along the pd+1 axes, order pd..0 when reverse. */
void plo_blur(plo_lattice *l, int reverse);
/* src/PermutohedralLatticeCPU.h:333-358 -- slice; normalize=0 skips the homogeneous division and
 * writes all vd channels per pixel (out has N*vd floats then), for adjointness tests. */
void plo_slice(plo_lattice *l, float *out, int normalize);
/* src/PermutohedralLatticeCPU.h:442-446 -- splat, blur, slice. */
void plo_filter(plo_lattice *l, float *output, const float *input, const float *positions,
                int reverse);
/* Same as plo_filter but with values that already carry the homogeneous channel (N*vd in,
 * N*vd out, no division): the linear operator slice*blur*splat itself. */
void plo_filter_raw(plo_lattice *l, float *output, const float *input_vd,
                    const float *positions, int reverse);

/* The reference computes the start cell of a lookup before it checks whether the index must
 * double (src/PermutohedralLatticeCPU.h:163-165 then :62), so the lookup that triggers a
 * doubling can miss a key that is present and enter it again as a second vertex: at most one
 * duplicate vertex per doubling.  on=1 reproduces that (bit-exact with the reference, vertex
 * count included); on=0 (default) is the intended algorithm, one vertex per distinct key,
 * which is what the HIP library is compared with. */
void plo_set_reference_growth_quirk(plo_lattice *l, int on);
/* number of index doublings during the last splat/blur */
int plo_num_growths(const plo_lattice *l);
/* the key whose lookup triggered each doubling (the lookups that, in the reference, probe from a
 * stale cell): out gets pd shorts per doubling, at most PLO_MAX_GROWTHS of them; returns how many */
#define PLO_MAX_GROWTHS 24
int plo_growth_keys(const plo_lattice *l, short *out);

int plo_num_vertices(const plo_lattice *l);
/* keys in first-touch order, M*pd shorts */
const short *plo_keys(const plo_lattice *l);
/* current vertex values, M*vd floats */
const float *plo_values(const plo_lattice *l);
/* replay rows: vertex index and weight of pixel n, vertex r at [n*(pd+1)+r] */
const int *plo_replay_vertex(const plo_lattice *l);
const float *plo_replay_weight(const plo_lattice *l);
/* seconds spent in the last splat / blur / slice */
void plo_stage_seconds(const plo_lattice *l, double *splat, double *blur, double *slice);

/* src/LatticeFilterKernel.cpp:111-179 -- the LatticeFilter op on channels-last tensors
 * [batch, s_1..s_k, C]; one lattice per batch item.  Returns 0, or -1 on bad arguments. */
int plo_lattice_filter_op(const float *input, const float *reference, float *output, int batch,
                          int n_spatial_dims, const int *spatial_dims, int n_input_channels,
                          int n_reference_channels, int bilateral, float theta_alpha,
                          float theta_beta, float theta_gamma, int reverse);

/* ------------------------------------------------------------------------------------------
 * T = double (the op registers it, src/LatticeFilterKernel.cpp:196-208): the same functions,
 * name by name, citing the same reference lines.  One difference is the reference's own: the
 * scaled coordinate of the elevation is a float for every T (`float cf`, :226).
 * ---------------------------------------------------------------------------------------- */
typedef struct plo_lattice_f64 plo_lattice_f64;
void plo_scale_factor_f64(int pd, double *scale);
void plo_embed_f64(int pd, const double *scale, const double *position, double *elevated);
void plo_simplex_f64(int pd, const double *elevated, double *rem0, short *rank);
void plo_barycentric_f64(int pd, const double *elevated, const double *rem0, const short *rank,
                         double *barycentric);
void plo_vertex_key_f64(int pd, const double *rem0, const short *rank, int remainder, short *key);
void plo_dump_simplex_f64(int pd, int N, const double *positions, short *rem0, short *rank,
                          short *keys, double *barycentric, double *elevated);
void plo_compute_positions_f64(const double *reference, double *positions, int num_super_pixels,
                               int reference_channels, int n_sdims, const int *sdims,
                               double spatial_std, double feature_std);
plo_lattice_f64 *plo_create_f64(int pd, int vd, int N);
void plo_destroy_f64(plo_lattice_f64 *l);
void plo_splat_f64(plo_lattice_f64 *l, const double *positions, const double *values);
void plo_blur_f64(plo_lattice_f64 *l, int reverse);
void plo_slice_f64(plo_lattice_f64 *l, double *out, int normalize);
void plo_filter_f64(plo_lattice_f64 *l, double *output, const double *input,
                    const double *positions, int reverse);
void plo_filter_raw_f64(plo_lattice_f64 *l, double *output, const double *input_vd,
                        const double *positions, int reverse);
void plo_set_reference_growth_quirk_f64(plo_lattice_f64 *l, int on);
int plo_num_growths_f64(const plo_lattice_f64 *l);
int plo_growth_keys_f64(const plo_lattice_f64 *l, short *out);
int plo_num_vertices_f64(const plo_lattice_f64 *l);
const short *plo_keys_f64(const plo_lattice_f64 *l);
const double *plo_values_f64(const plo_lattice_f64 *l);
const int *plo_replay_vertex_f64(const plo_lattice_f64 *l);
const double *plo_replay_weight_f64(const plo_lattice_f64 *l);
void plo_stage_seconds_f64(const plo_lattice_f64 *l, double *splat, double *blur, double *slice);
int plo_lattice_filter_op_f64(const double *input, const double *reference, double *output,
                              int batch, int n_spatial_dims, const int *spatial_dims,
                              int n_input_channels, int n_reference_channels, int bilateral,
                              float theta_alpha, float theta_beta, float theta_gamma, int reverse);

#ifdef __cplusplus
}
#endif
#endif

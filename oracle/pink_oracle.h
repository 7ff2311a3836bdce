/*
 * pink_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, CPU-only restatement of the reference (HITS-AIN/PINK v2.5) CPU
 * path for one training / mapping step of the rotation-invariant SOM.  It is
 * the checker the HIP kernels are compared with.  Nothing in the shipped
 * library links, loads or calls it; only the tests, the smoke check and the
 * benchmark's cpu_baseline leg do.
 *
 * Every function names the reference file:line it follows.  Float arithmetic
 * is written so that, compiled with -ffp-contract=off on x86-64, it rounds
 * exactly where the reference's C++ rounds.
 *
 * Parity pins (see tests/test_oracle_*.py):
 *   - rotated images, region SSD (float and integer), circular region rule,
 *     layouts' distances, neighbourhood functors, mt19937 filler:
 *       compared bit-for-bit with the real reference headers compiled into
 *       oracle/_ref/libpink_ref.so, and with the reference tests' golden vectors.
 *   - min-over-rotations loop, BMU search, neuron update, mapper sqrt tail
 *     (Trainer.h / Mapper.h / generate_euclidean_distance_matrix.h need a
 *     CMake-generated header and are not compiled): pinned by the reference
 *     tests' known answers (290, {6,7,10,11}, 3-D best rotation, heatmap
 *     2.0/1.0/0.0, circular {0,.5,.2,.7}/{0,1,2,3}, update kernel vector)
 *     and by brute force in float64 / exact integers on small inputs.
 *   - visiting order of the shuffled data iterator (libstdc++ 11's std::shuffle
 *     over std::mt19937): compared with the reference's DataIteratorShuffled in
 *     oracle/_ref, with orders taken from it (tests/golden/shuffle_orders.json)
 *     and with the reference's own iterator test (seed 2, two entries).
 *   - integer (uint8/uint16) distance modes: the reference CPU path has none;
 *     the contract is the reference CPU functor evaluated in exact integers on
 *     arrays quantised as the reference's device conversion does
 *     (q = T(x * factor), saturated to [0, factor]).
 */
#ifndef PINK_ORACLE_H
#define PINK_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* UtilitiesLib/DataType.h:16-21 */
enum { PINK_ORACLE_FLOAT = 0, PINK_ORACLE_UINT16 = 1, PINK_ORACLE_UINT8 = 2 };
/* UtilitiesLib/EuclideanDistanceShape.h:14-18 */
enum { PINK_ORACLE_QUADRATIC = 0, PINK_ORACLE_CIRCULAR = 1 };
/* UtilitiesLib/Layout.h:13-17 */
enum { PINK_ORACLE_CARTESIAN = 0, PINK_ORACLE_HEXAGONAL = 1 };
/* UtilitiesLib/DistributionFunctor.h: Step, Gaussian, UnityGaussian, MexicanHat */
enum { PINK_ORACLE_STEP = 0, PINK_ORACLE_GAUSSIAN = 1, PINK_ORACLE_UNITY_GAUSSIAN = 2, PINK_ORACLE_MEXICAN_HAT = 3 };

typedef struct pink_oracle_shape {
    uint32_t som_size;    /* N: number of neurons                                   */
    uint32_t channels;    /* C: 1 for 2-D data, depth for channel-first 3-D data    */
    uint32_t image_dim;   /* I: image edge                                          */
    uint32_t neuron_dim;  /* D: neuron edge                                         */
    uint32_t num_rot;     /* 1 or a multiple of 4                                   */
    uint32_t use_flip;    /* 0 / 1                                                  */
    uint32_t ed_dim;      /* edge (quadratic) or diameter (circular) of the region  */
    uint32_t ed_shape;    /* PINK_ORACLE_QUADRATIC / _CIRCULAR                      */
    uint32_t ed_type;     /* PINK_ORACLE_FLOAT / _UINT16 / _UINT8                   */
} pink_oracle_shape;

/* ---- image primitives ---------------------------------------------------- */
void pink_oracle_resize(const float *src, float *dst, uint32_t src_h, uint32_t src_w,
                        uint32_t dst_h, uint32_t dst_w);
void pink_oracle_rotate_90(const float *src, float *dst, uint32_t h, uint32_t w);
void pink_oracle_flip(const float *src, float *dst, uint32_t h, uint32_t w);
void pink_oracle_rotate_bilinear(const float *src, float *dst, uint32_t src_h, uint32_t src_w,
                                 uint32_t dst_h, uint32_t dst_w, float alpha);

/* All num_rot*(flip?2:1) variants of one image, layout [k][c][x][y], each D*D. */
void pink_oracle_rotated_images(const float *image, uint32_t channels, uint32_t image_dim,
                                uint32_t neuron_dim, uint32_t num_rot, int use_flip, float *out);

/* ---- distance region ------------------------------------------------------ */
/* Offsets (into one C*D*D neuron) of the region elements in the reference's
 * summation order.  Returns the count; offsets may be NULL to only count. */
uint32_t pink_oracle_region(uint32_t channels, uint32_t neuron_dim, uint32_t ed_dim,
                            uint32_t ed_shape, uint32_t *offsets);

float   pink_oracle_ssd_f32(const float *a, const float *b, uint32_t channels, uint32_t neuron_dim,
                            uint32_t ed_dim, uint32_t ed_shape);
int64_t pink_oracle_ssd_int(const int32_t *a, const int32_t *b, uint32_t channels, uint32_t neuron_dim,
                            uint32_t ed_dim, uint32_t ed_shape);

/* q = T(x * factor), factor = 255 (UINT8) or 65535 (UINT16), saturated. */
int32_t pink_oracle_quantise(float x, uint32_t ed_type);
uint32_t pink_oracle_quant_factor(uint32_t ed_type);

/* d[n] = min_r SSD(som[n], rot[r]); best[n] = first r attaining it.
 * Float mode: dist_f32 only (ssd_int may be NULL).  Integer modes: ssd_int holds the
 * exact integer SSD and dist_f32 = float(double(ssd) / double(factor^2)). */
void pink_oracle_distance_matrix(const pink_oracle_shape *s, const float *som, const float *rotated,
                                 float *dist_f32, int64_t *ssd_int, uint32_t *best_rot);
/* The same matrix, one functor call per pair as the reference makes them (the definition the
 * sixteen-rotations-at-a-time form above is checked against, bit for bit). */
void pink_oracle_distance_matrix_pairwise(const pink_oracle_shape *s, const float *som, const float *rotated,
                                          float *dist_f32, int64_t *ssd_int, uint32_t *best_rot);
/* Float mode with the reference's own parallel structure (generate_euclidean_distance_matrix.h:45-56):
 * `omp parallel for` over the rotations of one neuron, one call through a function pointer and one
 * `omp critical` section per pair.  With several threads equal distances go to the thread that enters
 * first, as in the reference.  What the benchmark's CPU baseline times. */
void pink_oracle_distance_matrix_reference_loop(const pink_oracle_shape *s, const float *som,
                                                const float *rotated, float *dist_f32, uint32_t *best_rot);

/* Which of the three evaluations above pink_oracle_train / pink_oracle_map use: 0 = sixteen variants at a time
 * (default), 1 = pairwise, 2 = the reference's loop structure (float mode only; -2 from train / map otherwise).
 * Returns 0, or -1 for an unknown form.  Process-wide. */
int pink_oracle_set_distance_form(int form);

/* ---- SOM-grid distances, neighbourhood functors, update factors ----------- */
uint32_t pink_oracle_hex_size(uint32_t dim);
float pink_oracle_cartesian_distance(const uint32_t *dims, uint32_t ndims, uint32_t i1, uint32_t i2);
float pink_oracle_hex_distance(uint32_t dim, uint32_t i1, uint32_t i2);
float pink_oracle_functor(uint32_t kind, float sigma_or_value, float damping, float distance);
/* F[i*N+j] = functor(dist(i,j)) if max_update_distance <= 0 or dist < max, else 0. */
void pink_oracle_update_factors(uint32_t layout, const uint32_t *dims, uint32_t ndims,
                                uint32_t functor_kind, float sigma_or_value, float damping,
                                float max_update_distance, float *factors);

/* ---- steps ---------------------------------------------------------------- */
uint32_t pink_oracle_bmu(const pink_oracle_shape *s, const float *dist_f32, const int64_t *ssd_int);
void pink_oracle_update(float *som, uint32_t som_size, uint32_t neuron_size, const float *rotated,
                        const uint32_t *best_rot, uint32_t bmu, const float *factors);

/* One Trainer::operator() call.  scratch_rot must hold R*C*D*D floats (or NULL:
 * allocated inside).  Optional outputs may be NULL. */
int pink_oracle_train_step(const pink_oracle_shape *s, float *som, const float *image,
                           const float *factors, float *scratch_rot, uint32_t *bmu_out,
                           float *dist_out, uint32_t *best_rot_out);
/* n images in order, sequential SOM semantics. */
int pink_oracle_train(const pink_oracle_shape *s, float *som, const float *images, uint32_t n_images,
                      const float *factors, uint32_t *bmu_out);
/* One Mapper::operator() call per image: heatmap = sqrt(min distance). */
int pink_oracle_map(const pink_oracle_shape *s, const float *som, const float *images, uint32_t n_images,
                    float *heatmap_out, uint32_t *best_rot_out);

/* ---- random filler -------------------------------------------------------- */
void pink_oracle_fill_random_uniform(float *a, size_t length, uint32_t seed);
void pink_oracle_mt19937_raw(uint32_t seed, uint32_t *out, size_t n);
/* Visiting order of the shuffled data iterator for `n` entries. */
void pink_oracle_shuffled_order(uint64_t seed, uint32_t n, uint32_t *order);

int pink_oracle_num_threads(void);
void pink_oracle_set_num_threads(int n);

#ifdef __cplusplus
}
#endif
#endif

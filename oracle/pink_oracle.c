/*
 * pink_oracle.c -- TEST INFRASTRUCTURE ONLY (see pink_oracle.h).
 *
 * CPU restatement of the reference CPU path, citing the reference file:line
 * each function follows.  Build with -ffp-contract=off (no FMA contraction):
 * the reference's x86-64 build rounds every float product and sum separately.
 */
#include "pink_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#ifndef M_PI
#define M_PI 3.14159265358979323846
#endif

/* ------------------------------------------------------------------------ */
/* ImageProcessingLib/resize.h:15-40 : centre crop / centre pad, integer margins. */
void pink_oracle_resize(const float *src, float *dst, uint32_t src_h, uint32_t src_w,
                        uint32_t dst_h, uint32_t dst_w)
{
    uint32_t src_wm = 0, dst_wm = 0, src_hm = 0, dst_hm = 0;
    if (src_w < dst_w) dst_wm = (dst_w - src_w) / 2;
    else if (src_w > dst_w) src_wm = (src_w - dst_w) / 2;
    if (src_h < dst_h) dst_hm = (dst_h - src_h) / 2;
    else if (src_h > dst_h) src_hm = (src_h - dst_h) / 2;
    uint32_t w = src_w < dst_w ? src_w : dst_w;
    uint32_t h = src_h < dst_h ? src_h : dst_h;
    for (uint32_t i = 0; i < h; ++i)
        for (uint32_t j = 0; j < w; ++j)
            dst[(size_t)(i + dst_hm) * dst_w + (j + dst_wm)] = src[(size_t)(i + src_hm) * src_w + (j + src_wm)];
}

/* ImageProcessingLib/rotate_90_degrees.h:15-26 : clockwise quarter turn. */
void pink_oracle_rotate_90(const float *src, float *dst, uint32_t h, uint32_t w)
{
    for (uint32_t x = 0; x < w; ++x)
        for (uint32_t y = 0; y < h; ++y)
            dst[(size_t)x * h + y] = src[(size_t)(h - y - 1) * w + x];
}

/* ImageProcessingLib/flip.h:14-30 : reverse the order of the rows. */
void pink_oracle_flip(const float *src, float *dst, uint32_t h, uint32_t w)
{
    for (uint32_t i = 0; i < h; ++i)
        memcpy(dst + (size_t)(h - 1 - i) * w, src + (size_t)i * w, (size_t)w * sizeof(float));
}

/* ImageProcessingLib/rotate.h:17-67.  x is the slow index of both images.
 * Where the reference reads one element past a row / past the image with an
 * interpolation weight of exactly 0 (rotate.h:50,62-63), the index is clamped
 * here: the product is +-0 either way for finite pixels. */
void pink_oracle_rotate_bilinear(const float *src, float *dst, uint32_t src_h, uint32_t src_w,
                                 uint32_t dst_h, uint32_t dst_w, float alpha)
{
    const float cos_alpha = cosf(alpha);
    const float sin_alpha = sinf(alpha);
    const float src_center_x = (float)(src_w - 1) * 0.5f;
    const float src_center_y = (float)(src_h - 1) * 0.5f;
    const float dst_center_x = (float)(dst_w - 1) * 0.5f;
    const float dst_center_y = (float)(dst_h - 1) * 0.5f;
    const float max_x = (float)(src_w - 1);
    const float max_y = (float)(src_h - 1);
    const size_t last = (size_t)src_w * src_h - 1;

    for (uint32_t dst_x = 0; dst_x < dst_w; ++dst_x) {
        for (uint32_t dst_y = 0; dst_y < dst_h; ++dst_y) {
            float px = (float)dst_x - dst_center_x;
            float py = (float)dst_y - dst_center_y;
            float t0 = px * cos_alpha;
            float t1 = py * sin_alpha;
            float sx = (t0 - t1) + src_center_x;
            float t2 = px * sin_alpha;
            float t3 = py * cos_alpha;
            float sy = (t2 + t3) + src_center_y;
            float v;
            if (sx < 0.0f || sx > max_x || sy < 0.0f || sy > max_y) {
                v = 0.0f;
            } else {
                uint32_t ix = (uint32_t)sx;
                uint32_t iy = (uint32_t)sy;
                float rx = sx - (float)ix;
                float ry = sy - (float)iy;
                float cx = 1.0f - rx;
                float cy = 1.0f - ry;
                size_t i00 = (size_t)ix * src_h + iy;
                size_t i01 = i00 + 1;
                size_t i10 = i00 + src_h;
                size_t i11 = i10 + 1;
                if (i01 > last) i01 = last;
                if (i10 > last) i10 = last;
                if (i11 > last) i11 = last;
                float a = (cx * cy) * src[i00];
                float b = (cx * ry) * src[i01];
                float c = (rx * cy) * src[i10];
                float d = (rx * ry) * src[i11];
                v = ((a + b) + c) + d;
            }
            dst[(size_t)dst_x * dst_h + dst_y] = v;
        }
    }
}

/* SelfOrganizingMapLib/generate_rotated_images.h:50-117 (2-D) and :121-200 (3-D,
 * channel-first).  Variant k = f*num_rot + q*(num_rot/4) + i; variant k holds its
 * channels contiguously: element (k*C + c)*D*D + x*D + y. */
void pink_oracle_rotated_images(const float *image, uint32_t channels, uint32_t image_dim,
                                uint32_t neuron_dim, uint32_t num_rot, int use_flip, float *out)
{
    const size_t nsz = (size_t)neuron_dim * neuron_dim;
    const size_t isz = (size_t)image_dim * image_dim;
    const uint32_t nrr = num_rot / 4;
    const float angle_step = (float)(2 * M_PI) / (float)num_rot;
    const size_t off1 = (size_t)nrr * channels * nsz;
    const size_t off2 = 2 * off1, off3 = 3 * off1;

    memset(out, 0, (size_t)num_rot * (use_flip ? 2 : 1) * channels * nsz * sizeof(float));

    for (uint32_t c = 0; c < channels; ++c) {
        float *cur = out + c * nsz;
        pink_oracle_resize(image + c * isz, cur, image_dim, image_dim, neuron_dim, neuron_dim);
        if (num_rot != 1) {
            pink_oracle_rotate_90(cur, cur + off1, neuron_dim, neuron_dim);
            pink_oracle_rotate_90(cur + off1, cur + off2, neuron_dim, neuron_dim);
            pink_oracle_rotate_90(cur + off2, cur + off3, neuron_dim, neuron_dim);
        }
    }

    #pragma omp parallel for schedule(static)
    for (uint32_t i = 1; i < nrr; ++i) {
        for (uint32_t c = 0; c < channels; ++c) {
            float *cur = out + ((size_t)i * channels + c) * nsz;
            pink_oracle_rotate_bilinear(image + c * isz, cur, image_dim, image_dim,
                                        neuron_dim, neuron_dim, (float)i * angle_step);
            pink_oracle_rotate_90(cur, cur + off1, neuron_dim, neuron_dim);
            pink_oracle_rotate_90(cur + off1, cur + off2, neuron_dim, neuron_dim);
            pink_oracle_rotate_90(cur + off2, cur + off3, neuron_dim, neuron_dim);
        }
    }

    if (use_flip) {
        float *flipped = out + (size_t)channels * num_rot * nsz;
        #pragma omp parallel for schedule(static)
        for (uint32_t i = 0; i < num_rot; ++i)
            for (uint32_t c = 0; c < channels; ++c)
                pink_oracle_flip(out + ((size_t)i * channels + c) * nsz,
                                 flipped + ((size_t)i * channels + c) * nsz, neuron_dim, neuron_dim);
    }
}

/* ------------------------------------------------------------------------ */
/* Region element offsets in summation order.
 * Quadratic: ImageProcessingLib/euclidean_distance.h:47-67 (2-D), :70-100 (3-D):
 *   rows and columns [beg, beg+e), beg = uint32((D-e)*0.5), channels outermost.
 * Circular: ImageProcessingLib/circular_euclidean_distance.h:37-60 (2-D), :63-88 (3-D):
 *   row i of e, global row i+(D-e)/2, delta = sqrt(2*(e/2)*(i+.5) - (i+.5)^2),
 *   columns [round(D/2 - delta), round(D/2 + delta)).  A negative radicand (last
 *   row of an odd diameter) makes delta NaN and the row empty (the loop test
 *   `j < NaN` is false).  The 3-D functor never adds the channel offset (:77-85):
 *   channel 0 is summed `channels` times; followed as written. */
uint32_t pink_oracle_region(uint32_t channels, uint32_t neuron_dim, uint32_t ed_dim,
                            uint32_t ed_shape, uint32_t *offsets)
{
    uint32_t n = 0;
    const uint32_t dim = neuron_dim;
    if (ed_shape == PINK_ORACLE_QUADRATIC) {
        uint32_t beg = (uint32_t)((double)(dim - ed_dim) * 0.5);
        uint32_t end = beg + ed_dim;
        for (uint32_t d = 0; d < channels; ++d)
            for (uint32_t i = beg; i < end; ++i)
                for (uint32_t j = beg; j < end; ++j) {
                    if (offsets) offsets[n] = d * dim * dim + i * dim + j;
                    ++n;
                }
    } else {
        uint32_t center = dim / 2;
        uint32_t radius = ed_dim / 2;
        for (uint32_t d = 0; d < channels; ++d)
            for (uint32_t i = 0; i < ed_dim; ++i) {
                double delta = sqrt((double)(2 * radius) * (i + 0.5) - pow(i + 0.5, 2));
                uint32_t gi = i + (dim - ed_dim) / 2;
                if (isnan(delta)) continue;
                double lo = round((double)center - delta);
                double hi = round((double)center + delta);
                for (uint32_t j = (uint32_t)lo; (double)j < hi; ++j) {
                    if (offsets) offsets[n] = gi * dim + j;
                    ++n;
                }
            }
    }
    return n;
}

/* Float SSD: `ed += std::pow(a - b, 2)` with T = float (euclidean_distance.h:60-64):
 * the difference is rounded to float, std::pow(float,int) squares it in double,
 * the sum is formed in double and rounded back to float at every step. */
static float ssd_f32_offsets(const float *a, const float *b, const uint32_t *off, uint32_t n)
{
    float ed = 0.0f;
    for (uint32_t k = 0; k < n; ++k) {
        float diff = a[off[k]] - b[off[k]];
        double sq = (double)diff * (double)diff;
        ed = (float)((double)ed + sq);
    }
    return ed;
}

/* Integer SSD: the same functor with T integral -- `ed += std::pow(a - b, 2)` is
 * ed = T(double(ed) + double(diff)^2), exact while every partial sum < 2^53. */
static int64_t ssd_int_offsets(const int32_t *a, const int32_t *b, const uint32_t *off, uint32_t n)
{
    int64_t ed = 0;
    for (uint32_t k = 0; k < n; ++k) {
        int32_t diff = a[off[k]] - b[off[k]];
        ed = (int64_t)((double)ed + (double)diff * (double)diff);
    }
    return ed;
}

float pink_oracle_ssd_f32(const float *a, const float *b, uint32_t channels, uint32_t neuron_dim,
                          uint32_t ed_dim, uint32_t ed_shape)
{
    uint32_t n = pink_oracle_region(channels, neuron_dim, ed_dim, ed_shape, NULL);
    uint32_t *off = (uint32_t *)malloc((size_t)(n ? n : 1) * sizeof(uint32_t));
    pink_oracle_region(channels, neuron_dim, ed_dim, ed_shape, off);
    float r = ssd_f32_offsets(a, b, off, n);
    free(off);
    return r;
}

int64_t pink_oracle_ssd_int(const int32_t *a, const int32_t *b, uint32_t channels, uint32_t neuron_dim,
                            uint32_t ed_dim, uint32_t ed_shape)
{
    uint32_t n = pink_oracle_region(channels, neuron_dim, ed_dim, ed_shape, NULL);
    uint32_t *off = (uint32_t *)malloc((size_t)(n ? n : 1) * sizeof(uint32_t));
    pink_oracle_region(channels, neuron_dim, ed_dim, ed_shape, off);
    int64_t r = ssd_int_offsets(a, b, off, n);
    free(off);
    return r;
}

/* CudaLib/euclidean_distance_kernel.h:44-57 : range = 2^digits - 1. */
uint32_t pink_oracle_quant_factor(uint32_t ed_type)
{
    return ed_type == PINK_ORACLE_UINT8 ? 255u : ed_type == PINK_ORACLE_UINT16 ? 65535u : 1u;
}

/* CudaLib/copy_and_transform_kernel.h:27-28 : dst = T(src * factor): a float
 * multiply by 255.0f / 65535.0f, then truncation.  Out-of-range conversion is
 * undefined in the reference; here it saturates to [0, factor] (NaN -> 0). */
int32_t pink_oracle_quantise(float x, uint32_t ed_type)
{
    uint32_t factor = pink_oracle_quant_factor(ed_type);
    float v = x * (float)factor;
    if (!(v > 0.0f)) return 0;
    if (v >= (float)factor) return (int32_t)factor;
    return (int32_t)v;
}

/* SelfOrganizingMapLib/generate_euclidean_distance_matrix.h:19-59 with one thread:
 * d[n] starts at rotation 0, later rotations replace it only when strictly
 * smaller, so the first index attaining the minimum wins.  The OpenMP split
 * here keeps a per-thread (min, lowest index) and merges by (value, index), which
 * gives the one-thread answer for any thread count.  One functor call per pair,
 * as the reference makes them; pink_oracle_distance_matrix below gives the same
 * bits faster and is checked against this form (tests/test_oracle_golden.py). */
void pink_oracle_distance_matrix_pairwise(const pink_oracle_shape *s, const float *som, const float *rotated,
                                          float *dist_f32, int64_t *ssd_int, uint32_t *best_rot)
{
    const uint32_t N = s->som_size;
    const uint32_t R = s->num_rot * (s->use_flip ? 2 : 1);
    const size_t nsz = (size_t)s->channels * s->neuron_dim * s->neuron_dim;
    uint32_t E = pink_oracle_region(s->channels, s->neuron_dim, s->ed_dim, s->ed_shape, NULL);
    uint32_t *off = (uint32_t *)malloc((size_t)(E ? E : 1) * sizeof(uint32_t));
    pink_oracle_region(s->channels, s->neuron_dim, s->ed_dim, s->ed_shape, off);

    if (s->ed_type == PINK_ORACLE_FLOAT) {
        for (uint32_t n = 0; n < N; ++n) {
            const float *pn = som + n * nsz;
            const float d0 = ssd_f32_offsets(pn, rotated, off, E);
            float dmin = d0;
            uint32_t bmin = 0;
            #pragma omp parallel
            {
                float dl = d0; uint32_t bl = 0;
                #pragma omp for schedule(static) nowait
                for (uint32_t r = 1; r < R; ++r) {
                    float t = ssd_f32_offsets(pn, rotated + r * nsz, off, E);
                    if (t < dl) { dl = t; bl = r; }
                }
                #pragma omp critical
                if (dl < dmin || (dl == dmin && bl < bmin)) { dmin = dl; bmin = bl; }
            }
            dist_f32[n] = dmin;
            best_rot[n] = bmin;
        }
    } else {
        /* quantise only the region elements (the rest is never read) */
        const uint32_t factor = pink_oracle_quant_factor(s->ed_type);
        int32_t *qs = (int32_t *)calloc(N * nsz, sizeof(int32_t));
        int32_t *qr = (int32_t *)calloc(R * nsz, sizeof(int32_t));
        #pragma omp parallel for schedule(static)
        for (uint32_t n = 0; n < N; ++n)
            for (uint32_t k = 0; k < E; ++k)
                qs[n * nsz + off[k]] = pink_oracle_quantise(som[n * nsz + off[k]], s->ed_type);
        #pragma omp parallel for schedule(static)
        for (uint32_t r = 0; r < R; ++r)
            for (uint32_t k = 0; k < E; ++k)
                qr[r * nsz + off[k]] = pink_oracle_quantise(rotated[r * nsz + off[k]], s->ed_type);
        #pragma omp parallel for schedule(static)
        for (uint32_t n = 0; n < N; ++n) {
            int64_t dmin = ssd_int_offsets(qs + n * nsz, qr, off, E);
            uint32_t bmin = 0;
            for (uint32_t r = 1; r < R; ++r) {
                int64_t t = ssd_int_offsets(qs + n * nsz, qr + r * nsz, off, E);
                if (t < dmin) { dmin = t; bmin = r; }
            }
            if (ssd_int) ssd_int[n] = dmin;
            dist_f32[n] = (float)((double)dmin / ((double)factor * (double)factor));
            best_rot[n] = bmin;
        }
        free(qs);
        free(qr);
    }
    free(off);
}

/* The same matrix with the reference's own parallel structure
 * (generate_euclidean_distance_matrix.h:45-56): every neuron opens one `omp parallel for` over the
 * rotations, every pair is one call through a function object (here a function pointer) and one
 * `omp critical` section that compares and stores.  Like the reference with more than one thread,
 * equal distances go to whichever thread enters first; what the benchmark's CPU baseline times.
 * Float mode only (the reference's CPU path has no other). */
typedef float (*pair_functor)(const float *, const float *, const uint32_t *, uint32_t);

void pink_oracle_distance_matrix_reference_loop(const pink_oracle_shape *s, const float *som,
                                                const float *rotated, float *dist_f32, uint32_t *best_rot)
{
    const uint32_t N = s->som_size;
    const uint32_t R = s->num_rot * (s->use_flip ? 2 : 1);
    const size_t nsz = (size_t)s->channels * s->neuron_dim * s->neuron_dim;
    uint32_t E = pink_oracle_region(s->channels, s->neuron_dim, s->ed_dim, s->ed_shape, NULL);
    uint32_t *off = (uint32_t *)malloc((size_t)(E ? E : 1) * sizeof(uint32_t));
    pink_oracle_region(s->channels, s->neuron_dim, s->ed_dim, s->ed_shape, off);
    volatile pair_functor functor = ssd_f32_offsets;

    for (uint32_t n = 0; n < N; ++n) {
        dist_f32[n] = functor(som + n * nsz, rotated, off, E);
        best_rot[n] = 0;
        #pragma omp parallel for
        for (uint32_t r = 1; r < R; ++r) {
            float t = functor(som + n * nsz, rotated + r * nsz, off, E);
            #pragma omp critical
            if (t < dist_f32[n]) { dist_f32[n] = t; best_rot[n] = r; }
        }
    }
    free(off);
}

/* Sixteen rotations side by side.  Every pair still runs the functor's own sequence of operations in
 * the functor's element order (float difference; square and sum in double; the sum rounded to float
 * after every element); only which pairs share a vector instruction changes, so the results are the
 * bits of ssd_f32_offsets / ssd_int_offsets.  rt = the region of the variants, element-major
 * (rt[k * ld + r]). */
#define PO_LANES 16
typedef float   po_f4 __attribute__((vector_size(16)));
typedef int32_t po_i4 __attribute__((vector_size(16)));
typedef double  po_d4 __attribute__((vector_size(32)));

__attribute__((target_clones("avx2", "default")))
static void ssd_f32_lanes(const float *a, const float *rt0, const float *rt1, uint32_t n, float *out0, float *out1)
{
    /* two blocks of sixteen variants (eight independent chains of four lanes: a chain's step is a
     * convert, an add and a convert back, a dozen cycles that the other chains fill) */
    po_f4 ed0 = {0}, ed1 = {0}, ed2 = {0}, ed3 = {0}, ed4 = {0}, ed5 = {0}, ed6 = {0}, ed7 = {0};
#define PO_STEP(ed, row, j) { po_f4 b; memcpy(&b, row + 4 * (j), sizeof b); po_f4 diff = av - b;         \
                         po_d4 wide = __builtin_convertvector(diff, po_d4);                            \
                         po_d4 sum = __builtin_convertvector(ed, po_d4) + wide * wide;                 \
                         ed = __builtin_convertvector(sum, po_f4); }
    for (uint32_t k = 0; k < n; ++k) {
        const float *r0 = rt0 + (size_t)k * PO_LANES, *r1 = rt1 + (size_t)k * PO_LANES;
        const po_f4 av = {a[k], a[k], a[k], a[k]};
        PO_STEP(ed0, r0, 0) PO_STEP(ed1, r0, 1) PO_STEP(ed2, r0, 2) PO_STEP(ed3, r0, 3)
        PO_STEP(ed4, r1, 0) PO_STEP(ed5, r1, 1) PO_STEP(ed6, r1, 2) PO_STEP(ed7, r1, 3)
    }
#undef PO_STEP
    memcpy(out1, &ed4, 16); memcpy(out1 + 4, &ed5, 16); memcpy(out1 + 8, &ed6, 16); memcpy(out1 + 12, &ed7, 16);
    memcpy(out0, &ed0, 16); memcpy(out0 + 4, &ed1, 16); memcpy(out0 + 8, &ed2, 16); memcpy(out0 + 12, &ed3, 16);
}

/* Integer pairs: double(ed) + double(diff)^2 is exact while every partial sum stays below 2^53
 * (the functor's own condition), so the sum stays in double until the end. */
__attribute__((target_clones("avx2", "default")))
static void ssd_int_lanes(const int32_t *a, const int32_t *rt, uint32_t n, int64_t *out)
{
    po_d4 ed[4] = {{0}, {0}, {0}, {0}};
    po_d4 ed0 = {0}, ed1 = {0}, ed2 = {0}, ed3 = {0};
#define PO_STEP(ed, j) { po_i4 b; memcpy(&b, row + 4 * (j), sizeof b); po_i4 diff = av - b;              \
                         po_d4 wide = __builtin_convertvector(diff, po_d4); ed = ed + wide * wide; }
    for (uint32_t k = 0; k < n; ++k) {
        const int32_t *row = rt + (size_t)k * PO_LANES;
        const po_i4 av = {a[k], a[k], a[k], a[k]};
        PO_STEP(ed0, 0) PO_STEP(ed1, 1) PO_STEP(ed2, 2) PO_STEP(ed3, 3)
    }
#undef PO_STEP
    ed[0] = ed0; ed[1] = ed1; ed[2] = ed2; ed[3] = ed3;
    for (int j = 0; j < PO_LANES; ++j) out[j] = (int64_t)ed[j / 4][j % 4];
}

/* generate_euclidean_distance_matrix.h:19-59, the answer of its one-thread run (first rotation
 * attaining the minimum), evaluated sixteen rotations at a time.  Bit-identical to
 * pink_oracle_distance_matrix_pairwise. */
void pink_oracle_distance_matrix(const pink_oracle_shape *s, const float *som, const float *rotated,
                                 float *dist_f32, int64_t *ssd_int, uint32_t *best_rot)
{
    const uint32_t N = s->som_size;
    const uint32_t R = s->num_rot * (s->use_flip ? 2 : 1);
    const size_t nsz = (size_t)s->channels * s->neuron_dim * s->neuron_dim;
    const uint32_t blocks = (R + PO_LANES - 1) / PO_LANES;
    const size_t ld = (size_t)blocks * PO_LANES;
    uint32_t E = pink_oracle_region(s->channels, s->neuron_dim, s->ed_dim, s->ed_shape, NULL);
    const size_t Ea = E ? E : 1;
    uint32_t *off = (uint32_t *)malloc(Ea * sizeof(uint32_t));
    pink_oracle_region(s->channels, s->neuron_dim, s->ed_dim, s->ed_shape, off);
    const int is_float = s->ed_type == PINK_ORACLE_FLOAT;
    const uint32_t factor = pink_oracle_quant_factor(s->ed_type);
    /* the region of the variants, sixteen variants at a time and element-major inside such a block
     * (rt[(block * E + k) * 16 + lane]), and the region of every neuron, gathered; 4-byte elements:
     * floats, or the quantised integers of the integer modes.  all[n * ld + r] = the pair's sum. */
    uint32_t *rt = (uint32_t *)calloc(Ea * ld, 4);
    uint32_t *sr = (uint32_t *)malloc((size_t)N * Ea * 4);
    int64_t *all = (int64_t *)malloc((size_t)N * ld * sizeof(int64_t));

    #pragma omp parallel
    {
        #pragma omp for schedule(static) nowait
        for (uint32_t r = 0; r < R; ++r)
            for (uint32_t k = 0; k < E; ++k) {
                float v = rotated[r * nsz + off[k]];
                uint32_t *dst = &rt[((size_t)(r / PO_LANES) * E + k) * PO_LANES + r % PO_LANES];
                if (is_float) memcpy(dst, &v, 4);
                else *dst = (uint32_t)pink_oracle_quantise(v, s->ed_type);
            }
        #pragma omp for schedule(static)
        for (uint32_t n = 0; n < N; ++n)
            for (uint32_t k = 0; k < E; ++k) {
                float v = som[n * nsz + off[k]];
                if (is_float) memcpy(&sr[(size_t)n * E + k], &v, 4);
                else sr[(size_t)n * E + k] = (uint32_t)pink_oracle_quantise(v, s->ed_type);
            }
        /* float: two blocks per call (an odd last block runs beside itself) */
        #pragma omp for schedule(dynamic, 1)
        for (uint32_t blk = 0; blk < blocks; blk += is_float ? 2 : 1) {
            const uint32_t blk1 = blk + 1 < blocks ? blk + 1 : blk;
            for (uint32_t n = 0; n < N; ++n) {
                int64_t *out = all + (size_t)n * ld + (size_t)blk * PO_LANES;
                int64_t *out1 = all + (size_t)n * ld + (size_t)blk1 * PO_LANES;
                if (is_float) ssd_f32_lanes((const float *)sr + (size_t)n * E,
                                            (const float *)rt + (size_t)blk * E * PO_LANES,
                                            (const float *)rt + (size_t)blk1 * E * PO_LANES, E,
                                            (float *)out, (float *)out1);
                else ssd_int_lanes((const int32_t *)sr + (size_t)n * E,
                                   (const int32_t *)rt + (size_t)blk * E * PO_LANES, E, out);
            }
        }
        #pragma omp for schedule(static)
        for (uint32_t n = 0; n < N; ++n) {
            uint32_t bmin = 0;
            if (is_float) {
                float fmin = 0.0f;
                for (uint32_t r = 0; r < R; ++r) {
                    const float t = ((const float *)(all + (size_t)n * ld + (size_t)(r / PO_LANES) * PO_LANES))[r % PO_LANES];
                    if (r == 0 || t < fmin) { fmin = t; bmin = r; }
                }
                dist_f32[n] = fmin;
            } else {
                int64_t imin = 0;
                for (uint32_t r = 0; r < R; ++r) {
                    const int64_t t = all[(size_t)n * ld + r];
                    if (r == 0 || t < imin) { imin = t; bmin = r; }
                }
                if (ssd_int) ssd_int[n] = imin;
                dist_f32[n] = (float)((double)imin / ((double)factor * (double)factor));
            }
            best_rot[n] = bmin;
        }
    }
    free(rt); free(sr); free(all); free(off);
}

/* ------------------------------------------------------------------------ */
/* SelfOrganizingMapLib/HexagonalLayout.h:62-65 */
uint32_t pink_oracle_hex_size(uint32_t dim)
{
    uint32_t radius = (dim - 1) / 2;
    return dim * dim - radius * (radius + 1);
}

/* SelfOrganizingMapLib/CartesianLayout.h:47-60,103-129 : position from index, then
 * Euclidean distance with a float accumulator. */
float pink_oracle_cartesian_distance(const uint32_t *dims, uint32_t ndims, uint32_t i1, uint32_t i2)
{
    uint32_t p1[3] = {0, 0, 0}, p2[3] = {0, 0, 0};
    const uint32_t idx[2] = {i1, i2};
    uint32_t *pp[2] = {p1, p2};
    for (int k = 0; k < 2; ++k) {
        uint32_t i = idx[k], *p = pp[k];
        if (ndims == 1) {
            p[0] = i;
        } else if (ndims == 2) {
            p[1] = i / dims[1];
            p[0] = i % dims[1];
        } else {
            uint32_t z = i / dims[0] / dims[1];
            p[2] = z;
            p[1] = (i - z * dims[0] * dims[1]) / dims[1];
            p[0] = i % dims[1];
        }
    }
    float distance = 0.0f;
    for (uint32_t i = 0; i < ndims; ++i) {
        float diff = (float)p1[i] - (float)p2[i];
        distance += (float)((double)diff * (double)diff);
    }
    return sqrtf(distance);
}

/* SelfOrganizingMapLib/HexagonalLayout.h:27-48 (row tables), :79-87 (position),
 * :90-104 (cube-metric distance on (q, r)). */
float pink_oracle_hex_distance(uint32_t dim, uint32_t i1, uint32_t i2)
{
    uint32_t radius = (dim - 1) / 2;
    uint32_t *row_offset = (uint32_t *)malloc((dim + 1) * sizeof(uint32_t));
    row_offset[0] = 0;
    for (uint32_t r = 0; r < dim; ++r) {
        uint32_t away = r > radius ? r - radius : radius - r;
        row_offset[r + 1] = row_offset[r] + (dim - away);
    }
    int32_t q[2], rr[2];
    const uint32_t idx[2] = {i1, i2};
    for (int k = 0; k < 2; ++k) {
        uint32_t r = 0;
        for (; r < dim; ++r) if (idx[k] < row_offset[r + 1]) break;
        uint32_t qq = idx[k] - row_offset[r];
        if (radius > r) qq += radius - r;
        q[k] = (int32_t)qq;
        rr[k] = (int32_t)r;
    }
    free(row_offset);
    int32_t dx = q[0] - q[1], dy = rr[0] - rr[1];
    if ((dx >= 0) == (dy >= 0)) return (float)abs(dx + dy);
    int32_t ax = abs(dx), ay = abs(dy);
    return (float)(ax > ay ? ax : ay);
}

/* UtilitiesLib/DistributionFunctor.cpp:19-59 */
float pink_oracle_functor(uint32_t kind, float sigma, float damping, float distance)
{
    switch (kind) {
    case PINK_ORACLE_STEP:
        return distance <= sigma ? 1.0f : 0.0f;
    case PINK_ORACLE_GAUSSIAN:
        return damping / (sigma * sqrtf(2.0f * (float)M_PI))
                       * expf(-0.5f * powf(distance / sigma, 2.0f));
    case PINK_ORACLE_UNITY_GAUSSIAN:
        return damping * expf(-0.5f * powf(distance / sigma, 2.0f));
    case PINK_ORACLE_MEXICAN_HAT: {
        float distance2 = distance * distance;
        float sigma2 = sigma * sigma;
        return 2.0f * damping / (sqrtf(3.0f * sigma) * powf((float)M_PI, 0.25f))
                    * (1.0f - distance2 / sigma2) * expf(-distance2 / (2.0f * sigma2));
    }
    }
    return 0.0f;
}

/* SelfOrganizingMapLib/Trainer.h:62,69-76 */
void pink_oracle_update_factors(uint32_t layout, const uint32_t *dims, uint32_t ndims,
                                uint32_t functor_kind, float sigma, float damping,
                                float max_update_distance, float *factors)
{
    uint32_t N;
    if (layout == PINK_ORACLE_HEXAGONAL) N = pink_oracle_hex_size(dims[0]);
    else { N = 1; for (uint32_t i = 0; i < ndims; ++i) N *= dims[i]; }
    for (uint32_t i = 0; i < N; ++i)
        for (uint32_t j = 0; j < N; ++j) {
            float distance = layout == PINK_ORACLE_HEXAGONAL
                           ? pink_oracle_hex_distance(dims[0], i, j)
                           : pink_oracle_cartesian_distance(dims, ndims, i, j);
            float f = 0.0f;
            if (max_update_distance <= 0 || distance < max_update_distance)
                f = pink_oracle_functor(functor_kind, sigma, damping, distance);
            factors[(size_t)i * N + j] = f;
        }
}

/* ------------------------------------------------------------------------ */
/* SelfOrganizingMapLib/Trainer.h:164-165 : std::min_element, first minimum.  In the
 * integer modes the comparison is made on the exact integer SSD. */
uint32_t pink_oracle_bmu(const pink_oracle_shape *s, const float *dist_f32, const int64_t *ssd_int)
{
    uint32_t bmu = 0;
    if (s->ed_type == PINK_ORACLE_FLOAT || !ssd_int) {
        for (uint32_t n = 1; n < s->som_size; ++n) if (dist_f32[n] < dist_f32[bmu]) bmu = n;
    } else {
        for (uint32_t n = 1; n < s->som_size; ++n) if (ssd_int[n] < ssd_int[bmu]) bmu = n;
    }
    return bmu;
}

/* SelfOrganizingMapLib/Trainer.h:167-179 : w -= (w - x) * f over the whole neuron,
 * skipped when f == 0. */
void pink_oracle_update(float *som, uint32_t som_size, uint32_t neuron_size, const float *rotated,
                        const uint32_t *best_rot, uint32_t bmu, const float *factors)
{
    #pragma omp parallel for schedule(static)
    for (uint32_t i = 0; i < som_size; ++i) {
        float factor = factors[(size_t)bmu * som_size + i];
        if (factor != 0.0f) {
            float *w = som + (size_t)i * neuron_size;
            const float *x = rotated + (size_t)best_rot[i] * neuron_size;
            for (uint32_t j = 0; j < neuron_size; ++j) {
                float diff = w[j] - x[j];
                float step = diff * factor;
                w[j] = w[j] - step;
            }
        }
    }
}

/* Which evaluation of the distance matrix pink_oracle_train / pink_oracle_map use: 0 = sixteen variants at
 * a time (default), 1 = one functor call per pair, 2 = the reference's own OpenMP structure (float mode
 * only: the reference's CPU path has no other; what the benchmark's CPU baseline times).  All three give the
 * same distances; with form 2 on several threads equal distances go to the thread that enters first. */
static int g_distance_form = 0;

int pink_oracle_set_distance_form(int form)
{
    if (form < 0 || form > 2) return -1;
    g_distance_form = form;
    return 0;
}

static int distance_matrix_by_form(const pink_oracle_shape *s, const float *som, const float *rotated,
                                   float *dist_f32, int64_t *ssd_int, uint32_t *best_rot)
{
    if (g_distance_form == 2) {
        if (s->ed_type != PINK_ORACLE_FLOAT) return -2;
        pink_oracle_distance_matrix_reference_loop(s, som, rotated, dist_f32, best_rot);
    } else if (g_distance_form == 1) {
        pink_oracle_distance_matrix_pairwise(s, som, rotated, dist_f32, ssd_int, best_rot);
    } else {
        pink_oracle_distance_matrix(s, som, rotated, dist_f32, ssd_int, best_rot);
    }
    return 0;
}

/* SelfOrganizingMapLib/Trainer.h:133-186 */
int pink_oracle_train_step(const pink_oracle_shape *s, float *som, const float *image,
                           const float *factors, float *scratch_rot, uint32_t *bmu_out,
                           float *dist_out, uint32_t *best_rot_out)
{
    const uint32_t N = s->som_size;
    const uint32_t R = s->num_rot * (s->use_flip ? 2 : 1);
    const size_t nsz = (size_t)s->channels * s->neuron_dim * s->neuron_dim;
    float *rot = scratch_rot ? scratch_rot : (float *)malloc(R * nsz * sizeof(float));
    float *dist = (float *)malloc(N * sizeof(float));
    int64_t *ssd = (int64_t *)malloc(N * sizeof(int64_t));
    uint32_t *best = (uint32_t *)calloc(N, sizeof(uint32_t));
    if (!rot || !dist || !ssd || !best) return -1;

    pink_oracle_rotated_images(image, s->channels, s->image_dim, s->neuron_dim, s->num_rot,
                               (int)s->use_flip, rot);
    if (distance_matrix_by_form(s, som, rot, dist, ssd, best)) { if (!scratch_rot) free(rot); free(dist); free(ssd); free(best); return -2; }
    uint32_t bmu = pink_oracle_bmu(s, dist, ssd);
    pink_oracle_update(som, N, (uint32_t)nsz, rot, best, bmu, factors);

    if (bmu_out) *bmu_out = bmu;
    if (dist_out) memcpy(dist_out, dist, N * sizeof(float));
    if (best_rot_out) memcpy(best_rot_out, best, N * sizeof(uint32_t));
    if (!scratch_rot) free(rot);
    free(dist); free(ssd); free(best);
    return 0;
}

/* Pink/main_generic.h:87-89 : images strictly in order, each sees the SOM left by
 * the previous one. */
int pink_oracle_train(const pink_oracle_shape *s, float *som, const float *images, uint32_t n_images,
                      const float *factors, uint32_t *bmu_out)
{
    const uint32_t R = s->num_rot * (s->use_flip ? 2 : 1);
    const size_t nsz = (size_t)s->channels * s->neuron_dim * s->neuron_dim;
    const size_t isz = (size_t)s->channels * s->image_dim * s->image_dim;
    float *rot = (float *)malloc(R * nsz * sizeof(float));
    if (!rot) return -1;
    for (uint32_t i = 0; i < n_images; ++i) {
        int rc = pink_oracle_train_step(s, som, images + i * isz, factors, rot,
                                        bmu_out ? bmu_out + i : NULL, NULL, NULL);
        if (rc) { free(rot); return rc; }
    }
    free(rot);
    return 0;
}

/* SelfOrganizingMapLib/Mapper.h:107-124 : heatmap = sqrt of the minimum distance. */
int pink_oracle_map(const pink_oracle_shape *s, const float *som, const float *images, uint32_t n_images,
                    float *heatmap_out, uint32_t *best_rot_out)
{
    const uint32_t N = s->som_size;
    const uint32_t R = s->num_rot * (s->use_flip ? 2 : 1);
    const size_t nsz = (size_t)s->channels * s->neuron_dim * s->neuron_dim;
    const size_t isz = (size_t)s->channels * s->image_dim * s->image_dim;
    float *rot = (float *)malloc(R * nsz * sizeof(float));
    uint32_t *best = (uint32_t *)malloc(N * sizeof(uint32_t));
    if (!rot || !best) return -1;
    for (uint32_t i = 0; i < n_images; ++i) {
        pink_oracle_rotated_images(images + i * isz, s->channels, s->image_dim, s->neuron_dim,
                                   s->num_rot, (int)s->use_flip, rot);
        float *d = heatmap_out + (size_t)i * N;
        memset(best, 0, N * sizeof(uint32_t));
        if (distance_matrix_by_form(s, som, rot, d, NULL, best)) { free(rot); free(best); return -2; }
        for (uint32_t n = 0; n < N; ++n) d[n] = sqrtf(d[n]);
        if (best_rot_out) memcpy(best_rot_out + (size_t)i * N, best, N * sizeof(uint32_t));
    }
    free(rot); free(best);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* std::mt19937 (32-bit Mersenne Twister, MT19937 parameters of the C++ standard,
 * [rand.predef]) as used by UtilitiesLib/Filler.h:17-25. */
typedef struct { uint32_t mt[624]; int idx; } mt19937_t;

static void mt_seed(mt19937_t *g, uint32_t seed)
{
    g->mt[0] = seed;
    for (int i = 1; i < 624; ++i)
        g->mt[i] = 1812433253u * (g->mt[i - 1] ^ (g->mt[i - 1] >> 30)) + (uint32_t)i;
    g->idx = 624;
}

static uint32_t mt_next(mt19937_t *g)
{
    if (g->idx >= 624) {
        for (int i = 0; i < 624; ++i) {
            uint32_t y = (g->mt[i] & 0x80000000u) | (g->mt[(i + 1) % 624] & 0x7fffffffu);
            uint32_t v = g->mt[(i + 397) % 624] ^ (y >> 1);
            if (y & 1u) v ^= 0x9908b0dfu;
            g->mt[i] = v;
        }
        g->idx = 0;
    }
    uint32_t y = g->mt[g->idx++];
    y ^= y >> 11;
    y ^= (y << 7) & 0x9d2c5680u;
    y ^= (y << 15) & 0xefc60000u;
    y ^= y >> 18;
    return y;
}

void pink_oracle_mt19937_raw(uint32_t seed, uint32_t *out, size_t n)
{
    mt19937_t g;
    mt_seed(&g, seed);
    for (size_t i = 0; i < n; ++i) out[i] = mt_next(&g);
}

/* UtilitiesLib/Filler.h:17-25 : std::uniform_real_distribution<float>(0.0) over
 * std::mt19937.  libstdc++ draws one 32-bit word per float
 * (generate_canonical<float,24>): float(word) / 2^32, and a result that rounds
 * up to 1.0f is replaced by the largest float below 1. */
void pink_oracle_fill_random_uniform(float *a, size_t length, uint32_t seed)
{
    mt19937_t g;
    mt_seed(&g, seed);
    for (size_t i = 0; i < length; ++i) {
        float v = (float)mt_next(&g) / 4294967296.0f;
        if (v >= 1.0f) v = nextafterf(1.0f, 0.0f);
        a[i] = v;
    }
}

/* A draw of std::uniform_int_distribution<size_t>(0, range - 1) from a 32-bit generator as
 * libstdc++ 11 makes it (bits/uniform_int_dist.h, the multiply-and-reject method taken when the
 * generator's range is exactly 2^32): high word of word * range, redrawn while the low word falls
 * under 2^32 mod range.  `range` below 2^32. */
static uint32_t uniform_below(mt19937_t *g, uint64_t range)
{
    uint64_t product = (uint64_t)mt_next(g) * range;
    uint32_t low = (uint32_t)product;
    if (low < range) {
        const uint32_t threshold = (uint32_t)(-(uint32_t)range) % (uint32_t)range;
        while (low < threshold) {
            product = (uint64_t)mt_next(g) * range;
            low = (uint32_t)product;
        }
    }
    return (uint32_t)(product >> 32);
}

static void swap_u32(uint32_t *a, uint32_t *b) { const uint32_t t = *a; *a = *b; *b = t; }

/* SelfOrganizingMapLib/DataIteratorShuffled.h:62-69 : iota, std::default_random_engine(seed)
 * (minstd_rand0: x = seed mod (2^31 - 1), 1 if that is 0; next x = 16807 x mod (2^31 - 1)), a
 * std::mt19937 seeded with its first draw, std::shuffle.  std::shuffle as libstdc++ 11 has it
 * (bits/stl_algo.h): while the square of the length fits the generator's range, two swap positions
 * come out of one draw (position i with one of [0, i], position i + 1 with one of [0, i + 1]; an even
 * length first swaps position 1 alone); otherwise one draw per position.  The order is a property of
 * that library version, as it is for the reference. */
void pink_oracle_shuffled_order(uint64_t seed, uint32_t n, uint32_t *order)
{
    for (uint32_t i = 0; i < n; ++i) order[i] = i;
    if (n == 0) return;
    uint64_t x = seed % 2147483647u;
    if (x == 0) x = 1;
    x = (16807u * x) % 2147483647u;
    mt19937_t g;
    mt_seed(&g, (uint32_t)x);
    const uint64_t generator_range = 4294967295u;
    if (generator_range / n >= n) {
        uint32_t i = 1;
        if (n % 2 == 0) {
            swap_u32(&order[i], &order[uniform_below(&g, 2)]);
            ++i;
        }
        while (i < n) {
            const uint64_t first_range = (uint64_t)i + 1, second_range = first_range + 1;
            const uint32_t both = uniform_below(&g, first_range * second_range);
            swap_u32(&order[i], &order[both / second_range]);
            swap_u32(&order[i + 1], &order[both % second_range]);
            i += 2;
        }
        return;
    }
    for (uint32_t i = 1; i < n; ++i) swap_u32(&order[i], &order[uniform_below(&g, (uint64_t)i + 1)]);
}

/* Number of threads for the OpenMP loops above (the reference's --numthreads, UtilitiesLib/InputData.cpp:485). */
void pink_oracle_set_num_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* Threads the OpenMP loops above will use (1 without OpenMP). */
int pink_oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

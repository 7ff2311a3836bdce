/*
 * pink_hip.h -- C ABI of the MI355X (gfx950) implementation of PINK's GPU
 * training and mapping step.
 *
 * One context replaces the device half of one reference
 *   pink::Trainer<SOMLayout, DataLayout, float, true>   (src/SelfOrganizingMapLib/Trainer.h:201-335)
 * or
 *   pink::Mapper <SOMLayout, DataLayout, float, true>   (src/SelfOrganizingMapLib/Mapper.h:129-230)
 * i.e. everything those classes reach in src/CudaLib: the spatial transformer
 * (CudaLib/generate_rotated_images.h:57-294), the distance matrix + argmin
 * (CudaLib/generate_euclidean_distance_matrix.h:26-270) and the BMU search +
 * neuron update (CudaLib/update_neurons.h:55-85).
 *
 * Conventions
 *   - plain pointers and sizes only; all `host_*` pointers are host memory, all
 *     `dev_*` pointers are device memory of the context's device;
 *   - every function returns PINK_HIP_OK (0) or a negative pink_hip_status and never
 *     terminates the process (the reference's gpuErrchk calls exit(),
 *     CudaLib/CudaLib.h:20-29); pink_hip_last_error() gives the message the C++
 *     caller turns into pink::exception;
 *   - a context owns one HIP stream and all its device buffers, shares no global
 *     state with other contexts, and must not be used from two threads at once;
 *   - results follow the reference CPU path: rotated pixels and the update arithmetic
 *     bit-for-bit; float32 distances in the CPU's summation order, one fused
 *     multiply-add per step where the CPU rounds to double and then to float (the two
 *     can differ by one unit in the last place of a partial sum, about once in 2^29
 *     steps; distances therefore agree to 1e-5 relative and are bit-equal in practice,
 *     trained weights to 1e-4); integer (uint8/uint16) distances as exact integer sums
 *     of squared differences of q = T(x * (2^bits - 1))
 *     (CudaLib/copy_and_transform_kernel.h:27-28); lowest index on ties everywhere.
 *     kernel_choice PINK_HIP_KERNEL_MFMA_F32 alone leaves the CPU's summation order.
 */
#ifndef PINK_HIP_H
#define PINK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PINK_HIP_ABI_VERSION 2

typedef enum pink_hip_status {
    PINK_HIP_OK = 0,
    PINK_HIP_EINVAL = -1,   /* bad argument; message as the reference's pink::exception */
    PINK_HIP_ENOMEM = -2,   /* host or device allocation failed                         */
    PINK_HIP_EDEVICE = -3,  /* a HIP call failed; message holds hipGetErrorString       */
    PINK_HIP_ESTATE = -4    /* call not valid for this context (e.g. train on a mapper) */
} pink_hip_status;

/* src/UtilitiesLib/DataType.h:16-21 */
typedef enum { PINK_HIP_FLOAT = 0, PINK_HIP_UINT16 = 1, PINK_HIP_UINT8 = 2 } pink_hip_data_type;
/* src/UtilitiesLib/EuclideanDistanceShape.h:14-18 */
typedef enum { PINK_HIP_QUADRATIC = 0, PINK_HIP_CIRCULAR = 1 } pink_hip_ed_shape;
/* src/UtilitiesLib/Interpolation.h:15-19 */
typedef enum { PINK_HIP_NEAREST_NEIGHBOR = 0, PINK_HIP_BILINEAR = 1 } pink_hip_interpolation;

/* src/UtilitiesLib/Layout.h:13-17 */
typedef enum { PINK_HIP_CARTESIAN = 0, PINK_HIP_HEXAGONAL = 1 } pink_hip_som_layout;
/* src/UtilitiesLib/DistributionFunctor.h: StepFunctor, GaussianFunctor, UnityGaussianFunctor, MexicanHatFunctor */
typedef enum { PINK_HIP_STEP = 0, PINK_HIP_GAUSSIAN = 1, PINK_HIP_UNITY_GAUSSIAN = 2, PINK_HIP_MEXICAN_HAT = 3 } pink_hip_functor;

/* Which distance kernel a context uses (debugging / measurement knob). */
typedef enum {
    PINK_HIP_KERNEL_AUTO = 0,      /* float32: sequential-fma vector-ALU kernel; uint8 mapper: int8 MFMA where it applies */
    PINK_HIP_KERNEL_VALU = 1,      /* integer modes on the vector ALU in exact int32/int64                */
    PINK_HIP_KERNEL_MFMA = 2,      /* uint8 mapper, int8 MFMA, symmetries applied to the image variants   */
    PINK_HIP_KERNEL_MFMA_SYM = 3,  /* uint8 mapper, int8 MFMA, symmetries applied to the SOM once         */
    PINK_HIP_KERNEL_MFMA_GEMM = 4, /* integer modes, trainer or mapper: int8 MFMA GEMM, one launch (uint16 as 4 byte-plane products) */
    PINK_HIP_KERNEL_MFMA_F32 = 5   /* float32, trainer or mapper, on request only: |a|^2 + |b|^2 - 2 a.b with float32 MFMA dot
                                      products -- not the CPU's summation order: distances agree to a relative tolerance, best
                                      rotations where candidates are not that close, trained weights drift */
} pink_hip_kernel_choice;

/*
 * The constructor arguments of Trainer<...,true> (Trainer.h:211-215) and
 * Mapper<...,true> (Mapper.h:134-137), flattened.  The SOM layout itself does not
 * reach the device: it only shapes `update_factors`, the N x N matrix
 * TrainerCommon precomputes (Trainer.h:62,69-76).
 */
typedef struct pink_hip_config {
    uint32_t som_size;        /* N  = som_layout.size()                                  */
    uint32_t channels;        /* C  = 1 for CartesianLayout<2> data, depth for <3>       */
    uint32_t image_dim;       /* I  : images are C x I x I, row-major, channel first     */
    uint32_t neuron_dim;      /* D  : neurons are C x D x D                              */
    uint32_t num_rot;         /* number_of_rotations: 1 or a multiple of 4               */
    uint32_t use_flip;        /* 0 / 1                                                   */
    uint32_t interpolation;   /* pink_hip_interpolation                                  */
    uint32_t ed_dim;          /* euclidean_distance_dim                                  */
    uint32_t ed_shape;        /* pink_hip_ed_shape                                       */
    uint32_t ed_type;         /* pink_hip_data_type (euclidean_distance_type)            */
    const float *update_factors; /* host, N*N floats, row = BMU; NULL makes a mapper     */
    int32_t  device;          /* HIP device ordinal                                      */
    uint32_t max_batch;       /* images per launch group when mapping; 0 = choose        */
    uint32_t kernel_choice;   /* pink_hip_kernel_choice                                  */
} pink_hip_config;

typedef struct pink_hip_ctx pink_hip_ctx;

/* Replaces the constructors Trainer.h:211-260 / Mapper.h:134-179 (device allocation,
 * cos/sin tables, circle tables, upload of the update factors).  Argument errors the
 * reference throws (Trainer.h:66-67, Mapper.h:59-66, CudaLib/generate_rotated_images.h:51,120)
 * are reported here with the same text.
 * Limits of this library (PINK_HIP_EINVAL): in the integer modes a sum of squared differences
 * must stay below 2^48 and the variants below 65536 (a key is sum << 16 | variant), i.e. uint16
 * regions of at most 65538 elements, uint8 regions of any practical size; an image or a neuron
 * holds fewer than 2^31 floats. */
int pink_hip_create(pink_hip_ctx **out, const pink_hip_config *cfg);
/* The argument checks of pink_hip_create alone (the throws of Trainer.h:66-67, Mapper.h:59-66 and
 * CudaLib/generate_rotated_images.h:51,120), without touching a device: for callers that, like the
 * reference's constructors, report argument errors before the first image is seen.  Message through
 * pink_hip_last_error(NULL). */
int pink_hip_check_config(const pink_hip_config *cfg);
/* Frees the context.  Images that pink_hip_train(ctx, images, n, NULL) queued and that no later call has
 * trained yet (fewer than one launch group) are discarded, not trained: call pink_hip_get_som,
 * pink_hip_update_counts or pink_hip_synchronize first to have them applied. */
void pink_hip_destroy(pink_hip_ctx *ctx);

/* Message of the last failing call on `ctx` (or of the last failing
 * pink_hip_create on this thread when ctx is NULL).  Never NULL. */
const char *pink_hip_last_error(const pink_hip_ctx *ctx);

/* Upload the SOM (N * C*D*D floats): the `d_som(som.get_data())` initialisers at
 * Trainer.h:218 and Mapper.h:140. */
int pink_hip_set_som(pink_hip_ctx *ctx, const float *host_som);
/* Trainer<...,true>::update_som() (Trainer.h:306-309): device SOM -> host. */
int pink_hip_get_som(pink_hip_ctx *ctx, float *host_som);

/* Trainer<...,true>::operator()(Data const&) (Trainer.h:263-304) applied to n_images
 * images in order with sequential SOM semantics (image k+1 sees the weights left by
 * image k, Pink/main_generic.h:87-89); n_images = 1 is exactly one operator() call.
 * bmu_out receives the best-matching neuron of each image, which the caller adds to
 * m_update_info (Trainer.h:302-303); the call then returns when they are there.
 * With bmu_out NULL and up to 128 KiB of images the call only copies the images into a
 * pinned buffer and returns (operator() returns nothing either); they are trained, in
 * order, a launch group (up to 64 images; 256 for small uint8 trainers) at a time: when the group is full or when any
 * other call on the context follows.  A loop of per-image calls then runs at the rate of
 * the kernels (the rotation of a group is one launch), not of per-image launches and
 * round trips, and leaves the weights of training call by call.  pink_hip_get_som,
 * pink_hip_update_counts and pink_hip_synchronize wait for that work; an error in it is
 * reported by the call that starts or waits for it. */
int pink_hip_train(pink_hip_ctx *ctx, const float *host_images, uint32_t n_images, uint32_t *host_bmu_out);
/* m_update_info (Trainer.h:79,94-95,302-303): how often each of the N neurons was the
 * best match, over all images this context has trained, counted on the device. */
int pink_hip_update_counts(pink_hip_ctx *ctx, uint32_t *host_counts_out);
/* Same with the images already on the device and the BMUs left on the device;
 * asynchronous on the context's stream (see pink_hip_synchronize).  A small uint8 trainer
 * (at most 64 neurons, 32 variants, 2048 elements per neuron) trains a launch group of up
 * to 256 images in ONE launch whose blocks stay on the device and exchange one word per
 * image; the host waits for each such launch and learns from it whether every block saw
 * the others in time (they do unless other work keeps the device's compute units busy for
 * seconds).  If not, nothing of the context has changed, the group is trained again with
 * one launch per image, and the context stays with that form.  The environment variable
 * PINK_HIP_RESIDENT_TRAINER=0, read when a context is created, selects the one launch per
 * image from the start. */
int pink_hip_train_device(pink_hip_ctx *ctx, const float *dev_images, uint32_t n_images, uint32_t *dev_bmu_out);

/* Mapper<...,true>::operator()(Data const&) (Mapper.h:181-208) for n_images images:
 * heatmap_out[i*N + n] = sqrt(min over rotations of the distance), already square-rooted
 * (Mapper.h:206); best_rot_out[i*N + n] = index of that rotation (may be NULL).
 * A call that brings 32 MB of images or more starts three helper threads in the context (kept until
 * pink_hip_destroy) that copy the input into pinned memory beside the calling thread. */
int pink_hip_map(pink_hip_ctx *ctx, const float *host_images, uint32_t n_images,
                 float *host_heatmap_out, uint32_t *host_best_rot_out);
int pink_hip_map_device(pink_hip_ctx *ctx, const float *dev_images, uint32_t n_images,
                        float *dev_heatmap_out, uint32_t *dev_best_rot_out);

/* pink_hip_map_device for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments and results as pink_hip_map_device, but the per-group buffers of the call (argmin keys,
 * packed variant operand, variant norms, float variants where a kernel of its own packs them) are taken
 * from a static device array of PINK_HIP_STATIC_SCRATCH_BYTES that every GPU holds from the moment the
 * library is loaded until the process ends, not from the context's own allocations; the call itself
 * allocates and frees nothing and clears the part of the array it uses with a kernel.  Images are
 * processed in groups of as many as fit the array (less its last KiB, which kernels that read ahead of
 * their operand may touch); PINK_HIP_EINVAL when a single image of the context
 * does not fit (the message says how many bytes it needs), PINK_HIP_ESTATE on a trainer, while
 * per-kernel timing is on (event records allocate), or on a context created with
 * PINK_HIP_KERNEL_MFMA_F32 (that measurement-only kernel choice keeps its operands in buffers of the
 * context).  All contexts on a GPU share the one array: calls
 * that overlap on the same GPU (two contexts, two streams) race; calls one after the other are fine. */
#define PINK_HIP_STATIC_SCRATCH_BYTES (32u << 20)
int pink_hip_map_device_static(pink_hip_ctx *ctx, const float *dev_images, uint32_t n_images,
                               float *dev_heatmap_out, uint32_t *dev_best_rot_out);

/* Wait for everything queued on the context's stream. */
int pink_hip_synchronize(pink_hip_ctx *ctx);

/* Debug taps used by the parity tests.
 * pink_hip_rotate: SpatialTransformerGPU alone (CudaLib/generate_rotated_images.h:57-294):
 *   variants_out holds R*C*D*D floats, variant k at ((k*C + c)*D + x)*D + y.
 * pink_hip_distance: rotate + generate_euclidean_distance_matrix for one image against
 *   the current SOM: dist_out[N] (float distance; integer modes: float(double(ssd)/factor^2)),
 *   ssd_out[N] (exact integer sum, integer modes only; may be NULL), best_rot_out[N]. */
int pink_hip_rotate(pink_hip_ctx *ctx, const float *host_image, float *host_variants_out);
int pink_hip_distance(pink_hip_ctx *ctx, const float *host_image, float *host_dist_out,
                      int64_t *host_ssd_out, uint32_t *host_best_rot_out);

/* Number of elements in the distance region (incl. channels) as the context counts it. */
uint32_t pink_hip_region_size(const pink_hip_ctx *ctx);
/* The distance kernel the context runs: PINK_HIP_KERNEL_VALU, _MFMA, _MFMA_SYM, _MFMA_GEMM or _MFMA_F32. */
uint32_t pink_hip_distance_kernel(const pink_hip_ctx *ctx);

/* Per-kernel timing with HIP events on the context's stream.  While enabled every
 * launch of the rotation, distance and update kernels is bracketed by two events
 * (launches of one kernel that follow each other directly, as a small float32
 * trainer's one launch per image does within a group, share one pair);
 * pink_hip_kernel_times synchronises and returns, per kernel class, the number of
 * launches and their summed duration in milliseconds since the last reset.
 * Index: 0 rotation, 1 operand packing, 2 distance, 3 update, 4 finalise. */
#define PINK_HIP_NUM_KERNEL_CLASSES 5
int pink_hip_set_profiling(pink_hip_ctx *ctx, int enable);
int pink_hip_kernel_times(pink_hip_ctx *ctx, uint64_t *launches_out, double *ms_out);

/* cuda_print_properties() / cuda_get_gpu_ids() (CudaLib/CudaLib.h:15-18): writes a
 * one-line description of every visible device into buf; returns the device count
 * or a negative status. */
int pink_hip_device_info(char *buf, size_t len);

/* Host-only helpers for the matrix a trainer context is created with: the loop in
 * TrainerCommon's constructor (Trainer.h:69-76) over SOMLayout::get_distance
 * (CartesianLayout.h:47-60,103-129 for 1/2/3 dimensions given as dims[0..ndims);
 * HexagonalLayout.h:79-104 with dims[0] = the odd edge length) and one of the
 * functors of UtilitiesLib/DistributionFunctor.cpp:19-59 (`sigma` is the step width
 * for PINK_HIP_STEP).  factors_out holds N*N floats, N = pink_hip_som_size(...). */
uint32_t pink_hip_som_size(uint32_t layout, const uint32_t *dims, uint32_t ndims);
/* SOMLayout::get_distance(i, j) for all pairs (N*N floats): what a caller with its own
 * distribution function (the std::function<float(float)> of Trainer.h:211) evaluates it on. */
int pink_hip_layout_distances(uint32_t layout, const uint32_t *dims, uint32_t ndims, float *distances_out);

/* Host-only helpers for the callers either side of the path.
 * pink_hip_shuffled_order: the order in which DataIteratorShuffled visits a data file of n entries
 * (DataIteratorShuffled.h:62-69: iota, std::default_random_engine(seed), std::mt19937 seeded with its
 * first draw, std::shuffle); the training loop uses seed + iteration (Pink/main_generic.h:83-84).
 * pink_hip_fill_random_uniform: fill_random_uniform of UtilitiesLib/Filler.h:16-25, the SOM
 * initialisation "random" (SOM.h:79-80): std::mt19937(seed), uniform_real_distribution<float>(0, 1). */
int pink_hip_shuffled_order(uint64_t seed, uint32_t n, uint32_t *order_out);
int pink_hip_fill_random_uniform(float *values_out, size_t length, uint32_t seed);
int pink_hip_make_update_factors(uint32_t layout, const uint32_t *dims, uint32_t ndims, uint32_t functor,
                                 float sigma, float damping, float max_update_distance, float *factors_out);

int pink_hip_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif

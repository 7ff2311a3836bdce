// pink_hip.hip -- HIP kernels (gfx950) and the C ABI declared in include/pink_hip.h.
//
// One context = the device half of one reference Trainer<...,true> / Mapper<...,true>
// (src/SelfOrganizingMapLib/Trainer.h:201-335, Mapper.h:129-230).  The kernels are
// written for CDNA4: 64-lane wavefronts, lanes own rotations so that every global
// access of the hot loop is a coalesced 256-byte row, neuron values arrive through
// DPP broadcasts or scalar loads, and the argmin over rotations is a packed 64-bit
// atomic minimum.
//
// Numerical contract (what the parity tests check against the CPU path):
//   * rotated pixels: every product and sum rounded separately, in the order of
//     ImageProcessingLib/rotate.h:37-63  -> bit-identical to the CPU;
//   * float32 distance: one lane owns one (neuron, rotation) pair and accumulates
//     fma(d, d, acc) over the region in the CPU's element order
//     (ImageProcessingLib/euclidean_distance.h:47-100: the CPU squares in double and
//     rounds the running sum to double, then to float, at every step; a fused
//     multiply-add rounds once, which differs from that by one unit in the last place
//     about once in 2^29 steps -- within the 1e-5 gate by orders of magnitude, and
//     bit-equal on the tests' seeds);
//   * integer distance: exact sums of squared differences of quantised values;
//   * update: w - ((w - x) * f), three roundings (SelfOrganizingMapLib/Trainer.h:175).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>
#include <string>
#include <type_traits>
#include <vector>

#include <condition_variable>
#include <memory>
#include <mutex>
#include <thread>

#include "mfma_u8_sym.h"
#include "pink_hip.h"

// Scratch of pink_hip_map_device_static, the entry point for callers that cannot allocate: the
// per-group buffers of a mapping call (argmin keys, the packed variant operand, variant norms, float
// variants where a kernel of its own packs them) live in this array instead of in buffers the
// context allocated.  Every GPU the library runs on holds its own copy at its own address until the
// process ends; host code reaches it only through the address hipGetSymbolAddress returns for the
// current device (the name below is a host-side stand-in, not a device address).
static __device__ __align__(256) unsigned char scratch[PINK_HIP_STATIC_SCRATCH_BYTES];

// Timestamp probes, in builds made with -DPINK_PROBE only (measurement builds; the shipped library has
// none): wave w of block b of kernel k stores the 100 MHz constant clock at the places marked
// PROBE(k, b, slot); pink_hip_probe_read copies the stamps of the last launch of each kernel out.
#ifdef PINK_PROBE
constexpr uint32_t kProbeKernels = 5, kProbeBlocks = 2048, kProbeWaves = 8, kProbeSlots = 8;
static __device__ unsigned long long g_probe[kProbeKernels * kProbeBlocks * kProbeWaves * kProbeSlots];
__device__ __forceinline__ void probe_stamp(uint32_t kernel, uint32_t block, uint32_t slot)
{
    if ((threadIdx.x & 63) == 0 && block < kProbeBlocks)
        g_probe[((kernel * kProbeBlocks + block) * kProbeWaves + ((threadIdx.x >> 6) & (kProbeWaves - 1))) * kProbeSlots + slot] =
            wall_clock64();
}
#define PROBE(kernel, block, slot) probe_stamp(kernel, block, slot)
#else
#define PROBE(kernel, block, slot) ((void)(kernel), (void)(block), (void)(slot))
#endif
constexpr uint32_t kProbeRotate = 0, kProbeGemm = 1, kProbeUpdate = 2, kProbeTrainF32 = 3, kProbeResident = 4;

namespace {

constexpr uint32_t kWave = 64;
constexpr uint32_t kEpadMultiple = 64;   // region length padded so k-loops need no tail
constexpr int kClsRotate = 0, kClsPack = 1, kClsDist = 2, kClsUpdate = 3, kClsFinal = 4;

thread_local std::string g_create_error;

inline uint32_t round_up(uint32_t v, uint32_t m) { return (v + m - 1) / m * m; }

// ---------------------------------------------------------------------------------
// Device helpers
// ---------------------------------------------------------------------------------

__device__ __forceinline__ unsigned long long wave_min_u64(unsigned long long v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        unsigned long long o = __shfl_xor(v, off, 64);
        v = o < v ? o : v;
    }
    return v;
}

// Minimum of a 32-bit value over the wave by DPP (within quads, rows of 16, then across the rows into lane 63):
// no LDS round trips, for waves that have their SIMD to themselves and pay for every instruction's latency.
__device__ __forceinline__ uint32_t wave_min_u32_dpp(uint32_t v)
{
#define PINK_DPP_MIN(ctrl, rows) \
    v = min(v, (uint32_t)__builtin_amdgcn_update_dpp((int)0xffffffffu, (int)v, ctrl, rows, 0xf, false))
    PINK_DPP_MIN(0xb1, 0xf);      // quad_perm [1, 0, 3, 2]
    PINK_DPP_MIN(0x4e, 0xf);      // quad_perm [2, 3, 0, 1]
    PINK_DPP_MIN(0x141, 0xf);     // row_half_mirror
    PINK_DPP_MIN(0x140, 0xf);     // row_mirror
    PINK_DPP_MIN(0x142, 0xa);     // row_bcast:15 into rows 1 and 3
    PINK_DPP_MIN(0x143, 0xc);     // row_bcast:31 into rows 2 and 3
#undef PINK_DPP_MIN
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// The smallest 64-bit value of the wave and the smallest index among the lanes that hold it, the same way: the
// high words, then the low words of the lanes that are still in, then their indices.
__device__ __forceinline__ void wave_first_min_u64_dpp(unsigned long long &v, uint32_t &idx)
{
    const uint32_t hi = (uint32_t)(v >> 32), lo = (uint32_t)v;
    const uint32_t mh = wave_min_u32_dpp(hi);
    const uint32_t ml = wave_min_u32_dpp(hi == mh ? lo : 0xffffffffu);
    idx = wave_min_u32_dpp(hi == mh && lo == ml ? idx : 0xffffffffu);
    v = ((unsigned long long)mh << 32) | ml;
}

// Sum of a 32-bit integer over the wave, the same way.
__device__ __forceinline__ int wave_sum_i32_dpp(int v)
{
#define PINK_DPP_ADD(ctrl, rows) v += __builtin_amdgcn_update_dpp(0, v, ctrl, rows, 0xf, false)
    PINK_DPP_ADD(0xb1, 0xf);      // pairs
    PINK_DPP_ADD(0x4e, 0xf);      // quads
    PINK_DPP_ADD(0x141, 0xf);     // halves of a row
    PINK_DPP_ADD(0x140, 0xf);     // rows
    PINK_DPP_ADD(0x142, 0xa);     // row 0 into 1, row 2 into 3
    PINK_DPP_ADD(0x143, 0xc);     // rows 0 + 1 into 2 and 3
#undef PINK_DPP_ADD
    return __builtin_amdgcn_readlane(v, 63);
}

// The key `bits << 32 | first + lane` of the lane with the smallest bits (the first such lane), lanes with
// valid == false left out; all ones when no lane is valid.
__device__ __forceinline__ unsigned long long wave_min_key_dpp(uint32_t bits, bool valid, uint32_t first)
{
    const uint32_t best = wave_min_u32_dpp(valid ? bits : 0xffffffffu);
    const unsigned long long hit = __ballot(valid && bits == best);
    return hit ? ((unsigned long long)best << 32) | (first + (uint32_t)__builtin_ctzll(hit)) : ~0ull;
}

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// Zero `n16` 16-byte words (a kernel, not a memset: a caller may be capturing the stream into a graph).
__global__ __launch_bounds__(256) void k_fill_zero(v4i *__restrict__ p, size_t n16)
{
    const v4i z = {0, 0, 0, 0};
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < n16; t += (size_t)gridDim.x * blockDim.x) p[t] = z;
}

// q = T(x * factor) truncated, saturated to [0, factor] (CudaLib/copy_and_transform_kernel.h:27-28)
__device__ __forceinline__ int32_t quantise(float x, float factor)
{
    const float v = __fmul_rn(x, factor);
    if (!(v > 0.0f)) return 0;
    if (v >= factor) return (int32_t)factor;
    return (int32_t)v;
}

// Value of base rotation `i` (angle i * 2pi / num_rot, 0 <= angle < 90 degrees) of one
// channel at neuron pixel (x, y).  i == 0 is the centre crop / centre pad of
// ImageProcessingLib/resize.h:15-40; i > 0 is ImageProcessingLib/rotate.h:31-65 with
// the operation order kept (no contraction).
__device__ __forceinline__ float base_pixel(const float *__restrict__ img, uint32_t I, uint32_t D,
                                            uint32_t i, float cs, float sn, uint32_t x, uint32_t y)
{
    if (i == 0) {
        if (I >= D) {
            uint32_t m = (I - D) / 2;
            return img[(size_t)(x + m) * I + (y + m)];
        }
        uint32_t m = (D - I) / 2;
        uint32_t sx = x - m, sy = y - m;           // wraps for x < m: caught by the range test
        return (sx < I && sy < I) ? img[(size_t)sx * I + sy] : 0.0f;
    }
    const float src_c = __fmul_rn((float)(I - 1), 0.5f);
    const float dst_c = __fmul_rn((float)(D - 1), 0.5f);
    const float px = __fsub_rn((float)x, dst_c);
    const float py = __fsub_rn((float)y, dst_c);
    const float sxf = __fadd_rn(__fsub_rn(__fmul_rn(px, cs), __fmul_rn(py, sn)), src_c);
    const float syf = __fadd_rn(__fadd_rn(__fmul_rn(px, sn), __fmul_rn(py, cs)), src_c);
    const float lim = (float)(I - 1);
    if (sxf < 0.0f || sxf > lim || syf < 0.0f || syf > lim) return 0.0f;
    const uint32_t ix = (uint32_t)sxf, iy = (uint32_t)syf;
    const float rx = __fsub_rn(sxf, (float)ix), ry = __fsub_rn(syf, (float)iy);
    const float cx = __fsub_rn(1.0f, rx), cy = __fsub_rn(1.0f, ry);
    // The neighbours one past the last row / column carry weight 0; clamp their index.
    const uint32_t last = I * I - 1;
    const uint32_t i00 = ix * I + iy;
    const uint32_t i01 = min(i00 + 1, last);
    const uint32_t i10 = min(i00 + I, last);
    const uint32_t i11 = min(i00 + I + 1, last);
    const float a = __fmul_rn(__fmul_rn(cx, cy), img[i00]);
    const float b = __fmul_rn(__fmul_rn(cx, ry), img[i01]);
    const float c = __fmul_rn(__fmul_rn(rx, cy), img[i10]);
    const float d = __fmul_rn(__fmul_rn(rx, ry), img[i11]);
    return __fadd_rn(__fadd_rn(__fadd_rn(a, b), c), d);
}

// base_pixel for U pixels of a base rotation i > 0 at once, without branches: the 4 U image taps are all
// requested before the first is used (a block's fill of its LDS tile is a chain of such round trips
// otherwise).  A pixel that maps outside the image reads clamped positions and comes out as 0, like
// base_pixel's early return; the arithmetic of the others is base_pixel's, operation for operation.
template <int U>
__device__ __forceinline__ void base_pixels(const float *__restrict__ img, uint32_t I, uint32_t D, float cs, float sn,
                                            const uint32_t (&x)[U], const uint32_t (&y)[U], float (&out)[U])
{
    const float src_c = __fmul_rn((float)(I - 1), 0.5f);
    const float dst_c = __fmul_rn((float)(D - 1), 0.5f);
    const float lim = (float)(I - 1);
    const uint32_t last = I * I - 1;
    float rx[U], ry[U], t00[U], t01[U], t10[U], t11[U];
    bool inside[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const float px = __fsub_rn((float)x[u], dst_c);
        const float py = __fsub_rn((float)y[u], dst_c);
        const float sxf = __fadd_rn(__fsub_rn(__fmul_rn(px, cs), __fmul_rn(py, sn)), src_c);
        const float syf = __fadd_rn(__fadd_rn(__fmul_rn(px, sn), __fmul_rn(py, cs)), src_c);
        inside[u] = !(sxf < 0.0f || sxf > lim || syf < 0.0f || syf > lim);
        const float sxc = inside[u] ? sxf : 0.0f, syc = inside[u] ? syf : 0.0f;
        const uint32_t ix = (uint32_t)sxc, iy = (uint32_t)syc;
        rx[u] = __fsub_rn(sxc, (float)ix);
        ry[u] = __fsub_rn(syc, (float)iy);
        const uint32_t i00 = ix * I + iy;
        t00[u] = img[i00];
        t01[u] = img[min(i00 + 1, last)];
        t10[u] = img[min(i00 + I, last)];
        t11[u] = img[min(i00 + I + 1, last)];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const float cx = __fsub_rn(1.0f, rx[u]), cy = __fsub_rn(1.0f, ry[u]);
        const float a = __fmul_rn(__fmul_rn(cx, cy), t00[u]);
        const float b = __fmul_rn(__fmul_rn(cx, ry[u]), t01[u]);
        const float c = __fmul_rn(__fmul_rn(rx[u], cy), t10[u]);
        const float d = __fmul_rn(__fmul_rn(rx[u], ry[u]), t11[u]);
        out[u] = inside[u] ? __fadd_rn(__fadd_rn(__fadd_rn(a, b), c), d) : 0.0f;
    }
}

// Quotient and remainder of a dividend below 2^24: the float reciprocal's estimate is within one of the
// quotient and is corrected (a quarter of the instructions of the general 32-bit division).
struct RcpDivisor {
    uint32_t d;
    float rcp;
    __device__ explicit RcpDivisor(uint32_t d_) : d(d_), rcp(1.0f / (float)max(d_, 1u)) {}
    __device__ __forceinline__ void divmod(uint32_t n, uint32_t &q, uint32_t &r) const
    {
        uint32_t e = (uint32_t)((float)n * rcp);
        int rem = (int)(n - e * d);
        if (rem < 0) { --e; rem += (int)d; }
        else if ((uint32_t)rem >= d) { ++e; rem -= (int)d; }
        q = e; r = (uint32_t)rem;
    }
};

// ---------------------------------------------------------------------------------
// Rotation: all num_rot * (flip ? 2 : 1) variants of a batch of images.
// Block (i, c, b) computes base rotation i of channel c of image b once, keeps it in
// LDS, and writes the 4 quarter turns and their flips as pure index permutations, each
// variant row-major so that consecutive lanes store consecutive addresses.
// Variant k = f * num_rot + q * (num_rot / 4) + i at rot[((b * R + k) * C + c) * D * D].
// Quarter turn q of base B (ImageProcessingLib/rotate_90_degrees.h:15-26 applied q times):
//   Q1[x][y] = B[D-1-y][x], Q2[x][y] = B[D-1-x][D-1-y], Q3[x][y] = B[y][D-1-x];
// flip (ImageProcessingLib/flip.h:14-30): F[x][y] = V[D-1-x][y].
// Block (0, 0, b) also resets the image's argmin keys.
// ---------------------------------------------------------------------------------
// Operand packing fused into the rotation kernel (blocks that hold their base rotation in LDS):
// the region of every variant goes straight from LDS into the distance kernel's operand, so the
// variants are not read back.  symoff[sym * Epad + e] = channel << 24 | position in the base
// rotation of region element e under symmetry sym = flip * 4 + quarter (PACK 2 / 3: the position alone, 16 bits).
//   PACK 1: float32 rows, opnd[(b * Rpad + k) * Epad + e]            (k = variant index)
//   PACK 2 / 3: uint8 / uint16 byte planes in MFMA fragment order (see mfma_int_gemm.inc) and
//               the row norms |V|^2; single channel only.
struct PackArgs {
    const uint32_t *symoff;
    void *opnd;            // float rows, or byte planes
    long long *norm;       // integer modes: [b][Rp]
    uint32_t E, Epad, rows_pad, KS;
};

template <int PACK, int TILE>
__global__ __launch_bounds__(1024) void k_rotate(const float *__restrict__ images, float *__restrict__ rot,
                                                const float *__restrict__ cos_t, const float *__restrict__ sin_t,
                                                unsigned long long *__restrict__ key, uint32_t N,
                                                uint32_t C, uint32_t I, uint32_t D, uint32_t num_rot,
                                                uint32_t use_flip, uint32_t Dp, PackArgs pk,
                                                uint32_t store_variants, uint32_t lo, uint32_t hi, uint32_t nch)
{
    // the base rotation, rows of Dp floats (odd): the quarter turns read it along columns, and an odd
    // stride keeps those reads in different banks (a stride of 64 would put all of them into one)
    // TILE 1: as described; 2: neurons too large for that, the image channel is in LDS instead and every
    // element is interpolated out of it where it is needed; 0: neither fits, the image is read from memory
    extern __shared__ float s_base[];
    __shared__ unsigned long long s_norm[8];
    constexpr bool use_lds = TILE == 1;
    // a block holds the base rotation of nch channels (TILE 1: one, or all of them when they fit LDS
    // together, which lets the byte planes of multi-channel data be packed here; else one), tile after tile
    const uint32_t i = blockIdx.x, c = blockIdx.y * nch, b = blockIdx.z;
    const uint32_t tile = D * Dp;
    const uint32_t nrr = num_rot / 4;
    const uint32_t R = num_rot * (use_flip ? 2u : 1u);
    const uint32_t DD = D * D;
    const float *img = images + ((size_t)b * C + c) * I * I;
    float *out = rot + (size_t)b * R * C * DD;
    const float cs = i ? cos_t[i] : 1.0f, sn = i ? sin_t[i] : 0.0f;
    const uint32_t nq = num_rot == 1 ? 1u : 4u, nf = use_flip ? 2u : 1u;

    const uint32_t probe_block = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
    PROBE(kProbeRotate, probe_block, 0);
    if (i == 0 && c == 0)
        for (uint32_t n = threadIdx.x; n < N; n += blockDim.x) key[(size_t)b * N + n] = ~0ull;
    if (PACK >= 2 && threadIdx.x < 8) s_norm[threadIdx.x] = 0;

    // Pixel (a, bb) of the base rotation: out of the LDS tile, or, for neurons too large for one,
    // computed where it is needed (every stored or packed element then costs one interpolation, which
    // is cheaper than strided stores of values computed once).  Positions arrive as a * Dp + bb.
    // (cc = channel within the block; TILE 0 and 2 have one channel per block)
    auto sample = [&](uint32_t cc, uint32_t a, uint32_t bb) {
        if constexpr (TILE == 1) return s_base[cc * tile + a * Dp + bb];
        else if constexpr (TILE == 2) return base_pixel(s_base, I, D, i, cs, sn, a, bb);
        else return base_pixel(img, I, D, i, cs, sn, a, bb);
    };
    const RcpDivisor by_Dp(Dp);
    auto sample_at = [&](uint32_t po) {               // po: position in the block's LDS tiles
        if constexpr (use_lds) return s_base[po];
        else {
            uint32_t a, bb;
            by_Dp.divmod(po, a, bb);
            return sample(0, a, bb);
        }
    };
    if constexpr (TILE == 2) {
        for (uint32_t p = threadIdx.x; p < I * I; p += blockDim.x) s_base[p] = img[p];
        __syncthreads();
    }
    if constexpr (use_lds) {
        // rows and columns [lo, hi) of the base rotation: all of it, or, when only the packed operand is
        // wanted, the square that the region reaches under the eight symmetries
        const uint32_t side = hi - lo;
        const RcpDivisor by_side(side);
        for (uint32_t cc = 0; cc < nch; ++cc) {
            const float *im = img + (size_t)cc * I * I;
            // Where 8 x 8 patches cover the square with little waste, a wave takes a patch per round and a thread two
            // pixels whose taps are all requested before the first is used: the taps of a patch lie in a dozen rows
            // of the image whatever the angle, where 64 pixels of one row spread over up to 64 sin(angle) rows, each
            // a cache line of its own for the gather.  Otherwise (and for the centre crop) pixel by pixel along rows.
            const uint32_t pw = (side + 7) / 8, cells = pw * pw * 64;
            if (i == 0 || cells * 8 > side * side * 9) {
                for (uint32_t p = threadIdx.x; p < side * side; p += blockDim.x) {
                    uint32_t qx, qy;
                    by_side.divmod(p, qx, qy);
                    s_base[cc * tile + (lo + qx) * Dp + lo + qy] = base_pixel(im, I, D, i, cs, sn, lo + qx, lo + qy);
                }
            } else {
                constexpr int kFillU = 2;
                const RcpDivisor by_pw(pw);
                for (uint32_t t = threadIdx.x; t < cells; t += blockDim.x * kFillU) {
                    uint32_t x[kFillU], y[kFillU];
                    float v[kFillU];
                    bool live[kFillU];
#pragma unroll
                    for (int u = 0; u < kFillU; ++u) {
                        const uint32_t cell = t + u * blockDim.x;
                        uint32_t px, py;
                        by_pw.divmod(cell >> 6, px, py);
                        const uint32_t qx = px * 8 + ((cell >> 3) & 7), qy = py * 8 + (cell & 7);
                        live[u] = cell < cells && qx < side && qy < side;
                        x[u] = lo + min(qx, side - 1); y[u] = lo + min(qy, side - 1);
                    }
                    base_pixels<kFillU>(im, I, D, cs, sn, x, y, v);
#pragma unroll
                    for (int u = 0; u < kFillU; ++u)
                        if (live[u]) s_base[cc * tile + x[u] * Dp + y[u]] = v[u];
                }
            }
        }
        __syncthreads();
    }
    PROBE(kProbeRotate, probe_block, 1);
    {
        // store_variants 0: none (a mapper whose distance operand is packed below never reads the variants);
        // 1: all; 2: the base rotation and its quarter turn, of which the other six are row and column
        // reversals (the update kernel reads them that way)
        const uint32_t nf_st = store_variants == 2 ? 1u : nf, nq_st = store_variants == 2 ? min(nq, 2u) : nq;
        const RcpDivisor by_D(D);
        for (uint32_t cc = 0; cc < (store_variants ? nch : 0u); ++cc)
            for (uint32_t p = threadIdx.x; p < DD; p += blockDim.x) {
                uint32_t x, y;
                if (DD <= (1u << 24)) by_D.divmod(p, x, y);        // (the reciprocal is exact below 2^24)
                else { x = p / D; y = p % D; }
                for (uint32_t f = 0; f < nf_st; ++f) {
                    const uint32_t xs = f ? D - 1 - x : x;
                    for (uint32_t q = 0; q < nq_st; ++q) {
                        uint32_t a, bb;
                        switch (q) {
                        case 0: a = xs; bb = y; break;
                        case 1: a = D - 1 - y; bb = xs; break;
                        case 2: a = D - 1 - xs; bb = D - 1 - y; break;
                        default: a = y; bb = D - 1 - xs; break;
                        }
                        const uint32_t k = f * num_rot + q * nrr + i;
                        out[((size_t)k * C + c + cc) * DD + p] = sample(cc, a, bb);
                    }
                }
            }
        PROBE(kProbeRotate, probe_block, 2);
        if constexpr (PACK == 1) {
            float *opnd = (float *)pk.opnd + (size_t)b * pk.rows_pad * pk.Epad;
            for (uint32_t f = 0; f < nf; ++f)
                for (uint32_t q = 0; q < nq; ++q) {
                    const uint32_t *so = pk.symoff + (size_t)(f * 4 + q) * pk.Epad;
                    float *row = opnd + (size_t)(f * num_rot + q * nrr + i) * pk.Epad;
                    for (uint32_t e = threadIdx.x; e < pk.E; e += blockDim.x) {
                        const uint32_t po = so[e], cc = (po >> 24) - c;      // (wraps below the block's first channel)
                        if (cc < nch) row[e] = sample_at(cc * tile + (po & 0xffffffu));
                    }
                }
        } else if constexpr (PACK >= 2) {
            // One work item = one 16-byte piece of one of the block's (up to 8) rows; the items of all
            // rows are dealt to the threads in one sequence, so the last round is the only partial one.
            // The rows of the block are adjacent in the operand: nsym neighbouring lanes store 16 nsym
            // consecutive bytes.
            // Four elements at a time: quantise (clamp, truncate), bytes gathered with v_perm, q - 128 (or
            // the two bytes of q - 32768 with the low one shifted by 128) = the bytes XOR 0x80, squares by
            // dot4: |256 h + l|^2 = 65536 h.h + 512 h.l + l.l.
            constexpr bool U16 = PACK == 3;
            constexpr uint32_t planes = U16 ? 2 : 1;
            const float factor = U16 ? 65535.0f : 255.0f;
            const size_t plane_stride = (size_t)(pk.rows_pad / 32) * pk.KS * 64;
            v4i *P = (v4i *)pk.opnd + (size_t)b * planes * plane_stride;
            const uint32_t pieces = pk.KS * 2, nsym = nf * nq;
            auto clamp_q = [&](uint32_t po) {
                const float v = fminf(fmaxf(__fmul_rn(sample_at(po), factor), 0.0f), factor);   // NaN -> 0
                return (uint32_t)v;
            };
            for (uint32_t item = threadIdx.x; item < nsym * pieces; item += blockDim.x) {
                const uint32_t si = item % nsym, piece = item / nsym;   // neighbouring lanes: the adjacent rows of one piece
                const uint32_t f = si / nq, q = si % nq, sym = f * 4 + q;
                const uint32_t r = i * nsym + si;             // operand row: the symmetries of a base rotation are adjacent
                // (16-bit table entries with LDS tiles: at most 40 448 floats; 32-bit without)
                const uint2 *so4 = (const uint2 *)((const unsigned short *)pk.symoff + (size_t)sym * pk.Epad + piece * 16);
                const uint4 *so4w = (const uint4 *)(pk.symoff + (size_t)sym * pk.Epad + piece * 16);
                v4i hi = {0, 0, 0, 0}, lo = {0, 0, 0, 0};
                int hh = 0, hl = 0, ll = 0;
#pragma unroll
                for (int w4 = 0; w4 < 4; ++w4) {
                    uint32_t p0, p1, p2, p3;
                    if constexpr (use_lds) {
                        const uint2 pv = so4[w4];
                        p0 = pv.x & 0xffffu; p1 = pv.x >> 16; p2 = pv.y & 0xffffu; p3 = pv.y >> 16;
                    } else {
                        const uint4 pv = so4w[w4];
                        p0 = pv.x; p1 = pv.y; p2 = pv.z; p3 = pv.w;
                    }
                    const uint32_t k0 = piece * 16 + w4 * 4;
                    const uint32_t valid = pk.E > k0 ? min(pk.E - k0, 4u) : 0u;
                    const uint32_t live = valid >= 4 ? 0xffffffffu : (1u << (8 * valid)) - 1u;
                    const uint32_t q0 = clamp_q(p0), q1 = clamp_q(p1), q2 = clamp_q(p2), q3 = clamp_q(p3);
                    if constexpr (U16) {
                        const uint32_t w01 = q0 | (q1 << 16), w23 = q2 | (q3 << 16);
                        const int h = (int)((__builtin_amdgcn_perm(w23, w01, 0x07050301u) ^ 0x80808080u) & live);
                        const int l = (int)((__builtin_amdgcn_perm(w23, w01, 0x06040200u) ^ 0x80808080u) & live);
                        hi[w4] = h; lo[w4] = l;
                        hh = __builtin_amdgcn_sdot4(h, h, hh, false);
                        hl = __builtin_amdgcn_sdot4(h, l, hl, false);
                        ll = __builtin_amdgcn_sdot4(l, l, ll, false);
                    } else {
                        const int h = (int)(((q0 | (q1 << 8) | (q2 << 16) | (q3 << 24)) ^ 0x80808080u) & live);
                        hi[w4] = h;
                        hh = __builtin_amdgcn_sdot4(h, h, hh, false);
                    }
                }
                const size_t frag = ((size_t)(r >> 5) * pk.KS + (piece >> 1)) * 64 + (r & 31) + 32 * (piece & 1);
                P[frag] = hi;
                if (U16) P[plane_stride + frag] = lo;
                const long long sq = U16 ? ((long long)hh << 16) + (long long)hl * 512 + ll : (long long)hh;
                if (sq) atomicAdd(&s_norm[sym], (unsigned long long)sq);
            }
            __syncthreads();
            if (threadIdx.x < 8) {
                const uint32_t f = threadIdx.x >> 2, q = threadIdx.x & 3;
                if (f < nf && q < nq)
                    pk.norm[(size_t)b * pk.rows_pad + i * nsym + f * nq + q] = (long long)s_norm[threadIdx.x];
            }
        }
    }
    PROBE(kProbeRotate, probe_block, 3);
}

// The base rotation and its quarter turn for images and neurons of any size (neither fits LDS): a
// block computes one 32 x 32 tile of base rotation i of one channel.  The pixels of the image that
// the tile's interpolations touch lie in a window of at most 50 x 50 (the tile turned by up to 90
// degrees, plus the neighbours), which goes to LDS first; the arithmetic is base_pixel's, tap by tap.
// The tile is written twice, row-major both times: as it is into variant i, and turned,
// Q1[x][y] = B[D-1-y][x], into variant nrr + i (through LDS, so that both stores run along rows).
// A sample whose neighbours the window does not hold (on the last row or column of the image, where
// base_pixel's clamped neighbour index leaves the row) is left to base_pixel itself.
constexpr uint32_t kRotTile = 32, kRotWindow = 52;

__global__ __launch_bounds__(256) void k_rotate_pair_tiled(const float *__restrict__ images, float *__restrict__ rot,
                                                           const float *__restrict__ cos_t, const float *__restrict__ sin_t,
                                                           unsigned long long *__restrict__ key, uint32_t N, uint32_t C,
                                                           uint32_t I, uint32_t D, uint32_t num_rot, uint32_t use_flip,
                                                           uint32_t tiles_per_row)
{
    __shared__ float s_win[kRotWindow * kRotWindow];
    __shared__ float s_out[kRotTile][kRotTile + 1];
    const uint32_t tile = blockIdx.x, i = blockIdx.y, c = blockIdx.z % C, b = blockIdx.z / C;
    const uint32_t a0 = (tile / tiles_per_row) * kRotTile, b0 = (tile % tiles_per_row) * kRotTile;
    const uint32_t nrr = num_rot / 4, R = num_rot * (use_flip ? 2u : 1u), DD = D * D;
    const float *img = images + ((size_t)b * C + c) * I * I;
    float *out = rot + (size_t)b * R * C * DD;
    const float cs = i ? cos_t[i] : 1.0f, sn = i ? sin_t[i] : 0.0f;
    const uint32_t tid = threadIdx.x;
    if (tile == 0 && i == 0 && c == 0)
        for (uint32_t n = tid; n < N; n += blockDim.x) key[(size_t)b * N + n] = ~0ull;

    const uint32_t a1 = min(a0 + kRotTile, D), b1 = min(b0 + kRotTile, D);        // the tile: rows [a0, a1), columns [b0, b1)
    // source window [wx0, wx1] x [wy0, wy1] of the tile's corners, one pixel of margin on every side
    const float src_c = __fmul_rn((float)(I - 1), 0.5f), dst_c = __fmul_rn((float)(D - 1), 0.5f);
    int wx0 = 0, wx1 = -1, wy0 = 0, wy1 = -1;
    if (i) {
        float lo_x = 3.0e38f, hi_x = -3.0e38f, lo_y = 3.0e38f, hi_y = -3.0e38f;
#pragma unroll
        for (int corner = 0; corner < 4; ++corner) {
            const float px = __fsub_rn((float)((corner & 1) ? a1 - 1 : a0), dst_c);
            const float py = __fsub_rn((float)((corner & 2) ? b1 - 1 : b0), dst_c);
            const float sxf = __fadd_rn(__fsub_rn(__fmul_rn(px, cs), __fmul_rn(py, sn)), src_c);
            const float syf = __fadd_rn(__fadd_rn(__fmul_rn(px, sn), __fmul_rn(py, cs)), src_c);
            lo_x = fminf(lo_x, sxf); hi_x = fmaxf(hi_x, sxf); lo_y = fminf(lo_y, syf); hi_y = fmaxf(hi_y, syf);
        }
        wx0 = max(0, (int)floorf(lo_x) - 1); wx1 = min((int)I - 1, (int)floorf(hi_x) + 2);
        wy0 = max(0, (int)floorf(lo_y) - 1); wy1 = min((int)I - 1, (int)floorf(hi_y) + 2);
        // a tile that maps beyond the image (neurons larger than the image) has an empty window: every
        // sample is then outside; a window beyond the LDS array cannot occur, and would send all samples
        // down the slow path
        if (wx1 < wx0 || wy1 < wy0 || wx1 - wx0 + 1 > (int)kRotWindow || wy1 - wy0 + 1 > (int)kRotWindow) { wx1 = wx0 - 1; wy1 = wy0 - 1; }
    }
    const int ww = wy1 - wy0 + 1, wh = wx1 - wx0 + 1;
    for (int p = (int)tid; p < ww * wh; p += (int)blockDim.x) {
        const int r = p / ww, q = p - r * ww;
        s_win[r * ww + q] = img[(size_t)(wx0 + r) * I + (wy0 + q)];
    }
    __syncthreads();

    const uint32_t tx = tid & 31, ty = tid >> 5;
    for (uint32_t rr = ty; rr < kRotTile; rr += 8) {
        const uint32_t x = a0 + rr, y = b0 + tx;
        float v = 0.0f;
        if (x < D && y < D) {
            bool done = false;
            if (i) {
                const float px = __fsub_rn((float)x, dst_c), py = __fsub_rn((float)y, dst_c);
                const float sxf = __fadd_rn(__fsub_rn(__fmul_rn(px, cs), __fmul_rn(py, sn)), src_c);
                const float syf = __fadd_rn(__fadd_rn(__fmul_rn(px, sn), __fmul_rn(py, cs)), src_c);
                const float lim = (float)(I - 1);
                if (sxf < 0.0f || sxf > lim || syf < 0.0f || syf > lim) {
                    done = true;                           // outside the image: 0
                } else {
                    const int ix = (int)sxf, iy = (int)syf;
                    if (ix >= wx0 && ix + 1 <= wx1 && iy >= wy0 && iy + 1 <= wy1) {
                        const float rx = __fsub_rn(sxf, (float)ix), ry = __fsub_rn(syf, (float)iy);
                        const float cx = __fsub_rn(1.0f, rx), cy = __fsub_rn(1.0f, ry);
                        const float *t = s_win + (ix - wx0) * ww + (iy - wy0);
                        const float ta = __fmul_rn(__fmul_rn(cx, cy), t[0]);
                        const float tb = __fmul_rn(__fmul_rn(cx, ry), t[1]);
                        const float tc = __fmul_rn(__fmul_rn(rx, cy), t[ww]);
                        const float td = __fmul_rn(__fmul_rn(rx, ry), t[ww + 1]);
                        v = __fadd_rn(__fadd_rn(__fadd_rn(ta, tb), tc), td);
                        done = true;
                    }
                }
            }
            if (!done) v = base_pixel(img, I, D, i, cs, sn, x, y);
            out[((size_t)i * C + c) * DD + (size_t)x * D + y] = v;
        }
        s_out[rr][tx] = v;
    }
    if (num_rot == 1) return;                               // a single rotation has no quarter turns
    __syncthreads();
    // Q1[x][y] = B[D-1-y][x]: row x = b0 + r of Q1 takes column r of the tile, rows a1-1 down to a0
    for (uint32_t r = ty; r < kRotTile; r += 8) {
        const uint32_t x = b0 + r, aa = a1 - 1 - tx;         // tile row read by this lane (wraps below a0)
        if (x < D && tx < a1 - a0) out[((size_t)(nrr + i) * C + c) * DD + (size_t)x * D + (D - 1 - aa)] = s_out[aa - a0][r];
    }
}

// Where a packing kernel finds variant r when only two of a base rotation's eight symmetries are
// stored (the base rotation and its quarter turn): the stored variant to read and the region offsets
// to read it with -- the region under the row and/or column reversal that turns the stored variant
// into variant r (see k_update).  off4 = null: every variant is stored, `off` is used as it is.
struct PairSource {
    const uint32_t *off4;      // [rows reversed * 2 + columns reversed][E]
    uint32_t num_rot, nrr, E;
};

__device__ __forceinline__ void pair_source(const PairSource &ps, uint32_t r, uint32_t &src, const uint32_t *&off)
{
    src = r;
    if (!ps.off4) return;
    const uint32_t f = r >= ps.num_rot ? 1u : 0u, rem = r - f * ps.num_rot;
    const uint32_t q = rem / ps.nrr, i = rem - q * ps.nrr;
    src = (q & 1) * ps.nrr + i;
    off = ps.off4 + (size_t)((f ^ (q >> 1)) * 2 + (q >> 1)) * ps.E;
}

// ---------------------------------------------------------------------------------
// Operand packing for the vector-ALU distance kernels.
//   somP[n][k]    = conv(som[n][off[k]])                      k < E, 0 beyond (row length Epad)
//   rotT[b][k][r] = conv(rot[b][r][off[k]])   k-major so that the 64 lanes of a wave
//                   (64 consecutive rotations) read one 256-byte row per k.
// conv: float32 copy, or quantisation q = T(x * factor) saturated to [0, factor]
// (CudaLib/copy_and_transform_kernel.h:27-28) held as int32.
// ---------------------------------------------------------------------------------

template <bool QUANT>
__global__ __launch_bounds__(256) void k_pack_som(const float *__restrict__ som, const uint32_t *__restrict__ off,
                                                  void *__restrict__ somP, uint32_t N, uint32_t S, uint32_t E,
                                                  uint32_t Epad, float factor)
{
    const size_t total = (size_t)N * Epad;
    for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (size_t)gridDim.x * blockDim.x) {
        const uint32_t n = (uint32_t)(t / Epad), k = (uint32_t)(t % Epad);
        const float v = k < E ? som[(size_t)n * S + off[k]] : 0.0f;
        if (QUANT) ((int32_t *)somP)[t] = k < E ? quantise(v, factor) : 0;
        else ((float *)somP)[t] = v;
    }
}

template <bool QUANT>
__global__ __launch_bounds__(256) void k_pack_rot(const float *__restrict__ rot, const uint32_t *__restrict__ off,
                                                  void *__restrict__ rotT, uint32_t R, uint32_t S, uint32_t E,
                                                  uint32_t Epad, uint32_t Rpad, float factor, PairSource ps)
{
    __shared__ float tile[32][33];
    const uint32_t b = blockIdx.z;
    const uint32_t k0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
    const uint32_t tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
    for (uint32_t rr = ty; rr < 32; rr += 8) {
        const uint32_t r = r0 + rr, k = k0 + tx;
        uint32_t src = r;
        const uint32_t *o = off;
        if (r < R) pair_source(ps, r, src, o);
        tile[rr][tx] = (r < R && k < E) ? rot[((size_t)b * R + src) * S + o[k]] : 0.0f;
    }
    __syncthreads();
    for (uint32_t kk = ty; kk < 32; kk += 8) {
        const uint32_t k = k0 + kk, r = r0 + tx;
        const float v = tile[tx][kk];
        const size_t o = ((size_t)b * Epad + k) * Rpad + r;
        if (QUANT) ((int32_t *)rotT)[o] = (r < R && k < E) ? quantise(v, factor) : 0;
        else ((float *)rotT)[o] = v;
    }
}

// Float32 operand of the DPP distance kernel: rotP[b][r][k] = rot[b][r][off[k]], the region of
// every variant contiguous in k (rows r >= R and elements k >= E are zero).
__global__ __launch_bounds__(256) void k_pack_rot_rows(const float *__restrict__ rot, const uint32_t *__restrict__ off,
                                                       float *__restrict__ rotP, uint32_t R, uint32_t S, uint32_t E,
                                                       uint32_t Epad, uint32_t Rpad, PairSource ps)
{
    const uint32_t b = blockIdx.z, r = blockIdx.y;
    const uint32_t k = blockIdx.x * 256 + threadIdx.x;
    if (k >= Epad) return;
    float v = 0.0f;
    if (r < R && k < E) {
        uint32_t src;
        const uint32_t *o = off;
        pair_source(ps, r, src, o);
        v = rot[((size_t)b * R + src) * S + o[k]];
    }
    rotP[((size_t)b * Rpad + r) * Epad + k] = v;
}

// ---------------------------------------------------------------------------------
// Distance + argmin over rotations on the vector ALU.
// One wave = 64 consecutive rotations x TN neurons.  Lane l owns rotation r0 + l and TN
// accumulators; the neuron values of the k-loop are wave-uniform (scalar loads).  Each
// (neuron, rotation) sum is accumulated sequentially over k by one lane -- no split-K, no
// cross-lane partial sums -- so the float32 result has the CPU's rounding sequence.
// The minimum over rotations is exact: a wave-level minimum of (value, rotation) keys,
// then one 64-bit atomic minimum per neuron.  Key = value << shift | rotation, with
// value = float bits (non-negative floats order like their bit patterns) or the integer sum.
// MODE 0: float32, 1: uint8 (int32 sums), 2: uint16 (int64 sums).
// ---------------------------------------------------------------------------------
template <int MODE, int TN>
__global__ __launch_bounds__(64) void k_dist_valu(const void *__restrict__ somP_, const void *__restrict__ rotT_,
                                                  unsigned long long *__restrict__ key, uint32_t N, uint32_t Epad,
                                                  uint32_t R, uint32_t Rpad)
{
    using OpT = typename std::conditional<MODE == 0, float, int32_t>::type;
    using AccT = typename std::conditional<MODE == 0, float, typename std::conditional<MODE == 1, int32_t, long long>::type>::type;
    const OpT *__restrict__ somP = (const OpT *)somP_;
    const OpT *__restrict__ rotT = (const OpT *)rotT_;
    const uint32_t lane = threadIdx.x;
    const uint32_t r = blockIdx.x * kWave + lane;
    const uint32_t n0 = blockIdx.y * TN;
    const uint32_t b = blockIdx.z;
    const OpT *rp = rotT + (size_t)b * Epad * Rpad + r;
    const OpT *np[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) np[j] = somP + (size_t)min(n0 + j, N - 1) * Epad;

    AccT acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[j] = 0;

    for (uint32_t k = 0; k < Epad; k += 8) {
        OpT bv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) bv[u] = rp[(size_t)(k + u) * Rpad];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const OpT a = np[j][k + u];
                if (MODE == 0) {
                    const float d = __fsub_rn((float)a, (float)bv[u]);
                    acc[j] = (AccT)__builtin_fmaf(d, d, (float)acc[j]);
                } else {
                    const int32_t d = (int32_t)a - (int32_t)bv[u];
                    acc[j] += (AccT)d * (AccT)d;
                }
            }
        }
    }

#pragma unroll
    for (int j = 0; j < TN; ++j) {
        unsigned long long kv;
        if (MODE == 0) kv = ((unsigned long long)__float_as_uint((float)acc[j]) << 32) | r;
        else kv = ((unsigned long long)acc[j] << 16) | r;
        if (r >= R) kv = ~0ull;
        kv = wave_min_u64(kv);
        if (lane == 0 && n0 + j < N) atomicMin(&key[(size_t)b * N + n0 + j], kv);
    }
}



// ---------------------------------------------------------------------------------
// Float32 distance + argmin of small problems (about one wave per SIMD): LDS-shared rotations, neuron
// values broadcast by DPP.
// A block of 4 waves shares 64 consecutive rotations.  Their packed regions (k contiguous per
// rotation) are staged through a double-buffered LDS tile of 64 rotations x 64 elements by
// coalesced 16-byte loads, so every rotation element leaves L2 once per 4 neurons; a lane
// reads its own rotation's row back 16 bytes at a time (row stride 68 words: conflict-free).
// Wave w owns neuron n0 + w, lane l owns rotation r0 + l.  The neuron's 64 values of a chunk come as ONE
// 16-byte load per lane -- element e in register e % 4 of lane e / 4 of every row of 16 lanes -- and reach
// all lanes of a row through the DPP operand of the subtract (`v_sub_f32_dpp ... row_newbcast:k`), so a pair
// element costs exactly one subtract and one fma and no scalar or LDS traffic for the neuron side.
// The sum of each (neuron, rotation) pair is still one lane's sequential fma chain over k in
// the CPU's element order (bit-faithful); only the argmin crosses lanes.
//
// A lone wave issues one instruction of any kind about every eight clocks, so what is not one of the 128
// subtracts and multiply-adds of a chunk costs as much as they do: the chunk loop is on an instruction diet
// (four register sets for the neuron that take turns without copies, addresses that are a uniform base
// advanced once per four chunks plus per-thread offsets that never change plus a constant, one wait per 16
// elements) and written as one assembly statement, generated by gen_ssd_steps.py, which says why.  The loads
// that run ahead are neither branched around nor clamped at the end of a row: they read up to kDistOverrun
// floats past it, which both operands are allocated with.
// ---------------------------------------------------------------------------------
constexpr uint32_t kDistKC = 64;
constexpr uint32_t kDistRow = kDistKC + 4;   // LDS row stride in floats

#include "ssd_steps.inc"

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr uint32_t kDistOverrun = 4 * kDistKC;       // floats that the loads running ahead may read past a row's end
__global__ __launch_bounds__(256, 2) void k_dist_f32_dpp(const float *__restrict__ somP, const float *__restrict__ rotT,
                                                         unsigned long long *__restrict__ key, uint32_t N, uint32_t Epad,
                                                         uint32_t R, uint32_t Rpad)
{
    __shared__ v4f s_rot[2][64 * kDistRow / 4];          // [stage][64 rotations][64 elements + 4]
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t r0 = blockIdx.x * kWave;
    const uint32_t n = blockIdx.y * 4 + wave;
    const uint32_t b = blockIdx.z;
    // thread t stages 4 vectors of a chunk: rotation t / 16 + 16 i (i < 4), elements 4 (t % 16) .. + 4
    const uint32_t lrow = tid >> 4, lcol = (tid & 15) * 4;
    const uint32_t lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) v4f *)&s_rot[0][0];
    float acc = 0.0f;
    ssd_lone_wave_loop(acc, (lrow * Epad + lcol) * 4, ((lrow + 16) * Epad + lcol) * 4, ((lrow + 32) * Epad + lcol) * 4,
                       ((lrow + 48) * Epad + lcol) * 4, (lane & 15) * 16, lds + (lrow * kDistRow + lcol) * 4,
                       lds + lane * kDistRow * 4, rotT + ((size_t)b * Rpad + r0) * Epad, somP + (size_t)min(n, N - 1) * Epad,
                       Epad / kDistKC);

    // (float bits of a sum of squares order like the floats; rotations past the last one are left out)
    const unsigned long long kv = wave_min_key_dpp(__float_as_uint(acc), r0 + lane < R, r0);
    if (lane == 0 && n < N) atomicMin(&key[(size_t)b * N + n], kv);
}

// One launch per image for small float32 trainers: the distances of image i against the SOM as image i - 1
// leaves it.  The update of image i - 1 costs a launch of its own about a third of the distance kernel's time
// (each of its blocks waits for the keys, searches the best match, then waits for its factor); here every
// wave applies it to its neuron on the fly instead -- w = w - ((w - x) * f) on each chunk of the neuron's
// operand row one chunk ahead of its use, x the same chunk of the row of the variant of image i - 1 that was
// closest to the neuron -- and stores the new row to the other of two operand buffers (all waves of a neuron
// store the same bytes; an untouched neuron's row is copied).  What a wave needs for it does not depend on the search: the
// keys of image i - 1 and the neuron's whole column of the factor matrix are requested together, the best
// match is the minimum over the wave, the factor comes out of the column by lane.  The neuron's full image
// (all elements, not only the region that the operand row holds) is not on this path: k_update_replay applies
// the updates of a group of images to it in one launch, in order.
struct PrevImage {
    const unsigned long long *key;      // keys of image i - 1 (null: nothing to apply)
    const float *rotT;                  // its packed variants
    const float *factors_t;             // the factor matrix transposed: a neuron's column is contiguous
    float *somP_next;
    uint32_t *bmu_out, *counts;
};

template <int NQ>     // neurons / 64, rounded up: keys and factors per lane in the search
__global__ __launch_bounds__(512) void k_train_f32_dpp(const float *__restrict__ somP, const float *__restrict__ rotT,
                                                          unsigned long long *__restrict__ key, uint32_t N, uint32_t Epad,
                                                          uint32_t R, uint32_t Rpad, PrevImage prev)
{
    __shared__ v4f s_rot[2][64 * kDistRow / 4];
    __shared__ float s_upd[8][2][64];          // per wave: the updated chunk on its way into the operand layout, two stages
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t r0 = blockIdx.x * kWave;
    // Four to eight waves = neurons per block.  The first four move the rotation rows; the others only
    // compute (where four neurons per block would make more blocks than the chip has CUs and fewer neurons per block
    // fewer, a CU with two blocks sets the pace for all: better every CU with one block and one or two SIMDs shared).
    const bool stages = wave < 4;
    const uint32_t n = blockIdx.y * (blockDim.x >> 6) + wave, nc = min(n, N - 1);
    const uint32_t lrow = (tid & 255) >> 4, lcol = (tid & 15) * 4;
    const uint32_t lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) v4f *)&s_rot[0][0];
    const uint32_t upd = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) float *)&s_upd[0][0][0];
    const uint32_t roff0 = (lrow * Epad + lcol) * 4, roff1 = ((lrow + 16) * Epad + lcol) * 4,
                   roff2 = ((lrow + 32) * Epad + lcol) * 4, roff3 = ((lrow + 48) * Epad + lcol) * 4;
    const uint32_t noff = (lane & 15) * 16, ldsw = lds + (lrow * kDistRow + lcol) * 4, ldsr = lds + lane * kDistRow * 4;
    const float *rp = rotT + (size_t)r0 * Epad, *np = somP + (size_t)nc * Epad;
    const uint32_t chunks = Epad / kDistKC;
    float acc = 0.0f;
    const uint32_t probe_block = blockIdx.y * gridDim.x + blockIdx.x;
    PROBE(kProbeTrainF32, probe_block, 0);
    if (prev.key == nullptr) {
        if (stages) ssd_lone_wave_loop(acc, roff0, roff1, roff2, roff3, noff, ldsw, ldsr, rp, np, chunks);
        else ssd_lone_wave_loop_unstaged(acc, noff, ldsr, np, chunks);
    } else {
        // (NQ keys and NQ factors per lane; every load is issued before the first is used, indices
        // past the end are clamped and dropped afterwards)
        const uint32_t *key32 = (const uint32_t *)prev.key;          // little endian: rotation, then the distance bits
        uint32_t dist[NQ];
        float fcol[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const uint32_t m = min(lane + 64 * q, N - 1);
            dist[q] = key32[2 * m + 1];
            fcol[q] = prev.factors_t[(size_t)nc * N + m];
        }
        const uint32_t r = key32[2 * nc];                            // the neuron's closest variant of image i - 1
        // Chunk 0 of the rotation rows, of the neuron and (as soon as r is there) of the variant are requested here,
        // ahead of the search: they travel while it runs, go to LDS stage 0 and to the loop as registers behind it.
        v4f first0 = {}, first1 = {}, first2 = {}, first3 = {};
        if (stages) {
            first0 = *(const v4f *)((const char *)rp + roff0); first1 = *(const v4f *)((const char *)rp + roff1);
            first2 = *(const v4f *)((const char *)rp + roff2); first3 = *(const v4f *)((const char *)rp + roff3);
        }
        const float w0 = np[lane];
        const float *xp = prev.rotT + (size_t)__builtin_amdgcn_readfirstlane((int)r) * Epad;
        const float x0 = xp[lane];
        PROBE(kProbeTrainF32, probe_block, 1);       // everything requested (the variant's address needed the key)
        // The best match: the smallest distance of the wave (a reduction over the lanes by DPP), then the first
        // neuron that has it.
        uint32_t dmin = 0xffffffffu;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            if (lane + 64 * q >= N) dist[q] = 0xffffffffu;
            dmin = min(dmin, dist[q]);
        }
        const uint32_t best = wave_min_u32_dpp(dmin);
        uint32_t bmu = 0;
        float f = 0.0f;
#pragma unroll
        for (int q = NQ - 1; q >= 0; --q) {
            const unsigned long long hit = __ballot(dist[q] == best && lane + 64 * q < N);
            if (hit) {
                const uint32_t at = (uint32_t)__builtin_ctzll(hit);
                bmu = at + 64 * q;
                f = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, fcol[q]), (int)at));
            }
        }
        if (blockIdx.x == 0 && n == 0 && lane == 0) {
            *prev.bmu_out = bmu;
            atomicAdd(&prev.counts[bmu], 1u);          // m_update_info[bmu]++ (Trainer.h:302-303)
        }
        float *wp = prev.somP_next + (size_t)nc * Epad;
        PROBE(kProbeTrainF32, probe_block, 2);       // best match and factor known
        if (f == 0.0f) {
            asm volatile("" ::"v"(first0), "v"(first1), "v"(first2), "v"(first3), "v"(w0), "v"(x0));   // (requested, not used)
            if (stages) ssd_lone_wave_loop_copy(acc, roff0, roff1, roff2, roff3, noff, ldsw, ldsr, rp, np, chunks, wp);
            else ssd_lone_wave_loop_copy_unstaged(acc, noff, ldsr, np, chunks, wp);
        } else if (stages) {
            v4f *stage0 = &s_rot[0][(lrow * kDistRow + lcol) / 4];
            stage0[0] = first0; stage0[16 * kDistRow / 4] = first1; stage0[32 * kDistRow / 4] = first2; stage0[48 * kDistRow / 4] = first3;
            ssd_lone_wave_loop_update(acc, roff0, roff1, roff2, roff3, noff, ldsw, ldsr, rp, np, chunks, xp, wp, f, lane * 4,
                                      upd + wave * 512 + lane * 4, upd + wave * 512 + (lane & 15) * 16, w0, x0);
        } else {
            ssd_lone_wave_loop_update_unstaged(acc, noff, ldsr, np, chunks, xp, wp, f, lane * 4, upd + wave * 512 + lane * 4,
                                               upd + wave * 512 + (lane & 15) * 16, w0, x0);
        }
    }
    PROBE(kProbeTrainF32, probe_block, 3);           // the chunk loop done
    const unsigned long long kv = wave_min_key_dpp(__float_as_uint(acc), r0 + lane < R, r0);
    if (lane == 0 && n < N) atomicMin(&key[n], kv);
    PROBE(kProbeTrainF32, probe_block, 4);
}

// The same distance for large problems (many waves per SIMD): the neuron values are scalar operands.
// A DPP operand halves the issue rate of the subtract (measured: 5.9 against 3.2 clocks per instruction
// with eight waves per SIMD), which a lone wave does not notice -- it issues only every other turn anyway --
// but a full SIMD does.  Here a wave reads its neurons' elements with scalar loads (the neuron is the same
// for all lanes) and `v_sub_f32 d, s, v` runs at the full rate; stages of 32 elements and few registers
// let eight blocks share a CU.  Same chains, same order, same results.
template <int TN, int KC, int MINB, int SW, bool NL>
__global__ __launch_bounds__(256, MINB) void k_dist_f32_sg(const float *__restrict__ somP, const float *__restrict__ rotT,
                                                           unsigned long long *__restrict__ key, uint32_t N, uint32_t Epad,
                                                           uint32_t R, uint32_t Rpad, uint32_t lane_tiles, uint32_t scal_groups)
{
    static_assert(KC == 64 || KC == 32, "stage width");
    static_assert(SW == 16 || SW == 8, "slab width");
    constexpr int ROW = KC + 4;
    constexpr int SLABS = KC / SW;
    constexpr int VPT = KC / 16;
    constexpr int TPR = KC / 4;
    constexpr int RSTEP = 256 / TPR;
    __shared__ v4f s_rot[2][64 * ROW / 4];
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t b = blockIdx.z;
    // Rows on the lanes (64 per block, through LDS) and rows as scalar operands (TN per wave): rotations and
    // neurons, or (NL) neurons and rotations -- whichever wastes fewer lanes on padding.  A chain is the same
    // sequence of operations either way (the difference changes sign, its square does not).
    // Workgroups go to the 8 XCDs round-robin by linear id and each XCD has its own L2: XCD k takes the k-th run of
    // consecutive (lane tile, scalar group) pairs, lane tile slowest, so it streams a few lane tiles instead of all of them
    // (the grid is padded to a multiple of 8; the blocks beyond the last pair leave at once, whole)
    const uint32_t per_xcd = gridDim.x / 8, pair = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (pair >= lane_tiles * scal_groups) return;
    const uint32_t lane_tile = pair / scal_groups, scal_group = pair - lane_tile * scal_groups;
    const uint32_t l0 = lane_tile * kWave;
    const uint32_t s0 = scal_group * (4 * TN) + wave * TN;
    const float *laneP = NL ? somP : rotT + (size_t)b * Rpad * Epad;
    const float *scalP = NL ? rotT + (size_t)b * Rpad * Epad : somP;
    const uint32_t lane_rows = NL ? N : Rpad;             // rows that exist on the lane side (loads are clamped to them)
    const uint32_t scal_rows = NL ? R : N;
    const float *np[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) np[j] = scalP + (size_t)min(s0 + j, scal_rows - 1) * Epad;
    float acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[j] = 0.0f;

    const uint32_t lrow = tid / TPR, lcol = (tid % TPR) * 4;
    const float *lp[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) lp[i] = laneP + (size_t)min(l0 + lrow + RSTEP * i, lane_rows - 1) * Epad + lcol;
    const uint32_t lds_w = (lrow * ROW + lcol) / 4;
    const uint32_t lds_wstep = RSTEP * ROW / 4;
    const uint32_t nchunks = Epad / KC;
    v4f st[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) s_rot[0][lds_w + i * lds_wstep] = *(const v4f *)(lp[i]);
    if (nchunks > 1) {
#pragma unroll
        for (int i = 0; i < VPT; ++i) st[i] = *(const v4f *)(lp[i] + KC);
    }
    __syncthreads();

    // Operands of a slab of SW elements wait in registers one slab ahead: the lane's SW rotation values
    // (vector registers, from LDS) and the wave's TN x SW neuron values (scalar registers), in two sets
    // that take turns.  Slab 0 of a chunk also moves the staged chunk c+1 into the other stage and requests
    // chunk c+2; the barrier stands before the last slab: by then every wave holds all of chunk c in
    // registers (its last slab prefetched) and has stored its part of chunk c+1, so the last slab may
    // prefetch slab 0 of chunk c+1 and the next chunk may overwrite this one's stage.
    float bv[2][SW];
    float an[2][TN][SW];
    auto fetch = [&](int set, uint32_t c, int sl) {
        const v4f *from = s_rot[c & 1] + lane * (ROW / 4) + sl * (SW / 4);
#pragma unroll
        for (int q = 0; q < SW / 4; ++q) {
            const v4f t4 = from[q];
            bv[set][4 * q] = t4.x; bv[set][4 * q + 1] = t4.y; bv[set][4 * q + 2] = t4.z; bv[set][4 * q + 3] = t4.w;
        }
        const uint32_t k = min(c * KC + sl * SW, Epad - SW);     // (past the end: values nobody uses)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < SW; ++e) an[set][j][e] = np[j][k + e];
    };
    fetch(0, 0, 0);
    for (uint32_t c = 0; c < nchunks; ++c) {
#pragma unroll
        for (int sl = 0; sl < SLABS; ++sl) {
            const int set = sl & 1;
            // this slab's operands were requested a slab ago; scalar loads return in any order, so the
            // counter can only be waited down to zero: do it before the next requests join it
            // (the builtin, not inline assembly: the compiler's own wait insertion must know of it, or it
            // waits again at the first use, after the new requests; 0xc07f = lgkmcnt(0), the others untouched)
            __builtin_amdgcn_s_waitcnt(0xc07f);
            if (sl + 1 < SLABS) fetch(set ^ 1, c, sl + 1);
            else fetch(set ^ 1, c + 1, 0);
            if (sl == 0) {
                if (c + 1 < nchunks) {
                    v4f *nx = s_rot[(c + 1) & 1];
#pragma unroll
                    for (int i = 0; i < VPT; ++i) nx[lds_w + i * lds_wstep] = st[i];
                }
                if (c + 2 < nchunks) {
                    const uint32_t k = (c + 2) * KC;
#pragma unroll
                    for (int i = 0; i < VPT; ++i) st[i] = *(const v4f *)(lp[i] + k);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int e = 0; e < SW; ++e)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const float d = NL ? __fsub_rn(bv[set][e], an[set][j][e]) : __fsub_rn(an[set][j][e], bv[set][e]);
                    acc[j] = __builtin_fmaf(d, d, acc[j]);
                }
            __builtin_amdgcn_sched_barrier(0);
            if (sl == SLABS - 2) __syncthreads();
        }
    }

    if constexpr (!NL) {
        const uint32_t r = l0 + lane;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            unsigned long long kv = ((unsigned long long)__float_as_uint(acc[j]) << 32) | r;
            if (r >= R) kv = ~0ull;
            kv = wave_min_u64(kv);
            if (lane == 0 && s0 + j < N) atomicMin(&key[(size_t)b * N + s0 + j], kv);
        }
    } else {
        // a lane is a neuron: the minimum over this wave's TN rotations in the lane, over the block's four waves in LDS
        __shared__ unsigned long long s_best[4][64];
        unsigned long long best = ~0ull;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const unsigned long long kv = ((unsigned long long)__float_as_uint(acc[j]) << 32) | (s0 + j);
            if (s0 + j < R && kv < best) best = kv;
        }
        s_best[wave][lane] = best;
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int w = 1; w < 4; ++w) best = s_best[w][lane] < best ? s_best[w][lane] : best;
            if (l0 + lane < N) atomicMin(&key[(size_t)b * N + l0 + lane], best);
        }
    }
}

// ---------------------------------------------------------------------------------
// uint8 distance on the matrix cores (mapping).
//
// Integer sums are order-independent, so the uint8 distance is recast exactly as
//   ssd(n, r) = |a'_n|^2 + |b'_r|^2 - 2 a'_n . b'_r,    x' = q(x) - 128 in [-128, 127],
// with the dot products on v_mfma_i32_32x32x32_i8 (int32 accumulation, exact).
//
// Operand layout ("fragment-major"): rows in tiles of 32, k in steps of 32; one
// (tile, k-step) fragment is 1 KiB = 64 lanes x 16 bytes, lane l holding row l % 32,
// k = kstep * 32 + (l / 32) * 16 .. + 16.  A wave loads a fragment with one fully
// coalesced 16-byte-per-lane access and feeds it to the MFMA unchanged.  Both operands
// use the same layout, so the k assignment inside a fragment cancels out.
//
// Rotation operand rows are ordered (base rotation i, symmetry) instead of by variant
// index: row = i * 8 + flip * 4 + quarter.  The 8 symmetries of a base rotation are
// then adjacent, one block owns whole fragments, and the true variant index
// k = flip * num_rot + quarter * (num_rot / 4) + i travels in the argmin key, so ties
// still resolve to the lowest variant index.
// ---------------------------------------------------------------------------------

// Rotation + quantisation + packing, no float variants written.  Block (tile, b): base
// rotations 4*tile .. 4*tile+3 of image b are evaluated only at the pixels some region
// element of some symmetry refers to (`need`), quantised and shifted into LDS; every
// operand byte is then a gather through the precomputed table
//   poff[sym][e] = position in the base rotation of region element e of symmetry sym
// (position S = a zero byte, used for the padding beyond E).
__global__ __launch_bounds__(256) void k_rotpack_u8(const float *__restrict__ images, v4i *__restrict__ Pb,
                                                    int *__restrict__ nb, const float *__restrict__ cos_t,
                                                    const float *__restrict__ sin_t,
                                                    const unsigned short *__restrict__ poff,
                                                    const uint32_t *__restrict__ need, uint32_t n_need, uint32_t C,
                                                    uint32_t I, uint32_t D, uint32_t S, uint32_t num_rot,
                                                    uint32_t use_flip, uint32_t nrr_eff, uint32_t KS, uint32_t RT)
{
    extern __shared__ signed char s_q[];              // 4 * (S + 1) quantised pixels, then 32 ints
    const uint32_t tile = blockIdx.x, b = blockIdx.y;
    const uint32_t stride = S + 1;
    int *s_nb = (int *)(s_q + ((4 * stride + 15) & ~15u));
    const uint32_t DD = D * D;
    const float *img = images + (size_t)b * C * I * I;

    if (threadIdx.x < 32) s_nb[threadIdx.x] = 0;
    if (threadIdx.x < 4) s_q[threadIdx.x * stride + S] = 0;
    for (uint32_t t = threadIdx.x; t < 4 * n_need; t += blockDim.x) {
        const uint32_t g = t / n_need, p = need[t % n_need];
        const uint32_t i = tile * 4 + g;
        signed char v = 0;
        if (i < nrr_eff) {
            const uint32_t c = p / DD, px = (p % DD) / D, py = p % D;
            const float cs = i ? cos_t[i] : 1.0f, sn = i ? sin_t[i] : 0.0f;
            v = (signed char)(quantise(base_pixel(img + (size_t)c * I * I, I, D, i, cs, sn, px, py), 255.0f) - 128);
        }
        s_q[g * stride + p] = v;
    }
    __syncthreads();

    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row = lane & 31, half = lane >> 5;
    const uint32_t g = row >> 3, sym = row & 7;
    const uint32_t Kp = KS * 32;
    const signed char *src = s_q + g * stride;
    const unsigned short *tab = poff + (size_t)sym * Kp + half * 16;
    int sq = 0;
    for (uint32_t ks = wave; ks < KS; ks += 4) {
        const unsigned short *tp = tab + ks * 32;
        v4i frag;
#pragma unroll
        for (int w4 = 0; w4 < 4; ++w4) {
            uint32_t word = 0;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int v = src[tp[w4 * 4 + u]];
                sq += v * v;
                word |= (uint32_t)(v & 0xff) << (8 * u);
            }
            frag[w4] = (int)word;
        }
        Pb[(((size_t)b * RT + tile) * KS + ks) * 64 + lane] = frag;
    }
    atomicAdd(&s_nb[row], sq);
    __syncthreads();
    if (threadIdx.x < 32) nb[((size_t)b * RT + tile) * 32 + threadIdx.x] = s_nb[threadIdx.x];
}

// SOM operand in the same fragment-major layout plus |a'_n|^2.  One block per neuron.
__global__ __launch_bounds__(256) void k_pack_som_u8(const float *__restrict__ som, const uint32_t *__restrict__ off,
                                                     signed char *__restrict__ Pa, int *__restrict__ na, uint32_t N,
                                                     uint32_t S, uint32_t E, uint32_t KS)
{
    __shared__ int s_sum[256];
    const uint32_t n = blockIdx.x;      // 0 .. NT*32-1, rows beyond N are zero
    const uint32_t Kp = KS * 32;
    int sq = 0;
    for (uint32_t k = threadIdx.x; k < Kp; k += 256) {
        int v = 0;
        if (n < N && k < E) v = quantise(som[(size_t)n * S + off[k]], 255.0f) - 128;
        sq += v * v;
        const uint32_t lane = (n & 31) + 32 * ((k & 31) >> 4);
        Pa[((((size_t)(n >> 5) * KS + (k >> 5)) * 64 + lane) << 4) + (k & 15)] = (signed char)v;
    }
    s_sum[threadIdx.x] = sq;
    __syncthreads();
    for (uint32_t s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) s_sum[threadIdx.x] += s_sum[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) na[n] = s_sum[0];
}

// Distance + argmin.  The whole SOM operand stays in LDS; a block walks over images, its
// 8 waves share the rotation tiles of one image.  Per (tile, k-step) a wave loads one
// rotation fragment from HBM (each byte of the operand is read exactly once) and issues NT
// MFMAs against the neuron fragments in LDS.  Rotations are the MFMA's row operand, so a
// lane ends up with 16 rotations of ONE neuron (column lane % 32) per accumulator set: the
// minimum over rotations is a running in-lane minimum, one shuffle across the two
// half-waves, and one LDS pass across the 8 waves -- no atomics.
template <int NT>
__global__ __launch_bounds__(512) void k_dist_mfma_u8(const v4i *__restrict__ Pa, const int *__restrict__ na,
                                                      const v4i *__restrict__ Pb, const int *__restrict__ nb,
                                                      unsigned long long *__restrict__ key, uint32_t N, uint32_t KS,
                                                      uint32_t RT, uint32_t B, uint32_t num_rot, uint32_t use_flip,
                                                      uint32_t nrr_eff)
{
    extern __shared__ v4i s_a[];                                   // NT * KS * 64 fragments' lanes
    unsigned long long *s_key = (unsigned long long *)(s_a + (size_t)NT * KS * 64);   // 8 waves x NT*32
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t col = lane & 31, half = lane >> 5;
    const uint32_t nrr = num_rot / 4;

    for (uint32_t t = threadIdx.x; t < NT * KS * 64; t += blockDim.x) s_a[t] = Pa[t];
    int na_l[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) na_l[nt] = na[nt * 32 + col];
    __syncthreads();

    for (uint32_t b = blockIdx.x; b < B; b += gridDim.x) {
        unsigned long long best[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) best[nt] = ~0ull;

        for (uint32_t rt = wave; rt < RT; rt += 8) {
            v16i acc[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int j = 0; j < 16; ++j) acc[nt][j] = 0;
            const v4i *pb = Pb + ((size_t)b * RT + rt) * KS * 64 + lane;
            for (uint32_t ks = 0; ks < KS; ks += 8) {
                v4i bf[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) bf[u] = pb[(size_t)min(ks + u, KS - 1) * 64];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    if (ks + u < KS) {
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
                            acc[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[u], s_a[((size_t)nt * KS + ks + u) * 64 + lane],
                                                                            acc[nt], 0, 0, 0);
                    }
                }
            }
            // accumulator j of lane l: rotation row 8*(j/4) + 4*(l/32) + j%4 of the tile, neuron column l%32
            const int *nbp = nb + ((size_t)b * RT + rt) * 32;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const uint32_t ib = j >> 2, q = j & 3;
                const uint32_t i = rt * 4 + ib;
                const bool valid = i < nrr_eff && (num_rot != 1 || q == 0) && (use_flip || half == 0);
                const uint32_t k = half * num_rot + q * nrr + i;
                const int nbv = nbp[8 * ib + 4 * half + q];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const int ssd = na_l[nt] + nbv - 2 * acc[nt][j];
                    const unsigned long long kv = valid ? (((unsigned long long)(uint32_t)ssd << 16) | k) : ~0ull;
                    best[nt] = kv < best[nt] ? kv : best[nt];
                }
            }
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const unsigned long long o = __shfl_xor(best[nt], 32, 64);
            best[nt] = o < best[nt] ? o : best[nt];
            if (half == 0) s_key[wave * (NT * 32) + nt * 32 + col] = best[nt];
        }
        __syncthreads();
        if (threadIdx.x < NT * 32) {
            unsigned long long m = s_key[threadIdx.x];
#pragma unroll
            for (int w = 1; w < 8; ++w) {
                const unsigned long long o = s_key[w * (NT * 32) + threadIdx.x];
                m = o < m ? o : m;
            }
            if (threadIdx.x < N) key[(size_t)b * N + threadIdx.x] = m;
        }
        __syncthreads();
    }
}

#include "mfma_int_gemm.inc"
#include "mfma_f32_gemm.inc"

// ---------------------------------------------------------------------------------
// BMU search fused with the neuron update (Trainer.h:164-179; CudaLib/update_neurons.h).
// Every block recomputes the best-matching neuron from the N keys (first minimum wins),
// then block (part, n) pulls its slice of neuron n toward that neuron's best variant:
//   w = w - ((w - x) * f),  f = factors[bmu * N + n], skipped when f == 0,
// and refreshes the region elements of the packed distance operand in the same pass.
// ---------------------------------------------------------------------------------
// Operand refresh of the integer GEMM path inside the update: the byte planes of the updated
// elements (fragment order of mfma_int_gemm.inc) and the row norm |V|^2, accumulated per block
// into `na_next` (zeroed by the distance kernel's finish step, which read the other buffer).
// How the update kernel finds a variant when only two of a base rotation's eight symmetries are stored
// (D = 0: every variant is stored).  Element counts stay below 2^24 (the base rotation fits LDS).
struct VariantPair {
    uint32_t D, num_rot, nrr;
};

struct UpdatePlanes {
    signed char *Pa;            // null: not this path
    long long *na_next;
    const long long *na_cur;
    uint32_t KS, Np, u16;
};

constexpr uint32_t kFactorColumnMax = 2048;      // neurons whose column of the factor matrix a block keeps in LDS

template <uint32_t U>     // elements per thread and round: all their loads are issued before the first store
__global__ __launch_bounds__(256) void k_update(float *__restrict__ som, const float *__restrict__ rot,
                                                const unsigned long long *__restrict__ key,
                                                const float *__restrict__ factors_t, uint32_t *__restrict__ bmu_out,
                                                uint32_t N, uint32_t S, uint32_t parts, uint32_t shift,
                                                void *__restrict__ somP, const uint32_t *__restrict__ inv,
                                                uint32_t Epad, float qfactor, UpdatePlanes up,
                                                uint32_t *__restrict__ counts, VariantPair vp)
{
    __shared__ unsigned long long s_val[256];
    __shared__ uint32_t s_idx[256];
    __shared__ float s_fcol[kFactorColumnMax];
    const uint32_t tid = threadIdx.x;
    // Block (part, n); or, where the update also refreshes the byte planes of the integer GEMM's operand, the blocks of
    // the four neurons whose 16-byte pieces share a 64-byte line of the planes on ONE XCD (workgroups go to the XCDs
    // round-robin by linear id): its L2 then merges the four neurons' pieces into whole lines, where four L2s would
    // each write the line back in parts.  The grid's x then counts (XCD, neuron in the four, group of eight fours).
    uint32_t n = blockIdx.y, part = blockIdx.x;
    if (up.Pa) {
        const uint32_t x = blockIdx.x, four = (x >> 5) * 8 + (x & 7);
        n = four * 4 + ((x >> 3) & 3);
        part = blockIdx.y;
        if (n >= N) return;
    }
    const uint32_t probe_block = n * parts + part;
    PROBE(kProbeUpdate, probe_block, 0);
    // The factor of this neuron depends on the best match, the neuron's column of the factor matrix does not: it is
    // requested with the keys (factors_t is the matrix transposed, so the column is contiguous) and waits in LDS.
    const float *__restrict__ fcol = factors_t + (size_t)n * N;
    const bool column_in_lds = N <= kFactorColumnMax;
    // What the block will read does not depend on the best-matching neuron, only whether it is
    // needed does: the first round of loads is issued ahead of the search, which then runs while
    // they are in flight (a neuron with factor 0 drops them).
    // (loads return in issue order: the keys go first, so the search below waits for them alone)
    unsigned long long bv = ~0ull;
    uint32_t bi = 0xffffffffu;
    for (uint32_t m = tid; m < N; m += 256) {
        const unsigned long long v = key[m] >> shift;
        if (column_in_lds) s_fcol[m] = fcol[m];
        if (v < bv) { bv = v; bi = m; }        // ascending index per thread: first minimum kept
    }
    const uint32_t r = (uint32_t)(key[n] & ((1ull << shift) - 1ull));
    // The variant: stored as such, or (vp.D != 0) read out of the stored base rotation (q even) or its
    // quarter turn (q odd) with rows and/or columns reversed:
    //   V(f, q)[x][y] = V(0, q & 1)[f ^ (q >> 1) ? D-1-x : x][q >> 1 ? D-1-y : y]
    const float *__restrict__ x = rot + (size_t)r * S;
    uint32_t rev_x = 0, rev_y = 0;
    if (vp.D) {
        const uint32_t f = r >= vp.num_rot ? 1u : 0u, rem = r - f * vp.num_rot;
        const uint32_t q = rem / vp.nrr, i = rem - q * vp.nrr;
        x = rot + (size_t)((q & 1) * vp.nrr + i) * S;
        rev_x = f ^ (q >> 1); rev_y = q >> 1;
    }
    float *__restrict__ w = som + (size_t)n * S;
    const uint32_t chunk = (S + parts - 1) / parts;
    const uint32_t j0 = part * chunk, j1 = min(S, j0 + chunk);
    // Where element j of the variant sits in the stored one: j itself unless rows and/or columns are read
    // reversed.  A thread's elements are 256 apart, so its (row, column) inside the channel plane moves by a fixed
    // step with carries instead of two divisions per element (the kernel was half bound by its vector ALU work).
    const bool reversed = vp.D != 0 && (rev_x | rev_y) != 0;
    const uint32_t D = max(vp.D, 1u);
    const RcpDivisor by_DD(D * D), by_D(D);
    // (a slice of a single round, small neurons spread over many blocks: the divisions are as cheap as the stepping)
    const bool stepping = reversed && j1 - j0 > 256 * U;
    const uint32_t step_x = 256u / D, step_y = 256u % D;
    uint32_t px = 0, py = 0;                      // of the next element this thread loads
    if (stepping) {
        uint32_t c, p;
        by_DD.divmod(j0 + tid, c, p);
        by_D.divmod(p, px, py);
    }
    // element (px, py) of a channel plane is read at (rev_x ? D-1-px : px, rev_y ? D-1-py : py): j + c0 + cx px + cy py
    const int cx = rev_x ? -2 * (int)D : 0, cy = rev_y ? -2 : 0;
    const int c0 = (rev_x ? (int)((D - 1) * D) : 0) + (rev_y ? (int)D - 1 : 0);
    float wv[U], xv[U];
    uint32_t kk[U];
    auto load_round = [&](uint32_t jb) {
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) {
            const uint32_t j = jb + 256 * u;
            uint32_t src = j;
            if (stepping) {
                src = (uint32_t)((int)j + c0 + __mul24(cx, (int)px) + __mul24(cy, (int)py));
                py += step_y;
                px += step_x + (py >= D ? 1u : 0u);
                py -= py >= D ? D : 0u;
                px -= px >= D ? D : 0u;            // (past the end of a channel plane: the next one)
                if (D < 32) while (px >= D) px -= D;       // (a step of 256 elements spans more than two rows)
            } else if (reversed) {
                uint32_t c, p, qx, qy;
                by_DD.divmod(j, c, p);
                by_D.divmod(p, qx, qy);
                src = j - p + (rev_x ? D - 1 - qx : qx) * D + (rev_y ? D - 1 - qy : qy);
            }
            if (j < j1) {
                wv[u] = w[j];
                xv[u] = x[src];
                kk[u] = inv ? inv[j] : 0xffffffffu;
            }
        }
    };
    load_round(j0 + tid);
    PROBE(kProbeUpdate, probe_block, 1);
    // first minimum of the block: within a wave by DPP, then across the four waves
    wave_first_min_u64_dpp(bv, bi);
    PROBE(kProbeUpdate, probe_block, 2);
    if ((tid & 63) == 0) { s_val[tid >> 6] = bv; s_idx[tid >> 6] = bi; }
    __syncthreads();
    bv = s_val[0]; bi = s_idx[0];
#pragma unroll
    for (int g = 1; g < 4; ++g) {
        const unsigned long long ov = s_val[g];
        const uint32_t oi = s_idx[g];
        if (ov < bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    const uint32_t bmu = bi;
    if (n == 0 && part == 0 && tid == 0) {
        *bmu_out = bmu;
        atomicAdd(&counts[bmu], 1u);           // m_update_info[bmu]++ (Trainer.h:302-303)
    }

    const float f = column_in_lds ? s_fcol[bmu] : fcol[bmu];

    PROBE(kProbeUpdate, probe_block, 3);
    if (f == 0.0f) {
        // untouched neuron: its operand row stands, its norm moves to the next buffer
        if (up.Pa && part == 0 && tid == 0) atomicAdd((unsigned long long *)&up.na_next[n], (unsigned long long)up.na_cur[n]);
        return;
    }
    long long sq = 0;
    const size_t plane_bytes = (size_t)(up.Np / 32) * up.KS * 64 * 16;
    signed char *row_planes = up.Pa + ((((size_t)(n >> 5) * up.KS) * 64 + (n & 31)) << 4);
    // keep the distance kernel's packed copy of the region current (inv = position of element j in
    // the region, for the byte planes its byte inside the neuron's row of fragments, or none)
    auto refresh = [&](uint32_t k, float nv) {
        if (k == 0xffffffffu) return;
        if (up.Pa) {
            // (k: the element's byte inside the neuron's row of fragments; values of at most 17 bits: 24-bit products)
            const int q = quantise(nv, qfactor);
            signed char *at = row_planes + k;
            if (up.u16) {
                const int c = q - 32768;
                const int h = c >> 8, l = (c & 255) - 128;
                at[0] = (signed char)h;
                at[plane_bytes] = (signed char)l;
                sq += __mul24(c - 128, c - 128);            // (256 h + l) squared
            } else {
                const int h = q - 128;
                at[0] = (signed char)h;
                sq += __mul24(h, h);
            }
        } else if (qfactor > 0.0f) {
            ((int32_t *)somP)[(size_t)n * Epad + k] = quantise(nv, qfactor);
        } else {
            ((float *)somP)[(size_t)n * Epad + k] = nv;
        }
    };
    // Four elements per thread and round: all their loads are issued before the first store, so a
    // thread keeps several cache lines in flight (the kernel lives on memory latency and bandwidth).
    for (uint32_t jb = j0 + tid; jb < j1; jb += 256 * U) {
        if (jb != j0 + tid) load_round(jb);
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) {
            const uint32_t j = jb + 256 * u;
            if (j < j1) {
                const float nv = __fsub_rn(wv[u], __fmul_rn(__fsub_rn(wv[u], xv[u]), f));
                w[j] = nv;
                refresh(kk[u], nv);
            }
        }
    }
    PROBE(kProbeUpdate, probe_block, 4);
    if (up.Pa) {
        // (f depends on the block only, so every thread of the block is here)
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) sq += __shfl_xor(sq, o, 64);
        __syncthreads();                                   // s_val was last read by the search above
        if ((tid & 63) == 0) s_val[tid >> 6] = (unsigned long long)sq;
        __syncthreads();
        if (tid == 0) atomicAdd((unsigned long long *)&up.na_next[n], s_val[0] + s_val[1] + s_val[2] + s_val[3]);
    }
    PROBE(kProbeUpdate, probe_block, 5);
}

// The update of a float32 trainer on the distance operand alone: block (part, n) finds the best match like k_update,
// then pulls its slice of neuron n's operand row toward the packed row of the neuron's closest variant (the same
// elements in the same order: no index arithmetic, 16-byte accesses).  The neurons' full images follow once per
// group of images (k_update_replay): the distance never reads them.
__global__ __launch_bounds__(256) void k_update_rows(float *__restrict__ somP, const float *__restrict__ rotT,
                                                     const unsigned long long *__restrict__ key, const float *__restrict__ factors_t,
                                                     uint32_t *__restrict__ bmu_out, uint32_t *__restrict__ counts, uint32_t N,
                                                     uint32_t Epad, uint32_t parts, uint32_t shift)
{
    __shared__ unsigned long long s_val[4];
    __shared__ uint32_t s_idx[4];
    __shared__ float s_fcol[kFactorColumnMax];
    const uint32_t tid = threadIdx.x, n = blockIdx.y, part = blockIdx.x;
    const float *__restrict__ fcol = factors_t + (size_t)n * N;      // the neuron's column of the factor matrix (see k_update)
    const bool column_in_lds = N <= kFactorColumnMax;
    unsigned long long bv = ~0ull;
    uint32_t bi = 0xffffffffu;
    for (uint32_t m = tid; m < N; m += 256) {
        const unsigned long long v = key[m] >> shift;
        if (column_in_lds) s_fcol[m] = fcol[m];
        if (v < bv) { bv = v; bi = m; }        // ascending index per thread: first minimum kept
    }
    const uint32_t r = (uint32_t)(key[n] & ((1ull << shift) - 1ull));
    // the slice's first round of loads does not depend on the search: requested ahead of it
    const uint32_t vecs = Epad / 4, chunk = (vecs + parts - 1) / parts;
    const uint32_t v0 = part * chunk, v1 = min(vecs, v0 + chunk);
    v4f *__restrict__ w = (v4f *)(somP + (size_t)n * Epad);
    const v4f *__restrict__ x = (const v4f *)(rotT + (size_t)r * Epad);
    constexpr uint32_t U = 4;
    v4f wv[U], xv[U];
    auto load_round = [&](uint32_t vb) {
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) {
            const uint32_t v = vb + 256 * u;
            if (v < v1) { wv[u] = w[v]; xv[u] = x[v]; }
        }
    };
    load_round(v0 + tid);
    wave_first_min_u64_dpp(bv, bi);
    if ((tid & 63) == 0) { s_val[tid >> 6] = bv; s_idx[tid >> 6] = bi; }
    __syncthreads();
    bv = s_val[0]; bi = s_idx[0];
#pragma unroll
    for (int g = 1; g < 4; ++g) {
        const unsigned long long ov = s_val[g];
        const uint32_t oi = s_idx[g];
        if (ov < bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    const uint32_t bmu = bi;
    if (n == 0 && part == 0 && tid == 0) {
        *bmu_out = bmu;
        atomicAdd(&counts[bmu], 1u);           // m_update_info[bmu]++ (Trainer.h:302-303)
    }
    const float f = column_in_lds ? s_fcol[bmu] : fcol[bmu];
    if (f == 0.0f) return;
    for (uint32_t vb = v0 + tid; vb < v1; vb += 256 * U) {
        if (vb != v0 + tid) load_round(vb);
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) {
            const uint32_t v = vb + 256 * u;
            if (v < v1) {
                v4f o;
                o.x = __fsub_rn(wv[u].x, __fmul_rn(__fsub_rn(wv[u].x, xv[u].x), f));
                o.y = __fsub_rn(wv[u].y, __fmul_rn(__fsub_rn(wv[u].y, xv[u].y), f));
                o.z = __fsub_rn(wv[u].z, __fmul_rn(__fsub_rn(wv[u].z, xv[u].z), f));
                o.w = __fsub_rn(wv[u].w, __fmul_rn(__fsub_rn(wv[u].w, xv[u].w), f));
                w[v] = o;
            }
        }
    }
}

// The neurons' full images after a group of images: thread (n, j) pulls element j of neuron n toward the
// closest variant of image 0, then of image 1, ... (Trainer.h:164-179; CudaLib/update_neurons.h), with the
// arithmetic of k_update.  The best match of image i is bmu[i]; the closest variant of the neuron is in its
// key.  Nothing here waits for a search: one launch replays what k_update does in one launch per image.  What
// an image contributes to neuron n -- factor, row of the stored variant, how it is read -- is worked out for
// all images side by side first (one thread each) and kept in LDS, so the loop over the images is one
// variant element and three operations per image with nothing that depends on the image before.
constexpr uint32_t kReplayMax = 256;         // images per launch
template <int EPT>       // elements per thread, 256 apart
__global__ __launch_bounds__(256) void k_update_replay(float *__restrict__ som, const float *__restrict__ rot,
                                                       const unsigned long long *__restrict__ key, const float *__restrict__ factors,
                                                       const uint32_t *__restrict__ bmu, uint32_t images, uint32_t N, uint32_t S,
                                                       uint32_t R, uint32_t shift, VariantPair vp)
{
    __shared__ float s_f[kReplayMax];
    __shared__ uint32_t s_row[kReplayMax];   // stored row of the group's variants * 4 + how it is read
    // (neurons vary fastest over the grid: the blocks that run side by side then read the same stretch of elements of
    // whatever variants their neurons were closest to -- a few MB that stay in L2 -- and not whole variants)
    // (several elements per thread: what an image costs the thread beside its elements -- its row, how it is read, its
    // factor, out of LDS -- is paid once for all of them)
    const uint32_t n = blockIdx.x, j = blockIdx.y * (256 * EPT) + threadIdx.x;
    if (threadIdx.x < images) {
        const uint32_t i = threadIdx.x;
        const uint32_t r = (uint32_t)(key[(size_t)i * N + n] & ((1ull << shift) - 1ull));
        uint32_t row = r, which = 0;
        if (vp.D) {
            // stored: the base rotation and its quarter turn; the others are those with rows and / or columns reversed
            const uint32_t fl = r >= vp.num_rot ? 1u : 0u, rem = r - fl * vp.num_rot;
            const uint32_t q = rem / vp.nrr, b = rem - q * vp.nrr;
            row = (q & 1) * vp.nrr + b;
            which = 2 * (fl ^ (q >> 1)) + (q >> 1);
        }
        s_f[i] = factors[(size_t)bmu[i] * N + n];
        s_row[i] = (i * R + row) * 4 + which;
    }
    __syncthreads();
    if (j >= S) return;
    uint32_t jj[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) jj[e] = min(j + 256 * e, S - 1);      // (past the end: the last element again, not stored)
    // where an element sits in a stored variant read as it is, with columns, rows or both reversed (see k_update)
    uint32_t src[EPT][4];
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        src[e][0] = src[e][1] = src[e][2] = src[e][3] = jj[e];
        if (vp.D) {
            const uint32_t D = vp.D, p = jj[e] % (D * D), x = p / D, y = p % D;
            src[e][1] = jj[e] - p + x * D + (D - 1 - y);
            src[e][2] = jj[e] - p + (D - 1 - x) * D + y;
            src[e][3] = jj[e] - p + (D - 1 - x) * D + (D - 1 - y);
        }
    }
    float w[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) w[e] = som[(size_t)n * S + jj[e]];
    for (uint32_t i0 = 0; i0 < images; i0 += 8) {
        float x[8][EPT], f[8];
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) {
            const uint32_t i = min(i0 + u, images - 1);
            const uint32_t rw = s_row[i], which = rw & 3;
            f[u] = i0 + u < images ? s_f[i] : 0.0f;
            const float *row = rot + (size_t)(rw >> 2) * S;
#pragma unroll
            for (int e = 0; e < EPT; ++e)
                x[u][e] = row[which == 0 ? src[e][0] : which == 1 ? src[e][1] : which == 2 ? src[e][2] : src[e][3]];
        }
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u)
            if (f[u] != 0.0f) {
#pragma unroll
                for (int e = 0; e < EPT; ++e) w[e] = __fsub_rn(w[e], __fmul_rn(__fsub_rn(w[e], x[u][e]), f[u]));
            }
    }
#pragma unroll
    for (int e = 0; e < EPT; ++e)
        if (j + 256 * e < S) som[(size_t)n * S + j + 256 * e] = w[e];
}

// ---------------------------------------------------------------------------------
// Small uint8 trainers (at most 64 neurons and 32 variants, e.g. 8 x 8 neurons of 28 x 28 pixels under
// the eight symmetries): the whole step of an image -- distances, best match, update, operand refresh --
// in ONE launch.  Two dependent launches cost such a trainer about 5 us each whatever they compute; the
// distance matrix itself is a few dozen MFMAs.  So every block (one per neuron) computes the WHOLE
// matrix again (four waves cut k four ways and meet in LDS), finds the best match and its own neuron's
// best variant, and updates its neuron.  Everything the update needs that does not depend on the search
// is requested at the start (the neuron's weights, its column of the factor matrix, all stored variants
// into LDS), so after the search nothing waits for memory.  Blocks run side by side and read all rows of
// the SOM operand while others rewrite theirs: the operand and its norms therefore alternate between two
// buffers, every block writing its whole row of the next one (an untouched neuron's row comes out the
// same bytes).  Arithmetic and tie rules are those of k_dist_gemm_int + k_update.
// ---------------------------------------------------------------------------------
struct SmallTrain {
    const long long *na_cur;
    long long *na_next;
    const long long *nb;            // norms of this image's variant rows
    const uint32_t *variant;        // operand row -> variant index
    uint32_t *bmu_out, *counts;
    uint32_t N, S, R, KS, nstored;  // nstored: variants k_rotate stored for this image (two per base rotation)
    VariantPair vp;
};

// Per neuron element j, prepared once per context (no divisions in the kernel):
//   src4[j]  = where element j of a variant sits in the stored one, for rows / columns read as stored or reversed:
//              16 bits for each of the four combinations (rows reversed) * 2 + (columns reversed);
//   kbyte[j] = byte of element j inside a row of 32-row fragments of the SOM operand, (k / 32) * 1024 +
//              (k / 16 % 2) * 512 + k % 16 for region position k, or all ones outside the region.
template <int EPT, int KSW>    // elements of a neuron per thread; k-steps per wave held in registers at a time
__global__ __launch_bounds__(256) void k_train_small_u8(float *__restrict__ som, const float *__restrict__ rot,
                                                        const v4i *__restrict__ Pa, signed char *__restrict__ Pa_next,
                                                        const v4i *__restrict__ Pb, const float *__restrict__ factors,
                                                        const unsigned long long *__restrict__ src4,
                                                        const uint32_t *__restrict__ kbyte, SmallTrain a)
{
    extern __shared__ float s_var[];                      // the stored variants of this image
    // [wave][column tile][lane][16 accumulators + 4]: a lane's accumulators in one place (16-byte accesses), lanes
    // 80 bytes apart (sixteen neighbouring lanes then cover every bank once)
    __shared__ v4i s_part[4][2][64][5];
    __shared__ uint32_t s_key[4][32];
    __shared__ float s_f[64];
    __shared__ int s_sq[4];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = blockIdx.x;
    const uint32_t N = a.N, S = a.S, KS = a.KS;
    const bool two = N > 32;

    // (1) Every request that does not depend on the search goes out before anything is waited for, the
    // operand fragments first (loads return in order: the MFMAs below then wait for them alone).
    // (no branches here or around the MFMAs: a k-step past the end is loaded from the last one and multiplied
    // by zeros, a SOM of one column tile multiplies that tile twice)
    v4i fb[KSW], fa0[KSW], fa1[KSW];
    const uint32_t tile1 = two ? KS : 0u;
    auto load_fragments = [&](uint32_t first) {
#pragma unroll
        for (int u = 0; u < KSW; ++u) {
            const uint32_t ks = min(first + 4 * u, KS - 1);
            fb[u] = Pb[(size_t)ks * 64 + lane];
            fa0[u] = Pa[(size_t)ks * 64 + lane];
            fa1[u] = Pa[(size_t)(tile1 + ks) * 64 + lane];
        }
    };
    load_fragments(wave);
    // This thread's part of the finish: column tile `ct`, eight of the 16 accumulator rows.  Sums stay below
    // 2^27 (at most 2048 elements of 8 bits) and variants below 32: keys are 32 bits, distance * 32 + variant.
    const uint32_t ct = wave & 1, col = lane & 31, m = ct * 32 + col;
    int na_m = 0, nb_r[8];
    uint32_t var_r[8];
    if (m < N) na_m = (int)a.na_cur[m];
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
        const uint32_t j = 8 * (wave >> 1) + jj, row = 8 * (j >> 2) + 4 * (lane >> 5) + (j & 3);     // < 32
        nb_r[jj] = (int)a.nb[row];
        var_r[jj] = a.variant[row];
    }
    float wv[EPT];
    uint32_t kb[EPT];
    unsigned long long sp[EPT];
#pragma unroll
    for (int u = 0; u < EPT; ++u) {
        const uint32_t j = min(tid + 256 * u, S - 1);     // (past the end: the last element again, dropped below)
        wv[u] = som[(size_t)n * S + j];
        kb[u] = kbyte[j];
        sp[u] = src4[j];
    }
    const float f_if = tid < N ? factors[(size_t)tid * N + n] : 0.0f;     // the factor, should neuron `tid` be the best match
    const uint32_t n_var = a.nstored * S;
    float sv[8];                                          // the first 2048 variant elements wait in registers
#pragma unroll
    for (int u = 0; u < 8; ++u) sv[u] = rot[min(tid + 256 * u, n_var - 1)];

    // (2) all dot products: this wave's k-steps, both column tiles
    v16i acc[2];
    for (uint32_t first = wave; first < KS; first += 4 * KSW) {
        const bool again = first != wave;
        if (again) load_fragments(first);
#pragma unroll
        for (int u = 0; u < KSW; ++u) {
            const v4i zero = {0, 0, 0, 0};
            const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const v4i b = first + 4 * u < KS ? fb[u] : zero;
            acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b, fa0[u], (u == 0 && !again) ? zero16 : acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b, fa1[u], (u == 0 && !again) ? zero16 : acc[1], 0, 0, 0);
        }
    }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g)
            s_part[wave][t][lane][g] = (v4i){acc[t][4 * g], acc[t][4 * g + 1], acc[t][4 * g + 2], acc[t][4 * g + 3]};
    if (tid < 64) s_f[tid] = f_if;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const uint32_t t = tid + 256 * u;
        if (t < n_var) s_var[t] = sv[u];
    }
    for (uint32_t t = tid + 2048; t < n_var; t += 256) s_var[t] = rot[t];
    __syncthreads();

    // (3) keys: accumulator j of lane l is variant row 8 (j / 4) + 4 (l / 32) + j % 4, neuron column l % 32
    uint32_t best = 0xffffffffu;
    {
        int dot[8];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            v4i t4 = s_part[0][ct][lane][2 * (wave >> 1) + h];
#pragma unroll
            for (int w = 1; w < 4; ++w) t4 += s_part[w][ct][lane][2 * (wave >> 1) + h];
            dot[4 * h] = t4.x; dot[4 * h + 1] = t4.y; dot[4 * h + 2] = t4.z; dot[4 * h + 3] = t4.w;
        }
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
            const uint32_t j = 8 * (wave >> 1) + jj, row = 8 * (j >> 2) + 4 * (lane >> 5) + (j & 3);
            const uint32_t kv = ((uint32_t)(na_m + nb_r[jj] - 2 * dot[jj]) << 5) | var_r[jj];
            if (row < a.R && m < N) best = min(best, kv);
        }
    }
    best = min(best, (uint32_t)__shfl_xor((int)best, 32, 64));
    if (lane < 32) s_key[wave][lane] = best;
    __syncthreads();
    // neuron c's key: the minimum of the two waves that hold its column tile; best match: first minimum of
    // the distances (Trainer.h:164-168), found by every wave for itself
    auto key_of = [&](uint32_t c) { return min(s_key[c >> 5][c & 31], s_key[(c >> 5) + 2][c & 31]); };
    const uint32_t dist = lane < N ? key_of(lane) >> 5 : 0xffffffffu, lowest = wave_min_u32_dpp(dist);
    const uint32_t bmu = (uint32_t)__builtin_ctzll(__ballot(dist == lowest));
    const uint32_t r = key_of(n) & 31u;
    const float f = s_f[bmu];
    if (n == 0 && tid == 0) {
        *a.bmu_out = bmu;
        atomicAdd(&a.counts[bmu], 1u);                    // m_update_info[bmu]++ (Trainer.h:302-303)
    }

    // (4) update (Trainer.h:175) and the neuron's row of the next SOM operand
    const uint32_t flip = r >= a.vp.num_rot ? 1u : 0u, rem = r - flip * a.vp.num_rot;
    const uint32_t q = rem / a.vp.nrr, i = rem - q * a.vp.nrr;
    const float *x = s_var + (size_t)((q & 1) * a.vp.nrr + i) * S;
    const uint32_t shift = 16 * (2 * (flip ^ (q >> 1)) + (q >> 1));       // rows reversed, columns reversed
    signed char *row_next = Pa_next + ((((size_t)(n >> 5) * KS) * 64 + (n & 31)) << 4);
    int sq = 0;
#pragma unroll
    for (int u = 0; u < EPT; ++u) {
        const uint32_t j = tid + 256 * u;
        if (j < S) {
            float nv = wv[u];
            if (f != 0.0f) {
                const uint32_t src = (uint32_t)(sp[u] >> shift) & 0xffffu;
                nv = __fsub_rn(nv, __fmul_rn(__fsub_rn(nv, x[src]), f));
                som[(size_t)n * S + j] = nv;
            }
            if (kb[u] != 0xffffffffu) {
                const int h = quantise(nv, 255.0f) - 128;
                row_next[kb[u]] = (signed char)h;
                sq += h * h;
            }
        }
    }
    sq = wave_sum_i32_dpp(sq);
    if (lane == 0) s_sq[wave] = sq;
    __syncthreads();
    if (tid == 0) a.na_next[n] = (long long)s_sq[0] + s_sq[1] + s_sq[2] + s_sq[3];
}

// ---------------------------------------------------------------------------------
// The same trainers with the kernel RESIDENT over a whole launch group: one block per neuron keeps its neuron
// -- weights in registers, its row of the SOM operand and the norm in LDS -- over all images of the group and
// computes only its own neuron's distances (the MFMA's 32 columns all hold the one neuron).  Per image the
// blocks exchange one 64-bit word each, (tag, smallest distance of the neuron), through slots a cache line
// apart: a block stores its word and its first wave polls the N slots until all carry the image's tag.  Nothing
// else crosses between blocks, so no fences: the payload rides in the atomic word.  Two sets of slots take turns
// (a block can be at most one image ahead of another).  The exchange costs about 1.4 us, where a launch boundary
// with the distance matrix worked out again in every block costs 5.
// Every wait is bounded: a wave that does not see all words within `spin_limit` polls raises `error` and marks its
// block's slots, polling waves leave when they see such a mark, a block that leaves stops publishing, so every
// block leaves.  The group's
// results go to the OTHER buffers (weights, operand, norms); the host looks at `error` after the launch and only
// then makes them the current ones, or trains the group again, image by image, from the untouched current ones.
// ---------------------------------------------------------------------------------
constexpr uint32_t kSlotStride = 16;                      // 64-bit words between two blocks' slots (128 bytes)
constexpr uint32_t kSlotWords = 2 * 64 * kSlotStride;     // two sets of 64 slots
constexpr uint32_t kGaveUpTag = 0xffffffffu;              // in a slot: its block has left the launch

struct ResidentTrain {
    const long long *na_cur;
    long long *na_next;
    const long long *nb;            // norms of the variant rows, first image; nb_stride apart
    const uint32_t *variant;        // operand row -> variant index
    uint32_t *bmu_out;              // one per image
    unsigned long long *slots;
    uint32_t *error;
    uint32_t N, S, R, KS, nstored, images, tag0, spin_limit;
    uint32_t rot_stride, pb_stride, nb_stride;      // per image: floats, 16-byte words, norms
    VariantPair vp;
};

// Eight waves per block: two share a SIMD without slowing each other, so each wave's part of every step is half as long.
constexpr uint32_t kResidentThreads = 512, kResidentWaves = kResidentThreads / 64;

template <int EPT, int KSW, int SV>    // elements of the neuron, k-steps and variant elements (first batch) per thread
__global__ __launch_bounds__(512) void k_train_small_u8_resident(const float *__restrict__ som, float *__restrict__ som_next,
                                                                 const float *__restrict__ rot, const v4i *__restrict__ Pa,
                                                                 signed char *__restrict__ Pa_next, const v4i *__restrict__ Pb,
                                                                 const float *__restrict__ factors,
                                                                 const unsigned long long *__restrict__ src4,
                                                                 const uint32_t *__restrict__ kbyte, ResidentTrain a)
{
    extern __shared__ float s_var[];                      // the stored variants of this image and of the next one
    __shared__ v4i s_op[128 + 1];                         // this neuron's operand row: [k-step][half of the k-step]; one spare
    __shared__ v4i s_part[kResidentWaves][2][4];          // [wave][half][16 accumulators]
    __shared__ int s_sq[kResidentWaves];
    __shared__ uint2 s_bmu_f;                             // the best match (all ones: leave) and this neuron's factor for it
    uint32_t &s_bmu = s_bmu_f.x;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = blockIdx.x;
    const uint32_t N = a.N, S = a.S, KS = a.KS, n_var = a.nstored * S;
    // (a launch that follows one that gave up leaves at once; one thread looks, so the whole block decides alike)
    if (tid == 0) s_bmu = __hip_atomic_load(a.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_bmu) return;

    // what stays for the whole group
    float wv[EPT];
    uint32_t cb[EPT], in_region[EPT];
    unsigned long long sp[EPT];
#pragma unroll
    for (int u = 0; u < EPT; ++u) {
        const uint32_t j = min(tid + kResidentThreads * u, S - 1);     // (past the end: the last element again, dropped at the end)
        wv[u] = som[(size_t)n * S + j];
        // byte inside the neuron's row of 32-row fragments, lanes 16 bytes apart; here inside s_op.  Elements outside
        // the region (and past the end) write the spare bytes and count nothing: no branches in the update
        const uint32_t kb = tid + kResidentThreads * u < S ? kbyte[j] : 0xffffffffu;
        in_region[u] = kb == 0xffffffffu ? 0u : 0xffffffffu;
        cb[u] = kb == 0xffffffffu ? 128u * 16u + (tid & 15u) : ((kb >> 9) << 4) | (kb & 15u);
        sp[u] = src4[j];
    }
    const float f_if = lane < N ? factors[(size_t)lane * N + n] : 0.0f;     // the factor, should neuron `lane` be the best match
    // (k-steps past the end hold zeros: a wave whose share of the k-steps ends early multiplies by them)
    if (tid < 128) {
        const v4i zero = {0, 0, 0, 0};
        s_op[tid] = tid < 2 * KS ? Pa[((size_t)(n >> 5) * KS + (tid >> 1)) * 64 + (tid & 1) * 32 + (n & 31)] : zero;
    }
    int na = (int)a.na_cur[n];
    const uint32_t row = lane & 31;                       // the operand row whose key this lane works out
    const uint32_t var_row = a.variant[row];
    const uint32_t acc_half = (row >> 2) & 1, acc_j = ((row >> 3) << 2) | (row & 3);     // where the MFMA leaves row `row`
    for (uint32_t t = tid; t < n_var; t += kResidentThreads) s_var[t] = rot[t];
    // variant r of an image: which stored variant it is read from and how (rows / columns reversed), worked out once
    // by lane r: offset of the stored variant in floats << 8 | shift into the packed source positions
    uint32_t dec_lane;
    {
        const uint32_t flip = row >= a.vp.num_rot ? 1u : 0u, rem = row - flip * a.vp.num_rot;
        const uint32_t q = rem / a.vp.nrr, b0 = rem - q * a.vp.nrr;
        dec_lane = ((((q & 1) * a.vp.nrr + b0) * S) << 8) | (16 * (2 * (flip ^ (q >> 1)) + (q >> 1)));
    }
    v4i fb[KSW];
    auto load_fragments = [&](const v4i *pb, uint32_t first) {
#pragma unroll
        for (int u = 0; u < KSW; ++u) fb[u] = pb[(size_t)min(first + kResidentWaves * u, KS - 1) * 64 + lane];
    };
    load_fragments(Pb, wave);
    int nb_row = (int)a.nb[row];
    // the variants of the image after next wait in registers for a whole image (asked for during one exchange,
    // put into LDS during the next)
    float sv[SV];
    auto load_variants = [&](const float *src) {
#pragma unroll
        for (int u = 0; u < SV; ++u) sv[u] = src[min(tid + kResidentThreads * u, n_var - 1)];
    };
    if (a.images > 1) load_variants(rot + a.rot_stride);
    __syncthreads();

    for (uint32_t i = 0; i < a.images; ++i) {
        const bool more = i + 1 < a.images;
        const v4i *pb = Pb + (size_t)i * a.pb_stride;
        float *var_cur = s_var + (i & 1) * n_var, *var_next = s_var + ((i + 1) & 1) * n_var;
        if (i + 2 == a.images) PROBE(kProbeResident, n, 0);

        // (1) this neuron against all variants: this wave's k-steps (the operand row out of LDS first: a lone
        // wave waits out every LDS read it issues between two MFMAs)
        // (the first batch whatever KS: a wave with no k-step of its own multiplies by the zero k-steps)
        v16i acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        for (uint32_t first = wave;;) {
            v4i fa[KSW];
#pragma unroll
            for (int u = 0; u < KSW; ++u) fa[u] = s_op[min(first + kResidentWaves * u, 63u) * 2 + (lane >> 5)];
#pragma unroll
            for (int u = 0; u < KSW; ++u) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[u], fa[u], acc, 0, 0, 0);
            first += kResidentWaves * KSW;
            if (first >= KS) break;
            load_fragments(pb, first);
        }
        if (i + 2 == a.images) PROBE(kProbeResident, n, 1);
        if ((lane & 31) == 0) {
#pragma unroll
            for (int g = 0; g < 4; ++g)
                s_part[wave][lane >> 5][g] = (v4i){acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
        }
        __syncthreads();
        if (i + 2 == a.images) PROBE(kProbeResident, n, 2);

        // (2) the neuron's key (every wave for itself) and its word into the exchange
        const int *part = (const int *)&s_part[0][acc_half][0] + acc_j;
        int dot = 0;                                          // the waves' k ranges
#pragma unroll
        for (uint32_t w = 0; w < kResidentWaves; ++w) dot += part[32 * w];
        const uint32_t key = row < a.R ? ((uint32_t)(na + nb_row - 2 * dot) << 5) | var_row : 0xffffffffu;
        const uint32_t best = wave_min_u32_dpp(key);
        const uint32_t tag = a.tag0 + i;
        unsigned long long *set = a.slots + (size_t)(i & 1) * 64 * kSlotStride;
        if (tid == 0)
            __hip_atomic_store(set + (size_t)n * kSlotStride, ((unsigned long long)tag << 32) | (best >> 5), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        if (i + 2 == a.images) PROBE(kProbeResident, n, 3);

        // (3) while the words travel: the next image's variants into LDS, the requests for the image after it, and the
        // part of the update that does not need the best match (the neuron's own best variant is known)
        if (more) {
#pragma unroll
            for (int u = 0; u < SV; ++u) {
                const uint32_t t = tid + kResidentThreads * u;
                if (t < n_var) var_next[t] = sv[u];
            }
            for (uint32_t t = tid + kResidentThreads * SV; t < n_var; t += kResidentThreads) var_next[t] = rot[(size_t)(i + 1) * a.rot_stride + t];
            load_fragments(pb + a.pb_stride, wave);
            nb_row = (int)a.nb[(size_t)(i + 1) * a.nb_stride + row];
            if (i + 2 < a.images) load_variants(rot + (size_t)(i + 2) * a.rot_stride);
        }
        const uint32_t dec = (uint32_t)__builtin_amdgcn_readlane((int)dec_lane, (int)(best & 31u));
        const float *x = var_cur + (dec >> 8);
        const uint32_t shift = dec & 0xffu;
        float diff[EPT];
#pragma unroll
        for (int u = 0; u < EPT; ++u) diff[u] = __fsub_rn(wv[u], x[(uint32_t)(sp[u] >> shift) & 0xffffu]);

        // (4) the first wave waits for all words
        if (wave == 0) {
            unsigned long long v = 0;
            uint32_t spins = 0;
            bool all_in = false, gave_up = false;
            // (one load per poll: a block that gives up says so in its own slots, with a tag no image has)
            while (!all_in && !gave_up) {
                v = lane < N ? __hip_atomic_load(set + (size_t)lane * kSlotStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                             : (unsigned long long)tag << 32;
                all_in = __all((uint32_t)(v >> 32) == tag) != 0;
                if (!all_in) gave_up = __any(++spins > a.spin_limit || (uint32_t)(v >> 32) == kGaveUpTag) != 0;
            }
            if (gave_up) {
                if (lane < 2)
                    __hip_atomic_store(a.slots + ((size_t)lane * 64 + n) * kSlotStride, (unsigned long long)kGaveUpTag << 32, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                if (lane == 0) {
                    __hip_atomic_store(a.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    s_bmu_f = make_uint2(0xffffffffu, 0u);
                }
            } else {
                // best match: first minimum of the distances (Trainer.h:164-168)
                const uint32_t dist = lane < N ? (uint32_t)v : 0xffffffffu, lowest = wave_min_u32_dpp(dist);
                const uint32_t bmu = (uint32_t)__builtin_ctzll(__ballot(dist == lowest));
                const uint32_t f_bits = (uint32_t)__builtin_amdgcn_readlane(__builtin_bit_cast(int, f_if), (int)bmu);
                if (lane == 0) s_bmu_f = make_uint2(bmu, f_bits);
            }
        }
        if (i + 2 == a.images) PROBE(kProbeResident, n, 4);
        __syncthreads();
        if (i + 2 == a.images) PROBE(kProbeResident, n, 5);
        const uint2 bmu_f = s_bmu_f;
        const uint32_t bmu = bmu_f.x;
        if (bmu == 0xffffffffu) return;                   // somebody gave up: every block leaves, nothing is written back
        const float f = __builtin_bit_cast(float, bmu_f.y);
        if (n == 0 && tid == 0) a.bmu_out[i] = bmu;

        // (5) the rest of the update (Trainer.h:175), the neuron's operand row and its norm
        if (f != 0.0f) {
            int sq = 0;
#pragma unroll
            for (int u = 0; u < EPT; ++u) {
                const float nv = __fsub_rn(wv[u], __fmul_rn(diff[u], f));
                wv[u] = nv;
                const int h = quantise(nv, 255.0f) - 128;
                ((signed char *)s_op)[cb[u]] = (signed char)h;
                sq += (h * h) & (int)in_region[u];
            }
            sq = wave_sum_i32_dpp(sq);
            if (lane == 0) s_sq[wave] = sq;
        }
        if (i + 2 == a.images) PROBE(kProbeResident, n, 6);
        __syncthreads();
        if (i + 2 == a.images) PROBE(kProbeResident, n, 7);
        if (f != 0.0f) {
            na = 0;
#pragma unroll
            for (uint32_t w = 0; w < kResidentWaves; ++w) na += s_sq[w];
        }
    }

    // the group's result, into the other buffers
#pragma unroll
    for (int u = 0; u < EPT; ++u) {
        const uint32_t j = tid + kResidentThreads * u;
        if (j < S) som_next[(size_t)n * S + j] = wv[u];
    }
    if (tid < 2 * KS)
        *(v4i *)(Pa_next + ((((size_t)(n >> 5) * KS) * 64 + (n & 31)) << 4) + (size_t)(tid >> 1) * 1024 + (tid & 1) * 512) = s_op[tid];
    if (tid == 0) a.na_next[n] = (long long)na;
}

// m_update_info[bmu]++ for the images of a group (Trainer.h:302-303), after a resident launch that went through.
__global__ __launch_bounds__(256) void k_count_best_matches(const uint32_t *__restrict__ bmu, uint32_t images, uint32_t *__restrict__ counts)
{
    const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t < images) atomicAdd(&counts[bmu[t]], 1u);
}

// Decode keys: distance (optionally square-rooted for the mapper, Mapper.h:206), exact
// integer sum, best rotation.  Integer modes: distance = float(double(ssd) / factor^2).
__global__ __launch_bounds__(256) void k_finalize(const unsigned long long *__restrict__ key, float *__restrict__ dist,
                                                  long long *__restrict__ ssd, uint32_t *__restrict__ best,
                                                  size_t total, uint32_t shift, uint32_t is_int, double factor2,
                                                  uint32_t do_sqrt)
{
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total) return;
    const unsigned long long kv = key[t];
    const unsigned long long v = kv >> shift;
    float d;
    if (is_int) {
        d = (float)((double)(long long)v / factor2);
        if (ssd) ssd[t] = (long long)v;
    } else {
        d = __uint_as_float((uint32_t)v);
    }
    // sqrt in double, then one rounding: the correctly rounded float square root
    // (std::sqrt(float) on the host, Mapper.h:206)
    if (do_sqrt) d = (float)sqrt((double)d);
    if (dist) dist[t] = d;
    if (best) best[t] = (uint32_t)(kv & ((1ull << shift) - 1ull));
}

// ---------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------
struct EventPair { hipEvent_t a, b; int cls; uint32_t launches; };

// Host threads that copy one buffer into another side by side (the caller takes a part too): what carries a large
// pageable input of a mapper into pinned memory faster than one thread can (a single thread moves about half of what the
// PCIe link takes).  copy() returns when every part has been copied.
class HostCopyPool {
public:
    explicit HostCopyPool(unsigned workers)
    {
        for (unsigned i = 0; i < workers; ++i) threads_.emplace_back([this, i] { loop(i); });
    }
    ~HostCopyPool()
    {
        {
            std::lock_guard<std::mutex> lock(m_);
            stop_ = true;
            ++generation_;
        }
        start_.notify_all();
        for (std::thread &t : threads_) t.join();
    }
    void copy(char *dst, const char *src, size_t bytes)
    {
        const size_t parts = threads_.size() + 1;
        {
            std::lock_guard<std::mutex> lock(m_);
            dst_ = dst; src_ = src; bytes_ = bytes;
            each_ = ((bytes + parts - 1) / parts + 4095) & ~(size_t)4095;
            pending_ = (unsigned)threads_.size();
            ++generation_;
        }
        start_.notify_all();
        part((unsigned)threads_.size());
        std::unique_lock<std::mutex> lock(m_);
        done_.wait(lock, [&] { return pending_ == 0; });
    }

private:
    void part(unsigned i) const
    {
        const size_t off = (size_t)i * each_;
        if (off < bytes_) memcpy(dst_ + off, src_ + off, std::min(each_, bytes_ - off));
    }
    void loop(unsigned i)
    {
        unsigned long long seen = 0;
        for (;;) {
            {
                std::unique_lock<std::mutex> lock(m_);
                start_.wait(lock, [&] { return generation_ != seen; });
                seen = generation_;
                if (stop_) return;
            }
            part(i);
            std::lock_guard<std::mutex> lock(m_);
            if (--pending_ == 0) done_.notify_one();
        }
    }
    std::vector<std::thread> threads_;
    std::mutex m_;
    std::condition_variable start_, done_;
    unsigned long long generation_ = 0;
    unsigned pending_ = 0;
    bool stop_ = false;
    char *dst_ = nullptr;
    const char *src_ = nullptr;
    size_t bytes_ = 0, each_ = 0;
};
constexpr size_t kBounceBytes = (size_t)8 << 20;          // pinned buffers the pool fills, two taking turns
constexpr size_t kRotateLdsMax = 158 * 1024;
enum : uint32_t { kStoreNone = 0, kStoreAll = 1, kStorePair = 2 };

}  // namespace

struct pink_hip_ctx {
    pink_hip_config cfg{};
    uint32_t N = 0, C = 0, I = 0, D = 0, S = 0, R = 0, nrr = 0, E = 0, Epad = 0, Rpad = 0;
    uint32_t isz = 0;          // floats per image
    uint32_t Bcap = 1;         // images per launch group
    uint32_t Dp = 0;           // row stride of the rotation kernel's LDS tile
    uint32_t base_lo = 0, base_hi = 0;   // rows and columns of a base rotation that the packed region reads
    uint32_t shift = 32;       // key = value << shift | rotation
    uint32_t factor = 1;       // 255 / 65535 in the integer modes
    bool trainer = false;
    bool wide_sums = false;    // integer sums need more than 31 bits
    bool use_lds = true;       // the rotation kernel keeps a block's base rotation in LDS
    bool image_lds = false;    // ... or, neurons too large for that, the image channel
    uint32_t rot_nch = 1;      // channels per block of the rotation kernel: 1, or all of them (tiles side by side in LDS)
    int device = 0;
    hipStream_t stream = nullptr;

    float *d_som = nullptr, *d_rot = nullptr, *d_cos = nullptr, *d_sin = nullptr, *d_factors = nullptr, *d_factors_t = nullptr;
    uint32_t *d_region = nullptr;
    unsigned long long *d_key = nullptr;
    void *d_somP = nullptr, *d_rotT = nullptr;
    // small float32 trainers: one launch per image, the SOM operand alternates between two buffers (d_somP is
    // always the current one), the best matches of a group of images in d_bmu_group (see k_train_f32_dpp)
    bool fused_f32_train = false;
    void *d_somP_alt = nullptr;
    uint32_t *d_bmu_group = nullptr;
    // the other float32 trainers on the vector ALU: per image the update of the SOM operand alone (k_update_rows), the
    // neurons' full images once per group
    bool rows_f32_train = false;
    uint32_t *d_bmu_scratch = nullptr;
    uint32_t *d_inv = nullptr;   // element of a neuron -> position in the region (none: ~0); null if not one-to-one
    float *d_dist = nullptr;
    long long *d_ssd = nullptr;
    uint32_t *d_best = nullptr;

    // uint8 mapping on the matrix cores
    bool mfma = false;
    uint32_t KS = 0, RT = 0, NT = 0, n_need = 0, nrr_eff = 1;
    size_t lds_dist = 0, lds_rotpack = 0, lds_max = 0;
    int num_cu = 256;
    signed char *d_Pa = nullptr, *d_Pb = nullptr;
    void *d_rtab = nullptr;                // geometry table of the base rotations (symmetric MFMA path)
    // Staging of the host-pointer entry points, kept across calls (the reference's per-image
    // operator() makes one call per image): device buffers for a chunk of images and their
    // results, and a pinned bounce buffer through which small transfers go.
    float *st_img = nullptr, *st_heat = nullptr;
    uint32_t *st_best = nullptr, *st_bmu = nullptr;
    size_t st_images = 0;                  // capacity of the staging buffers, in images
    char *st_pin = nullptr;                // kPinBytes in (as a whole, or as a ring of kPinSlots slots), kPinBytes out
    hipEvent_t st_ev[8] = {};              // per slot: the copy out of it has run
    uint32_t st_slot = 0;
    bool st_ring_busy = false;             // a call returned with copies out of the ring still queued
    // per-image training calls that hand nothing back wait here until a launch group is full (or any other call comes)
    char *pend_pin[2] = {nullptr, nullptr};
    hipEvent_t pend_ev[2] = {nullptr, nullptr};
    uint32_t pend_count = 0, pend_cur = 0, pend_cap = 0;
    hipStream_t copy_stream = nullptr;     // host -> device copies of the next images while the kernels of the last run
    hipEvent_t copy_ev[2] = {};
    // mappers, large pageable inputs: host threads fill two pinned buffers in turn, the copies to the device leave from those
    std::unique_ptr<HostCopyPool> copy_pool;
    char *bounce[2] = {nullptr, nullptr};
    hipEvent_t bounce_ev[2] = {};
    uint32_t *d_counts = nullptr;          // trainer: how often each neuron was the best match
    uint32_t *d_symoff = nullptr;          // [8][Epad] region positions under the 8 symmetries: packing fused into k_rotate
    bool fused_pack = false;
    bool pair_pack = false;                // no LDS tile of any kind: two symmetries stored, the packing kernels read the rest out of them
    uint32_t *d_region4 = nullptr;         // the region under the four row/column reversals (pair_pack)
    bool pair_variants = false;            // trainer: k_rotate stores two of the eight symmetries of a base rotation
    bool fused_som = false;                // integer GEMM trainer: k_update refreshes the SOM planes and norms itself
    uint32_t na_cur = 0;                   // which half of d_gna holds the norms of the current SOM operand
    int *d_na = nullptr, *d_nb = nullptr;
    unsigned short *d_poff = nullptr;
    uint32_t *d_need = nullptr;
    // uint8 mapping with the symmetries on the SOM side
    bool mfma_sym = false;
    uint32_t Ku = 0, KSs = 0, RTP = 0, slices = 0, groups = 1, all_sym = 0, sym_tiles = 8;
    uint32_t *d_upos = nullptr, *d_aoff = nullptr;
    unsigned char *d_kmask = nullptr;

    // integer distances as an int8 MFMA GEMM, one launch: every block owns an output tile over the whole k range
    // (training, SOMs of any size)
    bool gemm = false;
    uint32_t gKS = 0, Np = 0, Rp = 0;
    bool g_tile32 = false;     // one image: a block per 32 x 32 tile instead of 64 x 64 (few tiles, long rows)
    v4i *d_gPa = nullptr, *d_gPb = nullptr;
    v4i *d_gPa_alt = nullptr;             // small uint8 trainers: the SOM operand alternates between two buffers
    uint32_t pa_cur = 0;                   // ... which of them holds the current SOM
    bool small_train = false;              // ... one launch per image (k_train_small_u8)
    // ... or one launch per group, the blocks exchanging a word per image (k_train_small_u8_resident): the group's
    // result goes to the other buffers (d_som_alt, the other operand, the other norms) and becomes current when the
    // launch reports that no block gave up waiting
    bool resident_train = false;
    float *d_som_alt = nullptr;
    unsigned long long *d_slots = nullptr;
    uint32_t *d_resident_error = nullptr, *h_resident_error = nullptr;
    uint32_t exchange_tag = 1, spin_limit = 1u << 21;
    unsigned long long *d_src4 = nullptr;  // ... its per-element tables (see the kernel)
    uint32_t *d_kbyte = nullptr;
    uint32_t *d_grow = nullptr, *d_gvariant = nullptr;   // variant index -> row of the variant operand, and back
    long long *d_gna = nullptr, *d_gnb = nullptr;

    unsigned char *static_scratch = nullptr;   // this device's copy of the file-scope scratch array

    // float32 distances recast as a GEMM on the matrix cores (kernel_choice PINK_HIP_KERNEL_MFMA_F32 only)
    bool f32gemm = false;
    uint32_t fKS = 0, fslices = 1, fks_per = 0;
    v4f *d_fPa = nullptr, *d_fPb = nullptr;
    double *d_fna = nullptr, *d_fnb = nullptr;
    float *d_fpart = nullptr;

    bool profiling = false;
    std::vector<EventPair> events;
    std::vector<hipEvent_t> event_pool;
    uint64_t prof_launches[PINK_HIP_NUM_KERNEL_CLASSES] = {0};
    double prof_ms[PINK_HIP_NUM_KERNEL_CLASSES] = {0};

    std::string err;
};

namespace {

int fail(pink_hip_ctx *ctx, int code, const std::string &msg)
{
    if (ctx) ctx->err = msg;
    else g_create_error = msg;
    return code;
}

#define HIP_TRY(ctx, call)                                                                          \
    do {                                                                                            \
        hipError_t e_ = (call);                                                                     \
        if (e_ != hipSuccess)                                                                       \
            return fail(ctx, e_ == hipErrorOutOfMemory ? PINK_HIP_ENOMEM : PINK_HIP_EDEVICE,        \
                        std::string(#call) + ": " + hipGetErrorString(e_));                         \
    } while (0)

struct Timed {
    pink_hip_ctx *ctx;
    int cls;
    uint32_t launches;      // launches of one kernel queued back to back between the two events
    hipEvent_t a = nullptr, b = nullptr;
    Timed(pink_hip_ctx *c, int k, uint32_t n = 1) : ctx(c), cls(k), launches(n)
    {
        if (!ctx->profiling) return;
        auto take = [&]() {
            hipEvent_t e = nullptr;
            if (!ctx->event_pool.empty()) { e = ctx->event_pool.back(); ctx->event_pool.pop_back(); }
            else if (hipEventCreate(&e) != hipSuccess) e = nullptr;
            return e;
        };
        a = take();
        b = take();
        if (a) (void)hipEventRecord(a, ctx->stream);
    }
    ~Timed()
    {
        if (!ctx->profiling || !a || !b) return;
        (void)hipEventRecord(b, ctx->stream);
        ctx->events.push_back({a, b, cls, launches});
    }
};

int drain_events(pink_hip_ctx *ctx)
{
    if (ctx->events.empty()) return PINK_HIP_OK;
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    for (auto &p : ctx->events) {
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, p.a, p.b) == hipSuccess) {
            ctx->prof_ms[p.cls] += ms;
            ctx->prof_launches[p.cls] += p.launches;
        }
        ctx->event_pool.push_back(p.a);
        ctx->event_pool.push_back(p.b);
    }
    ctx->events.clear();
    return PINK_HIP_OK;
}

// Offsets of the distance region inside one C*D*D neuron, in the CPU's summation order.
// Quadratic: ImageProcessingLib/euclidean_distance.h:47-100.  Circular:
// ImageProcessingLib/circular_euclidean_distance.h:37-88 -- including its integer
// radius e/2, the empty last row of an odd diameter (NaN radicand) and, for
// multi-channel data, the missing channel offset (channel 0 counted C times).
std::vector<uint32_t> build_region(uint32_t C, uint32_t D, uint32_t e, uint32_t shape)
{
    std::vector<uint32_t> off;
    if (shape == PINK_HIP_QUADRATIC) {
        const uint32_t beg = static_cast<uint32_t>((D - e) * 0.5);
        for (uint32_t c = 0; c < C; ++c)
            for (uint32_t i = beg; i < beg + e; ++i)
                for (uint32_t j = beg; j < beg + e; ++j) off.push_back(c * D * D + i * D + j);
    } else {
        const uint32_t center = D / 2, radius = e / 2;
        for (uint32_t c = 0; c < C; ++c)
            for (uint32_t i = 0; i < e; ++i) {
                const double delta = std::sqrt(2 * radius * (i + 0.5) - std::pow(i + 0.5, 2));
                if (std::isnan(delta)) continue;
                const uint32_t gi = i + (D - e) / 2;
                const double hi = std::round(center + delta);
                for (uint32_t j = static_cast<uint32_t>(std::round(center - delta)); j < hi; ++j)
                    off.push_back(gi * D + j);
            }
    }
    return off;
}

template <typename T>
int dev_alloc(pink_hip_ctx *ctx, T **p, size_t count)
{
    HIP_TRY(ctx, hipMalloc((void **)p, (count ? count : 1) * sizeof(T)));
    return PINK_HIP_OK;
}

#define TRY(expr)                         \
    do {                                  \
        int rc_ = (expr);                 \
        if (rc_ != PINK_HIP_OK) return rc_; \
    } while (0)

int launch_check(pink_hip_ctx *ctx, const char *what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(ctx, PINK_HIP_EDEVICE, std::string(what) + ": " + hipGetErrorString(e));
    return PINK_HIP_OK;
}

bool is_int(const pink_hip_ctx *ctx) { return ctx->cfg.ed_type != PINK_HIP_FLOAT; }

// --- launch groups ---------------------------------------------------------------

// The SOM operand of the integer GEMM path that holds the current SOM (small uint8 trainers alternate between two).
static inline v4i *cur_gPa(const pink_hip_ctx *ctx) { return ctx->pa_cur ? ctx->d_gPa_alt : ctx->d_gPa; }

// Matrix-core float32 path: fragments and norms of the SOM rows (after every change of the packed rows).
int run_pack_frag_som(pink_hip_ctx *ctx)
{
    hipLaunchKernelGGL(k_pack_frag_f32, dim3(ctx->Np / 32, 1), dim3(256), 0, ctx->stream, (const float *)ctx->d_somP, ctx->d_fPa,
                       ctx->d_fna, ctx->N, ctx->Epad, (size_t)0, (size_t)0, ctx->Np);
    return launch_check(ctx, "k_pack_frag_f32");
}

int run_pack_som(pink_hip_ctx *ctx)
{
    Timed t(ctx, kClsPack);
    if (ctx->gemm) {
        if (ctx->cfg.ed_type == PINK_HIP_UINT16)
            hipLaunchKernelGGL(k_pack_planes<true>, dim3(ctx->N, 1), dim3(1024), 2 * ctx->gKS * 32, ctx->stream, ctx->d_som, ctx->d_region,
                               cur_gPa(ctx), ctx->d_gna + (size_t)ctx->na_cur * ctx->Np, ctx->N, ctx->Np, ctx->S, ctx->E, ctx->gKS, nullptr, PairSource{});
        else
            hipLaunchKernelGGL(k_pack_planes<false>, dim3(ctx->N, 1), dim3(1024), ctx->gKS * 32, ctx->stream, ctx->d_som, ctx->d_region,
                               cur_gPa(ctx), ctx->d_gna + (size_t)ctx->na_cur * ctx->Np, ctx->N, ctx->Np, ctx->S, ctx->E, ctx->gKS, nullptr, PairSource{});
        return launch_check(ctx, "k_pack_planes");
    }
    if (ctx->mfma_sym) {
        HIP_TRY(ctx, pink_sym::pack_som(ctx->stream, ctx->d_som, ctx->d_aoff, ctx->d_Pa, ctx->d_na, ctx->N, ctx->S, ctx->KSs,
                                        ctx->slices * ctx->sym_tiles * 32));
        return PINK_HIP_OK;
    }
    if (ctx->mfma) {
        hipLaunchKernelGGL(k_pack_som_u8, dim3(ctx->NT * 32), dim3(256), 0, ctx->stream, ctx->d_som, ctx->d_region,
                           ctx->d_Pa, ctx->d_na, ctx->N, ctx->S, ctx->E, ctx->KS);
        return launch_check(ctx, "k_pack_som_u8");
    }
    const size_t total = (size_t)ctx->N * ctx->Epad;
    const uint32_t blocks = (uint32_t)std::min<size_t>((total + 255) / 256, 8192);
    if (is_int(ctx))
        hipLaunchKernelGGL(k_pack_som<true>, dim3(blocks), dim3(256), 0, ctx->stream, ctx->d_som, ctx->d_region,
                           ctx->d_somP, ctx->N, ctx->S, ctx->E, ctx->Epad, (float)ctx->factor);
    else
        hipLaunchKernelGGL(k_pack_som<false>, dim3(blocks), dim3(256), 0, ctx->stream, ctx->d_som, ctx->d_region,
                           ctx->d_somP, ctx->N, ctx->S, ctx->E, ctx->Epad, 1.0f);
    TRY(launch_check(ctx, "k_pack_som"));
    return ctx->f32gemm ? run_pack_frag_som(ctx) : PINK_HIP_OK;
}

// store: kStoreNone, kStoreAll or kStorePair (see k_rotate)
int run_rotate(pink_hip_ctx *ctx, const float *dev_images, uint32_t B, uint32_t store)
{
    const bool store_variants = store != kStoreNone;
    Timed t(ctx, kClsRotate);
    if (ctx->pair_pack && store == kStorePair) {
        const uint32_t tiles_per_row = (ctx->D + kRotTile - 1) / kRotTile;
        hipLaunchKernelGGL(k_rotate_pair_tiled, dim3(tiles_per_row * tiles_per_row, std::max(ctx->nrr, 1u), ctx->C * B), dim3(256), 0,
                           ctx->stream, dev_images, ctx->d_rot, ctx->d_cos, ctx->d_sin, ctx->d_key, ctx->N, ctx->C, ctx->I, ctx->D,
                           ctx->cfg.num_rot, ctx->cfg.use_flip, tiles_per_row);
        return launch_check(ctx, "k_rotate_pair_tiled");
    }
    const dim3 grid(std::max(ctx->nrr, 1u), ctx->C / ctx->rot_nch, B);
    const size_t lds = ctx->use_lds ? (size_t)ctx->rot_nch * ctx->D * ctx->Dp * sizeof(float)
                     : ctx->image_lds ? (size_t)ctx->I * ctx->I * sizeof(float) : 0;
    // about four neuron pixels per thread: large neurons get large blocks, whose many waves per LDS
    // footprint hide the latency of the gathers (measured: 1024 threads 35 % faster than 256 at 3 x 70 x 70)
    uint32_t threads = 256;
    while (threads < 1024 && threads * 4 < ctx->D * ctx->D) threads *= 2;
    PackArgs pk{};
    int pack = 0;
    if (ctx->fused_pack) {
        pk.symoff = ctx->d_symoff;
        pk.E = ctx->E;
        pk.Epad = ctx->Epad;
        if (ctx->gemm) {
            pack = ctx->cfg.ed_type == PINK_HIP_UINT16 ? 3 : 2;
            pk.opnd = ctx->d_gPb; pk.norm = ctx->d_gnb; pk.rows_pad = ctx->Rp; pk.KS = ctx->gKS;
        } else {
            pack = 1;
            pk.opnd = ctx->d_rotT; pk.rows_pad = ctx->Rpad;
        }
    }
#define LAUNCH_ROTATE_(P_, L_)                                                                                     \
    hipLaunchKernelGGL((k_rotate<P_, L_>), grid, dim3(threads), lds, ctx->stream, dev_images, ctx->d_rot, ctx->d_cos, ctx->d_sin, \
                       ctx->d_key, ctx->N, ctx->C, ctx->I, ctx->D, ctx->cfg.num_rot, ctx->cfg.use_flip,               \
                       ctx->Dp, pk, store,                   \
                       store_variants ? 0u : ctx->base_lo, store_variants ? ctx->D : ctx->base_hi, ctx->rot_nch)
#define LAUNCH_ROTATE(P_)                         \
    do {                                          \
        if (ctx->use_lds) LAUNCH_ROTATE_(P_, 1);  \
        else if (ctx->image_lds) LAUNCH_ROTATE_(P_, 2); \
        else LAUNCH_ROTATE_(P_, 0);               \
    } while (0)
    switch (pack) {
    case 1: LAUNCH_ROTATE(1); break;
    case 2: LAUNCH_ROTATE(2); break;
    case 3: LAUNCH_ROTATE(3); break;
    default: LAUNCH_ROTATE(0); break;
    }
#undef LAUNCH_ROTATE
#undef LAUNCH_ROTATE_
    return launch_check(ctx, "k_rotate");
}

int run_pack_rot(pink_hip_ctx *ctx, uint32_t B)
{
    if (ctx->f32gemm) {
        // the float rows (written by k_rotate or packed below) also go into fragments, with their norms
        if (!ctx->fused_pack) {
            Timed t(ctx, kClsPack);
            PairSource ps{};
            if (ctx->pair_pack) { ps.off4 = ctx->d_region4; ps.num_rot = ctx->cfg.num_rot; ps.nrr = std::max(ctx->nrr, 1u); ps.E = ctx->E; }
            hipLaunchKernelGGL(k_pack_rot_rows, dim3((ctx->Epad + 255) / 256, ctx->Rpad, B), dim3(256), 0, ctx->stream,
                               ctx->d_rot, ctx->d_region, (float *)ctx->d_rotT, ctx->R, ctx->S, ctx->E, ctx->Epad, ctx->Rpad, ps);
            TRY(launch_check(ctx, "k_pack_rot_rows"));
        }
        Timed t(ctx, kClsPack);
        hipLaunchKernelGGL(k_pack_frag_f32, dim3(ctx->Rp / 32, B), dim3(256), 0, ctx->stream, (const float *)ctx->d_rotT, ctx->d_fPb,
                           ctx->d_fnb, ctx->R, ctx->Epad, (size_t)ctx->Epad * ctx->Rpad, (size_t)(ctx->Rp / 32) * ctx->fKS * 64, ctx->Rp);
        return launch_check(ctx, "k_pack_frag_f32");
    }
    if (ctx->fused_pack) return PINK_HIP_OK;              // k_rotate wrote the operand already
    Timed t(ctx, kClsPack);
    PairSource ps{};
    if (ctx->pair_pack) { ps.off4 = ctx->d_region4; ps.num_rot = ctx->cfg.num_rot; ps.nrr = std::max(ctx->nrr, 1u); ps.E = ctx->E; }
    if (ctx->gemm) {
        // long rows: large blocks, so that a CU (a few blocks by their LDS rows) still runs all its waves
        const uint32_t pack_threads = ctx->gKS * 32 >= 4096 ? 1024 : 256;
        if (ctx->cfg.ed_type == PINK_HIP_UINT16)
            hipLaunchKernelGGL(k_pack_planes<true>, dim3(ctx->R, B), dim3(pack_threads), 2 * ctx->gKS * 32, ctx->stream, ctx->d_rot, ctx->d_region,
                               ctx->d_gPb, ctx->d_gnb, ctx->R, ctx->Rp, ctx->S, ctx->E, ctx->gKS, ctx->d_grow, ps);
        else
            hipLaunchKernelGGL(k_pack_planes<false>, dim3(ctx->R, B), dim3(pack_threads), ctx->gKS * 32, ctx->stream, ctx->d_rot, ctx->d_region,
                               ctx->d_gPb, ctx->d_gnb, ctx->R, ctx->Rp, ctx->S, ctx->E, ctx->gKS, ctx->d_grow, ps);
        return launch_check(ctx, "k_pack_planes");
    }
    if (!is_int(ctx)) {
        hipLaunchKernelGGL(k_pack_rot_rows, dim3((ctx->Epad + 255) / 256, ctx->Rpad, B), dim3(256), 0, ctx->stream,
                           ctx->d_rot, ctx->d_region, (float *)ctx->d_rotT, ctx->R, ctx->S, ctx->E, ctx->Epad, ctx->Rpad, ps);
        return launch_check(ctx, "k_pack_rot_rows");
    }
    const dim3 grid(ctx->Epad / 32, ctx->Rpad / 32, B);
    if (is_int(ctx))
        hipLaunchKernelGGL(k_pack_rot<true>, grid, dim3(256), 0, ctx->stream, ctx->d_rot, ctx->d_region, ctx->d_rotT,
                           ctx->R, ctx->S, ctx->E, ctx->Epad, ctx->Rpad, (float)ctx->factor, ps);
    else
        hipLaunchKernelGGL(k_pack_rot<false>, grid, dim3(256), 0, ctx->stream, ctx->d_rot, ctx->d_region, ctx->d_rotT,
                           ctx->R, ctx->S, ctx->E, ctx->Epad, ctx->Rpad, 1.0f, ps);
    return launch_check(ctx, "k_pack_rot");
}

template <int MODE>
void launch_dist(pink_hip_ctx *ctx, uint32_t slot, uint32_t B)
{
    // Neurons per wave: as many as keep at least ~2 waves per SIMD in flight.
    const uint32_t rblocks = ctx->Rpad / kWave;
    const size_t target_waves = 2048;
    uint32_t tn = 8;
    while (tn > 1 && (size_t)rblocks * ((ctx->N + tn - 1) / tn) * B < target_waves) tn >>= 1;
    const dim3 grid(rblocks, (ctx->N + tn - 1) / tn, B);
    const void *rotT = (const char *)ctx->d_rotT + (size_t)slot * ctx->Epad * ctx->Rpad * 4;
    unsigned long long *key = ctx->d_key + (size_t)slot * ctx->N;
#define LAUNCH_TN(T_)                                                                                           \
    hipLaunchKernelGGL((k_dist_valu<MODE, T_>), grid, dim3(64), 0, ctx->stream, ctx->d_somP, rotT, key,        \
                       ctx->N, ctx->Epad, ctx->R, ctx->Rpad)
    switch (tn) {
    case 8: LAUNCH_TN(8); break;
    case 4: LAUNCH_TN(4); break;
    case 2: LAUNCH_TN(2); break;
    default: LAUNCH_TN(1); break;
    }
#undef LAUNCH_TN
}

// Distance + argmin of B images starting at image slot `slot` of the current launch group.
void launch_dist_f32(pink_hip_ctx *ctx, uint32_t slot, uint32_t B)
{
    // A block is 64 rows on its lanes x (4 waves x TN) rows as per-wave operands.  While the blocks of one
    // neuron per wave are all resident at once (four per CU; measured up to 225 neurons x 720 rotations):
    // rotations on the lanes, neuron values by DPP broadcast, deep register prefetch.  More work than that:
    // per-wave operands as scalar registers, the largest TN that still leaves the chip about four waves per
    // SIMD (a value read from LDS then serves TN chains), and on the lanes whichever of rotations and neurons
    // loses fewer lanes to padding (360 rotations fill 5.6 tiles of 64, 1600 neurons exactly 25).
    const uint32_t rblocks = ctx->Rpad / kWave, nblocks = (ctx->N + kWave - 1) / kWave;
    auto groups = [](uint32_t rows, uint32_t tn) { return (rows + 4 * tn - 1) / (4 * tn); };
    const bool scalar_operands = (size_t)rblocks * groups(ctx->N, 1) * B > (size_t)4 * ctx->num_cu;
    const float *rotT = (const float *)ctx->d_rotT + (size_t)slot * ctx->Epad * ctx->Rpad;
    unsigned long long *key = ctx->d_key + (size_t)slot * ctx->N;
    if (!scalar_operands) {
        hipLaunchKernelGGL(k_dist_f32_dpp, dim3(rblocks, groups(ctx->N, 1), B), dim3(256), 0, ctx->stream,
                           (const float *)ctx->d_somP, rotT, key, ctx->N, ctx->Epad, ctx->R, ctx->Rpad);
        return;
    }
    // lanes computed, padding included, per image: rotations on the lanes / neurons on the lanes (TN = 2 for the comparison)
    const size_t work_rot = (size_t)rblocks * kWave * groups(ctx->N, 2) * 8, work_neu = (size_t)nblocks * kWave * groups(ctx->R, 2) * 8;
    const bool neurons_on_lanes = work_neu * 100 < work_rot * 98;
    const uint32_t lane_blocks = neurons_on_lanes ? nblocks : rblocks, scal_rows = neurons_on_lanes ? ctx->R : ctx->N;
    const uint32_t tn = (size_t)lane_blocks * groups(scal_rows, 4) * B >= (size_t)4 * ctx->num_cu ? 4 : 2;
    const uint32_t scal_groups = groups(scal_rows, tn);
    const dim3 grid((lane_blocks * scal_groups + 7) / 8 * 8, 1, B);        // (see the kernel: an XCD takes a run of pairs)
#define LAUNCH_SG(...)                                                                                             \
    hipLaunchKernelGGL((k_dist_f32_sg<__VA_ARGS__>), grid, dim3(256), 0, ctx->stream, (const float *)ctx->d_somP,  \
                       (const float *)ctx->d_rotT + (size_t)slot * ctx->Epad * ctx->Rpad, key, ctx->N, ctx->Epad, ctx->R, ctx->Rpad, \
                       lane_blocks, scal_groups)
    // (TN = 4: 8-element slabs, 4 x 8 x 2 sets of scalar registers)
    if (neurons_on_lanes) { if (tn == 4) LAUNCH_SG(4, 32, 6, 8, true); else LAUNCH_SG(2, 32, 6, 16, true); }
    else { if (tn == 4) LAUNCH_SG(4, 32, 6, 8, false); else LAUNCH_SG(2, 32, 6, 16, false); }
#undef LAUNCH_SG
}

// Distances of B images starting at image slot `slot`: one launch, every block takes the whole k range of its
// tile and finishes it.  Several images (mapping) fill the chip with 64 x 64 tiles; one image (training) with few
// tiles and long rows takes 32 x 32 tiles (measured against 64 x 64 tiles with k cut across blocks and a second
// kernel that adds the partial sums up, images/s of the whole training step: 253 tiles x 135 k-steps uint16 +17 %,
// 299 x 64 uint16 +27 %, 414 x 64 uint16 +25 %, 299 x 128 uint8 +13 %, equal from 23 to 184 tiles).
template <bool U16>
void launch_dist_gemm(pink_hip_ctx *ctx, uint32_t slot, uint32_t B)
{
    const uint32_t planes = U16 ? 2 : 1;
    const v4i *pb = ctx->d_gPb + (size_t)slot * planes * (ctx->Rp / 32) * ctx->gKS * 64;
    const bool tile32 = B == 1 && ctx->g_tile32;
    const uint32_t side = tile32 ? 32u : 64u;
    // The 8 XCDs (each with its own L2) take rectangles of the tile grid: the split xr x xc = 8 with the fewest
    // operand rows per XCD (a tile row of variants and a tile column of neurons cost the same bytes).
    const uint32_t row_tiles = ctx->Rp / side, col_tiles = ctx->Np / side;
    uint32_t xc = 1, cost = ~0u;
    for (uint32_t c = 1; c <= 8; c *= 2) {
        const uint32_t r = 8 / c, v = (row_tiles + r - 1) / r + (col_tiles + c - 1) / c;
        if (v < cost) { cost = v; xc = c; }
    }
    const uint32_t rect_h = (row_tiles + 8 / xc - 1) / (8 / xc), rect_w = (col_tiles + xc - 1) / xc;
    const uint32_t tiles_per_xcd = rect_h * rect_w;
    const uint32_t ks_per = (ctx->gKS + 3) / 4;
    GemmFinish fin{};
    fin.key = ctx->d_key + (size_t)slot * ctx->N;
    fin.na = ctx->d_gna + (size_t)ctx->na_cur * ctx->Np;
    fin.na_other = ctx->d_gna + (size_t)(ctx->na_cur ^ 1) * ctx->Np;
    fin.nb = ctx->d_gnb + (size_t)slot * ctx->Rp;
    fin.variant = ctx->d_gvariant;
    fin.N = ctx->N; fin.R = ctx->R;
    const uint32_t real_tiles = ((ctx->R + side - 1) / side) * ((ctx->N + side - 1) / side);
    if (tile32 && real_tiles <= (uint32_t)ctx->num_cu) {
        // one block per CU at most: every XCD takes the same number of consecutive real tiles (see the kernel)
        const uint32_t per_xcd = (real_tiles + 7) / 8;
        hipLaunchKernelGGL((k_dist_gemm_int<U16, 1>), dim3(8 * per_xcd, 1), dim3(256), 0, ctx->stream, cur_gPa(ctx), pb,
                           ctx->Np, ctx->Rp, ctx->gKS, ks_per, per_xcd, 0u, 1u, fin);
    } else if (tile32)
        hipLaunchKernelGGL((k_dist_gemm_int<U16, 1>), dim3(8 * tiles_per_xcd, 1), dim3(256), 0, ctx->stream, cur_gPa(ctx), pb,
                           ctx->Np, ctx->Rp, ctx->gKS, ks_per, rect_h, rect_w, xc, fin);
    else
        hipLaunchKernelGGL((k_dist_gemm_int<U16, 2>), dim3(8 * tiles_per_xcd, B), dim3(256), 0, ctx->stream, cur_gPa(ctx), pb,
                           ctx->Np, ctx->Rp, ctx->gKS, ks_per, rect_h, rect_w, xc, fin);
}

// Distances of B images starting at image slot `slot` on the matrix cores, float32.
int run_dist_f32gemm(pink_hip_ctx *ctx, uint32_t slot, uint32_t B)
{
    const uint32_t tiles = (ctx->Rp / 64) * (ctx->Np / 64);
    const uint32_t slices = B > 1 ? 1 : ctx->fslices;
    const uint32_t ks_per = B > 1 ? (ctx->fKS + 3) / 4 : ctx->fks_per;
    GemmFinishF32 fin{};
    fin.na = ctx->d_fna;
    fin.nb = ctx->d_fnb + (size_t)slot * ctx->Rp;
    fin.N = ctx->N; fin.R = ctx->R;
    unsigned long long *key = ctx->d_key + (size_t)slot * ctx->N;
    if (slices == 1) fin.key = key;
    const v4f *pb = ctx->d_fPb + (size_t)slot * (ctx->Rp / 32) * ctx->fKS * 64;
    hipLaunchKernelGGL(k_dist_gemm_f32, dim3(tiles * slices, B), dim3(256), 65536, ctx->stream, (const v4f *)ctx->d_fPa, pb, ctx->d_fpart,
                       ctx->Np, ctx->Rp, ctx->fKS, ks_per, slices, fin);
    TRY(launch_check(ctx, "k_dist_gemm_f32"));
    if (slices == 1) return PINK_HIP_OK;
    const uint32_t rows_per_chunk = 32;
    hipLaunchKernelGGL(k_dist_finish_f32, dim3((ctx->N + 31) / 32, (ctx->R + rows_per_chunk - 1) / rows_per_chunk), dim3(256), 0,
                       ctx->stream, (const float *)ctx->d_fpart, (const double *)ctx->d_fna, fin.nb, key, ctx->N, ctx->Np, ctx->R,
                       ctx->Rp, slices, rows_per_chunk);
    return launch_check(ctx, "k_dist_finish_f32");
}

int run_dist(pink_hip_ctx *ctx, uint32_t slot, uint32_t B)
{
    Timed t(ctx, kClsDist);
    if (ctx->f32gemm) return run_dist_f32gemm(ctx, slot, B);
    if (ctx->gemm) {
        if (ctx->cfg.ed_type == PINK_HIP_UINT16) launch_dist_gemm<true>(ctx, slot, B);
        else launch_dist_gemm<false>(ctx, slot, B);
        return launch_check(ctx, "k_dist_gemm_int");
    }
    // the vector-ALU kernels below read d_somP / d_rotT: never reached without them
    if (!ctx->d_somP || !ctx->d_rotT) return fail(ctx, PINK_HIP_ESTATE, "distance operands were not allocated");
    switch (ctx->cfg.ed_type) {
    case PINK_HIP_FLOAT: launch_dist_f32(ctx, slot, B); break;
    case PINK_HIP_UINT8:
        if (ctx->wide_sums) launch_dist<2>(ctx, slot, B);
        else launch_dist<1>(ctx, slot, B);
        break;
    default: launch_dist<2>(ctx, slot, B); break;
    }
    return launch_check(ctx, "k_dist");
}

int run_update(pink_hip_ctx *ctx, uint32_t slot, uint32_t *dev_bmu_out)
{
    Timed t(ctx, kClsUpdate);
    // about 1024 blocks; a small SOM (every block repeats the search for the best match) does better with about 128
    const uint32_t target_blocks = (size_t)ctx->N * ctx->S >= ((size_t)1 << 20) ? 1024u : 128u;
    uint32_t parts = (target_blocks + ctx->N - 1) / ctx->N;
    parts = std::max(1u, std::min(parts, (ctx->S + 255) / 256));
    UpdatePlanes up{};
    if (ctx->fused_som) {
        up.Pa = (signed char *)cur_gPa(ctx);
        up.na_cur = ctx->d_gna + (size_t)ctx->na_cur * ctx->Np;
        up.na_next = ctx->d_gna + (size_t)(ctx->na_cur ^ 1) * ctx->Np;
        up.KS = ctx->gKS; up.Np = ctx->Np; up.u16 = ctx->cfg.ed_type == PINK_HIP_UINT16;
    }
    VariantPair vp{};
    if (ctx->pair_variants) { vp.D = ctx->D; vp.num_rot = ctx->cfg.num_rot; vp.nrr = std::max(ctx->nrr, 1u); }
    // (see the kernel: with the byte planes, the four neurons that share lines of them on one XCD)
    const dim3 grid = up.Pa ? dim3(32 * ((ctx->N + 31) / 32), parts) : dim3(parts, ctx->N);
#define LAUNCH_UPDATE(U_)                                                                                        \
    hipLaunchKernelGGL(k_update<U_>, grid, dim3(256), 0, ctx->stream, ctx->d_som,                                  \
                       ctx->d_rot + (size_t)slot * ctx->R * ctx->S, ctx->d_key + (size_t)slot * ctx->N, ctx->d_factors_t, \
                       dev_bmu_out, ctx->N, ctx->S, parts, ctx->shift, ctx->d_somP,                                \
                       ctx->fused_som ? ctx->d_kbyte : ctx->gemm ? nullptr : ctx->d_inv, ctx->Epad,                \
                       is_int(ctx) ? (float)ctx->factor : 0.0f, up, ctx->d_counts, vp)
    // a slice of several rounds keeps eight elements per thread in flight (cfg2 -6 %, cfg3 -3 % against four);
    // a slice of one round is faster with four (cfg0 +8 % with eight)
    // ... and in rounds of equal length: a slice of 2809 elements takes two rounds of six per thread, not eight and three
    // (cfg2: 15.2 -> 14.6 us; eleven or twelve per thread, a single round, 15.8 and 16.1)
    const uint32_t chunk = (ctx->S + parts - 1) / parts;
    uint32_t per_thread = 4;
    if (chunk > 1024) {
        const uint32_t rounds = (chunk + 2047) / 2048;
        per_thread = std::min(8u, std::max(4u, (chunk + 256 * rounds - 1) / (256 * rounds)));
    }
    switch (per_thread) {
    case 4: LAUNCH_UPDATE(4); break;
    case 5: LAUNCH_UPDATE(5); break;
    case 6: LAUNCH_UPDATE(6); break;
    case 7: LAUNCH_UPDATE(7); break;
    default: LAUNCH_UPDATE(8); break;
    }
#undef LAUNCH_UPDATE
    if (ctx->fused_som) ctx->na_cur ^= 1;                  // the norms of the updated SOM are in the other buffer now
    return launch_check(ctx, "k_update");
}

// Distances of the image in slot `slot` against the SOM with the update of the image before it applied on the
// way (small float32 trainers, k_train_f32_dpp); that image's best match goes to *bmu_prev.
int run_train_f32(pink_hip_ctx *ctx, uint32_t slot, bool has_prev, uint32_t *bmu_prev)
{
    PrevImage prev{};
    if (has_prev) {
        prev.key = ctx->d_key + (size_t)(slot - 1) * ctx->N;
        prev.rotT = (const float *)ctx->d_rotT + (size_t)(slot - 1) * ctx->Epad * ctx->Rpad;
        prev.factors_t = ctx->d_factors_t;
        prev.somP_next = (float *)ctx->d_somP_alt;
        prev.bmu_out = bmu_prev;
        prev.counts = ctx->d_counts;
    }
    // neurons (waves) per block: four, or the five to eight that make the launch one block per CU where four do not
    // (measured: 2 to 4 % per image; two blocks of five on a CU do not run side by side -- 28 against 21 us)
    const uint32_t rblocks = ctx->Rpad / kWave;
    uint32_t per_block = 4;
    if (rblocks * ((ctx->N + 3) / 4) > (uint32_t)ctx->num_cu)
        for (uint32_t w = 5; w <= 8 && per_block == 4; ++w)
            if (rblocks * ((ctx->N + w - 1) / w) <= (uint32_t)ctx->num_cu) per_block = w;
#define LAUNCH_TRAIN_F32(NQ_)                                                                                          \
    hipLaunchKernelGGL(k_train_f32_dpp<NQ_>, dim3(rblocks, (ctx->N + per_block - 1) / per_block), dim3(64 * per_block), 0, ctx->stream, \
                       (const float *)ctx->d_somP, (const float *)ctx->d_rotT + (size_t)slot * ctx->Epad * ctx->Rpad,   \
                       ctx->d_key + (size_t)slot * ctx->N, ctx->N, ctx->Epad, ctx->R, ctx->Rpad, prev)
    if (ctx->N <= 128) LAUNCH_TRAIN_F32(2); else LAUNCH_TRAIN_F32(4);
#undef LAUNCH_TRAIN_F32
    if (has_prev) std::swap(ctx->d_somP, ctx->d_somP_alt);        // the updated operand is the current one now
    return launch_check(ctx, "k_train_f32_dpp");
}

// The update of the image in slot `slot` on the float32 distance operand alone (k_update_rows).
int run_update_rows(pink_hip_ctx *ctx, uint32_t slot, uint32_t *dev_bmu_out)
{
    Timed t(ctx, kClsUpdate);
    const uint32_t vecs = ctx->Epad / 4;
    const uint32_t target_blocks = (size_t)ctx->N * ctx->Epad >= ((size_t)1 << 20) ? 1024u : 128u;
    uint32_t parts = (target_blocks + ctx->N - 1) / ctx->N;
    parts = std::max(1u, std::min(parts, (vecs + 255) / 256));
    hipLaunchKernelGGL(k_update_rows, dim3(parts, ctx->N), dim3(256), 0, ctx->stream, (float *)ctx->d_somP,
                       (const float *)ctx->d_rotT + (size_t)slot * ctx->Epad * ctx->Rpad, ctx->d_key + (size_t)slot * ctx->N,
                       ctx->d_factors_t, dev_bmu_out, ctx->d_counts, ctx->N, ctx->Epad, parts, ctx->shift);
    return launch_check(ctx, "k_update_rows");
}

// The updates of the first `images` images of the current group applied to the neurons' full images, in order.
int run_update_replay(pink_hip_ctx *ctx, uint32_t images, const uint32_t *dev_bmu)
{
    Timed t(ctx, kClsUpdate);
    VariantPair vp{};
    if (ctx->pair_variants) { vp.D = ctx->D; vp.num_rot = ctx->cfg.num_rot; vp.nrr = std::max(ctx->nrr, 1u); }
    for (uint32_t first = 0; first < images; first += kReplayMax) {
        const uint32_t count = std::min(kReplayMax, images - first);
#define LAUNCH_REPLAY(EPT_)                                                                                                   \
    hipLaunchKernelGGL(k_update_replay<EPT_>, dim3(ctx->N, (ctx->S + 256 * EPT_ - 1) / (256 * EPT_)), dim3(256), 0, ctx->stream, \
                       ctx->d_som, ctx->d_rot + (size_t)first * ctx->R * ctx->S, ctx->d_key + (size_t)first * ctx->N,            \
                       ctx->d_factors, dev_bmu + first, count, ctx->N, ctx->S, ctx->R, ctx->shift, vp)
        // (large SOMs: several elements per thread -- 1600 neurons of 3 x 70 x 70: 13.6 us per image with one, 10.2 with
        // two, 9.0 with four; small ones need the blocks -- 100 neurons of 45 x 45: 0.42, 0.46)
        const size_t weights = (size_t)ctx->N * ctx->S;
        if (weights >= ((size_t)1 << 22)) LAUNCH_REPLAY(4);
        else if (weights >= ((size_t)1 << 20)) LAUNCH_REPLAY(2);
        else LAUNCH_REPLAY(1);
#undef LAUNCH_REPLAY
        TRY(launch_check(ctx, "k_update_replay"));
    }
    return PINK_HIP_OK;
}

// Distances, best match and update of the image in slot `slot` in one launch (small uint8 trainers).
int run_train_small(pink_hip_ctx *ctx, uint32_t slot, uint32_t *dev_bmu_out)
{
    Timed t(ctx, kClsUpdate);
    SmallTrain a{};
    a.na_cur = ctx->d_gna + (size_t)ctx->na_cur * ctx->Np;
    a.na_next = ctx->d_gna + (size_t)(ctx->na_cur ^ 1) * ctx->Np;
    a.nb = ctx->d_gnb + (size_t)slot * ctx->Rp;
    a.variant = ctx->d_gvariant;
    a.bmu_out = dev_bmu_out; a.counts = ctx->d_counts;
    a.N = ctx->N; a.S = ctx->S; a.R = ctx->R; a.KS = ctx->gKS;
    a.nstored = std::min(2 * std::max(ctx->nrr, 1u), ctx->R);
    a.vp.D = ctx->D; a.vp.num_rot = ctx->cfg.num_rot; a.vp.nrr = std::max(ctx->nrr, 1u);
    const v4i *pa = cur_gPa(ctx);
    signed char *pa_next = (signed char *)(ctx->pa_cur ? ctx->d_gPa : ctx->d_gPa_alt);
    const v4i *pb = ctx->d_gPb + (size_t)slot * (ctx->Rp / 32) * ctx->gKS * 64;
    const float *rot = ctx->d_rot + (size_t)slot * ctx->R * ctx->S;
    const size_t lds = (size_t)a.nstored * ctx->S * sizeof(float);
#define LAUNCH_SMALL(...)                                                                                        \
    hipLaunchKernelGGL((k_train_small_u8<__VA_ARGS__>), dim3(ctx->N), dim3(256), lds, ctx->stream, ctx->d_som, rot, pa, pa_next, pb, \
                       ctx->d_factors, ctx->d_src4, ctx->d_kbyte, a)
    // (elements per thread, k-steps a wave holds at a time: one batch of operand loads up to 32 k-steps)
    if (ctx->S <= 1024) LAUNCH_SMALL(4, 8); else LAUNCH_SMALL(8, 8);
#undef LAUNCH_SMALL
    ctx->pa_cur ^= 1;
    ctx->na_cur ^= 1;
    return launch_check(ctx, "k_train_small_u8");
}

// The first `images` images of the current group in one resident launch (small uint8 trainers).  `went_through`
// false: a block gave up waiting for the others (the device was not free to hold all blocks at once); nothing of
// the context has changed then, the context stops using this form, and the caller trains the group image by image.
int run_train_small_resident(pink_hip_ctx *ctx, uint32_t images, uint32_t *dev_bmu, bool *went_through)
{
    *went_through = false;
    if (ctx->exchange_tag > 0xfffffff0u - images) {        // the tags wrap: back to 1, over slots that hold none
        HIP_TRY(ctx, hipMemsetAsync(ctx->d_slots, 0, kSlotWords * sizeof(unsigned long long), ctx->stream));
        ctx->exchange_tag = 1;
    }
    ResidentTrain a{};
    a.na_cur = ctx->d_gna + (size_t)ctx->na_cur * ctx->Np;
    a.na_next = ctx->d_gna + (size_t)(ctx->na_cur ^ 1) * ctx->Np;
    a.nb = ctx->d_gnb;
    a.variant = ctx->d_gvariant;
    a.bmu_out = dev_bmu;
    a.slots = ctx->d_slots;
    a.error = ctx->d_resident_error;
    a.N = ctx->N; a.S = ctx->S; a.R = ctx->R; a.KS = ctx->gKS;
    a.nstored = std::min(2 * std::max(ctx->nrr, 1u), ctx->R);
    a.images = images; a.tag0 = ctx->exchange_tag; a.spin_limit = ctx->spin_limit;
    a.rot_stride = ctx->R * ctx->S;
    a.pb_stride = (ctx->Rp / 32) * ctx->gKS * 64;
    a.nb_stride = ctx->Rp;
    a.vp.D = ctx->D; a.vp.num_rot = ctx->cfg.num_rot; a.vp.nrr = std::max(ctx->nrr, 1u);
    ctx->exchange_tag += images;
    const v4i *pa = cur_gPa(ctx);
    signed char *pa_next = (signed char *)(ctx->pa_cur ? ctx->d_gPa : ctx->d_gPa_alt);
    const size_t lds = (size_t)2 * a.nstored * ctx->S * sizeof(float);
    {
        Timed t(ctx, kClsUpdate);
#define LAUNCH_RESIDENT(...)                                                                                          \
    hipLaunchKernelGGL((k_train_small_u8_resident<__VA_ARGS__>), dim3(ctx->N), dim3(kResidentThreads), lds, ctx->stream, ctx->d_som, \
                       ctx->d_som_alt, ctx->d_rot, pa, pa_next, ctx->d_gPb, ctx->d_factors, ctx->d_src4, ctx->d_kbyte, a)
        // (elements of a neuron per thread, k-steps per wave in one batch, variant elements per thread in registers)
        const bool few_variant_elements = (size_t)a.nstored * ctx->S <= 4 * kResidentThreads;
        if (ctx->S <= 1024 && few_variant_elements) LAUNCH_RESIDENT(2, 4, 4);
        else if (ctx->S <= 1024) LAUNCH_RESIDENT(2, 4, 8);
        else LAUNCH_RESIDENT(4, 8, 8);
#undef LAUNCH_RESIDENT
        TRY(launch_check(ctx, "k_train_small_u8_resident"));
    }
    HIP_TRY(ctx, hipMemcpyAsync(ctx->h_resident_error, ctx->d_resident_error, sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    if (*ctx->h_resident_error) {
        ctx->resident_train = false;
        HIP_TRY(ctx, hipMemsetAsync(ctx->d_resident_error, 0, sizeof(uint32_t), ctx->stream));
        HIP_TRY(ctx, hipMemsetAsync(ctx->d_slots, 0, kSlotWords * sizeof(unsigned long long), ctx->stream));
        return PINK_HIP_OK;
    }
    std::swap(ctx->d_som, ctx->d_som_alt);
    ctx->pa_cur ^= 1;
    ctx->na_cur ^= 1;
    hipLaunchKernelGGL(k_count_best_matches, dim3((images + 255) / 256), dim3(256), 0, ctx->stream, dev_bmu, images, ctx->d_counts);
    TRY(launch_check(ctx, "k_count_best_matches"));
    *went_through = true;
    return PINK_HIP_OK;
}

int run_finalize(pink_hip_ctx *ctx, uint32_t B, float *dev_dist, long long *dev_ssd, uint32_t *dev_best, bool do_sqrt)
{
    Timed t(ctx, kClsFinal);
    const size_t total = (size_t)B * ctx->N;
    const double f2 = (double)ctx->factor * (double)ctx->factor;
    hipLaunchKernelGGL(k_finalize, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, ctx->stream, ctx->d_key,
                       dev_dist, dev_ssd, dev_best, total, ctx->shift, is_int(ctx) ? 1u : 0u, f2, do_sqrt ? 1u : 0u);
    return launch_check(ctx, "k_finalize");
}

int free_all(pink_hip_ctx *ctx)
{
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    for (auto &p : ctx->events) { (void)hipEventDestroy(p.a); (void)hipEventDestroy(p.b); }
    for (auto e : ctx->event_pool) (void)hipEventDestroy(e);
    void *bufs[] = {ctx->d_som, ctx->d_rot, ctx->d_cos, ctx->d_sin, ctx->d_factors, ctx->d_factors_t, ctx->d_region, ctx->d_key,
                    ctx->d_somP, ctx->d_somP_alt, ctx->d_bmu_group, ctx->d_rotT, ctx->d_bmu_scratch, ctx->d_dist, ctx->d_ssd, ctx->d_best,
                    ctx->d_Pa, ctx->d_Pb, ctx->d_na, ctx->d_nb, ctx->d_poff, ctx->d_need, ctx->d_inv,
                    ctx->d_upos, ctx->d_aoff, ctx->d_kmask, ctx->d_gPa, ctx->d_gPa_alt, ctx->d_som_alt, ctx->d_slots, ctx->d_resident_error, ctx->d_src4, ctx->d_kbyte, ctx->d_gPb, ctx->d_gna, ctx->d_gnb, ctx->d_rtab, ctx->d_symoff, ctx->d_grow, ctx->d_gvariant, ctx->d_region4};
    for (void *p : bufs) if (p) (void)hipFree(p);
    for (void *p : {(void *)ctx->st_img, (void *)ctx->st_heat, (void *)ctx->st_best, (void *)ctx->st_bmu}) if (p) (void)hipFree(p);
    if (ctx->st_pin) (void)hipHostFree(ctx->st_pin);
    if (ctx->h_resident_error) (void)hipHostFree(ctx->h_resident_error);
    for (int i = 0; i < 2; ++i) {
        if (ctx->pend_pin[i]) (void)hipHostFree(ctx->pend_pin[i]);
        if (ctx->pend_ev[i]) (void)hipEventDestroy(ctx->pend_ev[i]);
    }
    for (hipEvent_t e : ctx->st_ev) if (e) (void)hipEventDestroy(e);
    for (hipEvent_t e : ctx->copy_ev) if (e) (void)hipEventDestroy(e);
    ctx->copy_pool.reset();
    for (int i = 0; i < 2; ++i) {
        if (ctx->bounce[i]) (void)hipHostFree(ctx->bounce[i]);
        if (ctx->bounce_ev[i]) (void)hipEventDestroy(ctx->bounce_ev[i]);
        ctx->bounce[i] = nullptr; ctx->bounce_ev[i] = nullptr;
    }
    if (ctx->copy_stream) (void)hipStreamDestroy(ctx->copy_stream);
    if (ctx->d_counts) (void)hipFree(ctx->d_counts);
    for (void *p : {(void *)ctx->d_fPa, (void *)ctx->d_fPb, (void *)ctx->d_fna, (void *)ctx->d_fnb, (void *)ctx->d_fpart})
        if (p) (void)hipFree(p);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    return PINK_HIP_OK;
}

// The address of the file-scope scratch array on the current device, asked for once per device.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
unsigned char *g_scratch_ptr[kMaxDevices] = {};

int resolve_static_scratch(pink_hip_ctx *ctx)
{
    if (ctx->device < 0 || ctx->device >= kMaxDevices) return fail(ctx, PINK_HIP_EINVAL, "device ordinal out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[ctx->device]) {
        void *p = nullptr;
        HIP_TRY(ctx, hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        g_scratch_ptr[ctx->device] = (unsigned char *)p;
    }
    ctx->static_scratch = g_scratch_ptr[ctx->device];
    return PINK_HIP_OK;
}

int init_ctx(pink_hip_ctx *ctx)
{
    const pink_hip_config &c = ctx->cfg;
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    TRY(resolve_static_scratch(ctx));
    HIP_TRY(ctx, hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking));

    // Rotation tables: cos/sin of i * 2pi/num_rot in float, as the CPU evaluates them
    // (SelfOrganizingMapLib/generate_rotated_images.h:69,94; ImageProcessingLib/rotate.h:20-21).
    std::vector<float> cs(std::max(ctx->nrr, 1u), 1.0f), sn(std::max(ctx->nrr, 1u), 0.0f);
    const float angle_step = static_cast<float>(2 * M_PI) / c.num_rot;
    for (uint32_t i = 1; i < ctx->nrr; ++i) {
        const float alpha = i * angle_step;
        cs[i] = std::cos(alpha);
        sn[i] = std::sin(alpha);
    }
    TRY(dev_alloc(ctx, &ctx->d_cos, cs.size()));
    TRY(dev_alloc(ctx, &ctx->d_sin, sn.size()));
    HIP_TRY(ctx, hipMemcpy(ctx->d_cos, cs.data(), cs.size() * sizeof(float), hipMemcpyHostToDevice));
    HIP_TRY(ctx, hipMemcpy(ctx->d_sin, sn.data(), sn.size() * sizeof(float), hipMemcpyHostToDevice));

    const std::vector<uint32_t> region = build_region(ctx->C, ctx->D, c.ed_dim, c.ed_shape);
    ctx->E = (uint32_t)region.size();
    if (ctx->E == 0) return fail(ctx, PINK_HIP_EINVAL, "Euclidean distance region is empty");
    ctx->Epad = round_up(ctx->E, kEpadMultiple);
    ctx->Rpad = round_up(ctx->R, kWave);
    if (is_int(ctx)) {
        // key = ssd << 16 | rotation: the sum must stay below 2^48 and R below 2^16.
        const double max_ssd = (double)ctx->factor * ctx->factor * ctx->E;
        if (ctx->R > 65536 || max_ssd >= 281474976710656.0)
            return fail(ctx, PINK_HIP_EINVAL, "distance region or rotation count too large for the integer distance modes");
        ctx->wide_sums = max_ssd >= 2147483648.0;          // uint8 beyond 33 025 elements: 64-bit sums like uint16
    }
    TRY(dev_alloc(ctx, &ctx->d_region, region.size()));
    HIP_TRY(ctx, hipMemcpy(ctx->d_region, region.data(), region.size() * sizeof(uint32_t), hipMemcpyHostToDevice));

    // uint8 mapping on the matrix cores: SOMs of up to 128 neurons whose packed operand fits in LDS.
    {
        hipDeviceProp_t prop;
        HIP_TRY(ctx, hipGetDeviceProperties(&prop, ctx->device));
        ctx->num_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        const size_t lds_max = std::min<size_t>(prop.sharedMemPerBlock, 160 * 1024) - 1024;
        ctx->lds_max = lds_max;
        ctx->nrr_eff = std::max(ctx->nrr, 1u);
        ctx->KS = ctx->Epad / 32;
        ctx->NT = (ctx->N + 31) / 32;
        ctx->RT = (ctx->nrr_eff + 3) / 4;
        ctx->lds_dist = (size_t)ctx->NT * ctx->KS * 1024 + (size_t)8 * ctx->NT * 32 * 8;
        ctx->lds_rotpack = (((size_t)4 * (ctx->S + 1) + 15) & ~(size_t)15) + 32 * sizeof(int);
        const bool fits = c.ed_type == PINK_HIP_UINT8 && !ctx->trainer && ctx->N <= 128 && ctx->S + 1 <= 65535 &&
                          ctx->lds_dist <= lds_max && ctx->lds_rotpack <= lds_max;
        if (c.kernel_choice == PINK_HIP_KERNEL_MFMA && !fits)
            return fail(ctx, PINK_HIP_EINVAL, "the MFMA distance kernel needs a uint8 mapper with at most 128 neurons "
                                              "whose packed SOM fits in LDS");
        ctx->mfma = fits && (c.kernel_choice == PINK_HIP_KERNEL_AUTO || c.kernel_choice == PINK_HIP_KERNEL_MFMA);
    }
    // Symmetries on the SOM side: needs the union of the symmetric images of the region to fit 64
    // k-steps held in registers and at most 256 base rotations per image (8 row tiles).
    {
        const uint32_t D = ctx->D, DD = D * D;
        std::vector<std::vector<uint32_t>> pos(8);      // pos[sym][e] = perm_sym(region[e])
        std::vector<char> in_union(ctx->S, 0);
        std::vector<bool> sym_valid(8);
        for (uint32_t sym = 0; sym < 8; ++sym) {
            const uint32_t f = sym >> 2, q = sym & 3;
            sym_valid[sym] = (c.num_rot != 1 || q == 0) && (c.use_flip || f == 0);
            pos[sym].resize(ctx->E);
            for (uint32_t e = 0; e < ctx->E; ++e) {
                const uint32_t ch = region[e] / DD, x = (region[e] % DD) / D, y = region[e] % D;
                const uint32_t xs = f ? D - 1 - x : x;
                uint32_t a, bb;
                switch (q) {
                case 0: a = xs; bb = y; break;
                case 1: a = D - 1 - y; bb = xs; break;
                case 2: a = D - 1 - xs; bb = D - 1 - y; break;
                default: a = y; bb = D - 1 - xs; break;
                }
                pos[sym][e] = ch * DD + a * D + bb;
                if (sym_valid[sym]) in_union[pos[sym][e]] = 1;
            }
        }
        std::vector<uint32_t> upos;
        std::vector<uint32_t> index_of(ctx->S, 0xffffffffu);
        for (uint32_t p = 0; p < ctx->S; ++p)     // packed as channel << 24 | x << 12 | y
            if (in_union[p]) {
                index_of[p] = (uint32_t)upos.size();
                upos.push_back(((p / DD) << 24) | (((p % DD) / D) << 12) | (p % D));
            }
        ctx->Ku = (uint32_t)upos.size();
        const uint32_t ks_need = (ctx->Ku + 31) / 32;
        ctx->KSs = (ks_need + 7) / 8 * 8;                  // 8 .. 32: two column tiles per wave; 40 .. 64: one
        ctx->sym_tiles = ctx->KSs <= 32 ? 8 : 4;           // column tiles per block (4 waves)
        ctx->RTP = (ctx->nrr_eff + 31) / 32;
        const uint32_t col_tiles = (8 * ctx->N + 31) / 32;
        ctx->slices = (col_tiles + ctx->sym_tiles - 1) / ctx->sym_tiles;
        ctx->groups = std::max(1u, (uint32_t)ctx->num_cu / ctx->slices);
        // a region element must not repeat (the multi-channel circular rule repeats channel 0)
        bool distinct = true;
        {
            std::vector<char> seen(ctx->S, 0);
            for (uint32_t e = 0; e < ctx->E; ++e) { if (seen[region[e]]) distinct = false; seen[region[e]] = 1; }
        }
        const size_t lds_img = pink_sym::lds_image_bytes(ctx->C, ctx->I);
        const bool fits_sym = c.ed_type == PINK_HIP_UINT8 && !ctx->trainer && distinct && ks_need <= 64 && ctx->RTP <= 8 &&
                              lds_img <= 150 * 1024 && D < 4096 && ctx->C < 256;
        if (c.kernel_choice == PINK_HIP_KERNEL_MFMA_SYM && !fits_sym)
            return fail(ctx, PINK_HIP_EINVAL, "the symmetric MFMA distance kernel needs a uint8 mapper, at most 2048 "
                                              "region elements (union over the symmetries) and at most 1024 rotations");
        ctx->mfma_sym = fits_sym && (c.kernel_choice == PINK_HIP_KERNEL_AUTO || c.kernel_choice == PINK_HIP_KERNEL_MFMA_SYM);
        if (ctx->mfma_sym) {
            ctx->mfma = false;
            const uint32_t Kp = ctx->KSs * 32;
            std::vector<uint32_t> aoff((size_t)8 * Kp, 0xffffffffu);
            std::vector<unsigned char> kmask(Kp, 0);
            for (uint32_t sym = 0; sym < 8; ++sym) {
                if (!sym_valid[sym]) continue;
                for (uint32_t e = 0; e < ctx->E; ++e) {
                    const uint32_t k = index_of[pos[sym][e]];
                    aoff[(size_t)sym * Kp + k] = region[e];
                    kmask[k] |= (unsigned char)(1u << sym);
                }
            }
            // all valid symmetries cover the whole union: one norm per base rotation serves them all
            unsigned char valid_bits = 0;
            for (uint32_t sym = 0; sym < 8; ++sym) if (sym_valid[sym]) valid_bits |= (unsigned char)(1u << sym);
            ctx->all_sym = 1;
            for (uint32_t k = 0; k < ctx->Ku; ++k) if ((kmask[k] & valid_bits) != valid_bits) ctx->all_sym = 0;
            upos.resize(Kp, 0u);                       // padded: the kernel reads whole 16-entry pieces
            TRY(dev_alloc(ctx, &ctx->d_upos, upos.size()));
            TRY(dev_alloc(ctx, &ctx->d_aoff, aoff.size()));
            TRY(dev_alloc(ctx, &ctx->d_kmask, kmask.size()));
            HIP_TRY(ctx, hipMemcpy(ctx->d_upos, upos.data(), upos.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
            HIP_TRY(ctx, hipMemcpy(ctx->d_aoff, aoff.data(), aoff.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
            HIP_TRY(ctx, hipMemcpy(ctx->d_kmask, kmask.data(), kmask.size(), hipMemcpyHostToDevice));
            HIP_TRY(ctx, pink_sym::configure(ctx->KSs, ctx->C, ctx->I));
            HIP_TRY(ctx, hipMalloc(&ctx->d_rtab, pink_sym::rot_table_bytes(ctx->KSs, ctx->RTP)));
            HIP_TRY(ctx, pink_sym::build_rot_table(ctx->stream, ctx->d_cos, ctx->d_sin, ctx->d_upos, ctx->Ku, ctx->I, ctx->D,
                                                   ctx->nrr_eff, ctx->KSs, ctx->RTP, ctx->d_rtab));
            HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
        }
    }
    if (ctx->mfma) {
        // poff[sym][e]: where region element e of symmetry sym = flip*4 + quarter sits in the base rotation.
        const uint32_t D = ctx->D, DD = D * D, Kp = ctx->KS * 32;
        std::vector<unsigned short> poff((size_t)8 * Kp, (unsigned short)ctx->S);
        std::vector<char> used(ctx->S, 0);
        for (uint32_t sym = 0; sym < 8; ++sym) {
            const uint32_t f = sym >> 2, q = sym & 3;
            const bool sym_valid = (c.num_rot != 1 || q == 0) && (c.use_flip || f == 0);
            for (uint32_t e = 0; e < ctx->E; ++e) {
                const uint32_t ch = region[e] / DD, x = (region[e] % DD) / D, y = region[e] % D;
                const uint32_t xs = f ? D - 1 - x : x;
                uint32_t a, bb;
                switch (q) {
                case 0: a = xs; bb = y; break;
                case 1: a = D - 1 - y; bb = xs; break;
                case 2: a = D - 1 - xs; bb = D - 1 - y; break;
                default: a = y; bb = D - 1 - xs; break;
                }
                const uint32_t p = ch * DD + a * D + bb;
                if (sym_valid) { poff[(size_t)sym * Kp + e] = (unsigned short)p; used[p] = 1; }
            }
        }
        std::vector<uint32_t> need;
        for (uint32_t p = 0; p < ctx->S; ++p) if (used[p]) need.push_back(p);
        ctx->n_need = (uint32_t)need.size();
        TRY(dev_alloc(ctx, &ctx->d_poff, poff.size()));
        TRY(dev_alloc(ctx, &ctx->d_need, need.size()));
        HIP_TRY(ctx, hipMemcpy(ctx->d_poff, poff.data(), poff.size() * sizeof(unsigned short), hipMemcpyHostToDevice));
        HIP_TRY(ctx, hipMemcpy(ctx->d_need, need.data(), need.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
        // (limits are per kernel, not per context: the most that any context may ask)
        HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_rotpack_u8, hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)ctx->lds_max));
        const void *fn = ctx->NT == 1 ? (const void *)k_dist_mfma_u8<1> : ctx->NT == 2 ? (const void *)k_dist_mfma_u8<2>
                       : ctx->NT == 3 ? (const void *)k_dist_mfma_u8<3> : (const void *)k_dist_mfma_u8<4>;
        HIP_TRY(ctx, hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)ctx->lds_max));
    }

    // Integer distances as an int8 GEMM: all that is left of the integer modes.  Small
    // problems pad their rows to one 64 x 64 tile; they are latency bound either way and the four
    // waves of a block still cut k four ways.
    {
        // the byte planes of a row are staged in LDS when a row is packed by a kernel of its own (128 KB), and the
        // uint16 accumulator that takes two byte products per element stays exact in int32 for 65 535 elements
        const bool applies = is_int(ctx) && !ctx->mfma && !ctx->mfma_sym && ctx->Epad < 65536;
        if (c.kernel_choice == PINK_HIP_KERNEL_MFMA_GEMM && !applies)
            return fail(ctx, PINK_HIP_EINVAL, "the MFMA GEMM distance kernel needs an integer distance type");
        ctx->gemm = applies && (c.kernel_choice == PINK_HIP_KERNEL_MFMA_GEMM ||
                                c.kernel_choice == PINK_HIP_KERNEL_AUTO);
        if (ctx->gemm) {
            // (limits are per kernel, not per context)
            HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_pack_planes<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 65536));
            HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_pack_planes<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
            ctx->gKS = ctx->Epad / 32;
            ctx->Np = round_up(ctx->N, 64);
            ctx->Rp = round_up(ctx->R, 64);
            const uint32_t tiles = (ctx->Np / 64) * (ctx->Rp / 64);
            // A launch of one image takes 32 x 32 tiles where 64 x 64 tiles would leave a wave more than about 16
            // k-steps (uint8: 64 MFMAs) or 11 (uint16: 176) while at least half of the CUs stay without a block.
            const uint32_t per_wave = c.ed_type == PINK_HIP_UINT16 ? 11u : 16u;
            ctx->g_tile32 = ctx->gKS > 4 * per_wave && 2 * tiles <= (uint32_t)ctx->num_cu;
        }
    }

    // Float32 distances on the matrix cores: only on request.
    if (c.kernel_choice == PINK_HIP_KERNEL_MFMA_F32) {
        if (is_int(ctx)) return fail(ctx, PINK_HIP_EINVAL, "the float32 matrix-core distance kernel needs the float distance type");
        ctx->f32gemm = true;
        HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_dist_gemm_f32, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
        ctx->fKS = ctx->Epad / 8;
        ctx->Np = round_up(ctx->N, 64);
        ctx->Rp = round_up(ctx->R, 64);
        const uint32_t tiles = (ctx->Np / 64) * (ctx->Rp / 64);
        // k is cut into slices (blocks per tile) to fill the chip about twice, a wave keeping at least four k-steps
        uint32_t slices = std::max(1u, 2u * (uint32_t)ctx->num_cu / tiles);
        slices = std::max(1u, std::min(slices, ctx->fKS / 16));
        ctx->fks_per = (ctx->fKS + 4 * slices - 1) / (4 * slices);
        ctx->fslices = (ctx->fKS + 4 * ctx->fks_per - 1) / (4 * ctx->fks_per);
    }

    ctx->Dp = ctx->D | 1u;     // odd (measured at D = 96: 20 % faster than a stride of 96; nothing to gain at 44, 70, 106)
    // the base rotation of a block lives in LDS: up to 158 of the CU's 160 KB (neurons up to 199 pixels wide)
    ctx->use_lds = (size_t)ctx->D * ctx->Dp * sizeof(float) <= kRotateLdsMax;
    // all channels of a base rotation in one block when their tiles fit together: multi-channel byte planes
    // can then be packed by the rotation kernel (an operand piece may span two channels)
    ctx->rot_nch = (ctx->use_lds && ctx->gemm && ctx->C > 1 && (size_t)ctx->C * ctx->D * ctx->Dp * sizeof(float) <= kRotateLdsMax)
                       ? ctx->C : 1u;
    ctx->image_lds = !ctx->use_lds && (size_t)ctx->I * ctx->I * sizeof(float) <= kRotateLdsMax;
    {
        const int lds = (int)kRotateLdsMax;          // per kernel, not per context: the most any context may ask
        HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_rotate<0, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_rotate<0, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_rotate<1, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_rotate<1, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_rotate<2, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_rotate<2, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_rotate<3, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_rotate<3, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    }
    // Operand packing inside the rotation kernel: float32 rows, or byte planes of single-channel
    // integer contexts, whenever the kernel keeps its base rotation in LDS.
    ctx->fused_pack = !ctx->mfma && !ctx->mfma_sym && ctx->C < 256 && (size_t)ctx->D * ctx->Dp < ((size_t)1 << 24) &&
                      (ctx->gemm ? (ctx->C == 1 || ctx->rot_nch == ctx->C) : !is_int(ctx));
    // Neither the base rotation nor the image fits LDS: interpolating every packed element out of global
    // memory is slow, so the rotation kernel stores two symmetries and packing kernels of their own read
    // all eight out of those, with coalesced accesses
    ctx->pair_pack = !ctx->use_lds && !ctx->image_lds && !ctx->mfma && !ctx->mfma_sym && ctx->S < (1u << 24);
    if (ctx->pair_pack) {
        ctx->fused_pack = false;
        const uint32_t D = ctx->D, DD = D * D;
        std::vector<uint32_t> region4((size_t)4 * ctx->E);
        for (uint32_t combo = 0; combo < 4; ++combo)
            for (uint32_t k = 0; k < ctx->E; ++k) {
                const uint32_t ch = region[k] / DD, x = (region[k] % DD) / D, y = region[k] % D;
                region4[(size_t)combo * ctx->E + k] = ch * DD + ((combo >> 1) ? D - 1 - x : x) * D + ((combo & 1) ? D - 1 - y : y);
            }
        TRY(dev_alloc(ctx, &ctx->d_region4, region4.size()));
        HIP_TRY(ctx, hipMemcpy(ctx->d_region4, region4.data(), region4.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
    }
    // Float variants of a whole launch group: for the update kernel and for a separate packing kernel.
    // The other contexts keep room for one image (pink_hip_rotate).
    ctx->pair_variants = ctx->trainer && (ctx->fused_pack || ctx->pair_pack) && ctx->S < (1u << 24);   // (the update kernel's divisions)
    const bool group_variants = ctx->trainer || !(ctx->mfma || ctx->mfma_sym || ctx->fused_pack);

    // Launch-group size: one image for a trainer; for a mapper as many as fit ~4 GiB.
    size_t per_image = ((size_t)ctx->R * ctx->S + (size_t)ctx->Epad * ctx->Rpad) * 4 + (size_t)ctx->N * 24;
    if (ctx->mfma) per_image = (size_t)ctx->RT * ctx->KS * 1024 + (size_t)ctx->RT * 128 + (size_t)ctx->N * 24;
    if (ctx->gemm)
        per_image = (size_t)ctx->R * ctx->S * 4 + (size_t)(c.ed_type == PINK_HIP_UINT16 ? 2 : 1) * (ctx->Rp / 32) * ctx->gKS * 1024 +
                    (size_t)ctx->Rp * 8 + (size_t)ctx->N * 24;
    if (ctx->mfma_sym) per_image = (size_t)ctx->RTP * pink_sym::unit_bytes(ctx->KSs) + (size_t)ctx->N * 24;
    else if (!ctx->mfma && !group_variants) per_image -= (size_t)ctx->R * ctx->S * 4;
    if (ctx->trainer) {
        // images whose variants are prepared ahead of the sequential distance/update chain
        size_t b = c.max_batch ? c.max_batch : 64;
        // small uint8 trainers (see k_train_small_u8_resident: one launch per group, the host waits for each): 256
        if (!c.max_batch && ctx->gemm && ctx->pair_variants && c.kernel_choice == PINK_HIP_KERNEL_AUTO && c.ed_type == PINK_HIP_UINT8 &&
            ctx->N <= 64 && ctx->R <= 32 && ctx->S <= 2048 && ctx->gKS <= 64)
            b = 256;
        const size_t budget = (size_t)2 << 30;
        while (b > 1 && b * per_image > budget) b >>= 1;
        if (!c.max_batch) {
            // a group's variants and operands are written by one launch and read back image by image: a group that
            // stays within the 256 MB last-level cache trains faster (measured: 10 x 10 float32 +2.6 % with 48
            // against 64 images, the hexagonal uint16 SOM +5 % with 16 against 32; groups below 16 cost the
            // rotation kernel more than they save)
            const size_t stored = ctx->pair_variants ? std::min<size_t>(2 * std::max(ctx->nrr, 1u), ctx->R) : ctx->R;
            const size_t touched = per_image - (ctx->R - stored) * ctx->S * 4;
            while (b > 16 && b * touched > ((size_t)224 << 20)) b -= std::min<size_t>(8, b - 16);
            // the integer GEMM trainers read a group's data with both of their per-image kernels and gain more from
            // the cache than the rotation kernel loses on smaller launches (hexagonal uint16 SOM: 30.6 us per image
            // with 16 images, 230 MB; 29.1-29.3 with 11 to 13; 29.7 with 8 to 10; 30.7 with 6)
            if (ctx->gemm) while (b > 8 && b * touched > ((size_t)192 << 20)) --b;
        }
        ctx->Bcap = (uint32_t)b;
    } else {
        size_t b = c.max_batch ? c.max_batch : ((ctx->mfma || ctx->mfma_sym) ? 2048 : 256);
        const size_t budget = (size_t)4 << 30;
        while (b > 1 && b * per_image > budget) b >>= 1;
        if (ctx->gemm && !c.max_batch) {
            // the GEMM reads a group's variant operand right after the rotation kernel wrote it: a group whose
            // operand stays within the 256 MB last-level cache maps faster than a larger one (measured: the
            // optimum is the largest power of two with at most ~190 MB, 128 images at 2048 uint8 elements)
            const size_t operand = (size_t)(c.ed_type == PINK_HIP_UINT16 ? 2 : 1) * (ctx->Rp / 32) * ctx->gKS * 1024;
            while (b > 16 && b * operand > ((size_t)192 << 20)) b >>= 1;
        }
        ctx->Bcap = (uint32_t)b;
    }
    const size_t B = ctx->Bcap;

    TRY(dev_alloc(ctx, &ctx->d_som, (size_t)ctx->N * ctx->S));
    HIP_TRY(ctx, hipMemset(ctx->d_som, 0, (size_t)ctx->N * ctx->S * sizeof(float)));
    TRY(dev_alloc(ctx, &ctx->d_rot, (group_variants ? B : 1) * ctx->R * ctx->S));
    TRY(dev_alloc(ctx, &ctx->d_key, B * ctx->N));
    if (ctx->mfma_sym) {
        TRY(dev_alloc(ctx, &ctx->d_Pa, (size_t)ctx->slices * ctx->sym_tiles * ctx->KSs * 1024));
        TRY(dev_alloc(ctx, &ctx->d_na, (size_t)ctx->slices * ctx->sym_tiles * 32));
        TRY(dev_alloc(ctx, &ctx->d_Pb, B * ctx->RTP * pink_sym::unit_bytes(ctx->KSs)));
    } else if (ctx->gemm) {
        const size_t planes = c.ed_type == PINK_HIP_UINT16 ? 2 : 1;
        const size_t a_vec = planes * (ctx->Np / 32) * ctx->gKS * 64, b_vec = planes * (ctx->Rp / 32) * ctx->gKS * 64;
        TRY(dev_alloc(ctx, &ctx->d_gPa, a_vec));
        TRY(dev_alloc(ctx, &ctx->d_gPb, B * b_vec));
        TRY(dev_alloc(ctx, &ctx->d_gna, (size_t)2 * ctx->Np));   // two halves, see na_cur
        TRY(dev_alloc(ctx, &ctx->d_gnb, B * ctx->Rp));
        {
            // rows of the variant operand: base rotation first, symmetry second
            const uint32_t nq = c.num_rot == 1 ? 1u : 4u, nf = c.use_flip ? 2u : 1u, nsym = nq * nf;
            const uint32_t nrr = std::max(c.num_rot / 4, 1u);
            std::vector<uint32_t> row_of(ctx->R), variant_of(ctx->Rp, 0u);
            for (uint32_t f = 0; f < nf; ++f)
                for (uint32_t q = 0; q < nq; ++q)
                    for (uint32_t i = 0; i < nrr; ++i) {
                        const uint32_t k = f * c.num_rot + q * nrr + i, r = i * nsym + f * nq + q;
                        row_of[k] = r;
                        variant_of[r] = k;
                    }
            TRY(dev_alloc(ctx, &ctx->d_grow, row_of.size()));
            TRY(dev_alloc(ctx, &ctx->d_gvariant, variant_of.size()));
            HIP_TRY(ctx, hipMemcpy(ctx->d_grow, row_of.data(), row_of.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
            HIP_TRY(ctx, hipMemcpy(ctx->d_gvariant, variant_of.data(), variant_of.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
        }
        // rows beyond N / R and elements beyond the region are never written: they must read as zero
        HIP_TRY(ctx, hipMemset(ctx->d_gPa, 0, a_vec * sizeof(v4i)));
        HIP_TRY(ctx, hipMemset(ctx->d_gPb, 0, B * b_vec * sizeof(v4i)));
    } else if (ctx->mfma) {
        TRY(dev_alloc(ctx, &ctx->d_Pa, (size_t)ctx->NT * ctx->KS * 1024));
        TRY(dev_alloc(ctx, &ctx->d_na, (size_t)ctx->NT * 32));
        TRY(dev_alloc(ctx, &ctx->d_Pb, B * ctx->RT * ctx->KS * 1024));
        TRY(dev_alloc(ctx, &ctx->d_nb, B * ctx->RT * 32));
    } else {
        // (the float distance kernel of small problems reads up to kDistOverrun floats past a row's end)
        TRY(dev_alloc(ctx, (uint32_t **)&ctx->d_somP, (size_t)ctx->N * ctx->Epad + kDistOverrun));
        TRY(dev_alloc(ctx, (uint32_t **)&ctx->d_rotT, B * ctx->Epad * ctx->Rpad + kDistOverrun));
        // rows beyond R and elements beyond the region must read as zero whoever fills the rest
        HIP_TRY(ctx, hipMemset(ctx->d_rotT, 0, B * ctx->Epad * ctx->Rpad * sizeof(uint32_t)));
        if (ctx->f32gemm) {
            TRY(dev_alloc(ctx, &ctx->d_fPa, (size_t)(ctx->Np / 32) * ctx->fKS * 64));
            TRY(dev_alloc(ctx, &ctx->d_fPb, B * (ctx->Rp / 32) * ctx->fKS * 64));
            TRY(dev_alloc(ctx, &ctx->d_fna, (size_t)ctx->Np));
            TRY(dev_alloc(ctx, &ctx->d_fnb, B * ctx->Rp));
            TRY(dev_alloc(ctx, &ctx->d_fpart, (size_t)ctx->fslices * ctx->Rp * ctx->Np));
        }
    }
    if (ctx->fused_pack) {
        const uint32_t D = ctx->D, DD = D * D;
        std::vector<uint32_t> symoff((size_t)8 * ctx->Epad, 0u);
        ctx->base_lo = D; ctx->base_hi = 0;
        for (uint32_t sym = 0; sym < 8; ++sym) {
            const uint32_t f = sym >> 2, q = sym & 3;
            for (uint32_t e = 0; e < ctx->E; ++e) {
                // variant pixel (x, y) of symmetry (f, q) is base-rotation pixel (a, bb): the flip
                // reverses the rows of the quarter turn (see k_rotate)
                const uint32_t ch = region[e] / DD, x = (region[e] % DD) / D, y = region[e] % D;
                const uint32_t xs = f ? D - 1 - x : x;
                uint32_t a, bb;
                switch (q) {
                case 0: a = xs; bb = y; break;
                case 1: a = D - 1 - y; bb = xs; break;
                case 2: a = D - 1 - xs; bb = D - 1 - y; break;
                default: a = y; bb = D - 1 - xs; break;
                }
                // float rows: channel and position in the channel's tile (LDS rows of Dp floats); byte planes:
                // position in the block's tiles, the channels' side by side
                symoff[(size_t)sym * ctx->Epad + e] = ctx->gemm ? ch * D * ctx->Dp + a * ctx->Dp + bb : (ch << 24) | (a * ctx->Dp + bb);
                ctx->base_lo = std::min({ctx->base_lo, a, bb});
                ctx->base_hi = std::max({ctx->base_hi, a + 1, bb + 1});
            }
        }
        if (ctx->base_hi <= ctx->base_lo) ctx->base_lo = ctx->base_hi = 0;       // empty region
        TRY(dev_alloc(ctx, &ctx->d_symoff, symoff.size()));
        if (ctx->gemm && ctx->use_lds) {        // (an LDS tile set has at most 40 448 floats)
            // byte-plane packing out of an LDS tile reads 16-bit entries (single channel, positions below 40 000)
            std::vector<unsigned short> narrow(symoff.begin(), symoff.end());
            HIP_TRY(ctx, hipMemcpy(ctx->d_symoff, narrow.data(), narrow.size() * sizeof(unsigned short), hipMemcpyHostToDevice));
        } else {
            HIP_TRY(ctx, hipMemcpy(ctx->d_symoff, symoff.data(), symoff.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
        }
    }
    TRY(dev_alloc(ctx, &ctx->d_bmu_scratch, 1));
    TRY(dev_alloc(ctx, &ctx->d_counts, ctx->N));
    HIP_TRY(ctx, hipMemset(ctx->d_counts, 0, (size_t)ctx->N * sizeof(uint32_t)));
    TRY(dev_alloc(ctx, &ctx->d_dist, B * ctx->N));
    TRY(dev_alloc(ctx, &ctx->d_ssd, B * ctx->N));
    TRY(dev_alloc(ctx, &ctx->d_best, B * ctx->N));
    if (ctx->trainer) {
        // element -> region position, when every region element is a distinct neuron element
        std::vector<uint32_t> inv(ctx->S, 0xffffffffu);
        bool one_to_one = true;
        for (uint32_t k = 0; k < ctx->E; ++k) {
            if (inv[region[k]] != 0xffffffffu) one_to_one = false;
            inv[region[k]] = k;
        }
        if (one_to_one) {
            TRY(dev_alloc(ctx, &ctx->d_inv, inv.size()));
            HIP_TRY(ctx, hipMemcpy(ctx->d_inv, inv.data(), inv.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
            ctx->fused_som = ctx->gemm;
        }
        if (ctx->fused_som) {
            // where an element of a neuron lands inside the neuron's row of 32-row fragments of the SOM operand
            // (see k_train_small_u8), or all ones outside the region
            std::vector<uint32_t> kbyte(ctx->S);
            for (uint32_t j = 0; j < ctx->S; ++j) {
                const uint32_t k = inv[j];
                kbyte[j] = k == 0xffffffffu ? k : (k >> 5) * 1024 + ((k >> 4) & 1) * 512 + (k & 15);
            }
            TRY(dev_alloc(ctx, &ctx->d_kbyte, kbyte.size()));
            HIP_TRY(ctx, hipMemcpy(ctx->d_kbyte, kbyte.data(), kbyte.size() * sizeof(uint32_t), hipMemcpyHostToDevice));
        }
        // one launch per image where the whole distance matrix is a few dozen MFMAs (see k_train_small_u8)
        const uint32_t nstored = std::min(2 * std::max(ctx->nrr, 1u), ctx->R);
        ctx->small_train = ctx->fused_som && ctx->pair_variants && c.kernel_choice == PINK_HIP_KERNEL_AUTO &&
                           c.ed_type == PINK_HIP_UINT8 && ctx->N <= 64 && ctx->R <= 32 && ctx->S <= 2048 && ctx->gKS <= 64 &&
                           (size_t)nstored * ctx->S * sizeof(float) <= 32768;
        if (ctx->small_train) {
            const size_t a_vec = (size_t)(ctx->Np / 32) * ctx->gKS * 64;
            TRY(dev_alloc(ctx, &ctx->d_gPa_alt, a_vec));
            HIP_TRY(ctx, hipMemset(ctx->d_gPa_alt, 0, a_vec * sizeof(v4i)));
            std::vector<unsigned long long> src4(ctx->S);
            const uint32_t D = ctx->D;
            for (uint32_t j = 0; j < ctx->S; ++j) {
                const uint32_t p = j % (D * D), qx = p / D, qy = p % D;
                unsigned long long packed = 0;
                for (uint32_t combo = 0; combo < 4; ++combo) {
                    const uint32_t src = j - p + ((combo >> 1) ? D - 1 - qx : qx) * D + ((combo & 1) ? D - 1 - qy : qy);
                    packed |= (unsigned long long)src << (16 * combo);
                }
                src4[j] = packed;
            }
            TRY(dev_alloc(ctx, &ctx->d_src4, src4.size()));
            HIP_TRY(ctx, hipMemcpy(ctx->d_src4, src4.data(), src4.size() * sizeof(unsigned long long), hipMemcpyHostToDevice));
            // (limits are per kernel, not per context)
            HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_train_small_u8<4, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, 32768));
            HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_train_small_u8<8, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, 32768));
            // resident over a launch group: every block needs a compute unit of its own for the whole launch
            ctx->resident_train = ctx->N <= (uint32_t)ctx->num_cu;
            if (const char *off = getenv("PINK_HIP_RESIDENT_TRAINER")) ctx->resident_train = ctx->resident_train && atoi(off) != 0;
            if (ctx->resident_train) {
                // (a test can make every wait give up at once, to see the group trained again image by image)
                if (const char *limit = getenv("PINK_HIP_RESIDENT_SPIN_LIMIT")) ctx->spin_limit = (uint32_t)strtoul(limit, nullptr, 10);
                // (... or start the tags of the exchange just below the value where they wrap, which 2^32 images take)
                if (const char *tag = getenv("PINK_HIP_RESIDENT_FIRST_TAG")) ctx->exchange_tag = std::max(1u, (uint32_t)strtoul(tag, nullptr, 10));
                TRY(dev_alloc(ctx, &ctx->d_som_alt, (size_t)ctx->N * ctx->S));
                TRY(dev_alloc(ctx, &ctx->d_slots, (size_t)kSlotWords));
                HIP_TRY(ctx, hipMemset(ctx->d_slots, 0, kSlotWords * sizeof(unsigned long long)));
                TRY(dev_alloc(ctx, &ctx->d_resident_error, 1));
                HIP_TRY(ctx, hipMemset(ctx->d_resident_error, 0, sizeof(uint32_t)));
                if (hipHostMalloc((void **)&ctx->h_resident_error, sizeof(uint32_t), hipHostMallocDefault) != hipSuccess) {
                    ctx->h_resident_error = nullptr;
                    return fail(ctx, PINK_HIP_ENOMEM, "pinned host allocation failed");
                }
                HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_train_small_u8_resident<2, 4, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
                HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_train_small_u8_resident<2, 4, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
                HIP_TRY(ctx, hipFuncSetAttribute((const void *)k_train_small_u8_resident<4, 8, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
            }
        }
        // one launch per image where the float32 distance kernel runs in its one-wave-per-SIMD form (see k_train_f32_dpp;
        // up to 256 neurons: measured with 512 allowed, 17 x 17 and 18 x 18 neurons at 720 variants train no faster this
        // way than with an update launch of their own -- with three to four waves per SIMD the launch saved is paid in
        // instructions)
        ctx->fused_f32_train = c.ed_type == PINK_HIP_FLOAT && !ctx->f32gemm && ctx->d_somP && ctx->d_inv && ctx->N <= 256 &&
                               (size_t)(ctx->Rpad / kWave) * ((ctx->N + 3) / 4) <= (size_t)4 * ctx->num_cu;
        ctx->rows_f32_train = !ctx->fused_f32_train && c.ed_type == PINK_HIP_FLOAT && !ctx->f32gemm && ctx->d_somP && ctx->d_inv &&
                              B <= kReplayMax;
        if (ctx->fused_f32_train) TRY(dev_alloc(ctx, (uint32_t **)&ctx->d_somP_alt, (size_t)ctx->N * ctx->Epad + kDistOverrun));
        if (ctx->fused_f32_train || ctx->rows_f32_train || ctx->resident_train) TRY(dev_alloc(ctx, &ctx->d_bmu_group, B));
        TRY(dev_alloc(ctx, &ctx->d_factors, (size_t)ctx->N * ctx->N));
        HIP_TRY(ctx, hipMemcpy(ctx->d_factors, c.update_factors, (size_t)ctx->N * ctx->N * sizeof(float),
                               hipMemcpyHostToDevice));
        {
            // the same matrix transposed: what a neuron receives for every possible best match, contiguous
            std::vector<float> t((size_t)ctx->N * ctx->N);
            for (uint32_t m = 0; m < ctx->N; ++m)
                for (uint32_t k = 0; k < ctx->N; ++k) t[(size_t)k * ctx->N + m] = c.update_factors[(size_t)m * ctx->N + k];
            TRY(dev_alloc(ctx, &ctx->d_factors_t, t.size()));
            HIP_TRY(ctx, hipMemcpy(ctx->d_factors_t, t.data(), t.size() * sizeof(float), hipMemcpyHostToDevice));
        }
    }
    HIP_TRY(ctx, hipDeviceSynchronize());   // set-up copies ran on the null stream
    TRY(run_pack_som(ctx));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return PINK_HIP_OK;
}

// rotate -> pack -> distance for B images already on the device; keys left in d_key.
int run_rotpack_mfma(pink_hip_ctx *ctx, const float *dev_images, uint32_t B)
{
    Timed t(ctx, kClsRotate);
    hipLaunchKernelGGL(k_rotpack_u8, dim3(ctx->RT, B), dim3(256), ctx->lds_rotpack, ctx->stream, dev_images,
                       (v4i *)ctx->d_Pb, ctx->d_nb, ctx->d_cos, ctx->d_sin, ctx->d_poff, ctx->d_need, ctx->n_need,
                       ctx->C, ctx->I, ctx->D, ctx->S, ctx->cfg.num_rot, ctx->cfg.use_flip, ctx->nrr_eff, ctx->KS,
                       ctx->RT);
    return launch_check(ctx, "k_rotpack_u8");
}

int run_dist_mfma(pink_hip_ctx *ctx, uint32_t B)
{
    Timed t(ctx, kClsDist);
    const dim3 grid(std::min<uint32_t>(B, (uint32_t)ctx->num_cu));
#define LAUNCH_NT(T_)                                                                                              \
    hipLaunchKernelGGL((k_dist_mfma_u8<T_>), grid, dim3(512), ctx->lds_dist, ctx->stream, (const v4i *)ctx->d_Pa,   \
                       ctx->d_na, (const v4i *)ctx->d_Pb, ctx->d_nb, ctx->d_key, ctx->N, ctx->KS, ctx->RT, B,      \
                       ctx->cfg.num_rot, ctx->cfg.use_flip, ctx->nrr_eff)
    switch (ctx->NT) {
    case 1: LAUNCH_NT(1); break;
    case 2: LAUNCH_NT(2); break;
    case 3: LAUNCH_NT(3); break;
    default: LAUNCH_NT(4); break;
    }
#undef LAUNCH_NT
    return launch_check(ctx, "k_dist_mfma_u8");
}

int run_rotpack_sym(pink_hip_ctx *ctx, const float *dev_images, uint32_t B)
{
    Timed t(ctx, kClsRotate);
    pink_sym::RotpackArgs g{};
    const size_t entries = (size_t)ctx->RTP * 32 * ctx->KSs * 32;
    g.images = dev_images; g.Pb = ctx->d_Pb; g.tab_w = ctx->d_rtab;
    g.tab_idx = (const uint32_t *)((const char *)ctx->d_rtab + entries * 16);
    g.kmask = ctx->d_kmask; g.Ku = ctx->Ku; g.all_sym = ctx->all_sym; g.C = ctx->C; g.I = ctx->I; g.nrr_eff = ctx->nrr_eff;
    g.KS = ctx->KSs; g.RTP = ctx->RTP; g.B = B;
    HIP_TRY(ctx, pink_sym::rotpack(ctx->stream, g));
    return PINK_HIP_OK;
}

int run_dist_sym(pink_hip_ctx *ctx, uint32_t B)
{
    Timed t(ctx, kClsDist);
    pink_sym::DistArgs g{};
    g.Pa = ctx->d_Pa; g.na = ctx->d_na; g.Pb = ctx->d_Pb; g.key = ctx->d_key; g.N = ctx->N; g.B = B;
    g.num_rot = ctx->cfg.num_rot; g.use_flip = ctx->cfg.use_flip; g.RTP = ctx->RTP; g.KS = ctx->KSs;
    g.slices = ctx->slices; g.groups = std::min(ctx->groups, B);
    HIP_TRY(ctx, pink_sym::dist(ctx->stream, g));
    return PINK_HIP_OK;
}

int distance_group(pink_hip_ctx *ctx, const float *dev_images, uint32_t B)
{
    if (ctx->mfma_sym) {
        TRY(run_rotpack_sym(ctx, dev_images, B));
        TRY(run_dist_sym(ctx, B));
        return PINK_HIP_OK;
    }
    if (ctx->mfma) {
        TRY(run_rotpack_mfma(ctx, dev_images, B));
        TRY(run_dist_mfma(ctx, B));
        return PINK_HIP_OK;
    }
    // the variants themselves are only read by the update kernel and by a separate packing kernel
    TRY(run_rotate(ctx, dev_images, B, ctx->fused_pack ? kStoreNone : ctx->pair_pack ? kStorePair : kStoreAll));
    TRY(run_pack_rot(ctx, B));
    TRY(run_dist(ctx, 0, B));
    return PINK_HIP_OK;
}

}  // namespace

// ---------------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------------
extern "C" {

int pink_hip_abi_version(void) { return PINK_HIP_ABI_VERSION; }

const char *pink_hip_last_error(const pink_hip_ctx *ctx) { return ctx ? ctx->err.c_str() : g_create_error.c_str(); }

int pink_hip_check_config(const pink_hip_config *cfg)
{
    if (!cfg) return fail(nullptr, PINK_HIP_EINVAL, "pink_hip_check_config: null argument");
    // SelfOrganizingMapLib/Trainer.h:66-67, Mapper.h:59-62
    if (cfg->num_rot == 0 || (cfg->num_rot != 1 && cfg->num_rot % 4 != 0))
        return fail(nullptr, PINK_HIP_EINVAL, "Number of rotations must be 1 or larger then 1 and divisible by 4");
    // SelfOrganizingMapLib/Mapper.h:63-66
    if (cfg->ed_dim > cfg->neuron_dim)
        return fail(nullptr, PINK_HIP_EINVAL, "Euclidean distance dimension larger than neuron dimension");
    // CudaLib/generate_rotated_images.h:119-121 (only bilinear interpolation exists on the device)
    if (cfg->num_rot > 4 && cfg->interpolation != PINK_HIP_BILINEAR)
        return fail(nullptr, PINK_HIP_EINVAL, "generate_rotated_images: unknown interpolation type");
    if (cfg->som_size == 0 || cfg->channels == 0 || cfg->image_dim == 0 || cfg->neuron_dim == 0 || cfg->ed_dim == 0)
        return fail(nullptr, PINK_HIP_EINVAL, "pink_hip_create: zero-sized SOM, image, neuron or distance region");
    if (cfg->ed_type > PINK_HIP_UINT8 || cfg->ed_shape > PINK_HIP_CIRCULAR)
        return fail(nullptr, PINK_HIP_EINVAL, "pink_hip_create: unknown distance type or shape");
    if ((uint64_t)cfg->image_dim * cfg->image_dim >= (1ull << 31) ||
        (uint64_t)cfg->channels * cfg->neuron_dim * cfg->neuron_dim >= (1ull << 31))
        return fail(nullptr, PINK_HIP_EINVAL, "pink_hip_create: image or neuron too large");
    return PINK_HIP_OK;
}

int pink_hip_create(pink_hip_ctx **out, const pink_hip_config *cfg)
{
    if (!out || !cfg) return fail(nullptr, PINK_HIP_EINVAL, "pink_hip_create: null argument");
    *out = nullptr;
    TRY(pink_hip_check_config(cfg));

    pink_hip_ctx *ctx = new (std::nothrow) pink_hip_ctx();
    if (!ctx) return fail(nullptr, PINK_HIP_ENOMEM, "pink_hip_create: out of host memory");
    ctx->cfg = *cfg;
    ctx->N = cfg->som_size;
    ctx->C = cfg->channels;
    ctx->I = cfg->image_dim;
    ctx->D = cfg->neuron_dim;
    ctx->S = cfg->channels * cfg->neuron_dim * cfg->neuron_dim;
    ctx->isz = cfg->channels * cfg->image_dim * cfg->image_dim;
    ctx->R = cfg->num_rot * (cfg->use_flip ? 2u : 1u);
    ctx->nrr = cfg->num_rot / 4;
    ctx->trainer = cfg->update_factors != nullptr;
    ctx->device = cfg->device;
    ctx->factor = cfg->ed_type == PINK_HIP_UINT8 ? 255u : cfg->ed_type == PINK_HIP_UINT16 ? 65535u : 1u;
    ctx->shift = cfg->ed_type == PINK_HIP_FLOAT ? 32u : 16u;

    int rc = init_ctx(ctx);
    if (rc != PINK_HIP_OK) {
        g_create_error = ctx->err;
        free_all(ctx);
        delete ctx;
        return rc;
    }
    ctx->cfg.update_factors = nullptr;   // the host matrix is not kept
    *out = ctx;
    return PINK_HIP_OK;
}

void pink_hip_destroy(pink_hip_ctx *ctx)
{
    if (!ctx) return;
    free_all(ctx);
    delete ctx;
}

// Training calls without a result (the reference's Trainer::operator() returns nothing) only copy their
// image into a pinned buffer; the images go to the device, and through rotation, distance and update, a
// launch group at a time: when the group is full, or when any other call on the context needs the state
// they produce.  The order of the images and every result are those of training them call by call.
int ensure_staging(pink_hip_ctx *ctx, size_t n);
int flush_pending(pink_hip_ctx *ctx)
{
    if (!ctx || !ctx->pend_count) return PINK_HIP_OK;
    const uint32_t n = ctx->pend_count, cur = ctx->pend_cur;
    ctx->pend_count = 0;
    ctx->pend_cur ^= 1;
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    TRY(ensure_staging(ctx, std::max<size_t>(n, ctx->pend_cap)));
    HIP_TRY(ctx, hipMemcpyAsync(ctx->st_img, ctx->pend_pin[cur], (size_t)n * ctx->isz * sizeof(float), hipMemcpyHostToDevice,
                                ctx->stream));
    HIP_TRY(ctx, hipEventRecord(ctx->pend_ev[cur], ctx->stream));
    return pink_hip_train_device(ctx, ctx->st_img, n, ctx->st_bmu);
}

int pink_hip_synchronize(pink_hip_ctx *ctx)
{
    if (!ctx) return PINK_HIP_EINVAL;
    TRY(flush_pending(ctx));
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return PINK_HIP_OK;
}

int pink_hip_set_som(pink_hip_ctx *ctx, const float *host_som)
{
    if (!ctx || !host_som) return fail(ctx, PINK_HIP_EINVAL, "pink_hip_set_som: null argument");
    TRY(flush_pending(ctx));                              // images trained before this call see the SOM before it
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    HIP_TRY(ctx, hipMemcpyAsync(ctx->d_som, host_som, (size_t)ctx->N * ctx->S * sizeof(float), hipMemcpyHostToDevice,
                                ctx->stream));
    TRY(run_pack_som(ctx));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return PINK_HIP_OK;
}

int pink_hip_get_som(pink_hip_ctx *ctx, float *host_som)
{
    if (!ctx || !host_som) return fail(ctx, PINK_HIP_EINVAL, "pink_hip_get_som: null argument");
    TRY(flush_pending(ctx));
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    HIP_TRY(ctx, hipMemcpyAsync(host_som, ctx->d_som, (size_t)ctx->N * ctx->S * sizeof(float), hipMemcpyDeviceToHost,
                                ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return PINK_HIP_OK;
}

int pink_hip_update_counts(pink_hip_ctx *ctx, uint32_t *host_counts_out)
{
    if (!ctx || !host_counts_out) return fail(ctx, PINK_HIP_EINVAL, "pink_hip_update_counts: null argument");
    if (!ctx->trainer) return fail(ctx, PINK_HIP_ESTATE, "pink_hip_update_counts: context was created without update factors");
    TRY(flush_pending(ctx));
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    HIP_TRY(ctx, hipMemcpyAsync(host_counts_out, ctx->d_counts, (size_t)ctx->N * sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return PINK_HIP_OK;
}

int pink_hip_train_device(pink_hip_ctx *ctx, const float *dev_images, uint32_t n_images, uint32_t *dev_bmu_out)
{
    if (!ctx || (!dev_images && n_images)) return fail(ctx, PINK_HIP_EINVAL, "pink_hip_train_device: null argument");
    if (!ctx->trainer) return fail(ctx, PINK_HIP_ESTATE, "pink_hip_train: context was created without update factors");
    TRY(flush_pending(ctx));                              // (none while flush_pending itself calls this)
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    // The variants of an image and their packed distance operand do not depend on the SOM: they
    // are produced for a group of images per launch.  Distance and update stay strictly sequential.
    for (uint32_t done = 0; done < n_images; done += ctx->Bcap) {
        const uint32_t B = std::min(ctx->Bcap, n_images - done);
        TRY(run_rotate(ctx, dev_images + (size_t)done * ctx->isz, B, ctx->pair_variants ? kStorePair : kStoreAll));
        TRY(run_pack_rot(ctx, B));
        if (ctx->fused_f32_train) {
            // every launch but the first applies the update of the image before it; the last image's update and,
            // ahead of it, all the others on the neurons' full images close the group
            uint32_t *bmu = dev_bmu_out ? dev_bmu_out + done : ctx->d_bmu_group;
            {
                // (per-kernel timing: one pair of events around the group's launches, which follow each other directly)
                Timed t(ctx, kClsDist, B);
                for (uint32_t b = 0; b < B; ++b) TRY(run_train_f32(ctx, b, b > 0, b > 0 ? bmu + b - 1 : nullptr));
            }
            if (B > 1) TRY(run_update_replay(ctx, B - 1, bmu));
            TRY(run_update(ctx, B - 1, bmu + B - 1));
            continue;
        }
        if (ctx->rows_f32_train) {
            uint32_t *bmu = dev_bmu_out ? dev_bmu_out + done : ctx->d_bmu_group;
            for (uint32_t b = 0; b < B; ++b) {
                TRY(run_dist(ctx, b, 1));
                TRY(run_update_rows(ctx, b, bmu + b));
            }
            TRY(run_update_replay(ctx, B, bmu));
            continue;
        }
        if (ctx->resident_train) {
            bool went_through = false;
            TRY(run_train_small_resident(ctx, B, dev_bmu_out ? dev_bmu_out + done : ctx->d_bmu_group, &went_through));
            if (went_through) continue;
        }
        for (uint32_t b = 0; b < B; ++b) {
            if (ctx->small_train) {
                TRY(run_train_small(ctx, b, dev_bmu_out ? dev_bmu_out + done + b : ctx->d_bmu_scratch));
                continue;
            }
            TRY(run_dist(ctx, b, 1));
            TRY(run_update(ctx, b, dev_bmu_out ? dev_bmu_out + done + b : ctx->d_bmu_scratch));
            if (!ctx->d_inv || (ctx->gemm && !ctx->fused_som)) TRY(run_pack_som(ctx));
            else if (ctx->f32gemm) { Timed t(ctx, kClsPack); TRY(run_pack_frag_som(ctx)); }
        }
    }
    return PINK_HIP_OK;
}

constexpr size_t kPinBytes = (size_t)1 << 20;
constexpr uint32_t kPinSlots = 8;
constexpr size_t kSlotBytes = kPinBytes / kPinSlots;

// Staging for `n` images per chunk (grown on demand, freed with the context).
int ensure_staging(pink_hip_ctx *ctx, size_t n)
{
    if (!ctx->st_pin) {
        if (hipHostMalloc((void **)&ctx->st_pin, 2 * kPinBytes, hipHostMallocDefault) != hipSuccess) {
            ctx->st_pin = nullptr;
            return fail(ctx, PINK_HIP_ENOMEM, "pinned host allocation failed");
        }
        for (hipEvent_t &e : ctx->st_ev) HIP_TRY(ctx, hipEventCreateWithFlags(&e, hipEventDisableTiming));
    }
    if (n <= ctx->st_images) return PINK_HIP_OK;
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    for (void *p : {(void *)ctx->st_img, (void *)ctx->st_heat, (void *)ctx->st_best, (void *)ctx->st_bmu})
        if (p) (void)hipFree(p);
    ctx->st_img = ctx->st_heat = nullptr;
    ctx->st_best = ctx->st_bmu = nullptr;
    ctx->st_images = 0;
    hipError_t e = hipMalloc((void **)&ctx->st_img, n * ctx->isz * sizeof(float));
    if (e == hipSuccess && ctx->trainer) e = hipMalloc((void **)&ctx->st_bmu, n * sizeof(uint32_t));
    if (e == hipSuccess && !ctx->trainer) e = hipMalloc((void **)&ctx->st_heat, n * ctx->N * sizeof(float));
    if (e == hipSuccess && !ctx->trainer) e = hipMalloc((void **)&ctx->st_best, n * ctx->N * sizeof(uint32_t));
    if (e != hipSuccess) return fail(ctx, PINK_HIP_ENOMEM, "staging allocation failed");
    ctx->st_images = n;
    return PINK_HIP_OK;
}

// Host -> device on the context's stream; small transfers go through the pinned buffer (one
// memcpy on the host, then a true asynchronous copy).
hipError_t stage_in(pink_hip_ctx *ctx, void *dev, const void *host, size_t bytes)
{
    if (bytes <= kPinBytes) {
        if (ctx->st_ring_busy) {                           // queued calls may still read the buffer
            const hipError_t e = hipStreamSynchronize(ctx->stream);
            if (e != hipSuccess) return e;
            ctx->st_ring_busy = false;
        }
        memcpy(ctx->st_pin, host, bytes);
        return hipMemcpyAsync(dev, ctx->st_pin, bytes, hipMemcpyHostToDevice, ctx->stream);
    }
    return hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, ctx->stream);
}

// `n` host images into the staging buffer and through `run(device images, first image, count)`,
// in pieces that grow from about 1 MB to 16 or 64 MB: the copy of a piece goes over a second stream
// while the kernels of the piece before it run (also from pageable memory, where the copy call
// returns when the piece has left the host buffer).  Small inputs take the pinned bounce buffer in one go.
extern "C++" {
template <typename Run>
int staged_run(pink_hip_ctx *ctx, const float *host_images, uint32_t n, Run run)
{
    const size_t img_bytes = (size_t)ctx->isz * sizeof(float);
    if ((size_t)n * img_bytes <= kPinBytes) {
        HIP_TRY(ctx, stage_in(ctx, ctx->st_img, host_images, n * img_bytes));
        return run(ctx->st_img, 0u, n);
    }
    if (!ctx->copy_stream) {
        HIP_TRY(ctx, hipStreamCreateWithFlags(&ctx->copy_stream, hipStreamNonBlocking));
        for (hipEvent_t &e : ctx->copy_ev) HIP_TRY(ctx, hipEventCreateWithFlags(&e, hipEventDisableTiming));
    }
    // whatever still reads the staging buffer (queued per-image calls) finishes first
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    ctx->st_ring_busy = false;
    // (a trainer's kernels take long enough per image for 16 MB pieces to hide all copies but the first behind them:
    // cfg0 40 k -> 51 k images/s with pageable buffers; a mapper's launch groups want the larger pieces)
    // Nothing hides the copy of the first piece, so the pieces start at about 1 MB and double up to that size.
    const auto whole_groups = [&](size_t bytes) {
        uint32_t images = (uint32_t)std::max<size_t>(1, bytes / img_bytes);
        if (images > ctx->Bcap) images -= images % ctx->Bcap;
        return images;
    };
    const uint32_t largest = whole_groups((size_t)(ctx->trainer ? 16 : 64) << 20);
    uint32_t piece = std::min(largest, std::max(whole_groups((size_t)1 << 20), std::min(ctx->Bcap, largest)));
    // A mapper's kernels are faster than the link, so its rate from host buffers is the rate of the copies, and a
    // copy out of pageable memory is one host thread's work (about half of what the link takes): inputs of 32 MB and
    // more go through two pinned buffers that four host threads fill side by side (cfg1 from pageable memory: 26 -> 42 GB/s,
    // 1.6 M -> 2.56 M images/s).
    // Set up all or nothing; a host that cannot give the threads or the pinned memory keeps the plain copies.
    const bool pooled = !ctx->trainer && (size_t)n * img_bytes >= ((size_t)32 << 20);
    if (pooled && !ctx->copy_pool) {
        char *pin[2] = {nullptr, nullptr};
        hipEvent_t ev[2] = {nullptr, nullptr};
        bool ok = true;
        for (int i = 0; i < 2 && ok; ++i)
            ok = hipHostMalloc((void **)&pin[i], kBounceBytes, hipHostMallocDefault) == hipSuccess &&
                 hipEventCreateWithFlags(&ev[i], hipEventDisableTiming) == hipSuccess;
        std::unique_ptr<HostCopyPool> pool;
        if (ok) {
            // (three workers and the caller; five or seven workers, buffers of 4 or 16 MB: the same 42 GB/s)
            try { pool.reset(new HostCopyPool(3)); } catch (...) { ok = false; }
        }
        if (ok) {
            ctx->copy_pool = std::move(pool);
            for (int i = 0; i < 2; ++i) { ctx->bounce[i] = pin[i]; ctx->bounce_ev[i] = ev[i]; }
        } else {
            (void)hipGetLastError();
            for (int i = 0; i < 2; ++i) {
                if (ev[i]) (void)hipEventDestroy(ev[i]);
                if (pin[i]) (void)hipHostFree(pin[i]);
            }
        }
    }
    uint32_t turn = 0, count = 0, bounce_turn = 0;
    for (uint32_t first = 0; first < n; first += count, turn ^= 1, piece = std::min(largest, 2 * piece)) {
        count = std::min(piece, n - first);
        float *dev = ctx->st_img + (size_t)first * ctx->isz;
        if (pooled && ctx->copy_pool) {
            const char *src = (const char *)(host_images + (size_t)first * ctx->isz);
            const size_t bytes = (size_t)count * img_bytes;
            for (size_t off = 0; off < bytes; off += kBounceBytes, bounce_turn ^= 1) {
                const size_t len = std::min(kBounceBytes, bytes - off);
                HIP_TRY(ctx, hipEventSynchronize(ctx->bounce_ev[bounce_turn]));       // its last copy to the device has run
                ctx->copy_pool->copy(ctx->bounce[bounce_turn], src + off, len);
                HIP_TRY(ctx, hipMemcpyAsync((char *)dev + off, ctx->bounce[bounce_turn], len, hipMemcpyHostToDevice, ctx->copy_stream));
                HIP_TRY(ctx, hipEventRecord(ctx->bounce_ev[bounce_turn], ctx->copy_stream));
            }
        } else
        HIP_TRY(ctx, hipMemcpyAsync(dev, host_images + (size_t)first * ctx->isz, count * img_bytes, hipMemcpyHostToDevice,
                                    ctx->copy_stream));
        HIP_TRY(ctx, hipEventRecord(ctx->copy_ev[turn], ctx->copy_stream));
        HIP_TRY(ctx, hipStreamWaitEvent(ctx->stream, ctx->copy_ev[turn], 0));
        TRY(run(dev, first, count));
    }
    return PINK_HIP_OK;
}
}  // extern "C++"

int pink_hip_train(pink_hip_ctx *ctx, const float *host_images, uint32_t n_images, uint32_t *host_bmu_out)
{
    if (!ctx || (!host_images && n_images)) return fail(ctx, PINK_HIP_EINVAL, "pink_hip_train: null argument");
    if (!ctx->trainer) return fail(ctx, PINK_HIP_ESTATE, "pink_hip_train: context was created without update factors");
    if (n_images == 0) return PINK_HIP_OK;
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    const size_t img_bytes = (size_t)ctx->isz * sizeof(float);
    if (!host_bmu_out && n_images * img_bytes <= kSlotBytes) {
        // Nothing to hand back (the reference's operator() returns nothing either): the images join the
        // pending launch group in pinned memory and the call returns; see flush_pending.
        if (!ctx->pend_pin[0]) {
            // both buffers and both events, or none of them: the context takes them only when all four exist
            char *pin[2] = {nullptr, nullptr};
            hipEvent_t ev[2] = {nullptr, nullptr};
            bool ok = true;
            for (int i = 0; i < 2 && ok; ++i)
                ok = hipHostMalloc((void **)&pin[i], (size_t)ctx->Bcap * img_bytes, hipHostMallocDefault) == hipSuccess &&
                     hipEventCreateWithFlags(&ev[i], hipEventDisableTiming) == hipSuccess;
            if (!ok) {
                (void)hipGetLastError();
                for (int i = 0; i < 2; ++i) {
                    if (ev[i]) (void)hipEventDestroy(ev[i]);
                    if (pin[i]) (void)hipHostFree(pin[i]);
                }
                return fail(ctx, PINK_HIP_ENOMEM, "pink_hip_train: pinned host buffers for queued images could not be set up");
            }
            ctx->pend_cap = ctx->Bcap;
            for (int i = 0; i < 2; ++i) { ctx->pend_pin[i] = pin[i]; ctx->pend_ev[i] = ev[i]; }
        }
        for (uint32_t done = 0; done < n_images;) {
            const uint32_t take = std::min(n_images - done, ctx->pend_cap - ctx->pend_count);
            if (ctx->pend_count == 0) HIP_TRY(ctx, hipEventSynchronize(ctx->pend_ev[ctx->pend_cur]));   // its last copy has run
            memcpy(ctx->pend_pin[ctx->pend_cur] + (size_t)ctx->pend_count * img_bytes, host_images + (size_t)done * ctx->isz,
                   (size_t)take * img_bytes);
            ctx->pend_count += take;
            done += take;
            if (ctx->pend_count == ctx->pend_cap) TRY(flush_pending(ctx));
        }
        return PINK_HIP_OK;
    }
    TRY(flush_pending(ctx));
    // Stage the images in chunks of at most ~1 GiB.
    const uint32_t chunk = (uint32_t)std::max<size_t>(1, std::min<size_t>(n_images, ((size_t)1 << 30) / img_bytes));
    TRY(ensure_staging(ctx, chunk));
    for (uint32_t done = 0; done < n_images; done += chunk) {
        const uint32_t n = std::min(chunk, n_images - done);
        TRY(staged_run(ctx, host_images + (size_t)done * ctx->isz, n, [&](const float *dev, uint32_t first, uint32_t count) {
            return pink_hip_train_device(ctx, dev, count, ctx->st_bmu + first);
        }));
        if (host_bmu_out) {
            const size_t out_bytes = n * sizeof(uint32_t);
            const bool small = out_bytes <= kPinBytes;
            HIP_TRY(ctx, hipMemcpyAsync(small ? (void *)(ctx->st_pin + kPinBytes) : (void *)(host_bmu_out + done), ctx->st_bmu,
                                        out_bytes, hipMemcpyDeviceToHost, ctx->stream));
            HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
            if (small) memcpy(host_bmu_out + done, ctx->st_pin + kPinBytes, out_bytes);
        } else {
            HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));      // the host images are the caller's again on return
        }
    }
    return PINK_HIP_OK;
}

int pink_hip_map_device(pink_hip_ctx *ctx, const float *dev_images, uint32_t n_images, float *dev_heatmap_out,
                        uint32_t *dev_best_rot_out)
{
    if (!ctx || (n_images && (!dev_images || !dev_heatmap_out)))
        return fail(ctx, PINK_HIP_EINVAL, "pink_hip_map_device: null argument");
    if (ctx->trainer) return fail(ctx, PINK_HIP_ESTATE, "pink_hip_map_device: context was created with update factors (a trainer)");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    for (uint32_t done = 0; done < n_images; done += ctx->Bcap) {
        const uint32_t B = std::min(ctx->Bcap, n_images - done);
        TRY(distance_group(ctx, dev_images + (size_t)done * ctx->isz, B));
        TRY(run_finalize(ctx, B, dev_heatmap_out + (size_t)done * ctx->N, nullptr,
                         dev_best_rot_out ? dev_best_rot_out + (size_t)done * ctx->N : nullptr, true));
    }
    return PINK_HIP_OK;
}

// The per-group buffers of a mapping call, per image, in the order they are carved out of the static
// scratch (every piece starts on a 256-byte boundary).
struct StaticPieces {
    size_t key = 0, Pb = 0, nb = 0, gPb = 0, gnb = 0, rot = 0, rotT = 0;
    size_t per_image() const { return key + Pb + nb + gPb + gnb + rot + rotT; }
};

static StaticPieces static_pieces(const pink_hip_ctx *ctx)
{
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    StaticPieces p;
    p.key = up((size_t)ctx->N * sizeof(unsigned long long));
    if (ctx->mfma_sym) {
        p.Pb = up((size_t)ctx->RTP * pink_sym::unit_bytes(ctx->KSs));
    } else if (ctx->mfma) {
        p.Pb = up((size_t)ctx->RT * ctx->KS * 1024);
        p.nb = up((size_t)ctx->RT * 32 * sizeof(int));
    } else if (ctx->gemm) {
        const size_t planes = ctx->cfg.ed_type == PINK_HIP_UINT16 ? 2 : 1;
        p.gPb = up(planes * (ctx->Rp / 32) * ctx->gKS * 1024);
        p.gnb = up((size_t)ctx->Rp * sizeof(long long));
    } else {
        p.rotT = up((size_t)ctx->Epad * ctx->Rpad * 4);
    }
    if (!ctx->mfma && !ctx->mfma_sym && !ctx->fused_pack) p.rot = up((size_t)ctx->R * ctx->S * sizeof(float));
    return p;
}

int pink_hip_map_device_static(pink_hip_ctx *ctx, const float *dev_images, uint32_t n_images, float *dev_heatmap_out,
                               uint32_t *dev_best_rot_out)
{
    if (!ctx || (n_images && (!dev_images || !dev_heatmap_out)))
        return fail(ctx, PINK_HIP_EINVAL, "pink_hip_map_device_static: null argument");
    if (ctx->trainer)
        return fail(ctx, PINK_HIP_ESTATE, "pink_hip_map_device_static: context was created with update factors (a trainer)");
    if (ctx->f32gemm)
        return fail(ctx, PINK_HIP_ESTATE, "pink_hip_map_device_static: the float32 matrix-core kernel choice keeps its operands "
                                          "in buffers of the context; not available through this entry point");
    if (ctx->profiling)
        return fail(ctx, PINK_HIP_ESTATE, "pink_hip_map_device_static: per-kernel timing creates events; switch it off");
    if (!ctx->static_scratch) return fail(ctx, PINK_HIP_ESTATE, "pink_hip_map_device_static: no static scratch on this device");
    const StaticPieces pc = static_pieces(ctx);
    const size_t per_image = pc.per_image();
    // (the float distance kernel of small problems reads up to kDistOverrun floats past the last row of its
    // operand, the piece carved last)
    const size_t capacity = PINK_HIP_STATIC_SCRATCH_BYTES - kDistOverrun * sizeof(float);
    if (per_image > capacity)
        return fail(ctx, PINK_HIP_EINVAL, "pink_hip_map_device_static: one image of this context needs " + std::to_string(per_image) +
                                          " bytes of scratch, the static scratch holds " + std::to_string(capacity));
    if (n_images == 0) return PINK_HIP_OK;
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    const uint32_t B = (uint32_t)std::min<size_t>({(size_t)ctx->Bcap, capacity / per_image, (size_t)n_images});

    // the scratch keeps what the last call (of any context on this GPU) left: rows beyond the last variant
    // and elements beyond the region must read as zero, so the part this call uses starts from zero
    const size_t used = (size_t)B * per_image;
    hipLaunchKernelGGL(k_fill_zero, dim3((uint32_t)std::min<size_t>((used / 16 + 255) / 256, 2048)), dim3(256), 0, ctx->stream,
                       (v4i *)ctx->static_scratch, used / 16);
    TRY(launch_check(ctx, "k_fill_zero"));

    // the kernels take the scratch where they take the context's own buffers in pink_hip_map_device
    struct Saved {
        unsigned long long *key; signed char *Pb; int *nb; v4i *gPb; long long *gnb; float *rot; void *rotT;
    } const saved{ctx->d_key, ctx->d_Pb, ctx->d_nb, ctx->d_gPb, ctx->d_gnb, ctx->d_rot, ctx->d_rotT};
    unsigned char *at = ctx->static_scratch;
    auto carve = [&](size_t bytes_per_image) { unsigned char *p = at; at += (size_t)B * bytes_per_image; return p; };
    ctx->d_key = (unsigned long long *)carve(pc.key);
    if (pc.Pb) ctx->d_Pb = (signed char *)carve(pc.Pb);
    if (pc.nb) ctx->d_nb = (int *)carve(pc.nb);
    if (pc.gPb) ctx->d_gPb = (v4i *)carve(pc.gPb);
    if (pc.gnb) ctx->d_gnb = (long long *)carve(pc.gnb);
    if (pc.rot) ctx->d_rot = (float *)carve(pc.rot);
    if (pc.rotT) ctx->d_rotT = carve(pc.rotT);
    int rc = PINK_HIP_OK;
    for (uint32_t done = 0; done < n_images && rc == PINK_HIP_OK; done += B) {
        const uint32_t b = std::min(B, n_images - done);
        rc = distance_group(ctx, dev_images + (size_t)done * ctx->isz, b);
        if (rc == PINK_HIP_OK)
            rc = run_finalize(ctx, b, dev_heatmap_out + (size_t)done * ctx->N, nullptr,
                              dev_best_rot_out ? dev_best_rot_out + (size_t)done * ctx->N : nullptr, true);
    }
    ctx->d_key = saved.key; ctx->d_Pb = saved.Pb; ctx->d_nb = saved.nb; ctx->d_gPb = saved.gPb; ctx->d_gnb = saved.gnb;
    ctx->d_rot = saved.rot; ctx->d_rotT = saved.rotT;
    return rc;
}

int pink_hip_map(pink_hip_ctx *ctx, const float *host_images, uint32_t n_images, float *host_heatmap_out,
                 uint32_t *host_best_rot_out)
{
    if (!ctx || (n_images && (!host_images || !host_heatmap_out)))
        return fail(ctx, PINK_HIP_EINVAL, "pink_hip_map: null argument");
    if (ctx->trainer) return fail(ctx, PINK_HIP_ESTATE, "pink_hip_map: context was created with update factors (a trainer)");
    if (n_images == 0) return PINK_HIP_OK;
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    const size_t img_bytes = (size_t)ctx->isz * sizeof(float);
    const uint32_t chunk = (uint32_t)std::max<size_t>(1, std::min<size_t>(n_images, ((size_t)1 << 30) / img_bytes));
    TRY(ensure_staging(ctx, chunk));
    for (uint32_t done = 0; done < n_images; done += chunk) {
        const uint32_t n = std::min(chunk, n_images - done);
        TRY(staged_run(ctx, host_images + (size_t)done * ctx->isz, n, [&](const float *dev, uint32_t first, uint32_t count) {
            return pink_hip_map_device(ctx, dev, count, ctx->st_heat + (size_t)first * ctx->N, ctx->st_best + (size_t)first * ctx->N);
        }));
        const size_t heat_bytes = (size_t)n * ctx->N * sizeof(float);       // the best rotations take as many bytes
        const bool small = 2 * heat_bytes <= kPinBytes;
        char *pin_out = ctx->st_pin + kPinBytes;
        float *heat_dst = host_heatmap_out + (size_t)done * ctx->N;
        uint32_t *best_dst = host_best_rot_out ? host_best_rot_out + (size_t)done * ctx->N : nullptr;
        HIP_TRY(ctx, hipMemcpyAsync(small ? (void *)pin_out : (void *)heat_dst, ctx->st_heat, heat_bytes, hipMemcpyDeviceToHost,
                                    ctx->stream));
        if (best_dst)
            HIP_TRY(ctx, hipMemcpyAsync(small ? (void *)(pin_out + heat_bytes) : (void *)best_dst, ctx->st_best, heat_bytes,
                                        hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
        if (small) {
            memcpy(heat_dst, pin_out, heat_bytes);
            if (best_dst) memcpy(best_dst, pin_out + heat_bytes, heat_bytes);
        }
    }
    return PINK_HIP_OK;
}

int pink_hip_rotate(pink_hip_ctx *ctx, const float *host_image, float *host_variants_out)
{
    if (!ctx || !host_image || !host_variants_out) return fail(ctx, PINK_HIP_EINVAL, "pink_hip_rotate: null argument");
    TRY(flush_pending(ctx));
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    float *d_img = nullptr;
    HIP_TRY(ctx, hipMalloc((void **)&d_img, (size_t)ctx->isz * sizeof(float)));
    hipError_t e = hipMemcpyAsync(d_img, host_image, (size_t)ctx->isz * sizeof(float), hipMemcpyHostToDevice, ctx->stream);
    int rc = PINK_HIP_OK;
    if (e == hipSuccess) rc = run_rotate(ctx, d_img, 1, kStoreAll);
    if (e == hipSuccess && rc == PINK_HIP_OK)
        e = hipMemcpyAsync(host_variants_out, ctx->d_rot, (size_t)ctx->R * ctx->S * sizeof(float), hipMemcpyDeviceToHost,
                           ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    (void)hipFree(d_img);
    if (e != hipSuccess) return fail(ctx, PINK_HIP_EDEVICE, std::string("pink_hip_rotate: ") + hipGetErrorString(e));
    return rc;
}

int pink_hip_distance(pink_hip_ctx *ctx, const float *host_image, float *host_dist_out, int64_t *host_ssd_out,
                      uint32_t *host_best_rot_out)
{
    if (!ctx || !host_image) return fail(ctx, PINK_HIP_EINVAL, "pink_hip_distance: null argument");
    TRY(flush_pending(ctx));
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    float *d_img = nullptr;
    HIP_TRY(ctx, hipMalloc((void **)&d_img, (size_t)ctx->isz * sizeof(float)));
    hipError_t e = hipMemcpyAsync(d_img, host_image, (size_t)ctx->isz * sizeof(float), hipMemcpyHostToDevice, ctx->stream);
    int rc = PINK_HIP_OK;
    if (e == hipSuccess) rc = distance_group(ctx, d_img, 1);
    if (e == hipSuccess && rc == PINK_HIP_OK) rc = run_finalize(ctx, 1, ctx->d_dist, ctx->d_ssd, ctx->d_best, false);
    const size_t n = ctx->N;
    if (e == hipSuccess && rc == PINK_HIP_OK && host_dist_out)
        e = hipMemcpyAsync(host_dist_out, ctx->d_dist, n * sizeof(float), hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess && rc == PINK_HIP_OK && host_ssd_out && is_int(ctx))
        e = hipMemcpyAsync(host_ssd_out, ctx->d_ssd, n * sizeof(long long), hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess && rc == PINK_HIP_OK && host_best_rot_out)
        e = hipMemcpyAsync(host_best_rot_out, ctx->d_best, n * sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    (void)hipFree(d_img);
    if (e != hipSuccess) return fail(ctx, PINK_HIP_EDEVICE, std::string("pink_hip_distance: ") + hipGetErrorString(e));
    return rc;
}

uint32_t pink_hip_region_size(const pink_hip_ctx *ctx) { return ctx ? ctx->E : 0; }

uint32_t pink_hip_distance_kernel(const pink_hip_ctx *ctx)
{
    if (!ctx) return 0;
    return ctx->mfma_sym ? PINK_HIP_KERNEL_MFMA_SYM : ctx->mfma ? PINK_HIP_KERNEL_MFMA
         : ctx->gemm ? PINK_HIP_KERNEL_MFMA_GEMM : ctx->f32gemm ? PINK_HIP_KERNEL_MFMA_F32 : PINK_HIP_KERNEL_VALU;
}

int pink_hip_set_profiling(pink_hip_ctx *ctx, int enable)
{
    if (!ctx) return PINK_HIP_EINVAL;
    TRY(flush_pending(ctx));
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    TRY(drain_events(ctx));
    ctx->profiling = enable != 0;
    for (int i = 0; i < PINK_HIP_NUM_KERNEL_CLASSES; ++i) { ctx->prof_launches[i] = 0; ctx->prof_ms[i] = 0.0; }
    return PINK_HIP_OK;
}

int pink_hip_kernel_times(pink_hip_ctx *ctx, uint64_t *launches_out, double *ms_out)
{
    if (!ctx) return PINK_HIP_EINVAL;
    TRY(flush_pending(ctx));
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    TRY(drain_events(ctx));
    for (int i = 0; i < PINK_HIP_NUM_KERNEL_CLASSES; ++i) {
        if (launches_out) launches_out[i] = ctx->prof_launches[i];
        if (ms_out) ms_out[i] = ctx->prof_ms[i];
    }
    return PINK_HIP_OK;
}

#ifdef PINK_PROBE
// (measurement builds only) the stamps of kernel `kernel`: [block][wave][slot] 100 MHz clock values, 0 = never written
int pink_hip_probe_read(uint32_t kernel, unsigned long long *host_out, int clear)
{
    const size_t n = (size_t)kProbeBlocks * kProbeWaves * kProbeSlots;
    if (kernel >= kProbeKernels) return PINK_HIP_EINVAL;
    if (hipDeviceSynchronize() != hipSuccess) return PINK_HIP_EDEVICE;
    if (hipMemcpyFromSymbol(host_out, HIP_SYMBOL(g_probe), n * 8, (size_t)kernel * n * 8, hipMemcpyDeviceToHost) != hipSuccess)
        return PINK_HIP_EDEVICE;
    if (clear) {
        std::vector<unsigned long long> z(n, 0ull);
        if (hipMemcpyToSymbol(HIP_SYMBOL(g_probe), z.data(), n * 8, (size_t)kernel * n * 8, hipMemcpyHostToDevice) != hipSuccess)
            return PINK_HIP_EDEVICE;
    }
    return PINK_HIP_OK;
}
#endif

int pink_hip_device_info(char *buf, size_t len)
{
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess) {
        g_create_error = std::string("hipGetDeviceCount: ") + hipGetErrorString(e);
        return PINK_HIP_EDEVICE;
    }
    std::string s;
    for (int d = 0; d < count; ++d) {
        hipDeviceProp_t p;
        if (hipGetDeviceProperties(&p, d) != hipSuccess) continue;
        char line[512];
        snprintf(line, sizeof line, "device %d: %s (%s), %d CUs, %d MHz, %.1f GiB, LDS/block %zu KiB\n", d, p.name,
                 p.gcnArchName, p.multiProcessorCount, p.clockRate / 1000, p.totalGlobalMem / 1073741824.0,
                 p.sharedMemPerBlock / 1024);
        s += line;
    }
    if (buf && len) {
        strncpy(buf, s.c_str(), len - 1);
        buf[len - 1] = '\0';
    }
    return count;
}

}  // extern "C"

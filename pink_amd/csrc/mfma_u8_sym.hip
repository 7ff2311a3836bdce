// mfma_u8_sym.hip -- uint8 mapping with the 8 symmetries moved to the SOM side.
// A translation unit of its own: it is compiled with MFMA accumulators in the architectural
// vector registers, so that the accumulation registers can hold the resident SOM fragments
// (see the build script); pink_hip.hip reaches it through the launchers in mfma_u8_sym.h.
//
// A mapper's SOM never changes, so the quarter turns and the flip are applied to the
// neurons once instead of to every image: with perm_s the map from variant coordinates to
// base-rotation coordinates of symmetry s,
//   ssd(n, variant (s, i)) = sum_{e in region} (q_n[off_e] - q_i[perm_s(off_e)])^2
//                          = sum_{p in P_s} (A_{n,s}[p] - q_i[p])^2,   P_s = perm_s(region),
// where q_i is the quantised base rotation i (0 <= angle < 90 degrees) and A_{n,s}[p] is the
// neuron element that symmetry s pairs with base position p.  Over the union U of the P_s,
// with A_{n,s} = 0 outside P_s (values shifted by -128),
//   ssd = |A_{n,s}|^2 + sum_{p in P_s} q'_i[p]^2 - 2 A_{n,s} . q'_i          (exact in int32).
// The image side shrinks to num_rot/4 rows per image (8x fewer bytes to produce and to
// stream); the SOM side grows to 8 rows per neuron, prepared once.
//
// Operands are fragment-major as in the other matrix-core path: rows in tiles of 32, k in
// steps of 32, a (tile, k-step) fragment = 64 lanes x 16 bytes, lane l = row l % 32,
// k-half l / 32.  SOM-side rows are m = n * 8 + s, so the 8 symmetries of a neuron sit in 8
// adjacent lanes of the MFMA's column operand.

#include <hip/hip_runtime.h>

#include <climits>
#include <cstdint>

#include "mfma_u8_sym.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// q = T(x * factor) saturated to [0, factor] (CudaLib/copy_and_transform_kernel.h:27-28)
__device__ __forceinline__ int32_t quantise(float x, float factor)
{
    const float v = __fmul_rn(x, factor);
    if (!(v > 0.0f)) return 0;
    if (v >= factor) return (int32_t)factor;
    return (int32_t)v;
}

// Row stride (floats) of an image in the rotation kernel's LDS: the I pixels, at least one zero
// column, and congruent to 5 modulo 8.  The banks of the four neighbours of a rotated position
// are (stride * row + column) mod 64; the lanes of a wave read the same position under 32
// neighbouring angles, i.e. a short arc of texels, and with stride = 1 mod 64 (I = 64 with a single
// pad column) every arc along the anti-diagonal would stay in one bank (measured at I = 64: strides 67 to 73
// are 19 % faster than 65).
inline uint32_t row_stride(uint32_t I)
{
    uint32_t W = I + 1;
    while (W % 8 != 5) ++W;
    return W;
}

// SOM operand.  One block per row m = n * 8 + s (rows beyond 8 N are zero).
// aoff[s][k] = neuron element paired with union position k under symmetry s, or ~0.
__global__ __launch_bounds__(256) void k_pack_som_sym_u8(const float *__restrict__ som, const uint32_t *__restrict__ aoff,
                                                         signed char *__restrict__ Pa, int *__restrict__ na, uint32_t N,
                                                         uint32_t S, uint32_t KS)
{
    __shared__ int s_sum[256];
    const uint32_t m = blockIdx.x, n = m >> 3, sym = m & 7;
    const uint32_t Kp = KS * 32;
    int sq = 0;
    for (uint32_t k = threadIdx.x; k < Kp; k += 256) {
        int v = 0;
        if (n < N) {
            const uint32_t o = aoff[(size_t)sym * Kp + k];
            if (o != 0xffffffffu) v = quantise(som[(size_t)n * S + o], 255.0f) - 128;
        }
        sq += v * v;
        const uint32_t lane = (m & 31) + 32 * ((k & 31) >> 4);
        Pa[((((size_t)(m >> 5) * KS + (k >> 5)) * 64 + lane) << 4) + (k & 15)] = (signed char)v;
    }
    s_sum[threadIdx.x] = sq;
    __syncthreads();
    for (uint32_t s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) s_sum[threadIdx.x] += s_sum[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) na[m] = s_sum[0];
}

// Image operand: base rotations only.
//
// Where a rotated pixel comes from does not depend on the image: for base rotation i and union
// position k the bilinear rule of ImageProcessingLib/rotate.h:31-65 reads four neighbours at a
// fixed place of the source image with fixed weights.  k_rot_table evaluates that geometry once
// per context, in the CPU's operation order:
//   tab_idx(i, k) = offset of the upper-left neighbour in the padded LDS image (channel included),
//   tab_w(i, k)   = (cx*cy, cx*ry, rx*cy, rx*ry), the four products the CPU forms first.
// Where the source position lies outside the image (value 0, rotate.h:40-44) or k is beyond the
// union, the entry points at a zero cell of the padding with four zero weights: 0 for finite pixels.
// Base rotation 0 is the centre crop / pad of ImageProcessingLib/resize.h:15-40: weight 1 on the
// copied pixel, 0 on the others (1*x + 0 + 0 + 0 == x for the finite inputs the quantisation is
// defined for).  The per-image work that is left is four products, three sums and the quantisation.
//   upos[k] = (channel << 24 | x << 12 | y) of union element k, k < Ku.
__global__ __launch_bounds__(256) void k_rot_table(const float *__restrict__ cos_t, const float *__restrict__ sin_t,
                                                   const uint32_t *__restrict__ upos, uint32_t Ku, uint32_t I,
                                                   uint32_t D, uint32_t nrr_eff, uint32_t Kp, uint32_t rows,
                                                   uint32_t W, uint32_t *__restrict__ tab_idx,
                                                   float4 *__restrict__ tab_w)
{
    const uint32_t t = blockIdx.x * 256 + threadIdx.x;
    if (t >= rows * Kp) return;
    const uint32_t i = t / Kp, k = t % Kp;
    const uint32_t CH = (I + 1) * W;                      // W = row stride of the LDS image
    uint32_t idx = I;                                     // row 0 of the extra column: 0.0
    float4 w = {0.0f, 0.0f, 0.0f, 0.0f};
    if (i < nrr_eff && k < Ku) {
        const uint32_t p = upos[k];
        const uint32_t c = p >> 24, x = (p >> 12) & 0xfff, y = p & 0xfff;
        if (i == 0) {
            if (I >= D) {
                const uint32_t m = (I - D) / 2;
                idx = c * CH + (x + m) * W + (y + m);
                w.x = 1.0f;
            } else {
                const uint32_t m = (D - I) / 2;
                const uint32_t sx = x - m, sy = y - m;     // wraps below the margin: caught by the range test
                if (sx < I && sy < I) { idx = c * CH + sx * W + sy; w.x = 1.0f; }
            }
        } else {
            const float cs = cos_t[i], sn = sin_t[i];
            const float src_c = __fmul_rn((float)(I - 1), 0.5f), dst_c = __fmul_rn((float)(D - 1), 0.5f);
            const float lim = (float)(I - 1);
            const float px = __fsub_rn((float)x, dst_c), py = __fsub_rn((float)y, dst_c);
            const float sxf = __fadd_rn(__fsub_rn(__fmul_rn(px, cs), __fmul_rn(py, sn)), src_c);
            const float syf = __fadd_rn(__fadd_rn(__fmul_rn(px, sn), __fmul_rn(py, cs)), src_c);
            if (!(sxf < 0.0f || sxf > lim || syf < 0.0f || syf > lim)) {
                // the neighbours one past the last row / column carry weight 0 and exist in the
                // padded LDS image (rotate.h:50,62-63 reads them out of bounds)
                const uint32_t ix = (uint32_t)sxf, iy = (uint32_t)syf;
                const float rx = __fsub_rn(sxf, (float)ix), ry = __fsub_rn(syf, (float)iy);
                const float cx = __fsub_rn(1.0f, rx), cy = __fsub_rn(1.0f, ry);
                idx = c * CH + ix * W + iy;
                w.x = __fmul_rn(cx, cy); w.y = __fmul_rn(cx, ry); w.z = __fmul_rn(rx, cy); w.w = __fmul_rn(rx, ry);
            }
        }
    }
    // rotation-interleaved so that the lanes of a wave, which hold the same piece of 32 consecutive
    // rotations, read consecutive 16-byte entries: weights [piece][j][i], offsets [piece][j / 4][i][j % 4]
    const uint32_t piece = k / 16, j = k % 16;
    tab_w[((size_t)piece * 16 + j) * rows + i] = w;
    tab_idx[(((size_t)piece * 4 + j / 4) * rows + i) * 4 + j % 4] = idx;
}

// Quotient and remainder by a divisor that is the same for the whole block, for dividends below
// 2^24 (element counts of an LDS tile): a shift and a mask for a power of two, else the float
// reciprocal's estimate, which is within one of the quotient, corrected.  The compiler's general
// 32-bit division costs about four times as many instructions.
struct BlockDivisor {
    uint32_t d, mask;
    int shift;              // >= 0: d = 1 << shift
    float rcp;
    __device__ explicit BlockDivisor(uint32_t d_) : d(d_), mask(d_ - 1), shift((d_ & (d_ - 1)) == 0 ? __builtin_ctz(d_) : -1),
                                                    rcp(1.0f / (float)d_) {}
    __device__ __forceinline__ void divmod(uint32_t n, uint32_t &q, uint32_t &r) const
    {
        if (shift >= 0) { q = n >> shift; r = n & mask; return; }
        uint32_t e = (uint32_t)((float)n * rcp);
        int rem = (int)(n - e * d);
        if (rem < 0) { --e; rem += (int)d; }
        else if ((uint32_t)rem >= d) { ++e; rem -= (int)d; }
        q = e; r = (uint32_t)rem;
    }
};

// Byte `byte` of `word` = q = uint8(x * 255), truncated and saturated to [0, 255] (NaN -> 0):
// multiply, truncate, then the saturating convert-and-pack (which alone would round to nearest).
__device__ __forceinline__ uint32_t pack_quantised_u8(float x, uint32_t byte, uint32_t word)
{
    return __builtin_amdgcn_cvt_pk_u8_f32(__builtin_truncf(__fmul_rn(x, 255.0f)), byte, word);
}

// A block handles one row tile (32 base rotations) of G images, which it keeps in LDS with one
// extra zero column per row and one extra zero row per channel.  A thread evaluates 16
// consecutive union positions of one rotation for every image -- a table entry is read once and
// applied G times --, stores them as one 16-byte piece of a fragment per image, and adds their
// squares to the 8 per-symmetry norms of that rotation according to kmask (bit s of kmask[k] set
// when union position k belongs to P_s).
template <int G>
__global__ __launch_bounds__(512) void k_rotpack_sym_u8(const float *__restrict__ images, v4i *__restrict__ Pb,
                                                        const uint32_t *__restrict__ tab_idx,
                                                        const float4 *__restrict__ tab_w,
                                                        const unsigned char *__restrict__ kmask, uint32_t Ku,
                                                        uint32_t all_sym, uint32_t C, uint32_t I, uint32_t nrr_eff,
                                                        uint32_t KS, uint32_t RTP, uint32_t B, uint32_t W)
{
    // C x (I + 1) rows of W pixels, zero padded, the G images interleaved per pixel: the four
    // neighbours of a position are four reads of G floats for all images, from one address
    extern __shared__ float s_img[];
    __shared__ int s_nb[G][32][8];
    const uint32_t UNIT_V = KS * 64 + 64;                 // 16-byte vectors per unit: fragments, then norm entries
    // Workgroups go to the 8 XCDs round-robin by linear id, and each XCD has its own L2.  The
    // id is decoded so that all blocks of one group of images share id % 8, i.e. one XCD: the
    // images then leave HBM once instead of once per XCD.
    const uint32_t lin = blockIdx.x;
    const uint32_t span = 8 * RTP;                        // ids covering 8 groups
    const uint32_t rt = (lin % span) / 8;
    const uint32_t b0 = ((lin / span) * 8 + (lin % 8)) * G;
    if (b0 >= B) return;
    const uint32_t ng = min((uint32_t)G, B - b0);
    const uint32_t CH = (I + 1) * W, II = I * I;
    const uint32_t nthreads = blockDim.x;
    for (uint32_t t = threadIdx.x; t < G * 32 * 8; t += nthreads) (&s_nb[0][0][0])[t] = 0;
    // Copy the batch into the padded tiles.  The loads of up to 8 elements per thread are issued
    // before the first is used, so the block pays the memory latency once, not once per image.
    {
        const float *src = images + (size_t)b0 * C * II;
        const uint32_t total = ng * C * II;
        const BlockDivisor by_II(II), by_I(I), by_C(C), by_rows(I + 1), by_G(G);
        if ((I & 3) == 0) {
            // rows are whole float4s: 16-byte loads, one division per vector
            const float4 *src4 = (const float4 *)src;
            const uint32_t total4 = total / 4;
            for (uint32_t base = 0; base < total4; base += 8 * nthreads) {
                float4 v[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t e = base + j * nthreads + threadIdx.x;
                    if (e < total4) v[j] = src4[e];
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t e = base + j * nthreads + threadIdx.x;
                    if (e < total4) {
                        uint32_t gc, rem, row, col, gi, c;
                        by_II.divmod(4 * e, gc, rem);
                        by_I.divmod(rem, row, col);
                        by_C.divmod(gc, gi, c);
                        float *d = s_img + (c * CH + row * W + col) * G + gi;
                        d[0] = v[j].x; d[G] = v[j].y; d[2 * G] = v[j].z; d[3 * G] = v[j].w;
                    }
                }
            }
        } else {
            for (uint32_t base = 0; base < total; base += 8 * nthreads) {
                float v[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t e = base + j * nthreads + threadIdx.x;
                    if (e < total) v[j] = src[e];
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t e = base + j * nthreads + threadIdx.x;
                    if (e < total) {
                        uint32_t gc, rem, row, col, gi, c;
                        by_II.divmod(e, gc, rem);
                        by_I.divmod(rem, row, col);
                        by_C.divmod(gc, gi, c);
                        s_img[(c * CH + row * W + col) * G + gi] = v[j];
                    }
                }
            }
        }
        for (uint32_t t = threadIdx.x; t < G * C * (I + 1); t += nthreads) {
            uint32_t gi, p, c, r;
            by_G.divmod(t, p, gi);
            by_rows.divmod(p, c, r);
            s_img[(c * CH + r * W + I) * G + gi] = 0.0f;  // extra column (the only pad column ever read)
            s_img[(c * CH + I * W + r) * G + gi] = 0.0f;  // extra row
        }
    }
    __syncthreads();

    // The two halves of a wave take the two pieces of one k-step for the 32 rotations of the tile:
    // a wave's 64 pieces are one whole fragment, written as 1 KiB of consecutive addresses.
    const uint32_t pieces = KS * 2;                       // 16-element pieces per row
    const uint32_t rows = RTP * 32;
    for (uint32_t t = threadIdx.x; t < 32 * pieces; t += blockDim.x) {
        const uint32_t g = t % 32, piece = t / 32;
        const uint32_t i = rt * 32 + g;                   // base rotation
        const uint32_t k0 = piece * 16;
        uint32_t word[G][4];
#pragma unroll
        for (int gi = 0; gi < G; ++gi)
#pragma unroll
            for (int w4 = 0; w4 < 4; ++w4) word[gi][w4] = 0;
        uint32_t live[4];                                 // byte masks of the positions inside the union
#pragma unroll
        for (int w4 = 0; w4 < 4; ++w4) {
            // (rows beyond the last base rotation are all zero: their products must not count)
            const int inside = i < nrr_eff ? (int)Ku - (int)(k0 + 4 * w4) : 0;
            live[w4] = inside >= 4 ? 0xffffffffu : inside <= 0 ? 0u : (1u << (8 * inside)) - 1u;
        }
        if (i < nrr_eff) {
            const uint4 *ti = (const uint4 *)tab_idx + (size_t)piece * 4 * rows + i;
            const float4 *tw = tab_w + (size_t)piece * 16 * rows + i;
#pragma unroll
            for (int w4 = 0; w4 < 4; ++w4) {
                const uint4 iv = ti[w4 * rows];
                const uint32_t ii[4] = {iv.x, iv.y, iv.z, iv.w};
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const float4 wv = tw[(4 * w4 + u) * rows];
                    typedef float vecG __attribute__((ext_vector_type(G)));
                    const float *tap = s_img + ii[u] * G;
                    // (all G images, also past the end of the batch: what is computed from LDS nobody
                    // filled is dropped below, and the loop stays free of branches)
                    float t00[G], t01[G], t10[G], t11[G];
                    if constexpr (G > 1) {
                        const vecG a = *(const vecG *)tap, b = *(const vecG *)(tap + G);
                        const vecG c = *(const vecG *)(tap + W * G), d = *(const vecG *)(tap + W * G + G);
#pragma unroll
                        for (int gi = 0; gi < G; ++gi) { t00[gi] = a[gi]; t01[gi] = b[gi]; t10[gi] = c[gi]; t11[gi] = d[gi]; }
                    } else {
                        t00[0] = tap[0]; t01[0] = tap[1]; t10[0] = tap[W]; t11[0] = tap[W + 1];
                    }
#pragma unroll
                    for (int gi = 0; gi < G; ++gi) {
                        const float a = __fmul_rn(wv.x, t00[gi]);
                        const float b = __fmul_rn(wv.y, t01[gi]);
                        const float c = __fmul_rn(wv.z, t10[gi]);
                        const float d = __fmul_rn(wv.w, t11[gi]);
                        const float v = __fadd_rn(__fadd_rn(__fadd_rn(a, b), c), d);
                        word[gi][w4] = pack_quantised_u8(v, u, word[gi][w4]);
                    }
                }
            }
        }
#pragma unroll
        for (int gi = 0; gi < G; ++gi) {
            if (gi < (int)ng) {
                v4i frag;
                int sq[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int w4 = 0; w4 < 4; ++w4) {
                    // q - 128 as a signed byte is q ^ 0x80; bytes beyond the union stay 0
                    const int sw = (int)((word[gi][w4] ^ 0x80808080u) & live[w4]);
                    frag[w4] = sw;
                    if (all_sym) sq[0] = __builtin_amdgcn_sdot4(sw, sw, sq[0], false);
                    else {
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const uint32_t k = k0 + w4 * 4 + u;
                            const int v = (int)(signed char)(sw >> (8 * u));
                            const uint32_t mk = kmask[min(k, Ku - 1)];
#pragma unroll
                            for (int s = 0; s < 8; ++s) sq[s] += (mk >> s) & 1 ? v * v : 0;
                        }
                    }
                }
                Pb[((size_t)(b0 + gi) * RTP + rt) * UNIT_V + (piece >> 1) * 64 + g + 32 * (piece & 1)] = frag;
                if (all_sym) {
                    if (sq[0]) atomicAdd(&s_nb[gi][g][0], sq[0]);
                } else {
#pragma unroll
                    for (int s = 0; s < 8; ++s) if (sq[s]) atomicAdd(&s_nb[gi][g][s], sq[s]);
                }
            }
        }
    }
    __syncthreads();
    for (uint32_t gi = 0; gi < ng && threadIdx.x < 256; ++gi) {
        // norm entries of the unit, [symmetry][row]: (15 - j) - 16 |row|^2 with j the accumulator
        // index the distance kernel's lanes hold this row in (see there).  Rows beyond the last base
        // rotation get a norm no real distance reaches: they never win the argmin.
        const uint32_t s = threadIdx.x >> 5, g = threadIdx.x & 31;
        // (16 times the stand-in must stay inside int32 and below 16 (ssd - |a|^2) of any real row:
        // real rows reach 16 * 9.96e7 at 2048 elements)
        const int norm = rt * 32 + g < nrr_eff ? (all_sym ? s_nb[gi][g][0] : s_nb[gi][g][s]) : (KS > 32 ? (1 << 27) - 1 : (1 << 26));
        const int j = 4 * (g >> 3) + (g & 3);
        int *entries = (int *)(Pb + ((size_t)(b0 + gi) * RTP + rt) * UNIT_V + KS * 64);
        entries[s * 32 + g] = (15 - j) - 16 * norm;
    }
}

// Distance + argmin.  A wave keeps its 64 SOM-side rows (8 neurons x 8 symmetries = 2 column
// tiles) for the WHOLE k range in registers (2 * KS fragments in the accumulation half of the
// register file, which the MFMA reads directly), so the SOM operand is read once per kernel.
// The image operand arrives in units of one row tile (32 base rotations, all k, then the tile's
// 8 x 32 norm entries) and goes through three LDS buffers: unit u is multiplied from buffer
// u % 3 while unit u+1 moves from the staging registers into the next buffer and the loads of unit
// u+2 are issued into those registers.  One barrier per unit, in the middle of its k loop, is all
// the synchronisation: the MFMA stream runs on across unit boundaries.
// Base rotations are the MFMA's row operand: after the k loop a lane holds, for each of its 2
// columns (one neuron, one symmetry), 16 base rotations of the tile; their running argmin is
// kept in-lane by vector-ALU work slotted between the MFMAs of the next unit (from a second
// accumulator set); per image there is one exchange between the half-waves and three among the 8
// symmetry lanes.  Every (image, neuron) key is produced by exactly one wave: plain stores, no atomics.
template <int KS>
__global__ __launch_bounds__(256, 1) void k_dist_mfma_sym_u8(const v4i *__restrict__ Pa, const int *__restrict__ na,
                                                             const v4i *__restrict__ Pb,
                                                             unsigned long long *__restrict__ key, uint32_t N,
                                                             uint32_t B, uint32_t num_rot, uint32_t use_flip,
                                                             uint32_t RTP, uint32_t groups)
{
    constexpr int FRAG_V = KS * 64;                        // 16-byte vectors of fragments per unit
    constexpr int UNIT_V = FRAG_V + 64;                    // ... plus 8 x 32 norm entries (in memory)
    constexpr int PER_T = KS / 4;                          // fragment vectors per thread
    constexpr int H = KS / 2, W0 = KS / 4;                 // k-steps of the barrier / the first LDS store
    extern __shared__ v4i s_b[];                           // 3 x FRAG_V
    __shared__ int s_n[4][256];                            // norm entries of units u % 4: [symmetry][row]
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t col = lane & 31, half = lane >> 5;
    const uint32_t slice = blockIdx.x / groups, grp = blockIdx.x % groups;
    const uint32_t ct0 = (slice * 4 + wave) * 2;           // first of this wave's two column tiles
    const uint32_t nrr = num_rot / 4;
    const uint32_t sym = col & 7;                          // same for both column tiles

    const bool sym_ok = (num_rot != 1 || (sym & 3) == 0) && (use_flip || (sym & 4) == 0);

    // A wave whose two column tiles lie beyond the last neuron (the SOM's rows are padded to a whole
    // number of blocks) has nothing to multiply: it only does its share of the staging, in step with
    // the others through the block's barriers, and leaves the matrix pipe (and its power) alone.
    // (A path of its own from the first instruction on, so that it shares no live values with the
    // multiplying path, whose register allocation has no room to spare.)
    if (__builtin_amdgcn_readfirstlane((int)(ct0 * 32 >= 8 * N))) {
        const uint32_t images = grp < B ? (B - grp + groups - 1) / groups : 0;
        const uint32_t units = images * RTP;
        if (units == 0) return;
        const v4i *from = Pb + (size_t)grp * RTP * UNIT_V + tid;
        const size_t stride = (size_t)groups * RTP * UNIT_V;
        uint32_t from_rt = 0, from_u = 0;
        auto advance = [&]() {
            ++from_u;
            if (++from_rt == RTP) { from_rt = 0; from += stride - (size_t)(RTP - 1) * UNIT_V; }
            else from += UNIT_V;
        };
        v4i held[PER_T];
        int held_n;
#pragma unroll
        for (int i = 0; i < PER_T; ++i) held[i] = from[256 * i];
        held_n = ((const int *)(from - tid + FRAG_V))[tid];
#pragma unroll
        for (int i = 0; i < PER_T; ++i) s_b[tid + 256 * i] = held[i];
        s_n[0][tid] = held_n;
        if (units > 1) advance();
#pragma unroll
        for (int i = 0; i < PER_T; ++i) held[i] = from[256 * i];
        held_n = ((const int *)(from - tid + FRAG_V))[tid];
        if (units > 2) advance();
        __syncthreads();
        uint32_t o_cur = 0, o_next = FRAG_V, o_free = 2 * FRAG_V;
        for (uint32_t u = 0; u < units; ++u) {
            v4i *dst = s_b + o_next + tid;
#pragma unroll
            for (int i = 0; i < PER_T; ++i) dst[256 * i] = held[i];
            s_n[(u + 1) & 3][tid] = held_n;
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
            for (int i = 0; i < PER_T; ++i) held[i] = from[256 * i];
            held_n = ((const int *)(from - tid + FRAG_V))[tid];
            if (from_u + 1 < units) advance();
            const uint32_t o = o_cur;
            o_cur = o_next; o_next = o_free; o_free = o;
        }
        return;
    }

    // The block's units: u -> image grp + (u / RTP) * groups, tile u % RTP.
    const uint32_t my_images = grp < B ? (B - grp + groups - 1) / groups : 0;
    const uint32_t nunits = my_images * RTP;
    if (nunits == 0) return;
    // source of the next unit to load, advanced without divisions
    const v4i *src = Pb + (size_t)grp * RTP * UNIT_V + tid;
    const size_t image_stride = (size_t)groups * RTP * UNIT_V;
    uint32_t src_rt = 0, src_u = 0;
    auto advance_src = [&]() {
        ++src_u;
        if (++src_rt == RTP) { src_rt = 0; src += image_stride - (size_t)(RTP - 1) * UNIT_V; }
        else src += UNIT_V;
    };
    v4i stage[PER_T];
    int stage_n;
    // unit 0 -> buffer 0, unit 1 -> staging registers
#pragma unroll
    for (int i = 0; i < PER_T; ++i) stage[i] = src[256 * i];
    stage_n = ((const int *)(src - tid + FRAG_V))[tid];
#pragma unroll
    for (int i = 0; i < PER_T; ++i) s_b[tid + 256 * i] = stage[i];
    s_n[0][tid] = stage_n;
    if (nunits > 1) advance_src();
#pragma unroll
    for (int i = 0; i < PER_T; ++i) stage[i] = src[256 * i];
    stage_n = ((const int *)(src - tid + FRAG_V))[tid];
    if (nunits > 2) advance_src();
    __syncthreads();


    // SOM-side fragments for the whole k range, and the row norms of this lane's two columns
    v4i a[2][KS];
    int na_l[2];
    uint32_t n_l[2];
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) a[ct][ks] = Pa[((size_t)(ct0 + ct) * KS + ks) * 64 + lane];
        na_l[ct] = na[(ct0 + ct) * 32 + col];
        n_l[ct] = ((ct0 + ct) * 32 + col) >> 3;
    }
    // pin the fragments to accumulation registers for the whole kernel: without this the compiler
    // prefers to re-load them from memory for every row tile
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+a"(a[ct][ks]));

    // maximum over the 16 lanes that hold one neuron: the 8 symmetry lanes (two quad exchanges and
    // a mirror of the half row, all in the data-parallel path) and the other half-wave (v_permlane32_swap:
    // no trip through LDS)
    auto max16 = [&](int v) -> int {
        v = max(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false));    // lane ^ 1
        v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false));    // lane ^ 2
        v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, false));   // 7 - lane in the half row
        // the other half-wave: one swap of the upper half of one copy with the lower half of another
        // leaves the lower half's value in all lanes of the first and the upper half's in the second
        const auto halves = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);
        return max((int)halves[0], (int)halves[1]);
    };

    // Bookkeeping.  The unit's norm entry of row j of this lane is  cj = (15 - j) - 16 |b_row|^2, so
    //   cand = 32 acc_j + cj = 16 (|a|^2 - ssd_j) + (15 - j)       (|a|^2 = this column's norm)
    // and the running signed maximum `m` of cand over the rows of a tile is the tile's minimum
    // distance with the lowest row on ties.  Tiles ascend in rotation, so a later tile replaces the
    // image's best so far (`best_m`, from tile `m_rt`) only with a strictly smaller distance: the
    // comparison leaves the row bits out.  16 ssd < 2^30 (checked on the host); rows beyond the last
    // base rotation carry |b|^2 = 2^26 and never win.
    int m[2] = {INT_MIN, INT_MIN}, best_m[2] = {INT_MIN, INT_MIN};
    uint32_t m_rt[2] = {0, 0};
    auto close_tile = [&](uint32_t rt) {
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) {
            if (rt == 0 || (m[ct] >> 4) > (best_m[ct] >> 4)) { best_m[ct] = m[ct]; m_rt[ct] = rt; }
            m[ct] = INT_MIN;
        }
    };
    uint32_t bk_rt = 0, bk_img = grp;                      // tile and image of the unit whose bookkeeping ends next
    auto finish_image = [&](uint32_t b) {
        // lexicographic minimum of (distance, variant) over the neuron's 16 lanes in two passes
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) {
            const uint32_t j = 15u - ((uint32_t)best_m[ct] & 15u);
            const int ssd = na_l[ct] - (best_m[ct] >> 4);
            const uint32_t i = m_rt[ct] * 32 + 8 * (j >> 2) + 4 * half + (j & 3);
            const uint32_t k = (sym >> 2) * num_rot + (sym & 3) * nrr + i;
            const int sv = sym_ok ? -ssd : INT_MIN;
            const int smax = max16(sv);
            const int kmax = max16(sv == smax ? -(int)k : INT_MIN);
            if (half == 0 && sym == 0 && n_l[ct] < N)
                key[(size_t)b * N + n_l[ct]] = ((unsigned long long)(uint32_t)(-smax) << 16) | (uint32_t)(-kmax);
        }
    };
    // this lane's 16 norm entries of unit u: rows 8g + 4*half .. +3, g = 0..3
    auto read_cj = [&](uint32_t u, int (&cj)[16]) {
        const v4i *nbt = (const v4i *)(&s_n[u & 3][sym * 32 + 4 * half]);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const v4i t = nbt[2 * g];
            cj[4 * g + 0] = t[0]; cj[4 * g + 1] = t[1]; cj[4 * g + 2] = t[2]; cj[4 * g + 3] = t[3];
        }
    };

    // LDS offsets (in vectors) of the buffers holding units u, u+1, u+2
    uint32_t off_cur = 0, off_next = FRAG_V, off_free = 2 * FRAG_V;

    v4i bf[4];
#pragma unroll
    for (int ks = 0; ks < 3 && ks < KS; ++ks) bf[ks] = s_b[ks * 64 + lane];

    // One unit, hand-scheduled per k-step (nothing crosses the scheduling barriers): the LDS read
    // of the fragment three k-steps ahead (running on into the next unit's buffer), two MFMAs of
    // unit u into `acc`, and a slice of the other work: one (column, row) pair of unit u-1's
    // bookkeeping from `acc_prev` / `cj_prev`, the staging registers (unit u+1) to the next buffer,
    // the barrier, the loads of unit u+2, and this unit's own norm entries for the next round.
    auto run_unit = [&](uint32_t u, v16i (&acc)[2], int (&cj)[16], const v16i (&acc_prev)[2], const int (&cj_prev)[16]) {
        const v4i *cur = s_b + off_cur + lane, *nxt = s_b + off_next + lane;
        v4i *dst = s_b + off_next + tid;
        const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        // The 32 (column, row) pairs of unit u-1: shift and add of the norm entry, one pair per slot, and
        // a three-way maximum for every two pairs of a column, two slots behind (a lone wave issues an
        // instruction only every other turn of its SIMD, so every instruction between two MFMAs counts:
        // one accumulation chain per column tile and v_max3 keep it at three quarters of an instruction
        // per MFMA).
        uint32_t cand[4];
        auto book = [&](int s0, int s1) {
#pragma unroll
            for (int sl = s0; sl < s1; ++sl) {
                if (sl >= 2 && sl < 34 && (sl & 1) == 0) {
                    const int e = sl - 2, ct = (e >> 2) & 1;
                    m[ct] = max(max(m[ct], (int)cand[e & 3]), (int)cand[(e + 1) & 3]);
                }
                if (sl < 32) {
                    const int e = sl, ct = (e >> 2) & 1, j = 4 * (e >> 3) + (e & 3);
                    cand[e & 3] = ((uint32_t)acc_prev[ct][j] << 5) + (uint32_t)cj_prev[j];
                }
            }
            // pins the slot where it stands
            asm volatile("" : "+v"(m[0]), "+v"(m[1]), "+v"(cand[0]), "+v"(cand[1]), "+v"(cand[2]), "+v"(cand[3]));
        };
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (ks == H) {
                // every wave has stored its part of unit u+1 (k-steps W0 .. H-1): wait for this wave's
                // LDS operations, then meet the others
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            }
            bf[(ks + 3) & 3] = ks + 3 < KS ? cur[(ks + 3) * 64] : nxt[(ks + 3 - KS) * 64];
            acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[ks & 3], a[0][ks], ks > 0 ? acc[0] : zero, 0, 0, 0);
            book((2 * ks) * 17 / KS, (2 * ks + 1) * 17 / KS);
            __builtin_amdgcn_sched_barrier(0);
            acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[ks & 3], a[1][ks], ks > 0 ? acc[1] : zero, 0, 0, 0);
            book((2 * ks + 1) * 17 / KS, (2 * ks + 2) * 17 / KS);
            // (past the last unit the staging moves data nobody reads: no branches in the k loop)
            if (ks >= W0 && ks < W0 + PER_T) dst[256 * (ks - W0)] = stage[ks - W0];
            if (ks == W0) s_n[(u + 1) & 3][tid] = stage_n;
            if (ks >= H && ks < H + PER_T) stage[ks - H] = src[256 * (ks - H)];
            if (ks == H) stage_n = ((const int *)(src - tid + FRAG_V))[tid];
            if (ks == KS - 2) read_cj(u, cj);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (src_u + 1 < nunits) advance_src();
        if (u > 0) {
            // (unit u - 1 = image bk_img, tile bk_rt: counted along, a division per unit costs more
            // than the rest of this epilogue)
            close_tile(bk_rt);
            if (++bk_rt == RTP) { finish_image(bk_img); bk_img += groups; bk_rt = 0; }
        } else {
            m[0] = m[1] = INT_MIN;                           // there was no unit before the first
        }
        const uint32_t o = off_cur;
        off_cur = off_next; off_next = off_free; off_free = o;
    };

    // two accumulator sets (units alternate), each two columns; the two columns' MFMAs alternate, so a
    // column's next MFMA finds the one before it finished
    v16i acc0[2], acc1[2];
    int cj0[16], cj1[16];
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc1[ct][j] = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) cj1[j] = 0;
    for (uint32_t u = 0; u < nunits; u += 2) {
        run_unit(u, acc0, cj0, acc1, cj1);
        if (u + 1 < nunits) run_unit(u + 1, acc1, cj1, acc0, cj0);
    }
    {
        // the last unit's bookkeeping
        const uint32_t u = nunits - 1;
#pragma unroll
        for (int j = 0; j < 16; ++j)
#pragma unroll
            for (int ct = 0; ct < 2; ++ct) {
                const int av = (u & 1) ? acc1[ct][j] : acc0[ct][j];
                const int cv = (u & 1) ? cj1[j] : cj0[j];
                m[ct] = max(m[ct], (int)(((uint32_t)av << 5) + (uint32_t)cv));
            }
        close_tile(bk_rt);
        finish_image(bk_img);                                // units end with the last tile of an image
    }
}

// The same for unions of up to 2048 elements (KS = 40 .. 64 k-steps): a wave's accumulation registers
// hold ONE column tile over the whole k range (4 neurons x 8 symmetries), a block 4 tiles; a unit is
// up to 64 KiB, so two LDS buffers take turns and a unit has two barriers: the first, early in
// the k loop, says that every wave has left the previous unit (whose buffer then receives unit u+1 from
// the staging registers), the second that those stores have landed (the fragment reads run on into the
// next buffer at the end of the k loop).  One MFMA per k-step and fragment read, two chains (even /
// odd k-steps); bookkeeping, half-wave exchange and keys as above.
template <int KS>
__global__ __launch_bounds__(256, 1) void k_dist_mfma_sym_u8_wide(const v4i *__restrict__ Pa, const int *__restrict__ na,
                                                                  const v4i *__restrict__ Pb,
                                                                  unsigned long long *__restrict__ key, uint32_t N,
                                                                  uint32_t B, uint32_t num_rot, uint32_t use_flip,
                                                                  uint32_t RTP, uint32_t groups)
{
    constexpr int FRAG_V = KS * 64;
    constexpr int UNIT_V = FRAG_V + 64;
    constexpr int PER_T = KS / 4;
    constexpr int W0 = 2, H2 = W0 + PER_T + 2, L0 = H2;    // first barrier and stores / second barrier / loads
    static_assert(KS % 8 == 0 && L0 + PER_T <= KS - 3, "k loop too short for the staging schedule");
    extern __shared__ v4i s_b[];                           // 2 x FRAG_V
    __shared__ int s_n[4][256];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t col = lane & 31, half = lane >> 5;
    const uint32_t slice = blockIdx.x / groups, grp = blockIdx.x % groups;
    const uint32_t ct = slice * 4 + wave;                  // this wave's column tile
    const uint32_t nrr = num_rot / 4;
    const uint32_t sym = col & 7;
    const bool sym_ok = (num_rot != 1 || (sym & 3) == 0) && (use_flip || (sym & 4) == 0);

    // a wave whose column tile lies beyond the last neuron only takes part in the staging (a path of
    // its own from here on, sharing no live values with the multiplying path)
    if (__builtin_amdgcn_readfirstlane((int)(ct * 32 >= 8 * N))) {
        const uint32_t images = grp < B ? (B - grp + groups - 1) / groups : 0;
        const uint32_t units = images * RTP;
        if (units == 0) return;
        const v4i *from = Pb + (size_t)grp * RTP * UNIT_V + tid;
        const size_t stride = (size_t)groups * RTP * UNIT_V;
        uint32_t from_rt = 0, from_u = 0;
        auto advance = [&]() {
            ++from_u;
            if (++from_rt == RTP) { from_rt = 0; from += stride - (size_t)(RTP - 1) * UNIT_V; }
            else from += UNIT_V;
        };
        v4i held[PER_T];
        int held_n;
#pragma unroll
        for (int i = 0; i < PER_T; ++i) held[i] = from[256 * i];
        held_n = ((const int *)(from - tid + FRAG_V))[tid];
#pragma unroll
        for (int i = 0; i < PER_T; ++i) s_b[tid + 256 * i] = held[i];
        s_n[0][tid] = held_n;
        if (units > 1) advance();
#pragma unroll
        for (int i = 0; i < PER_T; ++i) held[i] = from[256 * i];
        held_n = ((const int *)(from - tid + FRAG_V))[tid];
        if (units > 2) advance();
        __syncthreads();
        uint32_t o_cur = 0, o_next = FRAG_V;
        for (uint32_t u = 0; u < units; ++u) {
            asm volatile("s_barrier" ::: "memory");
            v4i *dst = s_b + o_next + tid;
#pragma unroll
            for (int i = 0; i < PER_T; ++i) dst[256 * i] = held[i];
            s_n[(u + 1) & 3][tid] = held_n;
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
            for (int i = 0; i < PER_T; ++i) held[i] = from[256 * i];
            held_n = ((const int *)(from - tid + FRAG_V))[tid];
            if (from_u + 1 < units) advance();
            const uint32_t o = o_cur;
            o_cur = o_next; o_next = o;
        }
        return;
    }

    const uint32_t my_images = grp < B ? (B - grp + groups - 1) / groups : 0;
    const uint32_t nunits = my_images * RTP;
    if (nunits == 0) return;
    const v4i *src = Pb + (size_t)grp * RTP * UNIT_V + tid;
    const size_t image_stride = (size_t)groups * RTP * UNIT_V;
    uint32_t src_rt = 0, src_u = 0;
    auto advance_src = [&]() {
        ++src_u;
        if (++src_rt == RTP) { src_rt = 0; src += image_stride - (size_t)(RTP - 1) * UNIT_V; }
        else src += UNIT_V;
    };
    v4i stage[PER_T];
    int stage_n;
#pragma unroll
    for (int i = 0; i < PER_T; ++i) stage[i] = src[256 * i];
    stage_n = ((const int *)(src - tid + FRAG_V))[tid];
#pragma unroll
    for (int i = 0; i < PER_T; ++i) s_b[tid + 256 * i] = stage[i];
    s_n[0][tid] = stage_n;
    if (nunits > 1) advance_src();
#pragma unroll
    for (int i = 0; i < PER_T; ++i) stage[i] = src[256 * i];
    stage_n = ((const int *)(src - tid + FRAG_V))[tid];
    if (nunits > 2) advance_src();
    __syncthreads();
    uint32_t off_cur = 0, off_next = FRAG_V;


    v4i a[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) a[ks] = Pa[((size_t)ct * KS + ks) * 64 + lane];
    const int na_l = na[ct * 32 + col];
    const uint32_t n_l = (ct * 32 + col) >> 3;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+a"(a[ks]));

    auto max16 = [&](int v) -> int {
        v = max(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false));
        v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false));
        v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, false));
        const auto halves = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);
        return max((int)halves[0], (int)halves[1]);
    };
    int m = INT_MIN, best_m = INT_MIN;
    uint32_t m_rt = 0;
    uint32_t bk_rt = 0, bk_img = grp;
    auto close_tile = [&](uint32_t rt) {
        if (rt == 0 || (m >> 4) > (best_m >> 4)) { best_m = m; m_rt = rt; }
        m = INT_MIN;
    };
    auto finish_image = [&](uint32_t b) {
        const uint32_t j = 15u - ((uint32_t)best_m & 15u);
        const int ssd = na_l - (best_m >> 4);
        const uint32_t i = m_rt * 32 + 8 * (j >> 2) + 4 * half + (j & 3);
        const uint32_t k = (sym >> 2) * num_rot + (sym & 3) * nrr + i;
        const int sv = sym_ok ? -ssd : INT_MIN;
        const int smax = max16(sv);
        const int kmax = max16(sv == smax ? -(int)k : INT_MIN);
        if (half == 0 && sym == 0 && n_l < N)
            key[(size_t)b * N + n_l] = ((unsigned long long)(uint32_t)(-smax) << 16) | (uint32_t)(-kmax);
    };
    auto read_cj = [&](uint32_t u, int (&cj)[16]) {
        const v4i *nbt = (const v4i *)(&s_n[u & 3][sym * 32 + 4 * half]);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const v4i t = nbt[2 * g];
            cj[4 * g + 0] = t[0]; cj[4 * g + 1] = t[1]; cj[4 * g + 2] = t[2]; cj[4 * g + 3] = t[3];
        }
    };

    v4i bf[4];
#pragma unroll
    for (int ks = 0; ks < 3; ++ks) bf[ks] = s_b[ks * 64 + lane];

    auto run_unit = [&](uint32_t u, v16i (&acc)[2], int (&cj)[16], const v16i (&acc_prev)[2], const int (&cj_prev)[16]) {
        const v4i *cur = s_b + off_cur + lane, *nxt = s_b + off_next + lane;
        v4i *dst = s_b + off_next + tid;
        const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        // the 16 rows of unit u-1 in three steps, one row behind the other (see the kernel above)
        uint32_t pair_sum[2], pair_cand[2];
        auto book = [&](int s0, int s1) {
#pragma unroll
            for (int sl = s0; sl < s1; ++sl) {
                if (sl >= 2 && sl < 18) m = max(m, (int)pair_cand[sl & 1]);
                if (sl >= 1 && sl < 17) pair_cand[(sl - 1) & 1] = (pair_sum[(sl - 1) & 1] << 5) + (uint32_t)cj_prev[sl - 1];
                if (sl < 16) pair_sum[sl & 1] = (uint32_t)(acc_prev[0][sl] + acc_prev[1][sl]);
            }
            asm volatile("" : "+v"(m), "+v"(pair_sum[0]), "+v"(pair_sum[1]), "+v"(pair_cand[0]), "+v"(pair_cand[1]));
        };
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (ks == W0) asm volatile("s_barrier" ::: "memory");          // every wave has left unit u-1
            if (ks == H2) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");   // unit u+1 is in LDS
            bf[(ks + 3) & 3] = ks + 3 < KS ? cur[(ks + 3) * 64] : nxt[(ks + 3 - KS) * 64];
            acc[ks & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[ks & 3], a[ks], ks > 1 ? acc[ks & 1] : zero, 0, 0, 0);
            book(ks * 18 / KS, (ks + 1) * 18 / KS);
            if (ks >= W0 && ks < W0 + PER_T) dst[256 * (ks - W0)] = stage[ks - W0];
            if (ks == W0) s_n[(u + 1) & 3][tid] = stage_n;
            if (ks >= L0 && ks < L0 + PER_T) stage[ks - L0] = src[256 * (ks - L0)];
            if (ks == L0) stage_n = ((const int *)(src - tid + FRAG_V))[tid];
            if (ks == KS - 2) read_cj(u, cj);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (src_u + 1 < nunits) advance_src();
        if (u > 0) {
            close_tile(bk_rt);
            if (++bk_rt == RTP) { finish_image(bk_img); bk_img += groups; bk_rt = 0; }
        } else {
            m = INT_MIN;
        }
        const uint32_t o = off_cur;
        off_cur = off_next; off_next = o;
    };

    v16i acc0[2], acc1[2];
    int cj0[16], cj1[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) { acc1[0][j] = acc1[1][j] = 0; cj1[j] = 0; }
    for (uint32_t u = 0; u < nunits; u += 2) {
        run_unit(u, acc0, cj0, acc1, cj1);
        if (u + 1 < nunits) run_unit(u + 1, acc1, cj1, acc0, cj0);
    }
    {
        const uint32_t u = nunits - 1;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int av = (u & 1) ? acc1[0][j] + acc1[1][j] : acc0[0][j] + acc0[1][j];
            const int cv = (u & 1) ? cj1[j] : cj0[j];
            m = max(m, (int)(((uint32_t)av << 5) + (uint32_t)cv));
        }
        close_tile(bk_rt);
        finish_image(bk_img);
    }
}

template <int KS>
hipError_t launch_dist(hipStream_t stream, const pink_sym::DistArgs &g, bool configure_only)
{
    const int lds = 3 * KS * 64 * 16;
    if (configure_only)
        return hipFuncSetAttribute((const void *)k_dist_mfma_sym_u8<KS>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    hipLaunchKernelGGL((k_dist_mfma_sym_u8<KS>), dim3(g.slices * g.groups), dim3(256), lds, stream, (const v4i *)g.Pa, g.na,
                       (const v4i *)g.Pb, g.key, g.N, g.B, g.num_rot, g.use_flip, g.RTP, g.groups);
    return hipGetLastError();
}

template <int KS>
hipError_t launch_dist_wide(hipStream_t stream, const pink_sym::DistArgs &g, bool configure_only)
{
    const int lds = 2 * KS * 64 * 16;
    if (configure_only)
        return hipFuncSetAttribute((const void *)k_dist_mfma_sym_u8_wide<KS>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    hipLaunchKernelGGL((k_dist_mfma_sym_u8_wide<KS>), dim3(g.slices * g.groups), dim3(256), lds, stream, (const v4i *)g.Pa,
                       g.na, (const v4i *)g.Pb, g.key, g.N, g.B, g.num_rot, g.use_flip, g.RTP, g.groups);
    return hipGetLastError();
}

hipError_t dispatch_dist(hipStream_t stream, const pink_sym::DistArgs &g, bool configure_only)
{
    switch (g.KS) {
    case 8: return launch_dist<8>(stream, g, configure_only);
    case 16: return launch_dist<16>(stream, g, configure_only);
    case 24: return launch_dist<24>(stream, g, configure_only);
    case 32: return launch_dist<32>(stream, g, configure_only);
    case 40: return launch_dist_wide<40>(stream, g, configure_only);
    case 48: return launch_dist_wide<48>(stream, g, configure_only);
    case 56: return launch_dist_wide<56>(stream, g, configure_only);
    case 64: return launch_dist_wide<64>(stream, g, configure_only);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

namespace pink_sym {

size_t unit_bytes(uint32_t KS) { return ((size_t)KS * 64 + 64) * 16; }

hipError_t pack_som(hipStream_t stream, const float *som, const uint32_t *aoff, signed char *Pa, int *na, uint32_t N,
                    uint32_t S, uint32_t KS, uint32_t rows)
{
    hipLaunchKernelGGL(k_pack_som_sym_u8, dim3(rows), dim3(256), 0, stream, som, aoff, Pa, na, N, S, KS);
    return hipGetLastError();
}

size_t lds_image_bytes(uint32_t C, uint32_t I) { return (size_t)C * (I + 1) * row_stride(I) * sizeof(float); }

// images per block of the rotation kernel: as many as let two blocks share a CU's LDS (one loads
// its images while the other computes), next to their norm counters
uint32_t images_per_block(size_t image_bytes)
{
    const size_t budget = 76 * 1024;                      // two blocks and their counters within 160 KiB
    return image_bytes * 4 <= budget ? 4 : image_bytes * 2 <= budget ? 2 : 1;
}

template <int G>
hipError_t launch_rotpack(hipStream_t stream, const RotpackArgs &g, bool configure_only)
{
    const size_t lds = (size_t)G * lds_image_bytes(g.C, g.I);
    // (the limit is per kernel, not per context: the most that any context may ask of this instantiation)
    if (configure_only)
        return hipFuncSetAttribute((const void *)k_rotpack_sym_u8<G>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   G == 1 ? 150 * 1024 : 76 * 1024);
    const uint32_t groups = (g.B + G - 1) / G;
    const uint32_t blocks = ((groups + 7) / 8) * 8 * g.RTP;           // 8 groups per span of ids, see the kernel
    hipLaunchKernelGGL(k_rotpack_sym_u8<G>, dim3(blocks), dim3(G >= 4 ? 512 : 256), lds, stream, g.images, (v4i *)g.Pb, g.tab_idx,
                       (const float4 *)g.tab_w, g.kmask, g.Ku, g.all_sym, g.C, g.I, g.nrr_eff, g.KS, g.RTP, g.B,
                       row_stride(g.I));
    return hipGetLastError();
}

hipError_t dispatch_rotpack(hipStream_t stream, const RotpackArgs &g, bool configure_only)
{
    switch (images_per_block(lds_image_bytes(g.C, g.I))) {
    case 4: return launch_rotpack<4>(stream, g, configure_only);
    case 2: return launch_rotpack<2>(stream, g, configure_only);
    default: return launch_rotpack<1>(stream, g, configure_only);
    }
}

hipError_t configure(uint32_t KS, uint32_t C, uint32_t I)
{
    RotpackArgs r{};
    r.C = C; r.I = I;
    hipError_t e = dispatch_rotpack(nullptr, r, true);
    if (e != hipSuccess) return e;
    DistArgs g{};
    g.KS = KS;
    return dispatch_dist(nullptr, g, true);
}

size_t rot_table_bytes(uint32_t KS, uint32_t RTP) { return (size_t)RTP * 32 * KS * 32 * (sizeof(uint32_t) + sizeof(float4)); }

hipError_t build_rot_table(hipStream_t stream, const float *cos_t, const float *sin_t, const uint32_t *upos, uint32_t Ku,
                           uint32_t I, uint32_t D, uint32_t nrr_eff, uint32_t KS, uint32_t RTP, void *table)
{
    const uint32_t rows = RTP * 32, Kp = KS * 32;
    float4 *tab_w = (float4 *)table;                                   // weights first: 16-byte aligned
    uint32_t *tab_idx = (uint32_t *)(tab_w + (size_t)rows * Kp);
    hipLaunchKernelGGL(k_rot_table, dim3((rows * Kp + 255) / 256), dim3(256), 0, stream, cos_t, sin_t, upos, Ku, I, D, nrr_eff,
                       Kp, rows, row_stride(I), tab_idx, tab_w);
    return hipGetLastError();
}

hipError_t rotpack(hipStream_t stream, const RotpackArgs &g) { return dispatch_rotpack(stream, g, false); }

hipError_t dist(hipStream_t stream, const DistArgs &g) { return dispatch_dist(stream, g, false); }

}  // namespace pink_sym

// Launchers of the uint8 mapping kernels that keep the SOM operand resident in registers
// (mfma_u8_sym.hip).  Host-side interface only: plain pointers, one call per kernel launch.
#ifndef PINK_AMD_MFMA_U8_SYM_H
#define PINK_AMD_MFMA_U8_SYM_H

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace pink_sym {

// Once per context: allow the rotation kernel its LDS image (C x (I+1) x (I+1) floats) and the
// distance kernel of this KS (8, 16, 24 or 32 k-steps) its three LDS buffers.
hipError_t configure(uint32_t KS, size_t lds_image_bytes);

// Bytes of one unit of the image operand: one row tile of 32 base rotations = KS fragments of
// 1 KiB, followed by 1 KiB of norm entries [8 symmetries][32 rows].
size_t unit_bytes(uint32_t KS);

// SOM operand, `rows` = padded number of (neuron, symmetry) rows, a multiple of 32.
hipError_t pack_som(hipStream_t stream, const float *som, const uint32_t *aoff, signed char *Pa, int *na, uint32_t N,
                    uint32_t S, uint32_t KS, uint32_t rows);

struct RotpackArgs {
    const float *images;        // B x C x I x I
    void *Pb;                   // B x RTP units
    const float *cos_t, *sin_t;
    const uint32_t *upos;
    const unsigned char *kmask;
    uint32_t Ku, all_sym, C, I, nrr_eff, D, KS, RTP, B;
};
hipError_t rotpack(hipStream_t stream, const RotpackArgs &args);

struct DistArgs {
    const void *Pa;             // SOM fragments
    const int *na;              // SOM row norms
    const void *Pb;             // image units
    unsigned long long *key;    // B x N
    uint32_t N, B, num_rot, use_flip, RTP, KS, slices, groups;
};
hipError_t dist(hipStream_t stream, const DistArgs &args);

}  // namespace pink_sym

#endif

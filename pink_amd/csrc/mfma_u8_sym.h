// Launchers of the uint8 mapping kernels that keep the SOM operand resident in registers
// (mfma_u8_sym.hip).  Host-side interface only: plain pointers, one call per kernel launch.
#ifndef PINK_AMD_MFMA_U8_SYM_H
#define PINK_AMD_MFMA_U8_SYM_H

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace pink_sym {

// LDS bytes of one image in the rotation kernel (padded rows).
size_t lds_image_bytes(uint32_t C, uint32_t I);

// Once per context: allow the rotation kernel its LDS images (lds_image_bytes each) and the
// distance kernel of this KS (8, 16, 24 or 32 k-steps) its three LDS buffers.
hipError_t configure(uint32_t KS, uint32_t C, uint32_t I);

// The geometry of the base rotations (source offset and bilinear weights per rotation and union
// position), built once per context into `table` (rot_table_bytes() bytes of device memory).
size_t rot_table_bytes(uint32_t KS, uint32_t RTP);
hipError_t build_rot_table(hipStream_t stream, const float *cos_t, const float *sin_t, const uint32_t *upos, uint32_t Ku,
                           uint32_t I, uint32_t D, uint32_t nrr_eff, uint32_t KS, uint32_t RTP, void *table);

// Bytes of one unit of the image operand: one row tile of 32 base rotations = KS fragments of
// 1 KiB, followed by 1 KiB of norm entries [8 symmetries][32 rows].
size_t unit_bytes(uint32_t KS);

// SOM operand, `rows` = padded number of (neuron, symmetry) rows, a multiple of 32.
hipError_t pack_som(hipStream_t stream, const float *som, const uint32_t *aoff, signed char *Pa, int *na, uint32_t N,
                    uint32_t S, uint32_t KS, uint32_t rows);

struct RotpackArgs {
    const float *images;        // B x C x I x I
    void *Pb;                   // B x RTP units
    const uint32_t *tab_idx;    // table built by build_rot_table: offsets ...
    const void *tab_w;          // ... and weights
    const unsigned char *kmask;
    uint32_t Ku, all_sym, C, I, nrr_eff, KS, RTP, B;
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

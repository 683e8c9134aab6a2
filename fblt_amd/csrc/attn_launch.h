/* Host-side launch functions of the attention kernel families. */
#ifndef FBLT_AMD_ATTN_LAUNCH_H
#define FBLT_AMD_ATTN_LAUNCH_H

#include "attn_device.h"

#include <vector>

/* Upper bound of head_dim the rows family takes (64 lanes x 16 float4). */
#define ATTN_ROWS_MAX_HEAD_DIM 4096u

/* One work item of the mfma family: 32 query rows of one problem. */
struct AttnTile {
    uint32_t prob;  /* index into the device descriptor array */
    uint32_t qtile; /* rows [32*qtile, 32*qtile+32)            */
};

/* A batch whose problems differ from the first one only by (sequence, head)
 * strides: problem i = seq * heads + head.  Travels in the kernel arguments,
 * so a launch needs no descriptor memory at all.  Strides are in elements. */
struct AttnAffine {
    AttnProb first;
    int64_t q_seq, q_head, k_seq, k_head, v_seq, v_head, o_seq, o_head;
    int64_t w_seq, w_head, lse_seq, lse_head, mask_seq, mask_head, range_seq, range_head;
    uint32_t count; /* problems                       */
    uint32_t heads; /* problems per sequence          */
    uint32_t nqt;   /* 32-row query tiles per problem */
    uint32_t reserved;
};

/* rows family: problems [base, base+count) of a device array share head_dim hd */
void attn_rows_launch(const AttnProb *dprobs, uint32_t base, uint32_t count, uint32_t hd, uint32_t max_nq,
                      hipStream_t s);
/* one problem, descriptor passed as a kernel argument (nothing staged) */
void attn_rows_launch_single(const AttnProb &single, hipStream_t s);
/* a strided batch, descriptors in the kernel arguments (declared below the AttnAffine struct) */

void attn_rows_launch_affine(const AttnAffine &aff, hipStream_t s);

/* mfma family */
bool attn_mfma_can(const AttnProb &d);
bool attn_mfma_takes(const AttnProb &d);
void attn_mfma_make_tiles(const AttnProb *host, uint32_t base, uint32_t count, std::vector<AttnTile> &tiles);
void attn_mfma_launch(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t ntiles, uint32_t hd, bool vec4,
                      bool dense, hipStream_t s);
void attn_mfma_launch_single(const AttnProb &single, hipStream_t s);
void attn_mfma_launch_affine(const AttnAffine &aff, hipStream_t s);

/* wide family: work items are 128-row groups or pairs of them (AttnTile.qtile
 * = two 16-bit group indices) */
bool attn_wide_can(const AttnProb &d);
uint32_t attn_wide_groups(const AttnProb &d);
void attn_wide_make_tiles(const AttnProb *host, uint32_t base, uint32_t count, std::vector<AttnTile> &tiles);
void attn_wide_launch(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t ntiles, uint32_t hd, bool dense,
                      hipStream_t s);
void attn_wide_launch_single(const AttnProb &single, hipStream_t s);
void attn_wide_launch_affine(const AttnAffine &aff, hipStream_t s);

/* fine family: 32-row tiles cut into 16 x 16 units over eight waves, K/V rows of a tile shared
 * through LDS; `span` = keys the longest tile of the launch needs */
bool attn_fine_can(const AttnProb &d);
uint32_t attn_fine_span(const AttnProb &d);
uint32_t attn_fine_fill_max(uint32_t hd);
void attn_fine_make_tiles(const AttnProb *host, uint32_t base, uint32_t count, std::vector<AttnTile> &tiles);
void attn_fine_launch(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t ntiles, uint32_t hd, uint32_t span,
                      hipStream_t s);
/* tall: workgroups of one 16-row tile and sixteen waves instead of 32 rows and eight waves */
void attn_fine_launch_single(const AttnProb &single, bool tall, hipStream_t s);
void attn_fine_launch_affine(const AttnAffine &aff, bool tall, hipStream_t s);
/* whole short problems of a strided batch, one workgroup each (attn_fine.hip) */
bool attn_whole_can(const AttnProb &d);
void attn_whole_launch_affine(const AttnAffine &aff, hipStream_t s);

/* once family: 16-row tiles whose keys are all in flight at once, exact softmax, weights in the same
 * sweep (attn_once.hip) */
bool attn_once_can(const AttnProb &d);
uint32_t attn_once_tiles_max(uint32_t hd);
uint32_t attn_once_span_tiles(const AttnProb &d);
void attn_once_make_tiles(const AttnProb *host, uint32_t base, uint32_t count, std::vector<AttnTile> &tiles);
void attn_once_launch(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t ntiles, uint32_t hd, uint32_t span_tiles,
                      bool dense, hipStream_t s);
void attn_once_launch_single(const AttnProb &single, hipStream_t s);
void attn_once_launch_affine(const AttnAffine &aff, hipStream_t s);

#endif

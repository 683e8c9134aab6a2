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

/* rows family: problems [base, base+count) of a device array share head_dim hd */
void attn_rows_launch(const AttnProb *dprobs, uint32_t base, uint32_t count, uint32_t hd, uint32_t max_nq,
                      hipStream_t s);
/* one problem, descriptor passed as a kernel argument (nothing staged) */
void attn_rows_launch_single(const AttnProb &single, hipStream_t s);

/* mfma family */
bool attn_mfma_can(const AttnProb &d);
bool attn_mfma_takes(const AttnProb &d);
void attn_mfma_make_tiles(const AttnProb *host, uint32_t base, uint32_t count, std::vector<AttnTile> &tiles);
void attn_mfma_launch(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t ntiles, uint32_t hd, hipStream_t s);
void attn_mfma_launch_single(const AttnProb &single, hipStream_t s);

#endif

/*
 * sampler_host.h -- host-side interface of sampler_abi.hip for other translation units of this
 * package (not part of the C ABI under include/): a sampling call enqueued stage by stage.
 */
#ifndef GEIST_SAMPLER_HOST_H
#define GEIST_SAMPLER_HOST_H

#include "../../include/geist_sampler_hip.h"

namespace gs_host {

enum : unsigned {
    STAGE_STREAM = 2u, /* the pass that streams the logits */
    STAGE_TAIL   = 4u, /* what follows per row */
    STAGE_ALL    = 6u,
};

/* geist_hip_sample_rows restricted to the stages in `stages` (same checks, same geometry, same
 * choice of path). *stream_kernel, when given, receives the name of the kernel of STAGE_STREAM. */
int sample_stages(geist_hip_sampler *s, const struct geist_hip_rows *rows,
                  const struct geist_hip_sample_params *params, const float *d_uniforms,
                  geist_hip_token_t *d_out, unsigned stages, const char **stream_kernel);

} // namespace gs_host
#endif

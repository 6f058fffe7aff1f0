/*
 * geist_sampler_dropin.h -- the reference's sampler interface, served by the MI355X path.
 *
 * libgeist_sampler_host.so exports, with the reference's own names and signatures, every
 * symbol of src/engine/sampler.h (geistlib 0.9.0): linking it in place of the reference's
 * sampler.o leaves head.c, step.c, arch_state.c, spec_head.c and tests/test_sampler_unit.c
 * unchanged. The logit row a caller passes lives in host memory, as in the reference; it is
 * uploaded, sampled by the HIP kernels and only the 4-byte token id returns. There is no CPU
 * path behind these symbols: a missing or failing device goes to the failure handler below,
 * which by default ends the process with a message.
 *
 * Threads: every entry point may be called from any number of threads at once
 * (src/engine/sampler.h:8). A workspace belongs to one thread at a time, as in the reference;
 * geist_sampler_argmax / _temperature keep a device context per calling thread, made on the
 * thread's first call and given back when the thread ends.
 *
 * A translation unit that already includes the reference's <geist.h> / sampler.h must not
 * include this file (the declarations would repeat); it is for callers built without the
 * reference tree.
 */
#ifndef GEIST_SAMPLER_DROPIN_H
#define GEIST_SAMPLER_DROPIN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef GEIST_VERSION_MAJOR /* the reference's <geist.h> is not in this translation unit */
/* include/geist.h:190 */
typedef int32_t geist_token_t;
/* include/geist.h:46-67 (the values this path can return) */
enum geist_status {
    GEIST_OK            = 0,
    GEIST_E_OOM         = 1,
    GEIST_E_INVALID_ARG = 2,
    GEIST_E_INTERNAL    = 3,
    GEIST_E_UNSUPPORTED = 7,
    GEIST_E_BACKEND     = 9,
};
#endif

#ifndef GEIST_INTERNAL_SAMPLER_H /* the reference's sampler.h is not in this translation unit */
/* src/engine/sampler.h:28-32 */
struct geist_rng {
    uint64_t state;
};
/* src/engine/sampler.h:50-57. Here `probs` points at host memory of n_vocab floats, as in the
 * reference, and the device workspace hangs off a hidden header in front of it. Callers treat
 * both fields as opaque, as the reference's callers do. */
struct geist_sampler_workspace {
    float *probs;
    size_t n_vocab;
};

/* src/engine/sampler.h:34-36, sampler.c:27-48 */
void     geist_rng_seed(struct geist_rng *rng, uint64_t seed);
uint64_t geist_rng_next_u64(struct geist_rng *rng);
float    geist_rng_next_unit(struct geist_rng *rng);
/* src/engine/sampler.h:38-40, sampler.c:52-62 */
geist_token_t geist_sampler_argmax(size_t n_vocab, const float *logits);
/* src/engine/sampler.h:42-47, sampler.c:106-132 */
geist_token_t geist_sampler_temperature(size_t n_vocab, const float *logits, float temperature,
                                        struct geist_rng *rng);
/* src/engine/sampler.h:59-61, sampler.c:136-157 */
enum geist_status geist_sampler_workspace_init(struct geist_sampler_workspace *ws, size_t n_vocab);
void              geist_sampler_workspace_destroy(struct geist_sampler_workspace *ws);
/* src/engine/sampler.h:63-67, sampler.c:178-228 */
geist_token_t geist_sampler_top_k_ws(struct geist_sampler_workspace *ws, const float *logits,
                                     int top_k, float temperature, struct geist_rng *rng);
/* src/engine/sampler.h:69-73, sampler.c:232-305 */
geist_token_t geist_sampler_top_p_ws(struct geist_sampler_workspace *ws, const float *logits,
                                     float top_p, float temperature, struct geist_rng *rng);
#endif

/* No counterpart in the reference, whose samplers cannot fail. What a sampling call returns
 * after a device failure when the installed handler returns. */
#define GEIST_SAMPLER_DROPIN_FAILED_TOKEN ((geist_token_t) -1)
/* `what` names the step that failed, `detail` is the device layer's message. */
typedef void (*geist_sampler_dropin_failure_fn)(const char *what, const char *detail, void *user);
/* Installs the process-wide handler of device failures inside the sampling calls; null restores
 * the default, which prints the message to stderr and calls abort(). A handler may log and
 * return (the call then returns GEIST_SAMPLER_DROPIN_FAILED_TOKEN and consumes the draw it had
 * taken), or not return (longjmp, exit). It is called on the thread whose call failed. */
void geist_sampler_dropin_on_failure(geist_sampler_dropin_failure_fn fn, void *user);

#ifdef __cplusplus
}
#endif
#endif /* GEIST_SAMPLER_DROPIN_H */

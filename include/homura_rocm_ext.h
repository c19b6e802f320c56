/*
 * homura_rocm_ext.h -- entry points of this library that have no counterpart in the reference's
 * C ABI. Nothing in the reference crate needs them; they serve measurement harnesses.
 */
#ifndef HOMURA_ROCM_EXT_H
#define HOMURA_ROCM_EXT_H

#include "homura_rocm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* The HIP stream (hipStream_t) every kernel of `ctx` is queued on, so that a harness can record
 * its own hipEvents around calls. The context keeps ownership. No counterpart in the reference. */
hmr_status hmr_ext_stream(hmr_context_t ctx, void **stream);

#ifdef __cplusplus
}
#endif

#endif /* HOMURA_ROCM_EXT_H */

/*
 * Bootstrap entry points of the zbal API, MI355X build
 * (reference app/zbal/src/include/zbal_bootstrap.h:30-45).
 *
 * This build is single-process: zbal_bootstrap() selects the HIP device
 * options->deviceId, records worldSize/rankId and opens no transport. The
 * "ranks" of a world larger than one are local HBM windows registered per
 * communicator (zbal_comm_register_peer_window).
 */
#ifndef ZBAL_BOOTSTRAP_H
#define ZBAL_BOOTSTRAP_H

#include "zbal_def.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Fill `options` with defaults (worldSize 1, rank 0, device 0). */
int32_t zbal_bootstrap_options_init(zbal_bootstrap_options_t *options);

/* Must precede zbal_comm_create; a second call without unbootstrap fails. `output` may be NULL. */
int32_t zbal_bootstrap(zbal_bootstrap_options_t *options, zbal_bootstrap_output_t *output);

/* Destroys every communicator and returns the library to the un-bootstrapped state. */
int32_t zbal_unbootstrap(uint32_t flags);

#ifdef __cplusplus
}
#endif

#endif /* ZBAL_BOOTSTRAP_H */

/*
 * Umbrella header of the zbal API, MI355X build
 * (reference app/zbal/src/include/zbal.h:28-58).
 */
#ifndef ZBAL_H_
#define ZBAL_H_

#include "zbal_bootstrap.h"
#include "zbal_operations.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Version string of this library. */
const char *zbal_version();

/* Route log lines to `func(level, text)`; NULL restores stderr. */
int32_t zbal_set_logger(void (*func)(int, const char *));

/* 0 debug, 1 info, 2 warn, 3 error; anything else returns -2. */
int32_t zbal_set_logger_level(int level);

/* Text of the calling thread's most recent failure ("" if none). */
const char *zbal_get_last_error_msg();

/* Same, and clears it. The returned pointer stays valid until the thread's next call of this function. */
const char *zbal_get_and_clear_last_error_msg();

#ifdef __cplusplus
}
#endif

#endif /* ZBAL_H_ */

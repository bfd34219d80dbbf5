/*
 * fastkron_ext.h -- additions of the gfx950 library that have no counterpart in the FastKron
 * reference header.  Nothing in include/fastkron.h depends on them.
 */
#pragma once
#include "fastkron.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Describes the launch plan of the most recent GeMKM/GeKMM call on `handle` as text:
 *   "<problem string>;<lo>-<hi>:<kernel name>;..."   (one entry per launch, in launch order)
 * Writes at most `bufLen` bytes including the terminating NUL and returns the length the full text
 * needs (excluding the NUL), or 0 when no call has been made.  Used by the benchmark to attribute
 * time to kernels and by tests to assert which kernels ran.  The reference only prints this
 * information under FASTKRON_LOG=INFO (reference src/kernel_db/kernel_db.cpp:282-285).
 */
size_t fastKronGetLastPlan(fastKronHandle handle, char* buf, size_t bufLen);

/*
 * Path of the text file tuned launch plans are loaded from and saved to (also settable with the
 * FASTKRON_TUNED_DB environment variable before fastKronInit).  NULL or "" switches persistence off.
 * The reference keeps tuning results in memory only (reference src/autotuner/autotuner.h:101-116).
 */
fastKronError fastKronSetTunedDB(fastKronHandle handle, const char* path);

#ifdef __cplusplus
}
#endif

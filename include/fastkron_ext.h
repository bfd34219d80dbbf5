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

/*
 * Plan-only mode (on != 0): GeMKM/GeKMM calls on `handle` run every argument check, the launch planner and each
 * chosen kernel's check of the concrete buffers (alignment, strides), but launch nothing and touch no device;
 * an MI355X is assumed when none has been initialised.  fastKronGetLastPlan then names the kernels and
 * fastKronGetLastLaunches lists the launches the call would have made, one text line per launch:
 *   "kernel=<name> lo=<lo> hi=<hi> M=<rows> batch=<n> Kin=<cols> Kout=<cols> in=<ptr> out=<ptr> y=<ptr>
 *    in_batch=<elems> out_batch=<elems> y_batch=<elems> f_batch=<elems>,<elems>,..."
 * Meant for host-side tests of the planner and for inspecting what a call will do.  The reference has no such
 * mode; its nearest counterpart is the kernel series printed under FASTKRON_LOG=INFO
 * (reference src/kernel_db/kernel_db.cpp:282-285).
 */
fastKronError fastKronSetPlanOnly(fastKronHandle handle, int on);
size_t fastKronGetLastLaunches(fastKronHandle handle, char* buf, size_t bufLen);

/*
 * sgemkm for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments and result as sgemkm
 * (include/fastkron.h) without temp1 / temp2: the two temporaries and the workspace for merged factors are parts of
 * one array that the library keeps in device memory on every GPU it is loaded on, for the life of the process
 * (2 * FASTKRON_STATIC_SCRATCH_TEMP_BYTES + 512 KiB).  The call itself allocates and frees nothing and never tunes.
 * A problem whose temporaries (gekmmSizes' tmpElems * 4 bytes) exceed FASTKRON_STATIC_SCRATCH_TEMP_BYTES is refused
 * with fastKronInvalidArgument and a message on stderr.  All calls on one GPU share the array: calls that overlap
 * on one GPU race, whatever their handles and streams.  fastKronInitHIP resolves the array's address on its GPU.
 */
#define FASTKRON_STATIC_SCRATCH_TEMP_BYTES (16u << 20)
fastKronError sgemkmStaticScratch(fastKronHandle handle, fastKronBackend backend, uint32_t M, uint32_t N,
                                  uint32_t Ps[], uint32_t Qs[], const float* X, fastKronOp opX,
                                  const float* const Fs[], fastKronOp opFs, float* Z, float alpha, float beta,
                                  const float* Y);

/*
 * Kernels whose workgroups wait for each other inside one launch (the two-phase 4x4^6 GeKMM kernel) keep their counters
 * in device memory of the handle and bound every wait; a wait that runs out sets an error word there and the results
 * of that launch are not valid.  fastKronGetSyncError synchronises the handle's stream, copies the word to *word
 * (0: no wait ever ran out) and clears it.  fastKronSetSyncHelpAfter sets, for every handle of the process, after how
 * many polls a waiting workgroup runs the missing work of others itself (default 100000, far beyond what a launch
 * needs when all its workgroups run; 0 makes every workgroup do so at once, which tests use to cover that path).
 * Neither has a counterpart in the reference, whose kernels never synchronise across workgroups.
 */
fastKronError fastKronGetSyncError(fastKronHandle handle, uint32_t* word);
fastKronError fastKronSetSyncHelpAfter(uint32_t polls);

/*
 * Measurement aid, no counterpart in the reference: launches on the handle's stream a copy kernel Z = 1.5 X + 0.5 Y over
 * 4096 x M fp32 matrices (M a multiple of 2048, at most 16384) that touches memory the way one of the 4x4^6 GeKMM kernels
 * does and computes nothing else.  pattern 0: contiguous 16-byte accesses; 1: 32-byte strips of 8 columns, all 4096
 * rows per workgroup; 2: 256-byte pieces in two phases with an intermediate T (4096 x M floats) passed through the
 * L2 and workgroups waiting for each other.  `python bench.py --pattern-ceilings` times them beside the kernels.
 */
fastKronError fastKronProbeCopyPattern(fastKronHandle handle, int pattern, const float* X, const float* Y, float* Z,
                                       float* T, uint32_t M);

#ifdef __cplusplus
}
#endif

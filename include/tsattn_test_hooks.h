/*
 * tsattn_test_hooks.h -- entry points of libtsattn.so that exist for the library's own tests only.
 * Not part of the drop-in boundary: nothing in the reference corresponds to them and no caller needs them.
 */
#ifndef TSATTN_TEST_HOOKS_H
#define TSATTN_TEST_HOOKS_H

#include "tsattn.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Diagnostic: copies the handle's per-sequence arrival counters (used by the single-split fused append of tsattn_decode;
 * every launch leaves them at zero) into dst, a device array of n int32, on the stream.  For tests of graph replays. */
int tsattn_debug_read_counters(tsattn_handle_t h, int32_t *dst, int n, void *stream);

#ifdef __cplusplus
}
#endif

#endif

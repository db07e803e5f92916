/*
 * tfhip_test.h -- test hooks of libtfhip.so: entry points that exist so that error paths can be exercised from the
 * host while every kernel still exits normally. Not part of the interface a TensorFrost build binds (tfhip.h); the
 * reference has no counterpart. Same conventions as tfhip.h (int status, tfhip_last_error()).
 */
#ifndef TFHIP_TEST_H
#define TFHIP_TEST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Writes `code` into the pinned word through which kernels report a bounded wait that they gave up, as such a kernel
 * would; the next call that waits for the stream (tfhip_sync, tfhip_d2h, tfhip_h2d, tfhip_free,
 * tfhip_event_elapsed_ms) returns TFHIP_ERR_HIP once and clears it. Lets the error path be tested without any
 * kernel misbehaving. */
int tfhip_test_raise_async_error(uint32_t code);
/* Runs the one-pass u32 scan with its first tile missing (tickets start at 1): no group ever publishes tile 0, so each
 * look-back that reaches it gives up after `spin_limit` (1 .. 4096) polls, writes the error word and goes on with the
 * partial prefix. Every group stores its tile and exits normally; out[0 .. tile) is left untouched and the results are
 * wrong by construction. The next waiting call reports the given-up wait. n must span 2 .. 32768 tiles of 32768. */
int tfhip_test_scan_u32_first_tile_absent(const uint32_t* in, uint32_t* out, size_t n, uint32_t spin_limit);

#ifdef __cplusplus
}
#endif
#endif /* TFHIP_TEST_H */

/*
 * pimhip_probe.h -- measurement aids of libpimhip.so.  Not part of the drop-in interface of pimhip.h and without any
 * counterpart in the reference: a benchmark and the tests of the launch geometry call them, an integration does not.
 * Conventions (device pointers, `stream`, return value) as in pimhip.h.
 */
#ifndef PIMHIP_PROBE_H_
#define PIMHIP_PROBE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Reads `bytes` bytes (a multiple of 16, 16-byte aligned) once with the streaming loads of the GEMV kernels and keeps
 * nothing: what one launch of it takes is the floor for any kernel that has to read those bytes, launch included.  The
 * benchmark reports each GEMV beside it. */
int pimhip_probe_stream_read(const void* data, int64_t bytes, void* stream);

/* Launches `blocks` workgroups of `threads` lanes; workgroup b stores the index of the XCD it runs on (the hardware's
 * XCC_ID) to out[b] (uint32).  What the per-XCD LSTM kernel (mode 4 of pimhip_lstm_plan_set_mode) relies on can be looked
 * at with it: consecutive workgroups go to consecutive XCDs. */
int pimhip_probe_xcc_map(void* out, int blocks, int threads, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* PIMHIP_PROBE_H_ */

// Measurement switches of the kernel sources, in one place.  Every one of them changes what a kernel computes or how
// it is instrumented, so none may be set in a product build: defining any of them without TQ_MEASUREMENT_BUILD is a
// compile error, and a library built with TQ_MEASUREMENT_BUILD refuses tq_create unless the environment holds
// TQ_ALLOW_MEASUREMENT_BUILD=1 (capi.hip), so that a measurement variant named by TQ_HIP_LIBRARY cannot be loaded
// by accident.
//
//   TQ_KNOCKOUT=<bits>   fp16 store kernels with one phase removed (turbo_kernels.hip)
//   TQ_TIMELINE          per-wavefront timestamps of the fused K+V store, read back with tq_dbg_read_timeline
//   TQ_PAIRTAB3=1        3-bit decode attention through the conflict-free pair table (attn_kernels.hip)
//   TQ_STREAM_SITES=<m>  non-temporal hints switched off per family of kernels (tq_device.h)
#pragma once

#ifndef TQ_KNOCKOUT
#define TQ_KNOCKOUT 0
#endif
#ifndef TQ_PAIRTAB3
#define TQ_PAIRTAB3 0
#endif
#ifndef TQ_STREAM_SITES
#define TQ_STREAM_SITES 0xFFFF
#endif

#if (TQ_KNOCKOUT != 0 || TQ_PAIRTAB3 != 0 || TQ_STREAM_SITES != 0xFFFF || defined(TQ_TIMELINE)) && !defined(TQ_MEASUREMENT_BUILD)
#error "measurement switch set in a product build: add -DTQ_MEASUREMENT_BUILD (make MEASURE=1) and load the result on purpose"
#endif

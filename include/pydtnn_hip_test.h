/*
 * Test-only entry points of libpydtnn_hip.so.  Not part of the product ABI: nothing in pydtnn_hip.h depends
 * on them and no caller outside the test suite should bind them.
 */
#ifndef PYDTNN_HIP_TEST_H
#define PYDTNN_HIP_TEST_H

#ifdef __cplusplus
extern "C" {
#endif

/* The implicit convolution entry points run a batch whose tensors exceed 2^29 floats as consecutive groups of
 * whole images.  This lowers that limit (1 .. 2^29 floats) so that small tensors take the same route in a
 * test; returns the previous value.  Process-wide and not synchronised with running calls: set it, run the
 * case, restore it, all from one thread. */
long pydtnn_hip_debug_set_tensor_floats_limit(long floats);

/* The form of the calling thread's most recent GEMM or streaming-convolution launch (a call that launches several
 * kernels reports its last GEMM): out = {kind, tile rows, tile columns, workgroups, tiles cut by the balanced
 * launch, reduction splits}.  kind: 0 none yet, 1 grid of whole tiles, 2 balanced launch (workgroups = what the
 * chip holds at once, plus a fixup launch of `cut tiles` workgroups), 3 NHWC streaming kernel, 4 NCHW streaming
 * kernel, 5 fused 3x3 + 1x1 streaming kernel.  A benchmark that quotes hardware counters collected for one form
 * checks with this that the library still picks it. */
#define PYDTNN_HIP_LAUNCH_NONE 0
#define PYDTNN_HIP_LAUNCH_TILES 1
#define PYDTNN_HIP_LAUNCH_BALANCED 2
#define PYDTNN_HIP_LAUNCH_STREAM_NHWC 3
#define PYDTNN_HIP_LAUNCH_STREAM_NCHW 4
#define PYDTNN_HIP_LAUNCH_PAIR 5
void pydtnn_hip_debug_last_launch(int out[6]);

#ifdef __cplusplus
}
#endif
#endif /* PYDTNN_HIP_TEST_H */

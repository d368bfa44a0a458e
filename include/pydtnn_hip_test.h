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

#ifdef __cplusplus
}
#endif
#endif /* PYDTNN_HIP_TEST_H */

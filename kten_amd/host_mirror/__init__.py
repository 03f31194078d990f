"""Host-side mirror of the reference's layers above a backend: the raw-tensor contract
(`raw_tensor`, `shape_functions`), the autograd layer that emits the raw-op sequences
(`autograd`), and the seeded workloads and inputs of the parity tests and the benchmark
(`workloads`, `inputs`). In a deployment all of this is the reference's unchanged Kotlin;
here it is the harness that drives a backend through the contract. It is shared by the HIP
backend (`kten_amd.hip_raw_tensor`) and by the CPU checker, so a comparison of the two does not
test this layer: the known answers transcribed from the reference's suite and the numpy checks of
tests/test_host_logic.py pin it on its own."""

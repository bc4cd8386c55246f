"""MI355X (gfx950) graph-operator kernels for NeutronBench-style GNN training.

The product is the C-ABI library ``lib/libntship.so`` (declared in ``include/nts_hip.h``).  This
package is the thin Python host layer used by the tests and the benchmark:

* ``abi``     ctypes binding of every exported entry point (raises if the library is missing);
* ``stream``  ``CudaStream``, a mirror of the reference's ``Cuda_Stream`` class over the ABI;
* ``ops``     mirrors of the reference's graph operators (forward()/backward() objects);
* ``layout``  device-resident full-graph chunks and sampled layers;
* ``synth``   seeded synthetic graphs / features of the benchmark shapes.

There is no CPU fallback: every operator calls the HIP library.
"""
__version__ = "0.1.0"

"""gfx950 implementations of the reference's Triton ops on the MoE path (``batchgen_kernels/triton``), under the
reference's module and function names.  Nothing here is Triton: every function is an argument checker over a
HIP kernel of libbgmoe.so."""

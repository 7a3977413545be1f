"""MI355X (gfx950) kernels for the sparse CSR code LAPIS generates: SpMV, CSR x dense
SpMM and the vector operations of conjugate gradients, behind the generated module's
own calling convention.

``lapis_amd.hip``         ctypes binding of the C-ABI kernel library (device pointers)
``lapis_amd.module``      ``LAPISModule``, the class a generated package exposes (host numpy buffers)
``lapis_amd.generators``  seeded synthetic CSR inputs of the benchmark configurations
``lapis_amd.build``       hipcc build of both shared libraries
"""

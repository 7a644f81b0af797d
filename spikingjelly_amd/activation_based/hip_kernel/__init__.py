"""HIP kernel backend: ctypes binding of ``libsjhip.so`` and the ``torch.library`` operators on
top of it.  Counterpart of the reference's ``cuda_kernel`` (CuPy) and ``triton_kernel`` packages
for the multi-step IF / LIF / PLIF path and spike bit-packing."""

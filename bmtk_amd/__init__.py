"""MI355X-native GLIF3 point-neuron hot path (bmtk PointNet / NEST ``glif_psc``).

Host code is Python over a C-ABI shared library of hand-written HIP kernels
(``bmtk_amd/csrc``).  There is no CPU fallback: importing works anywhere, but
every compute entry point raises if the HIP library or a GPU is missing.
"""
__version__ = "0.1.0"

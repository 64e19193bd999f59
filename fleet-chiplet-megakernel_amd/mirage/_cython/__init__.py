"""Compiled (Cython) binding of libfleet_mk.so: `core.CyGraph`, the counterpart of the reference's
python/mirage/_cython/core.pyx for this library.  Built in tree by fleet-chiplet-megakernel_amd/build.py."""

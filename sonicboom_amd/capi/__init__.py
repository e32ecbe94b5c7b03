"""The C interface: ``sonicboom_amd.h``, its implementation ``capi.cpp`` (hosts this package
in an interpreter), the C++ command line ``sb_gen.cpp`` over it, and ``build.py``."""

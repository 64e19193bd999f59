// Single translation unit of libfleet_mk.so: the gfx950 persistent kernel and the C-ABI host
// library that lowers task graphs and launches it.
#include "mk_kernel.hip"
#include "mk_host.cpp"

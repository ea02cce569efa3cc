// Umbrella translation unit of the hybrid-decoder extension: the
// sequence-mixer kernels plus the elementwise templates they share with the
// main extension, compiled into a library of their own so that serving a
// hybrid model builds nothing else.
#include "elementwise.hip"
#include "seqmix.hip"
#include "latent_moe.hip"
#include "scan_mix.hip"
#include "memory_mix.hip"
#include "hybrid_bindings.cpp"

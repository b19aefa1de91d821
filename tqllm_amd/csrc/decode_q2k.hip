// Decode kernels of one bank format (see decode_kernels.cuh).
#include "decode_kernels.cuh"
template struct tqmoe::DecodeLaunch<TQMOE_Q2_K>;

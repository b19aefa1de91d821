// Decode kernels and grouped fp16 products of one bank format (see decode_kernels.cuh, prefill_f16_kernels.cuh).
#include "decode_kernels.cuh"
#include "prefill_f16_kernels.cuh"
template struct tqmoe::DecodeLaunch<TQMOE_IQ2_XS>;
template struct tqmoe::F16Launch<TQMOE_IQ2_XS>;

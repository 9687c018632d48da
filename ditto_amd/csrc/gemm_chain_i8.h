// Arguments and launcher of the int8 requantised GEMM chain kernel (gemm_chain_i8.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ditto {

struct I8ChainArgs {
  const int8_t* a;
  const int8_t* b;
  const int8_t* d;
  const float* scale;   // [L] or null
  float scale_uniform;  // used when scale == null
  int wrap;             // middle result = the accumulator's low byte (the wrapping astype("int8")) instead of requantised
  int relu;             // wrap only: max(acc, 0) first
  int out_i8;           // e is int8: the low byte of every result (the chain's closing astype("int8"))
  int32_t* e;
  long long a_bs, b_bs, d_bs, e_bs;  // batch strides, elements
  int a_rs, b_rs, d_rs, e_rs;        // row strides, elements
  int M, N, K, L, batch;
  int mblocks;
  int Lp;  // L rounded up to the weight-chunk width
};

// dynamic LDS bytes of the kernel for a padded L, mt = 1|2 row tiles of 32 per workgroup and a
// ring of nst = 2..4 staged chunks
int i8_chain_lds_bytes_host(int Lp, int mt, int nst);
// threads per workgroup of the kernel
int i8_chain_threads();
hipError_t launch_gemm_chain_i8(const I8ChainArgs& args, int mt, int nst, hipStream_t stream);

}  // namespace ditto

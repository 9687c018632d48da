// Arguments and launcher of the fp32 / fp64 GEMM chain kernel (gemm_chain_f32.hip).
#pragma once
#include <hip/hip_runtime.h>

namespace ditto {

struct F32ChainArgs {
  const void* a;  // float or double (f64)
  const void* b;
  const void* c;
  void* f;
  long long a_bs, b_bs, c_bs, f_bs;  // batch strides, elements
  int a_rs, b_rs, c_rs, f_rs;        // row strides, elements
  int M, N, K, L, batch;
  int mblocks;  // workgroups (32 rows each) per batch entry
  int b_lk;     // B stored [L][K]
  int relu;
  int relu_out;  // ReLU on the output
  int softmax;   // inter path: softmax over L of scale * (A.B)
  float softmax_scale;
  int f64;       // elements are doubles
};

int f32_chain_lds_bytes_host(int K, int N, int f64);
int f32_chain_max_dim();  // largest K and N the kernel takes
hipError_t launch_gemm_chain_f32(const F32ChainArgs& args, hipStream_t stream);

}  // namespace ditto

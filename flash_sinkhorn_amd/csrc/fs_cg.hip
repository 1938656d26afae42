// Conjugate-gradient bookkeeping on the device: the vector updates, dot products and the
// convergence decision of one CG iteration in one single-workgroup launch, so that a CG loop
// costs its matrix-vector products plus one small launch per iteration and the host reads the
// state back only when it wants to know whether to go on.
#include <hip/hip_runtime.h>

#include "flash_sinkhorn_hip.h"

namespace fs {
namespace {

constexpr int kCgThreads = 1024;

// state[0] = r.z of the current residual, [1] = |r0|, [2] = tolerance, [3] = |r| after the last
// update, [4] = done (0/1), [5] = converged (0/1), [6] = iterations performed, [7] unused
__device__ double block_sum(double v, double* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  __syncthreads();  // red may still be read from the previous call
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  double t = 0.0;
  for (int w = 0; w < kCgThreads / 64; ++w) t += red[w];
  return t;
}

__global__ __launch_bounds__(kCgThreads) void cg_init_kernel(const float* __restrict__ b,
                                                             float* __restrict__ sol,
                                                             float* __restrict__ res,
                                                             float* __restrict__ dir,
                                                             float* __restrict__ state, long long m,
                                                             float rtol, float atol) {
  __shared__ double red[kCgThreads / 64];
  double acc = 0.0;
  for (long long i = threadIdx.x; i < m; i += kCgThreads) {
    const float v = b[i];
    sol[i] = 0.f;
    res[i] = v;
    dir[i] = v;
    acc += (double)v * (double)v;
  }
  const double rz = block_sum(acc, red);
  if (threadIdx.x == 0) {
    const float r0 = (float)sqrt(rz);
    state[0] = (float)rz;
    state[1] = r0;
    state[2] = fmaxf(atol, rtol * r0);
    state[3] = r0;
    state[4] = 0.f;
    state[5] = 0.f;
    state[6] = 0.f;
    state[7] = 0.f;
  }
}

__global__ __launch_bounds__(kCgThreads) void cg_update_kernel(const float* __restrict__ a_dir,
                                                               float* __restrict__ sol,
                                                               float* __restrict__ res,
                                                               float* __restrict__ dir,
                                                               float* __restrict__ state,
                                                               long long m) {
  __shared__ double red[kCgThreads / 64];
  if (state[4] != 0.f) return;  // finished earlier: every later update leaves the vectors alone
  double acc = 0.0;
  for (long long i = threadIdx.x; i < m; i += kCgThreads) acc += (double)dir[i] * (double)a_dir[i];
  const double curvature = block_sum(acc, red);
  if (curvature == 0.0) {  // uniform: every thread holds the same sum
    if (threadIdx.x == 0) state[4] = 1.f;
    return;
  }
  const float rz = state[0];
  const float tol = state[2];
  const float step = (float)((double)rz / curvature);
  acc = 0.0;
  for (long long i = threadIdx.x; i < m; i += kCgThreads) {
    sol[i] += step * dir[i];
    const float r = res[i] - step * a_dir[i];
    res[i] = r;
    acc += (double)r * (double)r;
  }
  const double rr = block_sum(acc, red);
  const float rnorm = (float)sqrt(rr);
  if (rnorm <= tol) {
    if (threadIdx.x == 0) {
      state[3] = rnorm;
      state[4] = 1.f;
      state[5] = 1.f;
      state[6] += 1.f;
    }
    return;
  }
  const float beta = (float)(rr / (double)rz);
  for (long long i = threadIdx.x; i < m; i += kCgThreads) dir[i] = res[i] + beta * dir[i];
  if (threadIdx.x == 0) {
    state[0] = (float)rr;
    state[3] = rnorm;
    state[6] += 1.f;
  }
}

}  // namespace
}  // namespace fs

extern "C" {

int fs_cg_init(const float* b, float* sol, float* res, float* dir, float* state, int64_t m,
               float rtol, float atol, void* stream) {
  if (!b || !sol || !res || !dir || !state) return FS_ERR_NULL_POINTER;
  if (m <= 0 || m > ((int64_t)1 << 31)) return FS_ERR_BAD_SIZE;
  hipLaunchKernelGGL(fs::cg_init_kernel, dim3(1), dim3(fs::kCgThreads), 0, (hipStream_t)stream, b,
                     sol, res, dir, state, (long long)m, rtol, atol);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

int fs_cg_update(const float* a_dir, float* sol, float* res, float* dir, float* state, int64_t m,
                 void* stream) {
  if (!a_dir || !sol || !res || !dir || !state) return FS_ERR_NULL_POINTER;
  if (m <= 0 || m > ((int64_t)1 << 31)) return FS_ERR_BAD_SIZE;
  hipLaunchKernelGGL(fs::cg_update_kernel, dim3(1), dim3(fs::kCgThreads), 0, (hipStream_t)stream,
                     a_dir, sol, res, dir, state, (long long)m);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

}  // extern "C"

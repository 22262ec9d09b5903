// Device functions used as parpy.external targets by the tests (the HIP counterpart of the
// reference's test/code/cuda_utils.h).
#pragma once

__device__ inline float clamp(float x, float lo, float hi) {
  if (x < lo) return lo;
  if (x > hi) return hi;
  return x;
}

// not callable from a kernel: no __device__ attribute
inline float clamp_non_device(float x, float lo, float hi) {
  if (x < lo) return lo;
  if (x > hi) return hi;
  return x;
}

__device__ inline double sum_row_ext(double* p, long long n) {
  double s = 0;
  for (long long i = 0; i < n; i++) s += p[i];
  return s;
}

// sum of the 64 values of one row, one per lane of a wavefront; every lane gets the result
__device__ inline float wave_sum(float* values) {
  float v = values[threadIdx.x];
  for (int i = 32; i > 0; i /= 2) v = v + __shfl_xor(v, i, 64);
  return v;
}

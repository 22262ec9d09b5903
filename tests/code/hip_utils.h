// Device functions that tests/test_calls.py binds with parpy.external.  They are deliberately
// small: what is under test is the call path (header inclusion, argument passing, pointer
// arguments, one call executed co-operatively by a whole wavefront), not the functions.
#pragma once

// scalar in, scalar out
__device__ inline float clamp(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }

// Host-only twin of clamp: declaring it as an external must be rejected when the kernel is built,
// because a kernel cannot call a function without the __device__ attribute.
inline float clamp_non_device(float x, float lo, float hi) { return x < lo ? lo : (x > hi ? hi : x); }

// pointer argument: sequential sum of the n doubles at p
__device__ inline double sum_row_ext(double* p, long long n) {
  double total = 0.0;
  while (n-- > 0) total += *p++;
  return total;
}

// Called by all 64 lanes of a wavefront at once (parallelize=threads(64)): lane l contributes
// values[l]; a butterfly over the lane index leaves the total in every lane.
__device__ inline float wave_sum(float* values) {
  float mine = values[threadIdx.x];
#pragma unroll
  for (int stride = 1; stride < 64; stride <<= 1) mine += __shfl_xor(mine, stride, 64);
  return mine;
}

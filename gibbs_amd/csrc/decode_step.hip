// End of a decode step that runs as a captured graph: everything that changes from one step to the
// next moves on the device, so that a replay needs no host work.
//   log[counter * n + i] = ids[i]      the token each request was just given (sampled into ids)
//   pos[i] += 1;  ctx[i] += 1          the next step's position and cached length
//   u[i] = u_all[(counter + 1) * n + i]  the next step's random draws (if sampling)
//   counter += 1
#include "common.h"

__global__ void advance_kernel(int* __restrict__ pos, int* __restrict__ ctx, const int* __restrict__ ids,
                               int* __restrict__ log, int* __restrict__ counter, float* __restrict__ u,
                               const float* __restrict__ u_all, int n, int capacity) {
  const int step = *counter;
  const int i = threadIdx.x + blockIdx.x * blockDim.x;
  if (i < n) {
    if (step < capacity) log[(size_t)step * n + i] = ids[i];
    pos[i] += 1;
    ctx[i] += 1;
    if (u && step + 1 < capacity) u[i] = u_all[(size_t)(step + 1) * n + i];
  }
  // every thread has read the counter before any can see the new value: one block only
  __syncthreads();
  if (i == 0) *counter = step + 1;
}

GIBBS_EXPORT int gibbs_advance(int* pos, int* ctx, const int* ids, int* log, int* counter, float* u,
                               const float* u_all, int n, int capacity, hipStream_t stream) {
  GIBBS_REQUIRE(n > 0 && n <= 1024, "advance: batch %d outside 1..1024", n);
  GIBBS_REQUIRE(capacity > 0, "advance: empty token log");
  advance_kernel<<<1, 1024, 0, stream>>>(pos, ctx, ids, log, counter, u, u_all, n, capacity);
  GIBBS_LAUNCH_STATUS("advance");
}

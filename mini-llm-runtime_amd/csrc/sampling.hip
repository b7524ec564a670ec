// Token choice from float logits, one workgroup per row:
//   temperature <= 0: the largest logit, ties -> lowest id;
//   temperature  > 0: inverse-CDF draw from softmax(logits / T) with the uniform number u[r]
//                     that the host derived from the request's own generator state.
// A row that holds a NaN or an infinity gives token -1 and sets status[0] |= 1,
// status[1] = min(status[1], row).  Max, exponentials and sums are 32-bit; every thread owns
// a contiguous range of the vocabulary and all sums run in ascending order, so a row's
// token depends on that row only.
#include <hip/hip_runtime.h>
#include <stdint.h>

#define THREADS 1024

__global__ __launch_bounds__(THREADS) void sample_kernel(const float* __restrict__ logits, int vocab,
                                                         const float* __restrict__ temperature,
                                                         const float* __restrict__ uniform,
                                                         int32_t* __restrict__ tokens,
                                                         int32_t* __restrict__ status) {
    __shared__ float vals[THREADS];
    __shared__ int idxs[THREADS];
    __shared__ int bad, chosen;
    const int r = blockIdx.x, t = threadIdx.x;
    const float* row = logits + (size_t)r * vocab;
    const int chunk = (vocab + THREADS - 1) / THREADS;
    const int begin = min(vocab, t * chunk), end = min(vocab, begin + chunk);
    if (t == 0) { bad = 0; chosen = -1; }
    __syncthreads();

    float best = -INFINITY;
    int best_i = 0x7fffffff;
    bool nonfinite = false;
    for (int i = begin; i < end; ++i) {
        const float x = row[i];
        if (!(fabsf(x) <= 3.402823466e38f)) nonfinite = true;
        if (x > best) { best = x; best_i = i; }
    }
    if (nonfinite) bad = 1;
    vals[t] = best;
    idxs[t] = best_i;
    __syncthreads();
    for (int s = THREADS / 2; s > 0; s >>= 1) {
        if (t < s) {
            const float ov = vals[t + s];
            const int oi = idxs[t + s];
            if (ov > vals[t] || (ov == vals[t] && oi < idxs[t])) { vals[t] = ov; idxs[t] = oi; }
        }
        __syncthreads();
    }
    const float row_max = vals[0];
    const int arg = idxs[0];
    if (bad) {
        if (t == 0) {
            tokens[r] = -1;
            atomicOr(&status[0], 1);
            atomicMin(&status[1], r);
        }
        return;
    }
    const float temp = temperature ? temperature[r] : 0.f;
    if (!(temp > 0.f)) {
        if (t == 0) tokens[r] = arg;
        return;
    }
    __syncthreads();
    const float inv_t = 1.0f / temp;
    float sum = 0.f;
    for (int i = begin; i < end; ++i) sum += expf((row[i] - row_max) * inv_t);
    vals[t] = sum;
    __syncthreads();
    if (t == 0) {                                   // inclusive scan in ascending order
        float c = 0.f;
        for (int i = 0; i < THREADS; ++i) { c += vals[i]; vals[i] = c; }
    }
    __syncthreads();
    const float target = uniform[r] * vals[THREADS - 1];
    const float lo = t ? vals[t - 1] : 0.f, hi = vals[t];
    if (target >= lo && target < hi && end > begin) {
        float c = lo;
        int pick = end - 1;
        for (int i = begin; i < end; ++i) {
            c += expf((row[i] - row_max) * inv_t);
            if (c > target) { pick = i; break; }
        }
        chosen = pick;
    }
    __syncthreads();
    if (t == 0) tokens[r] = chosen >= 0 ? chosen : arg;
}

__global__ void reset_status_kernel(int32_t* status) {
    status[0] = 0;
    status[1] = 0x7fffffff;
}

extern "C" int mlr_sample(const float* logits, int rows, int vocab, const float* temperature,
                          const float* uniform, int32_t* tokens, int32_t* status, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0) return -1;
    reset_status_kernel<<<1, 1, 0, stream>>>(status);
    sample_kernel<<<rows, THREADS, 0, stream>>>(logits, vocab, temperature, uniform, tokens, status);
    return (int)hipGetLastError();
}

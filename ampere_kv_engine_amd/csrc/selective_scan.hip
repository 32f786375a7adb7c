// A selective scan with its short causal convolution.  What a request carries from token to token lies in its slot, in
// float32: S [channels, n_state], then the convolution's last taps - 1 inputs [taps - 1, channels], oldest first.
//
//   x_t = silu(sum_k w[c, k] * in[t - (taps - 1 - k)] + b[c])                (inputs before the sequence's start are 0)
//   S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;   y_c = sum_n S[c, n] C_n + D_c x_c;   out = y * silu(z)
// with dt = softplus(dt_raw).  Step sizes, decays, exponentials, the state and the sums are float32.

#include "common.h"
#include "api_parts.h"

using namespace akv;

namespace {

__device__ __forceinline__ float silu(float v) { return v / (1.f + expf(-v)); }
__device__ __forceinline__ float softplus(float v) { return v > 20.f ? v : log1pf(expf(v)); }

// ---- convolution over the portion and what the slot remembers of the tokens before it --------------------------------
template <typename T, typename TW>
__global__ __launch_bounds__(256) void conv_silu_kernel(const T* __restrict__ x, long x_stride, const TW* __restrict__ weight,
                                                        const TW* __restrict__ bias, const float* __restrict__ state,
                                                        long state_stride, long conv_at,
                                                        const int* __restrict__ seq_of_token,
                                                        const int* __restrict__ q_start, const int* __restrict__ seq_slots,
                                                        T* __restrict__ out, int channels, int taps) {
  const int n = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int r = seq_of_token[n];
  const int first = q_start[r];
  const float* kept = state + static_cast<long>(seq_slots[r]) * state_stride + conv_at;   // [taps - 1][channels]
  float acc = to_float(bias[c]);
  for (int k = 0; k < taps; ++k) {
    const int row = n - (taps - 1 - k);
    float v;
    if (row >= first) {
      v = to_float(x[row * x_stride + c]);
    } else {
      const int back = first - row;                  // 1 .. taps - 1 tokens before the portion
      v = kept[static_cast<long>(taps - 1 - back) * channels + c];
    }
    acc = fmaf(to_float(weight[static_cast<long>(c) * taps + k]), v, acc);
  }
  out[static_cast<long>(n) * channels + c] = from_float<T>(silu(acc));
}

// After the convolution has read the old inputs: the slot keeps the last taps - 1 of (old inputs, the portion's).
template <typename T>
__global__ __launch_bounds__(256) void conv_state_update_kernel(const T* __restrict__ x, long x_stride,
                                                                float* __restrict__ state, long state_stride,
                                                                long conv_at, const int* __restrict__ q_start,
                                                                const int* __restrict__ seq_slots, int channels,
                                                                int taps) {
  const int r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int first = q_start[r], count = q_start[r + 1] - first;
  float* kept = state + static_cast<long>(seq_slots[r]) * state_stride + conv_at;
  // entry k of the new state is input number count - (taps - 1) + k of the portion; negative numbers reach into the
  // old state at taps - 1 + that number, which is at least k: ascending k never reads what it has already replaced
  for (int k = 0; k < taps - 1; ++k) {
    const int index = count - (taps - 1) + k;
    const float v = index >= 0 ? to_float(x[(first + index) * x_stride + c])
                               : kept[static_cast<long>(taps - 1 + index) * channels + c];
    kept[static_cast<long>(k) * channels + c] = v;
  }
}

// ---- the scan: a thread owns a channel of a request, its row of S in registers, and walks the portion's tokens ------
// Tokens are taken kScanAhead at a time: their inputs are asked for together (a token's own arithmetic is short, and
// one trip to memory per token would be all a long portion's time), and the wave lays the tokens' B and C, which all
// channels share, into LDS once.
constexpr int kScanAhead = 8;

template <typename T, int NS>
__global__ __launch_bounds__(64) void selective_scan_kernel(const T* __restrict__ x, const float* __restrict__ dt,
                                                            const float* __restrict__ bc, const T* __restrict__ z,
                                                            long z_stride, const float* __restrict__ a,
                                                            const float* __restrict__ d, float* __restrict__ state,
                                                            long state_stride, const int* __restrict__ q_start,
                                                            const int* __restrict__ seq_slots, T* __restrict__ out,
                                                            int channels, int n_state) {
  extern __shared__ float shared_bc[];                // [kScanAhead][2 * n_state]
  const int r = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const bool works = c < channels;
  const int cc = works ? c : channels - 1;            // (a lane beyond the channels keeps the wave's steps and stores nothing)
  float* kept = state + static_cast<long>(seq_slots[r]) * state_stride + static_cast<long>(cc) * n_state;
  float S[NS], A[NS];
#pragma unroll
  for (int n = 0; n < NS; ++n) {
    S[n] = n < n_state ? kept[n] : 0.f;
    A[n] = n < n_state ? a[static_cast<long>(cc) * n_state + n] : 0.f;
  }
  const float skip = d[cc];
  const int first = q_start[r], last = q_start[r + 1];
  const int row = 2 * n_state;
  for (int t0 = first; t0 < last; t0 += kScanAhead) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();                  // the tokens before have been read by every lane
    for (int e = threadIdx.x; e < kScanAhead * row; e += blockDim.x) {
      const int t = min(t0 + e / row, last - 1);
      shared_bc[e] = bc[static_cast<long>(t) * row + e % row];
    }
    float xv[kScanAhead], step[kScanAhead], gate[kScanAhead];
#pragma unroll
    for (int u = 0; u < kScanAhead; ++u) {
      const long t = min(t0 + u, last - 1);
      xv[u] = to_float(x[t * channels + cc]);
      step[u] = dt[t * channels + cc];
      gate[u] = to_float(z[t * z_stride + cc]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int u = 0; u < kScanAhead; ++u) {
      if (t0 + u >= last) break;
      const float h = softplus(step[u]);
      const float* B = shared_bc + u * row;
      const float* C = B + n_state;
      const float drive = h * xv[u];
      float y = 0.f;
#pragma unroll
      for (int n = 0; n < NS; ++n) {
        if (n < n_state) {
          S[n] = fmaf(expf(h * A[n]), S[n], drive * B[n]);
          y = fmaf(S[n], C[n], y);
        }
      }
      y = fmaf(skip, xv[u], y);
      if (works) out[static_cast<long>(t0 + u) * channels + c] = from_float<T>(y * silu(gate[u]));
    }
  }
  if (!works) return;
#pragma unroll
  for (int n = 0; n < NS; ++n)
    if (n < n_state) kept[n] = S[n];
}

}  // namespace

extern "C" {

int akv_conv_silu(const void* x, long x_stride, int dtype, const void* weight, const void* bias, int w_dtype,
                  const float* state, long state_stride, long conv_at, const int* seq_of_token, const int* q_start,
                  const int* seq_slots, void* out, int tokens, int channels, int taps, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (taps < 1 || channels <= 0) return -2;
  const dim3 grid(tokens, (channels + 255) / 256);
#define AKV_CONV(T, TW)                                                                                            \
  conv_silu_kernel<T, TW><<<grid, 256, 0, stream>>>(static_cast<const T*>(x), x_stride, static_cast<const TW*>(weight), \
                                                    static_cast<const TW*>(bias), state, state_stride, conv_at,     \
                                                    seq_of_token, q_start, seq_slots, static_cast<T*>(out), channels, taps)
  if (dtype == kF32 && w_dtype == kF32) AKV_CONV(float, float);
  else if (dtype == kBF16 && w_dtype == kBF16) AKV_CONV(bf16_t, bf16_t);
  else if (dtype == kBF16 && w_dtype == kF32) AKV_CONV(bf16_t, float);
  else return -1;
#undef AKV_CONV
  return AKV_LAUNCH_STATUS();
}

int akv_conv_state_update(const void* x, long x_stride, int dtype, float* state, long state_stride, long conv_at,
                          const int* q_start, const int* seq_slots, int seqs, int channels, int taps,
                          hipStream_t stream) {
  if (seqs <= 0 || taps <= 1) return 0;
  const dim3 grid(seqs, (channels + 255) / 256);
  AKV_DISPATCH(dtype, T, conv_state_update_kernel<T><<<grid, 256, 0, stream>>>(
                             static_cast<const T*>(x), x_stride, state, state_stride, conv_at, q_start, seq_slots, channels,
                             taps));
  return AKV_LAUNCH_STATUS();
}

int akv_selective_scan(const void* x, int dtype, const float* dt, const float* bc, const void* z, long z_stride,
                       const float* a, const float* d, float* state, long state_stride, const int* q_start,
                       const int* seq_slots, void* out, int seqs, int channels, int n_state, hipStream_t stream) {
  if (seqs <= 0) return 0;
  if (n_state <= 0 || n_state > 256) return -2;
  const dim3 grid(seqs, (channels + 63) / 64);
#define AKV_SCAN(T, NS)                                                                                             \
  selective_scan_kernel<T, NS><<<grid, 64, kScanAhead * 2 * n_state * 4, stream>>>(static_cast<const T*>(x), dt, bc, static_cast<const T*>(z), \
                                                        z_stride, a, d, state, state_stride, q_start, seq_slots,    \
                                                        static_cast<T*>(out), channels, n_state)
  AKV_DISPATCH(dtype, T, {
    if (n_state <= 8) AKV_SCAN(T, 8);
    else if (n_state <= 16) AKV_SCAN(T, 16);
    else if (n_state <= 32) AKV_SCAN(T, 32);
    else if (n_state <= 64) AKV_SCAN(T, 64);
    else if (n_state <= 128) AKV_SCAN(T, 128);
    else AKV_SCAN(T, 256);
  });
#undef AKV_SCAN
  return AKV_LAUNCH_STATUS();
}
}

// Mixers whose requests carry a float32 state of fixed size from token to token:
//   retention - S [dim, vdim] per head, S <- decay S + k v^T, o = S^T q, with rotary positions on q and k, the unit norm of o
//   per head and the gate silu(g) in the same kernel;
//   a gated linear recurrence - S [channels], S <- a S + sqrt(1 - a^2) i u with a = exp(rate r), r and i sigmoids of
//   block-diagonal products, the output S * gelu_tanh(y).
// Everything but the loads of the projections is float32.  A request's tokens are taken in the order of their positions
// whatever the step's cutting, and a token's sums run in a fixed order, so cuttings agree to rounding.

#include "common.h"
#include "api_parts.h"

using namespace akv;

namespace {

__device__ __forceinline__ float silu(float v) { return v / (1.f + expf(-v)); }
__device__ __forceinline__ float sigmoid(float v) { return 1.f / (1.f + expf(-v)); }
__device__ __forceinline__ float gelu_tanh(float v) {
  return 0.5f * v * (1.f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
}

// ---- retention ------------------------------------------------------------------------------------------------------
// A block is a (request, head).  Thread (p, v) owns S[p R + r][v], r < R, in registers.  Tokens are taken TB at a time:
// their rotated queries and keys and their values go to LDS, every thread runs its share of the TB recurrence steps and
// leaves its shares of the outputs, which are then added over p, normed and gated, a wave a token.
template <typename T, int R>
__global__ __launch_bounds__(1024) void retention_kernel(
    const T* __restrict__ projected, long stride, int heads, int dim, int vdim, int rot_dims,
    const float* __restrict__ table, int table_positions, float key_scale, const float* __restrict__ decay, float eps,
    float* __restrict__ state, long state_stride, const int* __restrict__ q_start, const int* __restrict__ seq_slots,
    const int* __restrict__ positions, T* __restrict__ out, int parts, int batch) {
  extern __shared__ float lds[];
  const int seq = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, threads = blockDim.x;
  const int first = q_start[seq], count = q_start[seq + 1] - first;
  const int p = tid / vdim, v = tid % vdim;
  const bool owner = p < parts;
  float* qs = lds;                          // [batch][dim]
  float* ks = qs + batch * dim;             // [batch][dim]
  float* vs = ks + batch * dim;             // [batch][vdim]
  float* shares = vs + batch * vdim;        // [batch][parts][vdim]
  float* os = shares + batch * parts * vdim;  // [batch][vdim]
  float* mine = state + static_cast<long>(seq_slots[seq]) * state_stride + static_cast<long>(h) * dim * vdim;
  const float keep = decay[h];
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = p * R + r;
    S[r] = owner && d < dim ? mine[static_cast<long>(d) * vdim + v] : 0.f;
  }
  const long q_at = static_cast<long>(h) * dim, k_at = static_cast<long>(heads) * dim + q_at;
  const long v_at = 2L * heads * dim + static_cast<long>(h) * vdim, g_at = v_at + static_cast<long>(heads) * vdim;
  const int half = rot_dims / 2;
  const int waves = threads / kWave, wave = tid / kWave, lane = tid & (kWave - 1);
  for (int base = 0; base < count; base += batch) {
    const int tb = min(batch, count - base);
    for (int index = tid; index < tb * dim; index += threads) {
      const int t = index / dim, d = index % dim;
      const T* row = projected + static_cast<long>(first + base + t) * stride;
      float qv = to_float(row[q_at + d]), kv = to_float(row[k_at + d]);
      if (d < rot_dims) {
        const int i = d < half ? d : d - half;
        const int pos = min(positions[first + base + t], table_positions - 1);
        const float c = table[(static_cast<long>(pos) * half + i) * 2], s = table[(static_cast<long>(pos) * half + i) * 2 + 1];
        const int other = d < half ? d + half : d - half;
        const float qo = to_float(row[q_at + other]), ko = to_float(row[k_at + other]);
        qv = d < half ? qv * c - qo * s : qv * c + qo * s;
        kv = d < half ? kv * c - ko * s : kv * c + ko * s;
      }
      qs[t * dim + d] = qv;
      ks[t * dim + d] = kv * key_scale;
    }
    for (int index = tid; index < tb * vdim; index += threads) {
      const int t = index / vdim, c = index % vdim;
      vs[index] = to_float(projected[static_cast<long>(first + base + t) * stride + v_at + c]);
    }
    __syncthreads();
    if (owner) {
      for (int t = 0; t < tb; ++t) {
        const float value = vs[t * vdim + v];
        float share = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int d = p * R + r;
          if (d < dim) {
            S[r] = fmaf(keep, S[r], ks[t * dim + d] * value);
            share = fmaf(S[r], qs[t * dim + d], share);
          }
        }
        shares[(t * parts + p) * vdim + v] = share;
      }
    }
    __syncthreads();
    for (int index = tid; index < tb * vdim; index += threads) {
      const int t = index / vdim, c = index % vdim;
      float o = 0.f;
      for (int part = 0; part < parts; ++part) o += shares[(t * parts + part) * vdim + c];
      os[index] = o;
    }
    __syncthreads();
    for (int t = wave; t < tb; t += waves) {
      float squares = 0.f;
      for (int c = lane; c < vdim; c += kWave) squares += os[t * vdim + c] * os[t * vdim + c];
      const float scale = rsqrtf(wave_sum(squares) / static_cast<float>(vdim) + eps);
      const long n = first + base + t;
      for (int c = lane; c < vdim; c += kWave) {
        const float g = to_float(projected[n * stride + g_at + c]);
        out[n * heads * vdim + static_cast<long>(h) * vdim + c] = from_float<T>(os[t * vdim + c] * scale * silu(g));
      }
    }
    __syncthreads();
  }
  if (owner) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = p * R + r;
      if (d < dim) mine[static_cast<long>(d) * vdim + v] = S[r];
    }
  }
}

// ---- gated linear recurrence ------------------------------------------------------------------------------------------
// A thread is a (request, channel).  Tokens eight at a time: everything that does not depend on the state - gates,
// decays, the fed values, gelu of the gating branch - is formed for the eight first, then the eight steps of S <- a S + f.
template <typename T>
__global__ __launch_bounds__(256) void gated_linear_scan_kernel(
    const T* __restrict__ u, const float* __restrict__ gates, const float* __restrict__ gate_bias,
    const float* __restrict__ rate, const T* __restrict__ y, long y_stride, int channels, int block_width,
    float* __restrict__ state, long state_stride, const int* __restrict__ q_start, const int* __restrict__ seq_slots,
    T* __restrict__ out) {
  const int seq = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int first = q_start[seq], count = q_start[seq + 1] - first;
  const int b = c / block_width, j = c % block_width;
  const long gate_at = static_cast<long>(b) * 2 * block_width + j;      // (recurrence gate; the input gate block_width on)
  const float bias_r = gate_bias[gate_at], bias_i = gate_bias[gate_at + block_width], slope = rate[c];
  float* mine = state + static_cast<long>(seq_slots[seq]) * state_stride + c;
  float S = *mine;
  constexpr int kStep = 8;
  for (int base = 0; base < count; base += kStep) {
    float a[kStep], f[kStep], gy[kStep];
#pragma unroll
    for (int t = 0; t < kStep; ++t) {
      const long n = first + min(base + t, count - 1);
      const float r = sigmoid(gates[n * 2 * channels + gate_at] + bias_r);
      const float i = sigmoid(gates[n * 2 * channels + gate_at + block_width] + bias_i);
      a[t] = expf(slope * r);
      f[t] = sqrtf(1.f - a[t] * a[t]) * i * to_float(u[n * channels + c]);
      gy[t] = gelu_tanh(to_float(y[n * y_stride + c]));
    }
#pragma unroll
    for (int t = 0; t < kStep; ++t) {
      if (base + t < count) {
        S = fmaf(a[t], S, f[t]);
        out[static_cast<long>(first + base + t) * channels + c] = from_float<T>(S * gy[t]);
      }
    }
  }
  *mine = S;
}

}  // namespace

extern "C" {

int akv_retention(const void* projected, long stride, int dtype, int seqs, int heads, int dim, int vdim, int rot_dims,
                  const float* table, int table_positions, float key_scale, const float* decay, float eps, float* state,
                  long state_stride, const int* q_start, const int* seq_slots, const int* positions, void* out,
                  hipStream_t stream) {
  if (seqs <= 0) return 0;
  if (heads <= 0 || dim <= 0 || vdim <= 0 || vdim > 1024 || rot_dims < 0 || rot_dims % 2 || rot_dims > dim) return -2;
  if (rot_dims > 0 && (table == nullptr || table_positions <= 0)) return -2;
  int per_thread = 0;
  for (int r : {4, 8, 16, 32, 64}) {
    if (static_cast<long>(vdim) * ((dim + r - 1) / r) <= 1024) {
      per_thread = r;
      break;
    }
  }
  if (per_thread == 0) return -2;
  const int parts = (dim + per_thread - 1) / per_thread;
  const int threads = (vdim * parts + kWave - 1) / kWave * kWave;
  int batch = 16;
  auto lds_of = [&](int tb) { return static_cast<size_t>(tb) * (2 * dim + 2 * vdim + parts * vdim) * 4; };
  while (batch > 1 && lds_of(batch) > 64 * 1024) batch /= 2;
  if (lds_of(batch) > 64 * 1024) return -2;
  const dim3 grid(seqs, heads);
#define AKV_RETENTION(R)                                                                                                \
  AKV_DISPATCH(dtype, T, retention_kernel<T, R><<<grid, threads, lds_of(batch), stream>>>(                             \
                             static_cast<const T*>(projected), stride, heads, dim, vdim, rot_dims, table, table_positions, \
                             key_scale, decay, eps, state, state_stride, q_start, seq_slots, positions,                 \
                             static_cast<T*>(out), parts, batch))
  switch (per_thread) {
    case 4: AKV_RETENTION(4); break;
    case 8: AKV_RETENTION(8); break;
    case 16: AKV_RETENTION(16); break;
    case 32: AKV_RETENTION(32); break;
    default: AKV_RETENTION(64); break;
  }
#undef AKV_RETENTION
  return AKV_LAUNCH_STATUS();
}

int akv_gated_linear_scan(const void* u, int dtype, const float* gates, const float* gate_bias, const float* rate,
                          const void* y, long y_stride, int seqs, int channels, int blocks, float* state,
                          long state_stride, const int* q_start, const int* seq_slots, void* out, hipStream_t stream) {
  if (seqs <= 0) return 0;
  if (channels <= 0 || blocks <= 0 || channels % blocks) return -2;
  const dim3 grid(seqs, (channels + 255) / 256);
  AKV_DISPATCH(dtype, T, gated_linear_scan_kernel<T><<<grid, 256, 0, stream>>>(
                             static_cast<const T*>(u), gates, gate_bias, rate, static_cast<const T*>(y), y_stride, channels,
                             channels / blocks, state, state_stride, q_start, seq_slots, static_cast<T*>(out)));
  return AKV_LAUNCH_STATUS();
}
}

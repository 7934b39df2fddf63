// Short causal convolution over time on every channel of a step's packed tokens, with the last
// taps - 1 inputs of each live sequence carried in a slot pool between steps:
//   y_t = (add_input ? u_t : 0) + sum_j w[j][c] * u_(t - taps + 1 + j),   zeros before position 0
// (the weights arrive tap-major, [taps, C], so that neighbouring channels are neighbouring loads).
// A token whose tap reaches before the step's first row of its sequence reads the carried inputs; a
// sequence that starts at position 0 ignores what its slot holds.
//
//   causal_conv_kernel        one thread per (token, channel); fp32 arithmetic
//   causal_conv_vec_kernel    the same with 16-byte accesses (8 bf16 / 4 fp32 channels per thread), for
//                             channel counts and row pitches that allow them
//   causal_conv_state_kernel  after it (stream order): the slot's new content from the step's rows and,
//                             for portions shorter than taps - 1, the slot's old content
//   causal_conv_short_kernel  steps whose portions are all short (decode rows): one thread per (sequence,
//                             channel) walks the portion's tokens and then writes the slot, in one launch
#include "hybrid_common.h"

namespace llmctl_hybrid {

constexpr int CONV_MAX_TAPS = 16;

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(const T* __restrict__ u, int64_t u_stride, const float* __restrict__ w,
                                                          const float* __restrict__ state, const int* __restrict__ seq_of,
                                                          const int* __restrict__ cu, const int* __restrict__ start,
                                                          const int* __restrict__ sslot, T* __restrict__ y, int64_t y_stride, int C,
                                                          int taps, int add_input) {
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int s = seq_of[t];
  const int li = (int)t - cu[s];  // index inside the step's portion
  const int p0 = start[s];        // position of the portion's first token
  const float* st = state + (int64_t)sslot[s] * (taps - 1) * C;
  const float* wc = w + c;  // tap j of this channel: wc[j * C]
  const float cur = ldf(u + t * u_stride + c);
  float acc = wc[(int64_t)(taps - 1) * C] * cur;
  for (int k = 1; k < taps; ++k) {
    const int i = li - k;
    float v = 0.f;
    if (i >= 0) v = ldf(u + (t - k) * u_stride + c);
    else if (p0 + i >= 0) v = st[(int64_t)(taps - 1 + i) * C + c];
    acc += wc[(int64_t)(taps - 1 - k) * C] * v;
  }
  if (add_input) acc += cur;
  stf(y + t * y_stride + c, acc);
}

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_vec_kernel(const T* __restrict__ u, int64_t u_stride, const float* __restrict__ w,
                                                              const float* __restrict__ state, const int* __restrict__ seq_of,
                                                              const int* __restrict__ cu, const int* __restrict__ start,
                                                              const int* __restrict__ sslot, T* __restrict__ y, int C, int taps,
                                                              int add_input) {
  constexpr int N = Vec16<T>::N;
  const int64_t t = blockIdx.x;
  const int c = (blockIdx.y * 256 + threadIdx.x) * N;
  if (c >= C) return;
  const int s = seq_of[t];
  const int li = (int)t - cu[s];
  const int p0 = start[s];
  const float* st = state + (int64_t)sslot[s] * (taps - 1) * C;
  float cur[N], acc[N], v[N], wk[N];
  Vec16<T>::load(u + t * u_stride + c, cur);
#pragma unroll
  for (int i = 0; i < N; i += 4) Vec16<float>::load(w + (int64_t)(taps - 1) * C + c + i, wk + i);
#pragma unroll
  for (int i = 0; i < N; ++i) acc[i] = wk[i] * cur[i];
  for (int k = 1; k < taps; ++k) {
    const int i0 = li - k;
    if (i0 >= 0) {
      Vec16<T>::load(u + (t - k) * u_stride + c, v);
    } else if (p0 + i0 >= 0) {
#pragma unroll
      for (int i = 0; i < N; i += 4) Vec16<float>::load(st + (int64_t)(taps - 1 + i0) * C + c + i, v + i);
    } else {
      continue;
    }
#pragma unroll
    for (int i = 0; i < N; i += 4) Vec16<float>::load(w + (int64_t)(taps - 1 - k) * C + c + i, wk + i);
#pragma unroll
    for (int i = 0; i < N; ++i) acc[i] += wk[i] * v[i];
  }
  if (add_input) {
#pragma unroll
    for (int i = 0; i < N; ++i) acc[i] += cur[i];
  }
  Vec16<T>::store(y + t * (int64_t)C + c, acc);
}

// Portions of at most CONV_SHORT tokens: thread (sequence, channel) keeps the last taps - 1 inputs in
// registers, walks the portion and writes the slot back; the convolution and the state update are one launch.
constexpr int CONV_SHORT = 4;
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_short_kernel(const T* __restrict__ u, int64_t u_stride, const float* __restrict__ w,
                                                                float* __restrict__ state, const int* __restrict__ cu,
                                                                const int* __restrict__ start, const int* __restrict__ sslot,
                                                                T* __restrict__ y, int C, int taps, int add_input) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int a = cu[s], n = cu[s + 1] - a;
  if (n <= 0) return;
  const int p0 = start[s];
  float* st = state + (int64_t)sslot[s] * (taps - 1) * C;
  float h[CONV_MAX_TAPS];  // h[j]: the input taps - 1 - j positions before the current token (h[taps-1] = current)
  for (int j = 0; j < taps - 1; ++j) h[j] = (p0 - (taps - 1) + j >= 0) ? st[(int64_t)j * C + c] : 0.f;
  const float* wc = w + c;
  for (int i = 0; i < n; ++i) {
    const float cur = ldf(u + (int64_t)(a + i) * u_stride + c);
    h[taps - 1] = cur;
    float acc = add_input ? cur : 0.f;
    for (int j = 0; j < taps; ++j) acc += wc[(int64_t)j * C] * h[j];
    stf(y + (int64_t)(a + i) * C + c, acc);
    for (int j = 0; j < taps - 1; ++j) h[j] = h[j + 1];
  }
  for (int j = 0; j < taps - 1; ++j) st[(int64_t)j * C + c] = h[j];
}

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_state_kernel(const T* __restrict__ u, int64_t u_stride, float* __restrict__ state,
                                                                const int* __restrict__ cu, const int* __restrict__ start,
                                                                const int* __restrict__ sslot, int C, int taps) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int a = cu[s], n = cu[s + 1] - a;
  if (n <= 0) return;
  const int p0 = start[s];
  float* st = state + (int64_t)sslot[s] * (taps - 1) * C;
  // entry j holds the input of position (p0 + n) - (taps - 1) + j; ascending j reads old entries
  // j + n > j only, so the update is safe in place
  for (int j = 0; j < taps - 1; ++j) {
    const int li = n - (taps - 1) + j;
    float v = 0.f;
    if (li >= 0) v = ldf(u + (int64_t)(a + li) * u_stride + c);
    else if (p0 + li >= 0) v = st[(int64_t)(j + n) * C + c];
    st[(int64_t)j * C + c] = v;
  }
}

// max_len: the longest portion of the step if the host knows it (0 = unknown)
at::Tensor causal_conv(const at::Tensor& u, const at::Tensor& w, at::Tensor state, const at::Tensor& seq_of, const at::Tensor& cu,
                       const at::Tensor& start, const at::Tensor& sslot, bool add_input, int64_t max_len) {
  check_rows(u, "u");
  const int64_t T = u.size(0), C = u.size(1);
  HYB_CHECK(w.is_cuda() && w.dim() == 2 && w.is_contiguous() && w.scalar_type() == at::kFloat && w.size(1) == C, "w: contiguous fp32 [taps, C]");
  const int64_t taps = w.size(0);
  HYB_CHECK(taps >= 1 && taps <= CONV_MAX_TAPS, "taps in [1, 16]");
  HYB_CHECK(state.is_cuda() && state.is_contiguous() && state.scalar_type() == at::kFloat && state.dim() == 3 && state.size(1) == taps - 1 && state.size(2) == C,
            "state: contiguous fp32 [slots, taps - 1, C]");
  auto i32 = [](const at::Tensor& t) { return t.is_cuda() && t.is_contiguous() && t.scalar_type() == at::kInt; };
  HYB_CHECK(i32(seq_of) && i32(cu) && i32(start) && i32(sslot), "seq_of, cu, start, slots: contiguous int32 GPU tensors");
  const int64_t ns = start.numel();
  HYB_CHECK(seq_of.numel() == T && cu.numel() == ns + 1 && sslot.numel() == ns, "seq_of [T], cu [n + 1], start [n], slots [n]");
  c10::DeviceGuard guard(u.device());
  at::Tensor y = at::empty({T, C}, u.options());
  if (T == 0) return y;
  const unsigned cb = (unsigned)((C + 255) / 256);
  HYB_CHECK(cb <= 65535, "too many channels for one launch");
  dispatch_act(u, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    if (max_len >= 1 && max_len <= CONV_SHORT) {
      causal_conv_short_kernel<Tt><<<dim3((unsigned)ns, cb), 256, 0, cur_stream()>>>(
          (const Tt*)u.data_ptr(), u.stride(0), w.data_ptr<float>(), state.data_ptr<float>(), cu.data_ptr<int>(), start.data_ptr<int>(),
          sslot.data_ptr<int>(), (Tt*)y.data_ptr(), (int)C, (int)taps, add_input ? 1 : 0);
      return;
    }
    constexpr int N = Vec16<Tt>::N;
    if (C % 8 == 0 && aligned16<Tt>(u) && reinterpret_cast<uintptr_t>(state.data_ptr()) % 16 == 0 && reinterpret_cast<uintptr_t>(w.data_ptr()) % 16 == 0)
      causal_conv_vec_kernel<Tt><<<dim3((unsigned)T, (unsigned)((C / N + 255) / 256)), 256, 0, cur_stream()>>>(
          (const Tt*)u.data_ptr(), u.stride(0), w.data_ptr<float>(), state.data_ptr<float>(), seq_of.data_ptr<int>(), cu.data_ptr<int>(),
          start.data_ptr<int>(), sslot.data_ptr<int>(), (Tt*)y.data_ptr(), (int)C, (int)taps, add_input ? 1 : 0);
    else
      causal_conv_kernel<Tt><<<dim3((unsigned)T, cb), 256, 0, cur_stream()>>>(
          (const Tt*)u.data_ptr(), u.stride(0), w.data_ptr<float>(), state.data_ptr<float>(), seq_of.data_ptr<int>(), cu.data_ptr<int>(),
          start.data_ptr<int>(), sslot.data_ptr<int>(), (Tt*)y.data_ptr(), C, (int)C, (int)taps, add_input ? 1 : 0);
    if (taps > 1)
      causal_conv_state_kernel<Tt><<<dim3((unsigned)ns, cb), 256, 0, cur_stream()>>>(
          (const Tt*)u.data_ptr(), u.stride(0), state.data_ptr<float>(), cu.data_ptr<int>(), start.data_ptr<int>(), sslot.data_ptr<int>(),
          (int)C, (int)taps);
  });
  return y;
}

}  // namespace llmctl_hybrid

// mLSTM matrix memory, token by token.  Per (sequence, head): state S [dk, dv], normaliser n [dk] and
// log-scale m, all fp32, carried in slot pools between steps.  Per token, with log gates
//   i = cap tanh((zi + bi) / cap),   f = logsigmoid(cap tanh((zf + bf) / cap)):
//   m' = max(f + m, i);  S = e^(f + m - m') S + e^(i - m') k v^T;  n likewise with k alone;
//   o = S^T q / (max(|n . q|, e^(-m')) + 1e-6),  q already scaled.
// One block per (sequence, head, tile of 64 value columns): 4 waves split the dk rows into slabs, a
// lane owns one column of its slab in registers; lane r of a slab also owns n[row r of the slab].
// Column sums over slabs and n . q go through LDS (two barriers per token, double-buffered).
#include "hybrid_common.h"

namespace llmctl_hybrid {

__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

template <typename T, int DS>  // DS: rows per slab held in registers (>= ceil(dk / 4))
__global__ __launch_bounds__(256) void mlstm_scan_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                                         int64_t row_stride, const float* __restrict__ gates,
                                                         const float* __restrict__ b_i, const float* __restrict__ b_f, float cap,
                                                         float qscale, float* __restrict__ Sp, float* __restrict__ np,
                                                         float* __restrict__ mp, const int* __restrict__ slots,
                                                         const int* __restrict__ cu, const int* __restrict__ start,
                                                         float* __restrict__ out, int H, int dk, int dv) {
  extern __shared__ float sm[];
  float* qk = sm;                    // [2][2 dk]
  float* part = sm + 4 * dk;         // [2][4][65]
  constexpr int NR = (DS + 63) / 64;  // n rows per lane
  const int sq = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * 64;
  const int a = cu[sq], b = cu[sq + 1];
  if (a == b) return;
  const int slab = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int rows = (dk + 3) / 4;     // rows per slab
  const int d0 = slab * rows;
  const int col = v0 + lane;
  const bool cok = col < dv;
  const int64_t slot = slots[sq];
  float* Sb = Sp + (slot * H + h) * (int64_t)dk * dv;
  float* nb = np + (slot * H + h) * (int64_t)dk;
  const bool fresh = start[sq] == 0;
  float S[DS], nr[NR];
#pragma unroll
  for (int r = 0; r < DS; ++r) S[r] = (!fresh && cok && r < rows && d0 + r < dk) ? Sb[(int64_t)(d0 + r) * dv + col] : 0.f;
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int r = lane + 64 * i;
    nr[i] = (!fresh && r < rows && d0 + r < dk) ? nb[d0 + r] : 0.f;
  }
  float m = fresh ? 0.f : mp[slot * H + h];
  const float bi = b_i[h], bf = b_f[h];
  for (int t = a; t < b; ++t) {
    const int buf = (t - a) & 1;
    float* qs = qk + buf * 2 * dk;
    float* ks = qs + dk;
    for (int d = threadIdx.x; d < dk; d += 256) {
      qs[d] = ldf(q + t * row_stride + h * dk + d) * qscale;
      ks[d] = ldf(k + t * row_stride + h * dk + d);
    }
    const float vv = cok ? ldf(v + t * row_stride + h * dv + col) : 0.f;
    const float ig = cap * tanhf((gates[(int64_t)t * 2 * H + h] + bi) / cap);
    const float fg = log_sigmoid(cap * tanhf((gates[(int64_t)t * 2 * H + H + h] + bf) / cap));
    const float mn = fmaxf(fg + m, ig);
    const float da = expf(fg + m - mn), db = expf(ig - mn);
    m = mn;
    __syncthreads();
    float num = 0.f;
    const float bv = db * vv;
#pragma unroll
    for (int r = 0; r < DS; ++r) {
      if (r < rows && d0 + r < dk) {
        S[r] = da * S[r] + ks[d0 + r] * bv;
        num += S[r] * qs[d0 + r];
      }
    }
    float nq = 0.f;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int r = lane + 64 * i;
      if (r < rows && d0 + r < dk) {
        nr[i] = da * nr[i] + db * ks[d0 + r];
        nq += nr[i] * qs[d0 + r];
      }
    }
    nq = wave_sum(nq);
    float* pp = part + (buf * 4 + slab) * 65;
    pp[lane] = num;
    if (lane == 0) pp[64] = nq;
    __syncthreads();
    if (slab == 0 && cok) {
      const float* p0 = part + buf * 4 * 65;
      const float tot = p0[lane] + p0[65 + lane] + p0[130 + lane] + p0[195 + lane];
      const float nqt = p0[64] + p0[65 + 64] + p0[130 + 64] + p0[195 + 64];
      out[((int64_t)t * H + h) * dv + col] = tot / (fmaxf(fabsf(nqt), expf(-mn)) + 1e-6f);
    }
  }
#pragma unroll
  for (int r = 0; r < DS; ++r)
    if (cok && r < rows && d0 + r < dk) Sb[(int64_t)(d0 + r) * dv + col] = S[r];
  if (blockIdx.z == 0) {
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int r = lane + 64 * i;
      if (r < rows && d0 + r < dk) nb[d0 + r] = nr[i];
    }
    if (threadIdx.x == 0) mp[slot * H + h] = m;
  }
}

static void check_thd(const at::Tensor& t, int64_t T, int64_t H, int64_t d, int64_t row_stride, const char* name) {
  HYB_CHECK(t.is_cuda() && t.dim() == 3 && t.size(0) == T && t.size(1) == H && t.size(2) == d && (d == 1 || t.stride(2) == 1) &&
                (H == 1 || t.stride(1) == d) && (T <= 1 || t.stride(0) == row_stride), name, ": [T, H, d] rows of one projection output");
}

at::Tensor mlstm_scan(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& gates, const at::Tensor& b_i,
                      const at::Tensor& b_f, double cap, double qscale, at::Tensor S, at::Tensor n, at::Tensor m,
                      const at::Tensor& slots, const at::Tensor& cu, const at::Tensor& start) {
  HYB_CHECK(q.is_cuda() && q.dim() == 3 && v.dim() == 3, "q, k [T, H, dk], v [T, H, dv]");
  const int64_t T = q.size(0), H = q.size(1), dk = q.size(2), dv = v.size(2);
  const int64_t rs = T > 1 ? q.stride(0) : 0;
  check_thd(q, T, H, dk, rs, "q");
  check_thd(k, T, H, dk, rs, "k");
  check_thd(v, T, H, dv, rs, "v");
  HYB_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(), "q, k, v share a dtype");
  HYB_CHECK(gates.is_cuda() && gates.is_contiguous() && gates.scalar_type() == at::kFloat && gates.dim() == 2 && gates.size(0) == T && gates.size(1) == 2 * H, "gates: contiguous fp32 [T, 2H]");
  HYB_CHECK(b_i.scalar_type() == at::kFloat && b_f.scalar_type() == at::kFloat && b_i.numel() == H && b_f.numel() == H && b_i.is_contiguous() && b_f.is_contiguous() && b_i.is_cuda() && b_f.is_cuda(), "gate biases: fp32 [H]");
  const int64_t ns = slots.numel();
  HYB_CHECK(S.is_cuda() && S.is_contiguous() && S.scalar_type() == at::kFloat && S.dim() == 4 && S.size(1) == H && S.size(2) == dk && S.size(3) == dv, "S: contiguous fp32 [slots, H, dk, dv]");
  HYB_CHECK(n.is_cuda() && n.is_contiguous() && n.scalar_type() == at::kFloat && n.dim() == 3 && n.size(0) == S.size(0) && n.size(1) == H && n.size(2) == dk, "n: contiguous fp32 [slots, H, dk]");
  HYB_CHECK(m.is_cuda() && m.is_contiguous() && m.scalar_type() == at::kFloat && m.dim() == 2 && m.size(0) == S.size(0) && m.size(1) == H, "m: contiguous fp32 [slots, H]");
  for (const at::Tensor* t : {&slots, &cu, &start}) HYB_CHECK(t->is_cuda() && t->is_contiguous() && t->scalar_type() == at::kInt, "slots / cu / start: int32");
  HYB_CHECK(cu.numel() == ns + 1 && start.numel() == ns, "cu [n + 1], start [n], slots [n]");
  HYB_CHECK(dk >= 1 && dk <= 512 && H <= 65535, "dk <= 512");
  c10::DeviceGuard guard(q.device());
  at::Tensor out = at::empty({T, H, dv}, q.options().dtype(at::kFloat));
  if (T == 0 || ns == 0) return out;
  const int rows = (int)((dk + 3) / 4);
  const size_t lds = (size_t)(4 * dk + 2 * 4 * 65) * sizeof(float);
  dim3 grid((unsigned)ns, (unsigned)H, (unsigned)((dv + 63) / 64));
  const int64_t row_stride = T > 1 ? q.stride(0) : H * dk;
  HYB_CHECK(T <= 1 || (k.stride(0) == row_stride && v.stride(0) == row_stride), "q, k, v: the same row stride");
  dispatch_act(q, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    auto launch = [&](auto kern) {
      kern<<<grid, 256, lds, cur_stream()>>>((const Tt*)q.data_ptr(), (const Tt*)k.data_ptr(), (const Tt*)v.data_ptr(), row_stride,
                                            gates.data_ptr<float>(), b_i.data_ptr<float>(), b_f.data_ptr<float>(), (float)cap, (float)qscale,
                                            S.data_ptr<float>(), n.data_ptr<float>(), m.data_ptr<float>(), slots.data_ptr<int>(),
                                            cu.data_ptr<int>(), start.data_ptr<int>(), out.data_ptr<float>(), (int)H, (int)dk, (int)dv);
    };
    if (rows <= 8) launch(mlstm_scan_kernel<Tt, 8>);
    else if (rows <= 16) launch(mlstm_scan_kernel<Tt, 16>);
    else if (rows <= 32) launch(mlstm_scan_kernel<Tt, 32>);
    else if (rows <= 64) launch(mlstm_scan_kernel<Tt, 64>);
    else launch(mlstm_scan_kernel<Tt, 128>);
  });
  return out;
}

}  // namespace llmctl_hybrid

// mLSTM matrix memory, token by token.  Per (sequence, head): state S [dk, dv], normaliser n [dk] and
// log-scale m, all fp32, carried in slot pools between steps.  Per token, with log gates
//   i = cap tanh((zi + bi) / cap),   f = logsigmoid(cap tanh((zf + bf) / cap)):
//   m' = max(f + m, i);  S = e^(f + m - m') S + e^(i - m') k v^T;  n likewise with k alone;
//   o = S^T q / (max(|n . q|, e^(-m')) + 1e-6),  q already scaled.
// A pre-pass turns the gate pre-activations into i and f for all tokens at once.  The scan has two forms:
//   * dk <= 128: one wave per (sequence, head, tile of 64 value columns), a lane owns one column of S
//     (all dk rows in registers); k and q are spread over the lanes and reach the column update as
//     scalar operands (v_readlane), n is spread over the lanes and n . q is one wave reduction: no LDS
//     and no barrier in the token loop; the next token's operands are loaded during the current update;
//   * dk <= 512: one block per (sequence, head, tile): 4 waves split the dk rows into slabs, column
//     sums over slabs and n . q go through LDS (two barriers per token, double-buffered).
#include "hybrid_common.h"

#include <type_traits>

namespace llmctl_hybrid {

__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// raw [T, 2H] -> (i, f): i = cap tanh((z_i + b_i) / cap), f = logsigmoid(cap tanh((z_f + b_f) / cap))
__global__ void mlstm_gates_kernel(const float* __restrict__ raw, const float* __restrict__ b_i, const float* __restrict__ b_f,
                                   float cap, float* __restrict__ out, int64_t T, int H) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T * 2 * H) return;
  const int c = (int)(i % (2 * H));
  if (c < H) out[i] = cap * tanhf((raw[i] + b_i[c]) / cap);
  else out[i] = log_sigmoid(cap * tanhf((raw[i] + b_f[c - H]) / cap));
}

// Sum over the wave on the VALU's data-parallel primitives (quad swaps, half-row and row mirrors), then
// the four row sums through scalar registers: no LDS round trips.
__device__ __forceinline__ float wave_sum_dpp(float v) {
  auto dpp = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xf, 0xf, true));
  };
  v += dpp(v, std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
  v += dpp(v, std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]
  v += dpp(v, std::integral_constant<int, 0x141>{});  // row_half_mirror
  v += dpp(v, std::integral_constant<int, 0x140>{});  // row_mirror
  auto rl = [](float x, int l) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), l)); };
  return (rl(v, 0) + rl(v, 16)) + (rl(v, 32) + rl(v, 48));
}

// One wave per (sequence, head, 64 value columns); DK = register rows (>= dk), a multiple of 16.
// k and q of the token go through a wave-private LDS line and come back as broadcast reads.
template <typename T, int DK>
__global__ __launch_bounds__(64) void mlstm_scan_wave_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                                             int64_t row_stride, const float* __restrict__ gates, float qscale,
                                                             float* __restrict__ Sp, float* __restrict__ np, float* __restrict__ mp,
                                                             const int* __restrict__ slots, const int* __restrict__ cu,
                                                             const int* __restrict__ start, float* __restrict__ out, int H, int dk,
                                                             int dv, float* __restrict__ fsum, int write_out) {
  constexpr int NR = (DK + 63) / 64;
  constexpr int DP = NR * 64;
  __shared__ __attribute__((aligned(16))) float kq[2][2 * DP];
  const int sq = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * 64;
  const int a = cu[sq], b = cu[sq + 1];
  if (a == b) return;
  const int lane = threadIdx.x;
  const int col = v0 + lane;
  const bool cok = col < dv;
  const int64_t slot = slots[sq];
  float* Sb = Sp + (slot * H + h) * (int64_t)dk * dv;
  float* nb = np + (slot * H + h) * (int64_t)dk;
  const int st = start[sq];  // 0: new sequence (zero state, m = 0); -1: zero state with m = -inf (a chunk's
  const bool fresh = st <= 0;  // own contribution, to be merged into the carried state); else: load the slot
  float S[DK], nr[NR];
#pragma unroll
  for (int d = 0; d < DK; ++d) S[d] = (!fresh && cok && d < dk) ? Sb[(int64_t)d * dv + col] : 0.f;
#pragma unroll
  for (int i = 0; i < NR; ++i) nr[i] = (!fresh && lane + 64 * i < dk) ? nb[lane + 64 * i] : 0.f;
  float m = fresh ? (st < 0 ? -INFINITY : 0.f) : mp[slot * H + h];
  float facc = 0.f;
  // operands of TBATCH tokens are loaded ahead, one batch in flight while the previous one is processed
  // (a single wave has nothing else to hide a load behind)
  constexpr int TBATCH = 8;
  float kn[TBATCH][NR], qn[TBATCH][NR], vn[TBATCH], ign[TBATCH], fgn[TBATCH];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int j = 0; j < TBATCH; ++j) {
      const int t = min(t0 + j, b - 1);
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        const int d = lane + 64 * i;
        kn[j][i] = d < dk ? ldf(k + t * row_stride + h * dk + d) : 0.f;
        qn[j][i] = d < dk ? ldf(q + t * row_stride + h * dk + d) * qscale : 0.f;
      }
      vn[j] = cok ? ldf(v + t * row_stride + h * dv + col) : 0.f;
      ign[j] = gates[(int64_t)t * 2 * H + h];
      fgn[j] = gates[(int64_t)t * 2 * H + H + h];
    }
  };
  fetch(a);
  for (int t0 = a; t0 < b; t0 += TBATCH) {
    float kc[TBATCH][NR], qc[TBATCH][NR], vc[TBATCH], igc[TBATCH], fgc[TBATCH];
#pragma unroll
    for (int j = 0; j < TBATCH; ++j) {
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        kc[j][i] = kn[j][i];
        qc[j][i] = qn[j][i];
      }
      vc[j] = vn[j];
      igc[j] = ign[j];
      fgc[j] = fgn[j];
    }
    if (t0 + TBATCH < b) fetch(t0 + TBATCH);
#pragma unroll
    for (int j = 0; j < TBATCH; ++j) {
      const int t = t0 + j;
      if (t < b) {
        float* ks = kq[j & 1];
        float* qs = ks + DP;
        float nq = 0.f;
        const float mn = fmaxf(fgc[j] + m, igc[j]);
        const float da = __expf(fgc[j] + m - mn), db = __expf(igc[j] - mn);
        m = mn;
        facc += fgc[j];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          ks[lane + 64 * i] = kc[j][i];
          qs[lane + 64 * i] = qc[j][i];
          nr[i] = da * nr[i] + db * kc[j][i];
          nq += nr[i] * qc[j][i];
        }
        __builtin_amdgcn_wave_barrier();
        const float bv = db * vc[j];
        float num[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = 0; d < DK; d += 4) {
          if (d < dk) {  // rows past dk hold zeros in k and q: a partly used group of four is harmless
            const float4 k4 = *reinterpret_cast<const float4*>(ks + d);
            const float4 q4 = *reinterpret_cast<const float4*>(qs + d);
            S[d] = da * S[d] + k4.x * bv;
            S[d + 1] = da * S[d + 1] + k4.y * bv;
            S[d + 2] = da * S[d + 2] + k4.z * bv;
            S[d + 3] = da * S[d + 3] + k4.w * bv;
            num[0] += S[d] * q4.x;
            num[1] += S[d + 1] * q4.y;
            num[2] += S[d + 2] * q4.z;
            num[3] += S[d + 3] * q4.w;
          }
        }
        nq = wave_sum_dpp(nq);
        if (cok && write_out)
          out[((int64_t)t * H + h) * dv + col] = ((num[0] + num[1]) + (num[2] + num[3])) / (fmaxf(fabsf(nq), __expf(-mn)) + 1e-6f);
        __builtin_amdgcn_wave_barrier();
      }
    }
  }
#pragma unroll
  for (int d = 0; d < DK; ++d)
    if (cok && d < dk) Sb[(int64_t)d * dv + col] = S[d];
  if (blockIdx.z == 0) {
#pragma unroll
    for (int i = 0; i < NR; ++i)
      if (lane + 64 * i < dk) nb[lane + 64 * i] = nr[i];
    if (lane == 0) {
      mp[slot * H + h] = m;
      if (fsum != nullptr) fsum[(int64_t)sq * H + h] = facc;
    }
  }
}

// Merge per-chunk contributions into carried states.  Sequence s has chunks [base[s], base[s+1]); chunk
// p's own contribution (run from a zero state with m = -inf) is (locS, locn, locm)[p] with summed log
// forget gates fsum[p].  For every chunk the state at its first token is written to (iS, in, im)[p]:
// the sequence's carried state for its first chunk, then m' = max(F + m, m_loc),
// S' = e^(F + m - m') S + e^(m_loc - m') S_loc.  One thread per state entry, chunks in order.
__global__ void mlstm_chunk_combine_kernel(const float* __restrict__ Sp, const float* __restrict__ np, const float* __restrict__ mp,
                                           const int* __restrict__ slots, const int* __restrict__ start, const int* __restrict__ base,
                                           const float* __restrict__ locS, const float* __restrict__ locn, const float* __restrict__ locm,
                                           const float* __restrict__ fsum, float* __restrict__ iS, float* __restrict__ in_,
                                           float* __restrict__ im, int H, int dk, int dv) {
  const int s = blockIdx.x, h = blockIdx.y;
  const int64_t per = (int64_t)dk * dv + dk;  // S entries, then n entries
  const int64_t e = (int64_t)blockIdx.z * blockDim.x + threadIdx.x;
  if (e >= per) return;
  const bool isn = e >= (int64_t)dk * dv;
  const int64_t eo = isn ? e - (int64_t)dk * dv : e;
  const int64_t stride = isn ? dk : (int64_t)dk * dv;
  const float* real = isn ? np : Sp;
  const float* loc = isn ? locn : locS;
  float* init = isn ? in_ : iS;
  const int64_t slot = slots[s];
  const bool fresh = start[s] == 0;
  float val = fresh ? 0.f : real[(slot * H + h) * stride + eo];
  float m = fresh ? 0.f : mp[slot * H + h];
  for (int p = base[s]; p < base[s + 1]; ++p) {
    init[((int64_t)p * H + h) * stride + eo] = val;
    if (e == 0) im[(int64_t)p * H + h] = m;
    if (p + 1 < base[s + 1]) {
      const float F = fsum[(int64_t)p * H + h], ml = locm[(int64_t)p * H + h];
      const float mn = fmaxf(F + m, ml);
      val = expf(F + m - mn) * val + expf(ml - mn) * loc[((int64_t)p * H + h) * stride + eo];
      m = mn;
    }
  }
}

template <typename T, int DS>  // DS: rows per slab held in registers (>= ceil(dk / 4))
__global__ __launch_bounds__(256) void mlstm_scan_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                                         int64_t row_stride, const float* __restrict__ gates,
                                                         float qscale, float* __restrict__ Sp, float* __restrict__ np,
                                                         float* __restrict__ mp, const int* __restrict__ slots,
                                                         const int* __restrict__ cu, const int* __restrict__ start,
                                                         float* __restrict__ out, int H, int dk, int dv, float* __restrict__ fsum,
                                                         int write_out) {
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
  for (int t = a; t < b; ++t) {
    const int buf = (t - a) & 1;
    float* qs = qk + buf * 2 * dk;
    float* ks = qs + dk;
    for (int d = threadIdx.x; d < dk; d += 256) {
      qs[d] = ldf(q + t * row_stride + h * dk + d) * qscale;
      ks[d] = ldf(k + t * row_stride + h * dk + d);
    }
    const float vv = cok ? ldf(v + t * row_stride + h * dv + col) : 0.f;
    const float ig = gates[(int64_t)t * 2 * H + h], fg = gates[(int64_t)t * 2 * H + H + h];
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
    if (slab == 0 && cok && write_out) {
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
                      const at::Tensor& slots, const at::Tensor& cu, const at::Tensor& start, bool slab,
                      const c10::optional<at::Tensor>& fsum, bool write_out) {
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
  const bool wave = !slab && dk <= 128;
  if (fsum.has_value())
    HYB_CHECK(wave && fsum->is_cuda() && fsum->is_contiguous() && fsum->scalar_type() == at::kFloat && fsum->numel() == ns * H,
              "fsum: fp32 [n, H], wave-per-tile form only (dk <= 128)");
  c10::DeviceGuard guard(q.device());
  at::Tensor out = at::empty({T, H, dv}, q.options().dtype(at::kFloat));
  if (T == 0 || ns == 0) return out;
  at::Tensor act = at::empty_like(gates);
  {
    const int64_t ng = T * 2 * H;
    mlstm_gates_kernel<<<dim3((unsigned)((ng + 255) / 256)), 256, 0, cur_stream()>>>(gates.data_ptr<float>(), b_i.data_ptr<float>(),
                                                                                    b_f.data_ptr<float>(), (float)cap, act.data_ptr<float>(), T, (int)H);
  }
  const int rows = (int)((dk + 3) / 4);
  const size_t lds = (size_t)(4 * dk + 2 * 4 * 65) * sizeof(float);
  dim3 grid((unsigned)ns, (unsigned)H, (unsigned)((dv + 63) / 64));
  const int64_t row_stride = T > 1 ? q.stride(0) : H * dk;
  HYB_CHECK(T <= 1 || (k.stride(0) == row_stride && v.stride(0) == row_stride), "q, k, v: the same row stride");
  dispatch_act(q, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    auto go = [&](auto kern, int threads, size_t shm) {
      kern<<<grid, threads, shm, cur_stream()>>>((const Tt*)q.data_ptr(), (const Tt*)k.data_ptr(), (const Tt*)v.data_ptr(), row_stride,
                                                act.data_ptr<float>(), (float)qscale, S.data_ptr<float>(), n.data_ptr<float>(),
                                                m.data_ptr<float>(), slots.data_ptr<int>(), cu.data_ptr<int>(), start.data_ptr<int>(),
                                                out.data_ptr<float>(), (int)H, (int)dk, (int)dv,
                                                fsum.has_value() ? fsum->data_ptr<float>() : nullptr, write_out ? 1 : 0);
    };
    auto launch = [&](auto kern) { go(kern, 256, lds); };
    if (!slab && dk <= 16) go(mlstm_scan_wave_kernel<Tt, 16>, 64, 0);
    else if (!slab && dk <= 32) go(mlstm_scan_wave_kernel<Tt, 32>, 64, 0);
    else if (!slab && dk <= 64) go(mlstm_scan_wave_kernel<Tt, 64>, 64, 0);
    else if (!slab && dk <= 128) go(mlstm_scan_wave_kernel<Tt, 128>, 64, 0);
    else if (rows <= 8) launch(mlstm_scan_kernel<Tt, 8>);
    else if (rows <= 16) launch(mlstm_scan_kernel<Tt, 16>);
    else if (rows <= 32) launch(mlstm_scan_kernel<Tt, 32>);
    else if (rows <= 64) launch(mlstm_scan_kernel<Tt, 64>);
    else launch(mlstm_scan_kernel<Tt, 128>);
  });
  return out;
}

void mlstm_chunk_combine(const at::Tensor& S, const at::Tensor& n, const at::Tensor& m, const at::Tensor& slots, const at::Tensor& start,
                         const at::Tensor& base, const at::Tensor& locS, const at::Tensor& locn, const at::Tensor& locm,
                         const at::Tensor& fsum, at::Tensor iS, at::Tensor in_, at::Tensor im) {
  HYB_CHECK(S.is_cuda() && S.dim() == 4 && locS.dim() == 4 && iS.sizes() == locS.sizes() && in_.sizes() == locn.sizes() && im.sizes() == locm.sizes(), "state pools");
  const int64_t H = S.size(1), dk = S.size(2), dv = S.size(3), P = locS.size(0), ns = slots.numel();
  HYB_CHECK(locS.size(1) == H && locS.size(2) == dk && locS.size(3) == dv && locn.size(0) == P && locm.size(0) == P && fsum.numel() == P * H, "chunk pools [P, H, ...]");
  for (const at::Tensor* t : std::initializer_list<const at::Tensor*>{&S, &n, &m, &locS, &locn, &locm, &fsum, &iS, &in_, &im})
    HYB_CHECK(t->is_cuda() && t->is_contiguous() && t->scalar_type() == at::kFloat, "contiguous fp32 GPU tensors");
  for (const at::Tensor* t : {&slots, &start, &base}) HYB_CHECK(t->is_cuda() && t->is_contiguous() && t->scalar_type() == at::kInt, "int32 metadata");
  HYB_CHECK(start.numel() == ns && base.numel() == ns + 1, "start [n], base [n + 1]");
  if (ns == 0 || P == 0) return;
  c10::DeviceGuard guard(S.device());
  const int64_t per = dk * dv + dk;
  dim3 grid((unsigned)ns, (unsigned)H, (unsigned)((per + 255) / 256));
  mlstm_chunk_combine_kernel<<<grid, 256, 0, cur_stream()>>>(S.data_ptr<float>(), n.data_ptr<float>(), m.data_ptr<float>(), slots.data_ptr<int>(),
      start.data_ptr<int>(), base.data_ptr<int>(), locS.data_ptr<float>(), locn.data_ptr<float>(), locm.data_ptr<float>(), fsum.data_ptr<float>(),
      iS.data_ptr<float>(), in_.data_ptr<float>(), im.data_ptr<float>(), (int)H, (int)dk, (int)dv);
}

}  // namespace llmctl_hybrid

// Latent attention over a paged cache of rows [latent (rank) | rotary key part (rot)], one row per
// token shared by all heads.  Queries arrive in the same layout (the unrotated query part already
// carried into the latent space), so a score is one dot product of width R = rank + rot and the value
// of a key is the first ``rank`` entries of its row.  Sliding window (key j visible to query i when
// 0 <= i - j < window) and a per-head softmax sink (exp(sink) in the denominator, no value).
//
//   latent_kv_write     RMS norm of the latent, rotary of the key part, write the cache row
//   latent_q_assemble   [q_lat | rotary(q_rot)] per head
//   latent_attn_prefill prompt portions: one query per lane, keys streamed as wave-uniform rows
//   latent_attn_decode  one query per sequence: one key per lane for the scores, lanes over the
//                       value entries for the weighted sum
// Scores, softmax and the accumulators are fp32; angles are fp32 (position * inverse frequency).
#include "hybrid_common.h"

namespace llmctl_hybrid {

template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
                                                              const int* __restrict__ pos, const float* __restrict__ inv_freq,
                                                              T* __restrict__ cache, const int64_t* __restrict__ slots, int rk,
                                                              int dr, int rot_dims, float eps) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const T* xr = x + t * x_stride;
  T* out = cache + slot * (int64_t)(rk + dr);
  float q = 0.f;
  for (int c = threadIdx.x; c < rk; c += 256) {
    const float v = ldf(xr + c);
    q += v * v;
  }
  const float rstd = 1.0f / sqrtf(block_sum<4>(q, red) / (float)rk + eps);
  for (int c = threadIdx.x; c < rk; c += 256) stf(out + c, ldf(xr + c) * rstd * w[c]);
  const int half = rot_dims / 2;
  const float p = (float)pos[t];
  for (int i = threadIdx.x; i < half; i += 256) {
    float s, c;
    sincosf(p * inv_freq[i], &s, &c);
    const float u = ldf(xr + rk + i), v = ldf(xr + rk + i + half);
    stf(out + rk + i, u * c - v * s);
    stf(out + rk + i + half, v * c + u * s);
  }
  for (int i = rot_dims + threadIdx.x; i < dr; i += 256) stf(out + rk + i, ldf(xr + rk + i));
}

template <typename T>
__global__ __launch_bounds__(256) void latent_q_assemble_kernel(const T* __restrict__ ql, int64_t ql_st, int64_t ql_sh,
                                                                const T* __restrict__ q, const int* __restrict__ pos,
                                                                const float* __restrict__ inv_freq, T* __restrict__ qa, int H,
                                                                int rk, int dn, int dr, int rot_dims) {
  const int64_t t = blockIdx.x;
  const int R = rk + dr, half = rot_dims / 2;
  const float p = (float)pos[t];
  for (int i = threadIdx.x; i < H * rk; i += 256) {
    const int h = i / rk, c = i - h * rk;
    qa[(t * H + h) * R + c] = ql[t * ql_st + h * ql_sh + c];
  }
  for (int i = threadIdx.x; i < H * half; i += 256) {
    const int h = i / half, c = i - h * half;
    float s, co;
    sincosf(p * inv_freq[c], &s, &co);
    const T* qr = q + (t * H + h) * (int64_t)(dn + dr) + dn;
    const float u = ldf(qr + c), v = ldf(qr + c + half);
    stf(qa + (t * H + h) * R + rk + c, u * co - v * s);
    stf(qa + (t * H + h) * R + rk + c + half, v * co + u * s);
  }
  const int rest = dr - rot_dims;
  for (int i = threadIdx.x; i < H * rest; i += 256) {
    const int h = i / rest, c = rot_dims + (i - h * rest);
    qa[(t * H + h) * R + rk + c] = q[(t * H + h) * (int64_t)(dn + dr) + dn + c];
  }
}

// ---------------------------------------------------------------------------------------- prefill
// grid (q tiles of 64, sequences, heads * value tiles); one wave per block, lane = query.
template <typename T, int VT>
__global__ __launch_bounds__(64) void latent_attn_prefill_kernel(const T* __restrict__ qa, const T* __restrict__ cache,
                                                                 const int* __restrict__ bt, int bt_stride, const int* __restrict__ cu,
                                                                 const int* __restrict__ ctx, const float* __restrict__ sink,
                                                                 T* __restrict__ out, int H, int R, int rk, int bs, int window,
                                                                 float scale, int nvt) {
  extern __shared__ float qT[];  // [R][64]
  const int n = blockIdx.y;
  const int h = blockIdx.z / nvt, v0 = (blockIdx.z % nvt) * VT;
  const int a = cu[n], qlen = cu[n + 1] - a;
  const int q0 = blockIdx.x * 64;
  if (q0 >= qlen) return;
  const int lane = threadIdx.x;
  const int p0 = ctx[n] - qlen;  // position of the sequence's first query row
  const bool live = q0 + lane < qlen;
  const int qp = p0 + q0 + lane;
  const int64_t qrow = ((int64_t)(a + q0 + (live ? lane : 0)) * H + h) * R;
  for (int d = 0; d < R; ++d) qT[d * 64 + lane] = live ? ldf(qa + qrow + d) : 0.f;
  const int last = p0 + min(q0 + 63, qlen - 1);
  int j0 = p0 + q0 - window + 1;
  if (j0 < 0) j0 = 0;
  float m = sink[h], l = 1.0f;  // the sink: exp(sink - m) with m = sink
  float acc[VT];
#pragma unroll
  for (int i = 0; i < VT; ++i) acc[i] = 0.f;
  const int* btn = bt + (int64_t)n * bt_stride;
  for (int j = j0; j <= last; ++j) {
    const T* row = cache + ((int64_t)btn[j / bs] * bs + j % bs) * R;
    float s = 0.f;
    for (int d = 0; d < R; ++d) s += qT[d * 64 + lane] * ldf(row + d);
    s *= scale;
    const int dist = qp - j;
    if (live && dist >= 0 && dist < window) {
      const float mn = fmaxf(m, s);
      const float corr = expf(m - mn), p = expf(s - mn);
      l = l * corr + p;
#pragma unroll
      for (int i = 0; i < VT; ++i) acc[i] = acc[i] * corr + p * ldf(row + min(v0 + i, R - 1));
      m = mn;
    }
  }
  if (!live) return;
  const float inv = 1.0f / l;
  T* o = out + ((int64_t)(a + q0 + lane) * H + h) * rk;
#pragma unroll
  for (int i = 0; i < VT; ++i)
    if (v0 + i < rk) stf(o + v0 + i, acc[i] * inv);
}

// ----------------------------------------------------------------------------------------- decode
// grid (sequences, heads); 4 waves, each takes chunks of 64 keys (one key per lane for the score).
template <typename T, int NA>
__global__ __launch_bounds__(256) void latent_attn_decode_kernel(const T* __restrict__ qa, const T* __restrict__ cache,
                                                                 const int* __restrict__ bt, int bt_stride, const int* __restrict__ ctx,
                                                                 const float* __restrict__ sink, T* __restrict__ out, int H, int R,
                                                                 int rk, int bs, int window, float scale) {
  extern __shared__ float sm[];
  float* qs = sm;                                   // [R]
  float* pw = qs + R + (R & 1);                     // [4][64]; the padding keeps ro 8-byte aligned
  int64_t* ro = reinterpret_cast<int64_t*>(pw + 256);  // [4][64]
  float* ml = reinterpret_cast<float*>(ro + 256);   // [4][2]
  float* ac = ml + 8;                               // [4][rk]
  const int n = blockIdx.x, h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int len = ctx[n];
  const int lo = max(0, len - window);
  const int nk = len - lo;
  const T* qr = qa + ((int64_t)n * H + h) * R;
  for (int d = threadIdx.x; d < R; d += 256) qs[d] = ldf(qr + d);
  __syncthreads();
  const int* btn = bt + (int64_t)n * bt_stride;
  float m = -INFINITY, l = 0.f;
  float acc[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i) acc[i] = 0.f;
  for (int c = wave * 64; c < nk; c += 256) {
    const int j = lo + c + lane;
    const bool ok = c + lane < nk;
    int64_t slot = 0;
    float s = -INFINITY;
    if (ok) {
      slot = (int64_t)btn[j / bs] * bs + j % bs;
      const T* row = cache + slot * R;
      float d0 = 0.f;
      for (int d = 0; d < R; ++d) d0 += qs[d] * ldf(row + d);
      s = d0 * scale;
    }
    const float mn = fmaxf(m, wave_max(s));  // at least one key of the chunk is valid: finite
    const float p = ok ? expf(s - mn) : 0.f;
    const float corr = expf(m - mn);         // m = -inf on the first chunk: 0
    l = l * corr + wave_sum(p);
    m = mn;
    pw[wave * 64 + lane] = p;
    ro[wave * 64 + lane] = slot;
    __builtin_amdgcn_wave_barrier();
    const int cnt = min(64, nk - c);
#pragma unroll
    for (int i = 0; i < NA; ++i) acc[i] *= corr;
    for (int jj = 0; jj < cnt; ++jj) {
      const float pj = pw[wave * 64 + jj];
      const T* row = cache + ro[wave * 64 + jj] * R;
#pragma unroll
      for (int i = 0; i < NA; ++i) {
        const int d = lane + 64 * i;
        if (d < rk) acc[i] += pj * ldf(row + d);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (lane == 0) {
    ml[wave * 2] = m;
    ml[wave * 2 + 1] = l;
  }
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int d = lane + 64 * i;
    if (d < rk) ac[wave * rk + d] = acc[i];
  }
  __syncthreads();
  const float sk = sink[h];
  float M = sk;
#pragma unroll
  for (int w = 0; w < 4; ++w) M = fmaxf(M, ml[w * 2]);
  float L = expf(sk - M);
  float f[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    f[w] = ml[w * 2 + 1] > 0.f ? expf(ml[w * 2] - M) : 0.f;
    L += ml[w * 2 + 1] * f[w];
  }
  T* o = out + ((int64_t)n * H + h) * rk;
  for (int d = threadIdx.x; d < rk; d += 256) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) v += ac[w * rk + d] * f[w];
    stf(o + d, v / L);
  }
}

// latent_attn_mfma.hip: the matrix-core form for bf16 shapes that fit it
bool latent_attn_mfma_ok(const at::Tensor& qa, int64_t rk);
void latent_attn_mfma(const at::Tensor& qa, const at::Tensor& cache, const at::Tensor& bt, const at::Tensor* cu, const at::Tensor& ctx,
                      int64_t window, const at::Tensor& sink, double scale, int64_t rk, int64_t max_q, at::Tensor& out);

// ------------------------------------------------------------------------------------------ host
static void check_cache(const at::Tensor& cache, const at::Tensor& like, int64_t R) {
  HYB_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 && cache.size(2) == R && cache.scalar_type() == like.scalar_type(),
            "cache: contiguous [blocks, block_size, rank + rot] of the activation dtype");
}

static void check_i32(const at::Tensor& t, const char* name) {
  HYB_CHECK(t.is_cuda() && t.is_contiguous() && t.scalar_type() == at::kInt, name, ": contiguous int32 GPU tensor");
}

void latent_kv_write(const at::Tensor& dkv, const at::Tensor& norm_w, double eps, const at::Tensor& pos, const at::Tensor& inv_freq,
                     int64_t rot_dims, at::Tensor cache, const at::Tensor& slots) {
  check_rows(dkv, "dkv");
  const int64_t T = dkv.size(0), R = dkv.size(1), rk = norm_w.numel();
  HYB_CHECK(rk >= 1 && rk <= R && norm_w.scalar_type() == at::kFloat && norm_w.is_contiguous(), "norm weight: fp32 [rank]");
  const int64_t dr = R - rk;
  HYB_CHECK(rot_dims % 2 == 0 && rot_dims <= dr && inv_freq.numel() == rot_dims / 2 && inv_freq.scalar_type() == at::kFloat && inv_freq.is_cuda() && inv_freq.is_contiguous(), "rotary: even dims <= rot part, fp32 inverse frequencies [dims/2]");
  check_cache(cache, dkv, R);
  check_i32(pos, "pos");
  HYB_CHECK(pos.numel() == T && slots.is_cuda() && slots.is_contiguous() && slots.scalar_type() == at::kLong && slots.numel() == T, "pos int32 [T], slots int64 [T]");
  if (T == 0) return;
  c10::DeviceGuard guard(dkv.device());
  dispatch_act(dkv, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    latent_kv_write_kernel<Tt><<<dim3((unsigned)T), 256, 0, cur_stream()>>>(
        (const Tt*)dkv.data_ptr(), dkv.stride(0), norm_w.data_ptr<float>(), pos.data_ptr<int>(), inv_freq.data_ptr<float>(),
        (Tt*)cache.data_ptr(), slots.data_ptr<int64_t>(), (int)rk, (int)dr, (int)rot_dims, (float)eps);
  });
}

at::Tensor latent_q_assemble(const at::Tensor& q_lat, const at::Tensor& q, const at::Tensor& pos, const at::Tensor& inv_freq,
                             int64_t rot_dims, int64_t dn) {
  HYB_CHECK(q.is_cuda() && q.is_contiguous() && q.dim() == 3, "q: contiguous [T, H, dn + rot]");
  const int64_t T = q.size(0), H = q.size(1), dr = q.size(2) - dn;
  HYB_CHECK(q_lat.is_cuda() && q_lat.dim() == 3 && q_lat.size(0) == T && q_lat.size(1) == H && (q_lat.size(2) == 1 || q_lat.stride(2) == 1) && q_lat.scalar_type() == q.scalar_type(), "q_lat: [T, H, rank], unit last stride, q's dtype");
  const int64_t rk = q_lat.size(2);
  HYB_CHECK(dr >= 0 && rot_dims % 2 == 0 && rot_dims <= dr && inv_freq.numel() == rot_dims / 2 && inv_freq.scalar_type() == at::kFloat && inv_freq.is_cuda() && inv_freq.is_contiguous(), "rotary: even dims <= rot part");
  check_i32(pos, "pos");
  HYB_CHECK(pos.numel() == T, "pos: int32 [T]");
  c10::DeviceGuard guard(q.device());
  at::Tensor qa = at::empty({T, H, rk + dr}, q.options());
  if (T == 0) return qa;
  dispatch_act(q, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    latent_q_assemble_kernel<Tt><<<dim3((unsigned)T), 256, 0, cur_stream()>>>(
        (const Tt*)q_lat.data_ptr(), q_lat.stride(0), q_lat.stride(1), (const Tt*)q.data_ptr(), pos.data_ptr<int>(),
        inv_freq.data_ptr<float>(), (Tt*)qa.data_ptr(), (int)H, (int)rk, (int)dn, (int)dr, (int)rot_dims);
  });
  return qa;
}

at::Tensor latent_attn_prefill(const at::Tensor& qa, const at::Tensor& cache, const at::Tensor& bt, const at::Tensor& cu,
                               const at::Tensor& ctx, int64_t window, const at::Tensor& sink, double scale, int64_t rk, int64_t max_q,
                               bool mfma) {
  HYB_CHECK(qa.is_cuda() && qa.is_contiguous() && qa.dim() == 3, "qa: contiguous [T, H, R]");
  const int64_t T = qa.size(0), H = qa.size(1), R = qa.size(2);
  check_cache(cache, qa, R);
  check_i32(bt, "block tables");
  check_i32(cu, "cu");
  check_i32(ctx, "ctx");
  const int64_t ns = ctx.numel();
  HYB_CHECK(bt.dim() == 2 && bt.size(0) == ns && cu.numel() == ns + 1, "block tables [n, max_blocks], cu [n + 1], ctx [n]");
  HYB_CHECK(sink.is_cuda() && sink.scalar_type() == at::kFloat && sink.is_contiguous() && sink.numel() == H, "sink: fp32 [H]");
  HYB_CHECK(rk >= 1 && rk <= R && window >= 1 && max_q >= 1, "rank <= R, window >= 1, max_q >= 1");
  HYB_CHECK((size_t)R * 64 * sizeof(float) <= 160 * 1024, "rank + rot too wide for the query tile in LDS");
  c10::DeviceGuard guard(qa.device());
  at::Tensor out = at::empty({T, H, rk}, qa.options());
  if (T == 0 || ns == 0) return out;
  if (mfma && latent_attn_mfma_ok(qa, rk)) {
    latent_attn_mfma(qa, cache, bt, &cu, ctx, window, sink, scale, rk, max_q, out);
    return out;
  }
  const int VT = rk <= 32 ? 32 : (rk <= 64 ? 64 : 128);
  const int nvt = (int)((rk + VT - 1) / VT);
  HYB_CHECK(H * nvt <= 65535 && ns <= 65535, "grid too large");
  dim3 grid((unsigned)((max_q + 63) / 64), (unsigned)ns, (unsigned)(H * nvt));
  const size_t lds = (size_t)R * 64 * sizeof(float);
  dispatch_act(qa, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    auto launch = [&](auto kern) {
      if (lds > 64 * 1024) HYB_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess, "LDS size");
      kern<<<grid, 64, lds, cur_stream()>>>((const Tt*)qa.data_ptr(), (const Tt*)cache.data_ptr(), bt.data_ptr<int>(), (int)bt.size(1),
                                           cu.data_ptr<int>(), ctx.data_ptr<int>(), sink.data_ptr<float>(), (Tt*)out.data_ptr(), (int)H,
                                           (int)R, (int)rk, (int)cache.size(1), (int)window, (float)scale, nvt);
    };
    if (VT == 32) launch(latent_attn_prefill_kernel<Tt, 32>);
    else if (VT == 64) launch(latent_attn_prefill_kernel<Tt, 64>);
    else launch(latent_attn_prefill_kernel<Tt, 128>);
  });
  return out;
}

at::Tensor latent_attn_decode(const at::Tensor& qa, const at::Tensor& cache, const at::Tensor& bt, const at::Tensor& ctx,
                              int64_t window, const at::Tensor& sink, double scale, int64_t rk, bool mfma) {
  HYB_CHECK(qa.is_cuda() && qa.is_contiguous() && qa.dim() == 3, "qa: contiguous [n, H, R]");
  const int64_t ns = qa.size(0), H = qa.size(1), R = qa.size(2);
  check_cache(cache, qa, R);
  check_i32(bt, "block tables");
  check_i32(ctx, "ctx");
  HYB_CHECK(bt.dim() == 2 && bt.size(0) == ns && ctx.numel() == ns, "block tables [n, max_blocks], ctx [n]");
  HYB_CHECK(sink.is_cuda() && sink.scalar_type() == at::kFloat && sink.is_contiguous() && sink.numel() == H, "sink: fp32 [H]");
  HYB_CHECK(rk >= 1 && rk <= R && window >= 1, "rank <= R, window >= 1");
  c10::DeviceGuard guard(qa.device());
  at::Tensor out = at::empty({ns, H, rk}, qa.options());
  if (ns == 0) return out;
  if (mfma && latent_attn_mfma_ok(qa, rk)) {
    latent_attn_mfma(qa, cache, bt, nullptr, ctx, window, sink, scale, rk, 1, out);
    return out;
  }
  HYB_CHECK(rk <= 512, "generic decode kernel: rank <= 512");
  const int64_t Rp = R + (R & 1);  // keeps the int64 array 8-byte aligned
  const size_t lds = (size_t)(Rp + 256) * 4 + 256 * 8 + 8 * 4 + (size_t)4 * rk * 4;
  HYB_CHECK(lds <= 64 * 1024 && H <= 65535, "rank + rot too wide");
  dim3 grid((unsigned)ns, (unsigned)H);
  dispatch_act(qa, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    if (rk <= 128)
      latent_attn_decode_kernel<Tt, 2><<<grid, 256, lds, cur_stream()>>>((const Tt*)qa.data_ptr(), (const Tt*)cache.data_ptr(), bt.data_ptr<int>(),
          (int)bt.size(1), ctx.data_ptr<int>(), sink.data_ptr<float>(), (Tt*)out.data_ptr(), (int)H, (int)R, (int)rk, (int)cache.size(1), (int)window, (float)scale);
    else
      latent_attn_decode_kernel<Tt, 8><<<grid, 256, lds, cur_stream()>>>((const Tt*)qa.data_ptr(), (const Tt*)cache.data_ptr(), bt.data_ptr<int>(),
          (int)bt.size(1), ctx.data_ptr<int>(), sink.data_ptr<float>(), (Tt*)out.data_ptr(), (int)H, (int)R, (int)rk, (int)cache.size(1), (int)window, (float)scale);
  });
  return out;
}

}  // namespace llmctl_hybrid

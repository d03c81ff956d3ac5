// Paged attention with a sliding window for any head size: key norm + K/V store, and the attention itself (one wavefront
// per (token row, query head): portions of prompts and single decoded tokens are the same launch). Scores, softmax and the
// output accumulation are 32-bit; the query norm and the sigmoid output gate are fused in.
#include "seq_common.h"

namespace {

constexpr int MAX_HEAD = 256;

// one wavefront per (token, kv head)
template <typename T>
__global__ void knorm_kvstore_kernel(const T* __restrict__ k, const T* __restrict__ v, int64_t stride, const T* __restrict__ knorm,
                                     float eps, int G, int d, int dv, const int32_t* __restrict__ slots, T* __restrict__ k_cache,
                                     T* __restrict__ v_cache) {
  const int64_t t = blockIdx.x;
  const int g = blockIdx.y, lane = threadIdx.x;
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const T* kp = k + t * stride + (int64_t)g * d;
  float kv[MAX_HEAD / 64];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < MAX_HEAD / 64; ++i) {
    const int c = lane + 64 * i;
    kv[i] = c < d ? ldf(kp + c) : 0.f;
    ss += kv[i] * kv[i];
  }
  float r = 1.f;
  if (knorm) r = rsqrtf(wave_sum(ss) / (float)d + eps);
  T* kc = k_cache + (slot * G + g) * d;
#pragma unroll
  for (int i = 0; i < MAX_HEAD / 64; ++i) {
    const int c = lane + 64 * i;
    if (c < d) stf(kc + c, knorm ? kv[i] * r * ldf(knorm + c) : kv[i]);
  }
  const T* vp = v + t * stride + (int64_t)g * dv;
  T* vc = v_cache + (slot * G + g) * dv;
  for (int c = lane; c < dv; c += 64) vc[c] = vp[c];
}

// one wavefront per (token, query head). Keys go in rounds of 64 (one per lane): score, running maximum, weights into LDS,
// then every lane accumulates its value columns over the round's keys.
template <typename T>
__global__ void window_attn_kernel(const T* __restrict__ q, int64_t q_stride, const T* __restrict__ qnorm, float eps,
                                   const T* __restrict__ gate, int64_t gate_stride, const T* __restrict__ k_cache,
                                   const T* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int64_t bt_stride,
                                   int block_size, const int32_t* __restrict__ cu_q, const int32_t* __restrict__ ctx0,
                                   const int32_t* __restrict__ tseq, int H, int G, int d, int dv, float scale, int window,
                                   T* __restrict__ out) {
  __shared__ float qs[MAX_HEAD];
  __shared__ float ps[64];
  __shared__ int64_t slot_s[64];
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int s = tseq[t];
  const int64_t pos = (int64_t)ctx0[s] + (t - cu_q[s]);
  const int g = h / (H / G);
  // query (+ norm) into LDS
  {
    const T* qp = q + t * q_stride + (int64_t)h * d;
    float qv[MAX_HEAD / 64];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAX_HEAD / 64; ++i) {
      const int c = lane + 64 * i;
      qv[i] = c < d ? ldf(qp + c) : 0.f;
      ss += qv[i] * qv[i];
    }
    const float r = qnorm ? rsqrtf(wave_sum(ss) / (float)d + eps) : 1.f;
#pragma unroll
    for (int i = 0; i < MAX_HEAD / 64; ++i) {
      const int c = lane + 64 * i;
      if (c < d) qs[c] = qnorm ? qv[i] * r * ldf(qnorm + c) : qv[i];
    }
  }
  __syncthreads();
  const int64_t lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  const int32_t* bt = block_tables + (int64_t)s * bt_stride;
  float m = -INFINITY, l = 0.f;
  float acc[MAX_HEAD / 64];
#pragma unroll
  for (int i = 0; i < MAX_HEAD / 64; ++i) acc[i] = 0.f;
  for (int64_t j0 = lo; j0 <= pos; j0 += 64) {
    const int64_t j = j0 + lane;
    const bool live = j <= pos;
    float sc = -INFINITY;
    int64_t slot = 0;
    if (live) {
      slot = (int64_t)bt[j / block_size] * block_size + j % block_size;
      const T* kp = k_cache + (slot * G + g) * d;
      float dot = 0.f;
      for (int c = 0; c < d; ++c) dot += qs[c] * ldf(kp + c);
      sc = dot * scale;
    }
    const float mn = fmaxf(m, wave_max(sc));          // finite: lane 0 of every round is live
    const float alpha = expf(m - mn);                 // 0 in the first round (m = -inf)
    const float p = live ? expf(sc - mn) : 0.f;
    l = l * alpha + wave_sum(p);
    m = mn;
    __syncthreads();                                  // the previous round's readers are done
    ps[lane] = p;
    slot_s[lane] = slot;
    __syncthreads();
    const int cnt = (int)((pos - j0 + 1) < 64 ? (pos - j0 + 1) : 64);
#pragma unroll
    for (int i = 0; i < MAX_HEAD / 64; ++i) {
      const int c = lane + 64 * i;
      if (c < dv) {
        float a = acc[i] * alpha;
        for (int jj = 0; jj < cnt; ++jj) a += ps[jj] * ldf(v_cache + (slot_s[jj] * G + g) * dv + c);
        acc[i] = a;
      }
    }
  }
  const float inv = 1.f / l;
#pragma unroll
  for (int i = 0; i < MAX_HEAD / 64; ++i) {
    const int c = lane + 64 * i;
    if (c < dv) {
      float o = acc[i] * inv;
      if (gate) {
        const float gv = ldf(gate + t * gate_stride + (int64_t)h * dv + c);
        o *= 1.f / (1.f + expf(-gv));
      }
      stf(out + (t * H + h) * dv + c, o);
    }
  }
}

}  // namespace

extern "C" int nvs_knorm_kvstore(const void* k, const void* v, int64_t stride, int dtype, const void* knorm, float eps, int G, int d,
                                 int dv, const int32_t* slots, int64_t n, void* k_cache, void* v_cache, void* stream) {
  NVS_REQUIRE(k && v && slots && k_cache && v_cache, "nvs_knorm_kvstore: null argument");
  NVS_REQUIRE(G > 0 && G <= 65535 && d > 0 && d <= MAX_HEAD && dv > 0 && dv <= MAX_HEAD && n >= 0, "nvs_knorm_kvstore: G %d d %d dv %d", G,
              d, dv);
  if (n == 0) return NVS_OK;
  NVS_DISPATCH(dtype, knorm_kvstore_kernel<T><<<dim3((unsigned)n, G), dim3(64), 0, (hipStream_t)stream>>>(
                          (const T*)k, (const T*)v, stride, (const T*)knorm, eps, G, d, dv, slots, (T*)k_cache, (T*)v_cache));
  return nvs_check_launch("nvs_knorm_kvstore");
}

extern "C" int nvs_window_attn(const void* q, int64_t q_stride, const void* qnorm, float eps, const void* gate, int64_t gate_stride,
                               int dtype, const void* k_cache, const void* v_cache, const int32_t* block_tables, int64_t bt_stride,
                               int block_size, const int32_t* cu_q, const int32_t* ctx0, const int32_t* tseq, int nseq, int64_t n, int H,
                               int G, int d, int dv, float scale, int window, void* out, void* stream) {
  NVS_REQUIRE(q && k_cache && v_cache && block_tables && cu_q && ctx0 && tseq && out, "nvs_window_attn: null argument");
  NVS_REQUIRE(H > 0 && H <= 65535 && G > 0 && H % G == 0 && d > 0 && d <= MAX_HEAD && dv > 0 && dv <= MAX_HEAD && block_size > 0 && n >= 0,
              "nvs_window_attn: H %d G %d d %d dv %d block %d", H, G, d, dv, block_size);
  if (n == 0 || nseq == 0) return NVS_OK;
  NVS_DISPATCH(dtype, window_attn_kernel<T><<<dim3((unsigned)n, H), dim3(64), 0, (hipStream_t)stream>>>(
                          (const T*)q, q_stride, (const T*)qnorm, eps, (const T*)gate, gate_stride, (const T*)k_cache, (const T*)v_cache,
                          block_tables, bt_stride, block_size, cu_q, ctx0, tseq, H, G, d, dv, scale, window, (T*)out));
  return nvs_check_launch("nvs_window_attn");
}

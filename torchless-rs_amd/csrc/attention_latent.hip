// The row-wise steps of an attention whose queries, keys and values come out of latents:
//
//   c_q = rms(W_dq h) * w_q ,  q = W_uq c_q
//   c   = rms(W_dkv h) * w_c , k = W_uk c ,  v = W_uv c        (per head, laid out head by head)
//   out = heads * logistic(W_g h)                               (a gate per CHANNEL of the heads)
//
// rms(t) = t / sqrt(mean(t^2) + eps).  The products are ordinary ones; between them run
// `latent_norms` (the fused down projection [c_q | c | g] in float: the two norms and the gate's
// logistic function, all in float, the latents rounded to the compute type once), `split_heads`
// (the up projections in float: q to rows, k and v to rows or, when every sequence brings one
// token, straight into the page of the row's position) and `mul_gate` after the attention.
#include "common.hpp"

namespace tl {

// proj[n, :] = [a (na) | b (nb) | g (ng)].  blockIdx.y: 0 norms a, 1 norms b, 2 gates.
template <typename T>
__global__ void __launch_bounds__(256)
latent_norms_kernel(const float* __restrict__ proj, int na, int nb, int ng, const float* __restrict__ wa,
                    const float* __restrict__ wb, float eps, T* __restrict__ a, T* __restrict__ b,
                    float* __restrict__ gate) {
  __shared__ float sh[4];
  const int n = blockIdx.x, section = blockIdx.y;
  const float* row = proj + (size_t)n * (na + nb + ng);
  if (section == 2) {
    for (int i = threadIdx.x; i < ng; i += 256) gate[(size_t)n * ng + i] = 1.0f / (1.0f + expf(-row[na + nb + i]));
    return;
  }
  const int off = section ? na : 0, len = section ? nb : na;
  const float* w = section ? wb : wa;
  T* out = (section ? b : a) + (size_t)n * len;
  float ss = 0.f;
  for (int i = threadIdx.x; i < len; i += 256) {
    const float t = row[off + i];
    ss += t * t;
  }
  ss = block_sum<256>(ss, sh);
  const float rms = sqrtf(ss / (float)len + eps);
  for (int i = threadIdx.x; i < len; i += 256) out[i] = from_f32<T>((row[off + i] / rms) * w[i]);
}

// qf[n, nq*dk] (row stride q_stride), kf[n, nkv*dk] and vf[n, nkv*dv] (row stride kv_stride each, so
// that k and v may be the two halves of one product) in float -> q, and k and v as rows or
// (pages != null: row n is sequence n) into the page of the row's position, values transposed.
// A workgroup takes HEADS_CHUNK consecutive outputs of a row's [q | k | v].
constexpr int HEADS_CHUNK = 1024;

template <typename T>
__global__ void __launch_bounds__(256)
split_heads_kernel(const float* __restrict__ qf, int q_stride, const float* __restrict__ kf,
                   const float* __restrict__ vf, int kv_stride, const int* __restrict__ row_pos, int nq, int nkv,
                   int dk, int dv, T* __restrict__ q, T* __restrict__ k, T* __restrict__ v,
                   const int* __restrict__ table, int table_stride, int ring_pages, T* __restrict__ pages, int chunk) {
  const int n = blockIdx.x;
  const int Q = nq * dk, K = nkv * dk, V = nkv * dv;
  const int e0 = blockIdx.y * chunk;
  const int e1 = min(Q + K + V, e0 + chunk);
  T* kd = nullptr;
  T* vd = nullptr;
  int r = 0;
  if (pages) {
    const int pos = row_pos[n];
    const int page = table[(size_t)n * table_stride + (pos / PAGE) % ring_pages];
    kd = pages + (size_t)page * nkv * PAGE * (dk + dv);
    vd = kd + (size_t)nkv * PAGE * dk;
    r = pos % PAGE;
  }
  for (int e = e0 + threadIdx.x; e < e1; e += 256) {
    if (e < Q) {
      q[(size_t)n * Q + e] = from_f32<T>(qf[(size_t)n * q_stride + e]);
    } else if (e < Q + K) {
      const int i = e - Q;
      const T t = from_f32<T>(kf[(size_t)n * kv_stride + i]);
      if (pages) kd[((size_t)(i / dk) * PAGE + r) * dk + i % dk] = t;
      else k[(size_t)n * K + i] = t;
    } else {
      const int i = e - Q - K;
      const T t = from_f32<T>(vf[(size_t)n * kv_stride + i]);
      if (pages) vd[(size_t)i * PAGE + r] = t;          // [kv head][dv][row]: channel i of the row is line i
      else v[(size_t)n * V + i] = t;
    }
  }
}

template <typename T>
__global__ void mul_gate_kernel(T* __restrict__ x, const float* __restrict__ gate, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) x[i] = from_f32<T>(to_f32(x[i]) * gate[i]);
}

}  // namespace tl

using namespace tl;

extern "C" {

int tl_latent_norms(const float* proj, int n, int na, int nb, int ng, const float* wa, const float* wb, float eps,
                    void* a, void* b, float* gate, int dt, hipStream_t st) {
  TL_REQUIRE(n >= 0 && na > 0 && nb > 0 && ng >= 0, "latent_norms: bad sizes n=%d a=%d b=%d g=%d", n, na, nb, ng);
  TL_REQUIRE(proj && wa && wb && a && b && (ng == 0 || gate), "latent_norms: a buffer is missing");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "latent_norms: unknown dtype code %d", dt);
  if (n == 0) return 0;
  const dim3 grid(n, ng ? 3 : 2);
  if (dt == DT_F32)
    latent_norms_kernel<float><<<grid, 256, 0, st>>>(proj, na, nb, ng, wa, wb, eps, (float*)a, (float*)b, gate);
  else
    latent_norms_kernel<bf16><<<grid, 256, 0, st>>>(proj, na, nb, ng, wa, wb, eps, (bf16*)a, (bf16*)b, gate);
  TL_LAUNCH_CHECK("latent_norms");
  return 0;
}

int tl_split_heads(const float* qf, int q_stride, const float* kf, const float* vf, int kv_stride, const int* row_pos,
                   int n, int nq, int nkv, int dk, int dv, void* q, void* k, void* v, int dt, const int* table,
                   int table_stride, int ring_pages, void* pages, hipStream_t st) {
  TL_REQUIRE(n >= 0 && nq > 0 && nkv > 0 && dk > 0 && dv > 0, "split_heads: bad sizes n=%d nq=%d nkv=%d dk=%d dv=%d",
             n, nq, nkv, dk, dv);
  TL_REQUIRE(q_stride >= nq * dk && kv_stride >= nkv * (dk > dv ? dk : dv), "split_heads: rows shorter than their heads");
  TL_REQUIRE(qf && kf && vf && q && (pages || (k && v)), "split_heads: a buffer is missing");
  TL_REQUIRE(pages == nullptr || (table && row_pos && table_stride > 0 && ring_pages > 0),
             "split_heads: pages without a page table");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "split_heads: unknown dtype code %d", dt);
  if (n == 0) return 0;
  // few rows: chunks of HEADS_CHUNK outputs, so that the row spreads over many workgroups; many rows: three workgroups a row
  const int total = nq * dk + nkv * (dk + dv);
  const int chunk = n >= 256 ? ((total + 2) / 3 + 255) / 256 * 256 : HEADS_CHUNK;
  const dim3 grid(n, (total + chunk - 1) / chunk);
  if (dt == DT_F32)
    split_heads_kernel<float><<<grid, 256, 0, st>>>(qf, q_stride, kf, vf, kv_stride, row_pos, nq, nkv, dk, dv, (float*)q,
                                                    (float*)k, (float*)v, table, table_stride, ring_pages, (float*)pages, chunk);
  else
    split_heads_kernel<bf16><<<grid, 256, 0, st>>>(qf, q_stride, kf, vf, kv_stride, row_pos, nq, nkv, dk, dv, (bf16*)q,
                                                   (bf16*)k, (bf16*)v, table, table_stride, ring_pages, (bf16*)pages, chunk);
  TL_LAUNCH_CHECK("split_heads");
  return 0;
}

// x[i] *= gate[i] over `total` elements (x in the compute type, gate float)
int tl_mul_gate(void* x, const float* gate, long long total, int dt, hipStream_t st) {
  TL_REQUIRE(total >= 0 && x && gate, "mul_gate: bad arguments");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "mul_gate: unknown dtype code %d", dt);
  if (total == 0) return 0;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dt == DT_F32) mul_gate_kernel<float><<<blocks, 256, 0, st>>>((float*)x, gate, (size_t)total);
  else mul_gate_kernel<bf16><<<blocks, 256, 0, st>>>((bf16*)x, gate, (size_t)total);
  TL_LAUNCH_CHECK("mul_gate");
  return 0;
}

}  // extern "C"

// Differential attention: every head holds TWO maps (two queries, two keys, each of d channels)
// over the same values; with a1 and a2 the two maps' softmax-weighted sums of the values,
//
//   o = a1 - lambda * a2 ;  out = o / sqrt(mean(o^2) + eps) * post       (per head, over its dv values)
//
// The maps run through the ordinary attention kernels: the cache keeps one key of 2d channels
// per KV head and position, [map 1 | map 2], and a query of map m is laid out as a head of 2d
// channels with its d channels in half m and zeros in the other, so that q' . k = q_m . k_m.  Query
// head 2h + m then shares the KV head of head h, and both maps read the same values.
//
// `diff_split`: a row of the fused projection [q (H*2*d) | k (G*2*d) | v (G*dv)] in float, its
// biases, the rotation of the first `rotary_dim` channels of EACH MAP in pairs (i, i + rotary_dim/2)
// by the angle pos * inv_freq[i], and the layouts above (k and v to rows, or straight into the
// page of the row's position when every sequence brings one token).
// `diff_combine`: the difference and its norm, in float, one wave per (row, head).
#include "common.hpp"

namespace tl {

constexpr int DIFF_MAX_D = 256;

// A workgroup takes SPLIT_CHUNK consecutive outputs of a row's [q (as laid out: 2 * Q) | k | v]: few rows
// (single-token steps) then still spread over many workgroups.
constexpr int SPLIT_CHUNK = 1024;

template <typename T>
__global__ void __launch_bounds__(256)
diff_split_kernel(const float* __restrict__ proj, const float* __restrict__ bias, const int* __restrict__ row_pos,
                  Rotation rot, int H, int G, int d, int dv, T* __restrict__ q, T* __restrict__ k, T* __restrict__ v,
                  const int* __restrict__ table, int table_stride, int ring_pages, T* __restrict__ pages, int chunk) {
  __shared__ float cs[DIFF_MAX_D / 2], sn[DIFF_MAX_D / 2];
  const int n = blockIdx.x;
  const int Q = 2 * H * d, K = 2 * G * d, V = G * dv;
  const int total = 2 * Q + K + V;
  const int e0 = blockIdx.y * chunk;
  const int e1 = min(total, e0 + chunk);
  const float* row = proj + (size_t)n * (Q + K + V);
  const int pos = row_pos[n];
  const int half = rot.rotary_dim / 2;
  if (e0 < 2 * Q + K) {           // some of this chunk is rotated
    for (int i = threadIdx.x; i < half; i += 256) sincosf((float)pos * rot.inv_freq[i], &sn[i], &cs[i]);
    __syncthreads();
  }
  auto at = [&](int i) { return row[i] + (bias ? bias[i] : 0.f); };
  // channel c of the map that starts at `base`, rotated
  auto rotated = [&](int base, int c) {
    if (c >= 2 * half) return at(base + c);
    float ra, rb;
    if (c < half) {
      rotate_pair(at(base + c), at(base + c + half), cs[c], sn[c], ra, rb);
      return ra;
    }
    rotate_pair(at(base + c - half), at(base + c), cs[c - half], sn[c - half], ra, rb);
    return rb;
  };
  T* kd = nullptr;
  T* vd = nullptr;
  int r = 0;
  if (pages) {
    const int page = table[(size_t)n * table_stride + (pos / PAGE) % ring_pages];
    kd = pages + (size_t)page * G * PAGE * (2 * d + dv);
    vd = kd + (size_t)G * PAGE * 2 * d;
    r = pos % PAGE;
  }
  for (int e = e0 + threadIdx.x; e < e1; e += 256) {
    if (e < 2 * Q) {
      // map u = 2h + m becomes the head u of 2d channels, its own channels in half m
      const int u = e / (2 * d), c = e % (2 * d), m = u % 2;
      const bool own = (c / d) == m;
      q[(size_t)n * 2 * Q + e] = from_f32<T>(own ? rotated(u * d, c % d) : 0.f);
    } else if (e < 2 * Q + K) {
      const int i = e - 2 * Q;
      const T t = from_f32<T>(rotated(Q + (i / d) * d, i % d));
      if (pages) kd[((size_t)(i / (2 * d)) * PAGE + r) * 2 * d + i % (2 * d)] = t;
      else k[(size_t)n * K + i] = t;
    } else {
      const int i = e - 2 * Q - K;
      const T t = from_f32<T>(at(Q + K + i));
      if (pages) vd[(size_t)i * PAGE + r] = t;
      else v[(size_t)n * V + i] = t;
    }
  }
}

// att[n, 2H, dv] (TA: the compute type, or float from a kernel that leaves its sums unrounded):
// head 2h is map 1 of head h, 2h + 1 its map 2.  One wave per (row, head).
template <typename TA, typename T>
__global__ void __launch_bounds__(64)
diff_combine_kernel(const TA* __restrict__ att, int H, int dv, float lambda, float eps, float post, T* __restrict__ out) {
  const int n = blockIdx.x / H, h = blockIdx.x % H;
  const TA* a1 = att + ((size_t)n * 2 * H + 2 * h) * dv;
  const TA* a2 = a1 + dv;
  float o[DIFF_MAX_D / WAVE];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < DIFF_MAX_D / WAVE; ++i) {
    const int c = threadIdx.x + WAVE * i;
    o[i] = c < dv ? to_f32(a1[c]) - lambda * to_f32(a2[c]) : 0.f;
    ss += o[i] * o[i];
  }
  ss = wave_sum(ss);
  const float rms = sqrtf(ss / (float)dv + eps);
  T* dst = out + ((size_t)n * H + h) * dv;
#pragma unroll
  for (int i = 0; i < DIFF_MAX_D / WAVE; ++i) {
    const int c = threadIdx.x + WAVE * i;
    if (c < dv) dst[c] = from_f32<T>((o[i] / rms) * post);
  }
}

}  // namespace tl

using namespace tl;

extern "C" {

int tl_diff_split(const float* proj, const float* bias, const int* row_pos, const float* inv_freq, int rotary_dim, int n,
                  int H, int G, int d, int dv, void* q, void* k, void* v, int dt, const int* table, int table_stride,
                  int ring_pages, void* pages, hipStream_t st) {
  TL_REQUIRE(n >= 0 && H > 0 && G > 0 && H % G == 0 && d > 0 && dv > 0, "diff_split: bad sizes n=%d H=%d G=%d d=%d dv=%d",
             n, H, G, d, dv);
  TL_REQUIRE(rotary_dim >= 0 && rotary_dim % 2 == 0 && rotary_dim <= d && rotary_dim <= DIFF_MAX_D,
             "diff_split: %d rotated channels of a map of %d (even, at most the map and %d)", rotary_dim, d, DIFF_MAX_D);
  TL_REQUIRE(rotary_dim == 0 || inv_freq, "diff_split: a rotation without frequencies");
  TL_REQUIRE(proj && row_pos && q && (pages || (k && v)), "diff_split: a buffer is missing");
  TL_REQUIRE(pages == nullptr || (table && table_stride > 0 && ring_pages > 0), "diff_split: pages without a page table");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "diff_split: unknown dtype code %d", dt);
  if (n == 0) return 0;
  const Rotation rot{inv_freq, rotary_dim, 0};
  // few rows: chunks of SPLIT_CHUNK outputs, so that the row spreads over many workgroups; many rows: three workgroups a row
  const int total = 4 * H * d + 2 * G * d + G * dv;
  const int chunk = n >= 256 ? ((total + 2) / 3 + 255) / 256 * 256 : SPLIT_CHUNK;
  const dim3 grid(n, (total + chunk - 1) / chunk);
  if (dt == DT_F32)
    diff_split_kernel<float><<<grid, 256, 0, st>>>(proj, bias, row_pos, rot, H, G, d, dv, (float*)q, (float*)k, (float*)v,
                                                   table, table_stride, ring_pages, (float*)pages, chunk);
  else
    diff_split_kernel<bf16><<<grid, 256, 0, st>>>(proj, bias, row_pos, rot, H, G, d, dv, (bf16*)q, (bf16*)k, (bf16*)v,
                                                  table, table_stride, ring_pages, (bf16*)pages, chunk);
  TL_LAUNCH_CHECK("diff_split");
  return 0;
}

int tl_diff_combine(const void* att, int att_dt, int n, int H, int dv, float lambda, float eps, float post, void* out,
                    int dt, hipStream_t st) {
  TL_REQUIRE(att_dt == dt || att_dt == DT_F32, "diff_combine: the maps are of the result's type or float");
  TL_REQUIRE(n >= 0 && H > 0 && dv > 0 && dv <= DIFF_MAX_D, "diff_combine: bad sizes n=%d H=%d dv=%d (values up to %d)",
             n, H, dv, DIFF_MAX_D);
  TL_REQUIRE((long long)n * H < 2147483647LL, "diff_combine: too many (row, head) pairs");
  TL_REQUIRE(att && out, "diff_combine: a buffer is missing");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "diff_combine: unknown dtype code %d", dt);
  if (n == 0) return 0;
  if (dt == DT_F32)
    diff_combine_kernel<float, float><<<n * H, 64, 0, st>>>((const float*)att, H, dv, lambda, eps, post, (float*)out);
  else if (att_dt == DT_F32)
    diff_combine_kernel<float, bf16><<<n * H, 64, 0, st>>>((const float*)att, H, dv, lambda, eps, post, (bf16*)out);
  else
    diff_combine_kernel<bf16, bf16><<<n * H, 64, 0, st>>>((const bf16*)att, H, dv, lambda, eps, post, (bf16*)out);
  TL_LAUNCH_CHECK("diff_combine");
  return 0;
}

}  // extern "C"

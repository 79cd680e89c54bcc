// Small row-wise steps that layers other than GPT-2's are put together from, all with 32-bit arithmetic:
//   * heads divided by their root mean square (queries and keys) and values blended with an earlier layer's values;
//   * a polynomial activation whose three powers are each divided by their root mean square over the row;
//   * attention outputs of all (query head, value head) pairs mixed over the query heads and gated per head;
//   * the residual stream as a weighted sum of this and every earlier layer's result.
#include "common.h"

// ------------------------------------------------------------------------------------------
// One wave per (token, item). Items 0 .. n_norm-1 are heads of `hd` elements that start at column item * hd of the row
// (queries, then keys: the two lie side by side): x <- x / sqrt(mean(x^2) + eps), in place. Items n_norm .. are value
// heads of `vd` elements in `v`: v <- (1 - lambda) v + lambda v_first, in place. Either part may be empty.
template <typename T>
__global__ void __launch_bounds__(64)
head_prepare_kernel(T* __restrict__ qk, long qk_stride, int n_norm, int hd, float eps, T* __restrict__ v, long v_stride,
                    const T* __restrict__ v_first, long vf_stride, int n_blend, int vd, const float* __restrict__ lambda) {
  const int t = blockIdx.x, item = blockIdx.y, lane = threadIdx.x;
  if (item < n_norm) {
    T* row = qk + (size_t)t * qk_stride + (size_t)item * hd;
    float ss = 0.f;
    for (int d = lane; d < hd; d += 64) {
      const float x = to_float<T>(row[d]);
      ss = fmaf(x, x, ss);
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)hd + eps);
    for (int d = lane; d < hd; d += 64) row[d] = from_float<T>(to_float<T>(row[d]) * r);
  } else {
    const int c = item - n_norm;
    if (c >= n_blend) return;
    const float lam = *lambda;
    T* row = v + (size_t)t * v_stride + (size_t)c * vd;
    const T* first = v_first + (size_t)t * vf_stride + (size_t)c * vd;
    for (int d = lane; d < vd; d += 64)
      row[d] = from_float<T>((1.0f - lam) * to_float<T>(row[d]) + lam * to_float<T>(first[d]));
  }
}

extern "C" int lev_head_prepare(void* qk, long qk_stride, int n_norm, int hd, float eps, void* v, long v_stride, const void* v_first,
                                long vf_stride, int n_blend, int vd, const float* lambda, int T, int dtype, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && n_norm >= 0 && n_blend >= 0, "head_prepare: bad counts T=%d heads=%d value heads=%d", T, n_norm, n_blend);
  LEV_REQUIRE(n_norm == 0 || (qk && hd > 0), "head_prepare: heads to normalise need a tensor and a size");
  LEV_REQUIRE(n_blend == 0 || (v && v_first && lambda && vd > 0), "head_prepare: values to blend need both tensors, a size and the weight");
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "head_prepare: unknown dtype %d", dtype);
  LEV_REQUIRE(n_norm + n_blend <= 65535, "head_prepare: too many heads (%d)", n_norm + n_blend);
  if (T == 0 || n_norm + n_blend == 0) return 0;
  dim3 grid(T, n_norm + n_blend);
  if (dtype == LEV_F32)
    head_prepare_kernel<float><<<grid, 64, 0, stream>>>((float*)qk, qk_stride, n_norm, hd, eps, (float*)v, v_stride, (const float*)v_first,
                                                       vf_stride, n_blend, vd, lambda);
  else
    head_prepare_kernel<bf16_t><<<grid, 64, 0, stream>>>((bf16_t*)qk, qk_stride, n_norm, hd, eps, (bf16_t*)v, v_stride,
                                                        (const bf16_t*)v_first, vf_stride, n_blend, vd, lambda);
  return lev_check_launch("head_prepare");
}

// ------------------------------------------------------------------------------------------
// out = c0 z / rms(z) + c1 z^2 / rms(z^2) + c2 z^3 / rms(z^3) + c3 over a row of F values, rms(u) = sqrt(mean(u^2) + eps).
// One block per row; the row is read twice (statistics, then the output), the second time from the cache. `out` may be `z`.
template <typename T, int NT>
__global__ void __launch_bounds__(NT)
poly_norm_kernel(const T* z, long z_stride, T* out, long o_stride, const float* __restrict__ coef, int F,
                 float eps) {
  __shared__ float red[NT / 64];
  const T* row = z + (size_t)blockIdx.x * z_stride;
  T* o = out + (size_t)blockIdx.x * o_stride;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int d = threadIdx.x; d < F; d += NT) {
    const float u = to_float<T>(row[d]);
    const float u2 = u * u, u3 = u2 * u;
    s2 += u2;
    s4 = fmaf(u2, u2, s4);
    s6 = fmaf(u3, u3, s6);
  }
  s2 = block_sum<NT>(s2, red);
  s4 = block_sum<NT>(s4, red);
  s6 = block_sum<NT>(s6, red);
  const float inv = 1.0f / (float)F;
  const float r1 = coef[0] / sqrtf(s2 * inv + eps), r2 = coef[1] / sqrtf(s4 * inv + eps), r3 = coef[2] / sqrtf(s6 * inv + eps);
  const float c3 = coef[3];
  for (int d = threadIdx.x; d < F; d += NT) {
    const float u = to_float<T>(row[d]);
    const float u2 = u * u;
    o[d] = from_float<T>(fmaf(u, r1, fmaf(u2, r2, fmaf(u2 * u, r3, c3))));
  }
}

extern "C" int lev_poly_norm(const void* z, long z_stride, void* out, long o_stride, const float* coef, int T, int F, float eps, int dtype,
                             hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && F > 0 && z_stride >= F && o_stride >= F, "poly_norm: bad sizes T=%d F=%d", T, F);
  LEV_REQUIRE(coef, "poly_norm: the four coefficients are missing");
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "poly_norm: unknown dtype %d", dtype);
  if (T == 0) return 0;
  if (dtype == LEV_F32)
    poly_norm_kernel<float, 256><<<T, 256, 0, stream>>>((const float*)z, z_stride, (float*)out, o_stride, coef, F, eps);
  else
    poly_norm_kernel<bf16_t, 256><<<T, 256, 0, stream>>>((const bf16_t*)z, z_stride, (bf16_t*)out, o_stride, coef, F, eps);
  return lev_check_launch("poly_norm");
}

// ------------------------------------------------------------------------------------------
// o [T][H][NV][VD] (float32) holds, for every query head g and value head c, the attention weights of g applied to the
// values of c. Head h of the result uses the values of its own value head c(h) = h / (H / KVH) with the weights of all
// query heads mixed by `talk` [H][H]:   a[t][h][:] = gate(t, h) * sum_g talk[h][g] * o[t][g][c(h)][:].
// talk == null: NV is 1 and the sum is o[t][h][0][:]. gate == null: 1, else sigmoid of the gate's entry.
template <typename T>
__global__ void __launch_bounds__(256)
head_talk_kernel(const float* __restrict__ o, const float* __restrict__ talk, const T* __restrict__ gate, long g_stride,
                 T* __restrict__ a, long a_stride, int H, int KVH, int NV, int VD) {
  const int t = blockIdx.x;
  const float* ot = o + (size_t)t * H * NV * VD;
  const int group = H / KVH;
  for (int e = threadIdx.x; e < H * VD; e += 256) {
    const int h = e / VD, d = e % VD;
    float s;
    if (talk) {
      const int c = h / group;
      s = 0.f;
      for (int g = 0; g < H; ++g) s = fmaf(talk[h * H + g], ot[((size_t)g * NV + c) * VD + d], s);
    } else {
      s = ot[(size_t)h * NV * VD + d];
    }
    if (gate) s *= 1.0f / (1.0f + expf(-to_float<T>(gate[(size_t)t * g_stride + h])));
    a[(size_t)t * a_stride + e] = from_float<T>(s);
  }
}

extern "C" int lev_head_talk(const float* o, const float* talk, const void* gate, long g_stride, void* a, long a_stride, int T, int H,
                             int KVH, int NV, int VD, int dtype, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && H > 0 && KVH > 0 && H % KVH == 0 && VD > 0, "head_talk: bad sizes T=%d heads=%d kv_heads=%d vd=%d", T, H, KVH, VD);
  LEV_REQUIRE(NV == (talk ? KVH : 1), "head_talk: %d outputs per query head; with a mixing matrix there are kv_heads=%d, without it one", NV, KVH);
  LEV_REQUIRE(a_stride >= (long)H * VD, "head_talk: the output's row stride is too small");
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "head_talk: unknown dtype %d", dtype);
  if (T == 0) return 0;
  if (dtype == LEV_F32)
    head_talk_kernel<float><<<T, 256, 0, stream>>>(o, talk, (const float*)gate, g_stride, (float*)a, a_stride, H, KVH, NV, VD);
  else
    head_talk_kernel<bf16_t><<<T, 256, 0, stream>>>(o, talk, (const bf16_t*)gate, g_stride, (bf16_t*)a, a_stride, H, KVH, NV, VD);
  return lev_check_launch("head_talk");
}

// ------------------------------------------------------------------------------------------
// streams [n][count] (float32) holds the results of earlier layers in its first n - 1 entries. x [count] is this layer's
// result: it is kept as entry n - 1, and x becomes sum_j w[j] * streams[j] (j = 0 .. n-1, added in that order).
__global__ void __launch_bounds__(256)
stream_average_kernel(float* __restrict__ streams, float* __restrict__ x, const float* __restrict__ w, int n, long count, int vec) {
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= count) return;
  if (vec && i + 4 <= count) {
    const float4 cur = *reinterpret_cast<const float4*>(x + i);
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int j = 0; j < n - 1; ++j) {
      const float wj = w[j];
      const float4 v = *reinterpret_cast<const float4*>(streams + (size_t)j * count + i);
      s.x = fmaf(wj, v.x, s.x); s.y = fmaf(wj, v.y, s.y); s.z = fmaf(wj, v.z, s.z); s.w = fmaf(wj, v.w, s.w);
    }
    const float wl = w[n - 1];
    s.x = fmaf(wl, cur.x, s.x); s.y = fmaf(wl, cur.y, s.y); s.z = fmaf(wl, cur.z, s.z); s.w = fmaf(wl, cur.w, s.w);
    *reinterpret_cast<float4*>(streams + (size_t)(n - 1) * count + i) = cur;
    *reinterpret_cast<float4*>(x + i) = s;
  } else {
    for (long e = i; e < count && e < i + 4; ++e) {
      const float cur = x[e];
      float s = 0.f;
      for (int j = 0; j < n - 1; ++j) s = fmaf(w[j], streams[(size_t)j * count + e], s);
      s = fmaf(w[n - 1], cur, s);
      streams[(size_t)(n - 1) * count + e] = cur;
      x[e] = s;
    }
  }
}

extern "C" int lev_stream_average(float* streams, float* x, const float* w, int n, long count, hipStream_t stream) {
  LEV_REQUIRE(n >= 1 && count >= 0 && streams && x && w, "stream_average: bad arguments n=%d count=%ld", n, count);
  if (count == 0) return 0;
  // 16-byte accesses where every stream starts on a 16-byte boundary
  const int vec = (((uintptr_t)x | (uintptr_t)streams) & 15) == 0 && count % 4 == 0;
  const long blocks = ((count + 3) / 4 + 255) / 256;
  LEV_REQUIRE(blocks <= 0x7fffffffL, "stream_average: too many elements (%ld)", count);
  stream_average_kernel<<<(unsigned)blocks, 256, 0, stream>>>(streams, x, w, n, count, vec);
  return lev_check_launch("stream_average");
}

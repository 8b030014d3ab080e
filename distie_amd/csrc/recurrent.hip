// Kernels of designs that put norms behind their sub-layers, run mixers side by side, keep a state whose decay is
// computed from the token (gated linear attention, a real-gated linear recurrent unit) and route tokens to experts.
// What such designs keep in 32-bit is float32 here in either precision: norm statistics, decays with their
// sigmoids, logarithms and exponentials, the gates of a recurrence, the states and every sum into them, router
// logits and weights.
//
// A step is a flattened batch: token t belongs to request token_request[t], whose new tokens are rows
// cu_q[b] .. cu_q[b+1]-1 and whose state is row state_slots[b] of a state tensor.
#include "common.h"

namespace {

__device__ __forceinline__ float sigmoid_exact(float x) { return 1.f / (1.f + expf(-x)); }
// ln(sigmoid(x)) and ln(1 + e^x) without overflow and without cancellation
__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

__device__ __forceinline__ float activate(float z, int kind) {   // the kinds of `distie_activation`; -1: z itself
  if (kind == 0) {
    const float p = fmaxf(z, 0.f);
    return p * p;
  }
  if (kind == 1) return z / (1.f + expf(-z));
  if (kind == 2) return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  if (kind == 3) return fmaxf(z, 0.f);
  return z;
}

// ---------------------------------------------------------------------------------------------------
// A chain of norms around the residual sum, one block a row; every stage but the first is optional:
//   y   = scale * (rms(t0) * w0 + rms(t1) * w1)      (w0 null: y = t0 as it is; t1 null: one term)
//   y   = rms(y) * post_w                            (the norm behind a sub-layer)
//   x  += y                                          (residual, float32, in place; null: y goes to y_out)
//   out = rms(x) * pre_w                             (the norm in front of the next sub-layer)
// rms(v) = v / sqrt(mean(v^2) + eps). A term may be partial sums (slices that lie `stride` apart, added in order).
// The row waits in LDS between the passes; a thread meets the same columns in every pass.
template <typename A, typename B, typename O>
__global__ void norm_chain_kernel(const A* __restrict__ t0, int slices0, int64_t stride0, const float* __restrict__ w0,
                                  const B* __restrict__ t1, int slices1, int64_t stride1, const float* __restrict__ w1,
                                  float term_eps, float scale, const float* __restrict__ post_w, float post_eps,
                                  float* __restrict__ residual, const float* __restrict__ pre_w, float pre_eps,
                                  O* __restrict__ out, float* __restrict__ y_out, int C) {
  extern __shared__ float row[];
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * C;
  float r0 = 1.f, r1 = 1.f;
  if (w0 != nullptr) {
    float q0 = 0.f, q1 = 0.f;
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
      const float a = sum_strided(t0 + base + c, slices0, stride0);
      q0 += a * a;
      if (t1 != nullptr) {
        const float b = sum_strided(t1 + base + c, slices1, stride1);
        q1 += b * b;
      }
    }
    r0 = 1.f / sqrtf(block_sum(q0, scratch) / C + term_eps);
    if (t1 != nullptr) r1 = 1.f / sqrtf(block_sum(q1, scratch) / C + term_eps);
  }
  float q = 0.f;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float y = sum_strided(t0 + base + c, slices0, stride0);
    if (w0 != nullptr) {
      y = y * r0 * w0[c];
      if (t1 != nullptr) y += sum_strided(t1 + base + c, slices1, stride1) * r1 * w1[c];
      y *= scale;
    }
    row[c] = y;
    q += y * y;
  }
  float rp = 1.f;
  if (post_w != nullptr) rp = 1.f / sqrtf(block_sum(q, scratch) / C + post_eps);
  float q2 = 0.f;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float y = row[c];
    if (post_w != nullptr) y = y * rp * post_w[c];
    if (residual != nullptr) {
      const float x = residual[base + c] + y;
      residual[base + c] = x;
      row[c] = x;
      q2 += x * x;
    } else {
      y_out[base + c] = y;
    }
  }
  if (residual == nullptr || pre_w == nullptr) return;
  const float rn = 1.f / sqrtf(block_sum(q2, scratch) / C + pre_eps);
  for (int c = threadIdx.x; c < C; c += blockDim.x) out[base + c] = from_float<O>(row[c] * rn * pre_w[c]);
}

// ---------------------------------------------------------------------------------------------------
// A state that decays by a factor of its own for every key channel and token, row after row:
//   alpha = sigmoid(z)^(1 / tau);   S <- diag(alpha) S + k v^T;   o = S^T (q * q_scale)     per head
// product [T, ld] holds q (H x D), k (H x D), v (H x E); z float32 [T, H * D]; state float32 [slots, H, D, E].
// A block owns 64 columns e of one head of one request and walks the request's rows in order; thread (e, part)
// keeps rows d = part, part + PARTS, ... of its column in registers, the PARTS partial sums of a column meet in LDS.
// The next row's values are asked for before this row's are used.
template <typename X, int PARTS, int ROWS>
__global__ void __launch_bounds__(64 * PARTS)
gated_decay_scan_kernel(const X* __restrict__ product, int64_t ld, const float* __restrict__ logits, float* __restrict__ state,
                        float* __restrict__ out, const int32_t* __restrict__ cu_q, const int32_t* __restrict__ state_slots,
                        int H, int D, int E, float q_scale, float tau) {
  __shared__ float q_s[PARTS * ROWS], k_s[PARTS * ROWS], a_s[PARTS * ROWS];
  __shared__ float partial[PARTS][64];
  const int b = blockIdx.x, head = blockIdx.y;
  const int lane = threadIdx.x % 64, part = threadIdx.x / 64;
  const int e = blockIdx.z * 64 + lane;
  const int first = cu_q[b], last = cu_q[b + 1];
  if (first >= last) return;
  float* own = state + (static_cast<int64_t>(state_slots[b]) * H + head) * D * E;
  float s[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int d = part + r * PARTS;
    s[r] = (d < D && e < E) ? own[static_cast<int64_t>(d) * E + e] : 0.f;
  }
  const int d_own = threadIdx.x;                      // the channel whose q, k and decay this thread fetches
  float nq = 0.f, nk = 0.f, nz = 0.f, nv = 0.f;
  auto fetch = [&](int t) {
    const X* row = product + static_cast<int64_t>(t) * ld;
    if (d_own < D) {
      nq = to_float(row[head * D + d_own]);
      nk = to_float(row[(H + head) * D + d_own]);
      nz = logits[(static_cast<int64_t>(t) * H + head) * D + d_own];
    }
    nv = e < E ? to_float(row[2 * H * D + head * E + e]) : 0.f;
  };
  fetch(first);
  for (int t = first; t < last; ++t) {
    __syncthreads();
    if (d_own < D) {
      q_s[d_own] = nq * q_scale;
      k_s[d_own] = nk;
      a_s[d_own] = expf(log_sigmoid(nz) / tau);
    }
    const float v = nv;
    if (t + 1 < last) fetch(t + 1);
    __syncthreads();
    float o = 0.f;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int d = part + r * PARTS;
      if (d < D) {
        s[r] = a_s[d] * s[r] + k_s[d] * v;
        o += s[r] * q_s[d];
      }
    }
    partial[part][lane] = o;
    __syncthreads();
    if (part == 0 && e < E) {
      float total = 0.f;
#pragma unroll
      for (int p = 0; p < PARTS; ++p) total += partial[p][lane];
      out[(static_cast<int64_t>(t) * H + head) * E + e] = total;
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int d = part + r * PARTS;
    if (d < D && e < E) own[static_cast<int64_t>(d) * E + e] = s[r];
  }
}

// ---------------------------------------------------------------------------------------------------
// The gates of a real-gated linear recurrent unit. u [T, ldu] holds R channels in B parts of n; in part b
//   r = sigmoid(ra[b] u_b + ra_b[b]),  i = sigmoid(ri[b] u_b + ri_b[b])          (ra[b], ri[b]: [n, n], [out, in])
//   a = exp(-rate * r * softplus(lam)),  x = sqrt(1 - a^2) * i * u     -> a_out, x_out float32 [T, R]
// A block owns 32 tokens x 64 output channels of one part, both gates at once; tiles of 32 inputs through LDS,
// float32 sums. 1 - a^2 is taken as -expm1(2 ln a), which keeps its digits where a is close to one.
constexpr int LG_TOKENS = 32, LG_OUT = 64, LG_K = 32;

template <typename X, typename W>
__global__ void __launch_bounds__(256)
lru_gates_kernel(const X* __restrict__ u, int64_t ldu, const W* __restrict__ ra, const float* __restrict__ ra_b,
                 const W* __restrict__ ri, const float* __restrict__ ri_b, const float* __restrict__ lam, float rate,
                 float* __restrict__ a_out, float* __restrict__ x_out, int T, int R, int n) {
  __shared__ float Us[LG_TOKENS][LG_K];
  __shared__ float Wa[LG_OUT][LG_K + 1], Wi[LG_OUT][LG_K + 1];
  const int t0 = blockIdx.x * LG_TOKENS, part = blockIdx.y, o0 = blockIdx.z * LG_OUT;
  const int tx = threadIdx.x % 64, ty = threadIdx.x / 64;
  const W* wa = ra + static_cast<int64_t>(part) * n * n;
  const W* wi = ri + static_cast<int64_t>(part) * n * n;
  float acc_a[8] = {}, acc_i[8] = {};
  for (int k0 = 0; k0 < n; k0 += LG_K) {
#pragma unroll
    for (int it = 0; it < LG_TOKENS * LG_K / 256; ++it) {
      const int idx = threadIdx.x + 256 * it;
      const int tok = idx / LG_K, kk = idx % LG_K;
      Us[tok][kk] = (t0 + tok < T && k0 + kk < n) ? to_float(u[static_cast<int64_t>(t0 + tok) * ldu + part * n + k0 + kk]) : 0.f;
    }
#pragma unroll
    for (int it = 0; it < LG_OUT * LG_K / 256; ++it) {
      const int idx = threadIdx.x + 256 * it;
      const int o = idx / LG_K, kk = idx % LG_K;
      const bool in = o0 + o < n && k0 + kk < n;
      Wa[o][kk] = in ? to_float(wa[static_cast<int64_t>(o0 + o) * n + k0 + kk]) : 0.f;
      Wi[o][kk] = in ? to_float(wi[static_cast<int64_t>(o0 + o) * n + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < LG_K; ++kk) {
      const float a = Wa[tx][kk], i = Wi[tx][kk];
#pragma unroll
      for (int m = 0; m < 8; ++m) {
        const float x = Us[ty * 8 + m][kk];
        acc_a[m] += a * x;
        acc_i[m] += i * x;
      }
    }
    __syncthreads();
  }
  if (o0 + tx >= n) return;
  const int c = part * n + o0 + tx;
  const float bias_a = ra_b[c], bias_i = ri_b[c];
  const float decay = -rate * softplus(lam[c]);
#pragma unroll
  for (int m = 0; m < 8; ++m) {
    const int t = t0 + ty * 8 + m;
    if (t >= T) break;
    const float r = sigmoid_exact(acc_a[m] + bias_a), i = sigmoid_exact(acc_i[m] + bias_i);
    const float log_a = decay * r;
    a_out[static_cast<int64_t>(t) * R + c] = expf(log_a);
    x_out[static_cast<int64_t>(t) * R + c] = sqrtf(-expm1f(2.f * log_a)) * i * to_float(u[static_cast<int64_t>(t) * ldu + c]);
  }
}

// h_t = a_t h_(t-1) + x_t for every channel over a request's rows in order; out = h * act(mul). One thread a
// (request, channel); the loads of four rows are under way together (they do not hang on h).
template <typename M, typename O>
__global__ void lru_scan_kernel(const float* __restrict__ a, const float* __restrict__ x, float* __restrict__ state,
                                const M* __restrict__ mul, int64_t ldm, int kind, O* __restrict__ out,
                                const int32_t* __restrict__ cu_q, const int32_t* __restrict__ state_slots, int R) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= R) return;
  const int first = cu_q[b], last = cu_q[b + 1];
  if (first >= last) return;
  float* own = state + static_cast<int64_t>(state_slots[b]) * R + c;
  float h = *own;
  for (int t = first; t < last; t += 4) {
    float av[4], xv[4], mv[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t r = min(t + k, last - 1);
      av[k] = a[r * R + c];
      xv[k] = x[r * R + c];
      mv[k] = mul != nullptr ? to_float(mul[r * ldm + c]) : 1.f;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (t + k >= last) break;
      h = av[k] * h + xv[k];
      out[static_cast<int64_t>(t + k) * R + c] = from_float<O>(mul != nullptr ? h * activate(mv[k], kind) : h);
    }
  }
  *own = h;
}

// ---------------------------------------------------------------------------------------------------
// The router of a mixture of experts, one block a token: z = W x + b in float32 (a wave an expert at a time), then
// the `top` largest z by one wave (the lower index among equals), largest first, and the softmax over those alone.
constexpr int ROUTE_MAX_EXPERTS = 1024;
constexpr int ROUTE_MAX_TOP = 32;

template <typename X, typename W>
__global__ void __launch_bounds__(256)
route_topk_kernel(const X* __restrict__ x, const W* __restrict__ weight, const float* __restrict__ bias,
                  int32_t* __restrict__ experts, float* __restrict__ gates, int C, int E, int top) {
  extern __shared__ float xs[];                       // the token's row as float32
  __shared__ float z[ROUTE_MAX_EXPERTS];
  __shared__ float chosen[ROUTE_MAX_TOP];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  for (int c = threadIdx.x; c < C; c += blockDim.x) xs[c] = to_float(x[t * C + c]);
  __syncthreads();
  for (int e = wave; e < E; e += 4) {
    const W* w = weight + static_cast<int64_t>(e) * C;
    float acc = 0.f;
    for (int c = lane; c < C; c += 64) acc += to_float(w[c]) * xs[c];
    acc = wave_sum(acc);
    if (lane == 0) z[e] = acc + (bias != nullptr ? bias[e] : 0.f);
  }
  __syncthreads();
  if (wave != 0) return;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = z[e];
      if (v > best || (v == best && e < at)) best = v, at = e;
    }
    // a NaN or a row of -inf never wins the comparison above: then the lowest index not yet taken does
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float other = __shfl_xor(best, o, 64);
      const int other_at = __shfl_xor(at, o, 64);
      if (other > best || (other == best && other_at < at)) best = other, at = other_at;
    }
    if (at == 0x7fffffff) at = k;                     // (unreachable for finite logits)
    if (lane == 0) {
      experts[t * top + k] = at;
      chosen[k] = best;
    }
    if (at % 64 == lane) z[at] = -INFINITY;           // the lane that reads this place takes it out itself
  }
  if (lane == 0) {
    const float peak = chosen[0];
    float total = 0.f;
    for (int k = 0; k < top; ++k) total += expf(chosen[k] - peak);
    for (int k = 0; k < top; ++k) gates[t * top + k] = expf(chosen[k] - peak) / total;
  }
}

// hidden [T, ld]: the columns [e * F, (e + 1) * F) of expert e times the row's weight for e, zero if e was not chosen
template <typename X>
__global__ void route_scale_kernel(X* __restrict__ hidden, int64_t ld, const int32_t* __restrict__ experts,
                                   const float* __restrict__ gates, int top, int F, int width) {
  const int64_t t = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) {
    const int e = c / F;
    float g = 0.f;
    for (int k = 0; k < top; ++k)
      if (experts[t * top + k] == e) g = gates[t * top + k];
    X* p = hidden + t * ld + c;
    *p = from_float<X>(to_float(*p) * g);
  }
}

__global__ void scale_f32_kernel(float* __restrict__ x, int64_t count, float scale) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < count) x[i] *= scale;
}

}  // namespace

extern "C" int distie_norm_chain(const void* t0, int t0_dtype, int slices0, const float* w0, const void* t1, int t1_dtype,
                                 int slices1, const float* w1, float term_eps, float scale, const float* post_w,
                                 float post_eps, float* residual, const float* pre_w, float pre_eps, void* out,
                                 int out_dtype, float* y_out, int T, int C, hipStream_t stream) {
  if (T <= 0) return 0;
  if (C < 1 || t0 == nullptr || slices0 < 1 || (t1 != nullptr && (slices1 < 1 || w0 == nullptr || w1 == nullptr)) ||
      (residual == nullptr && y_out == nullptr) || (residual != nullptr && pre_w != nullptr && out == nullptr) ||
      static_cast<size_t>(C) * sizeof(float) > 64 * 1024)
    return DISTIE_BAD_ARGUMENT;
  if (t1 == nullptr) t1_dtype = t0_dtype, slices1 = 1;
  if (out == nullptr) out_dtype = DISTIE_F32;
  const int threads = C >= 2048 ? 512 : (C >= 512 ? 256 : (C >= 128 ? 128 : 64));
  const int64_t stride = static_cast<int64_t>(T) * C;
  DISTIE_DISPATCH(t0_dtype, A, DISTIE_DISPATCH(t1_dtype, B, DISTIE_DISPATCH(out_dtype, O,
      norm_chain_kernel<A, B, O><<<T, threads, static_cast<size_t>(C) * sizeof(float), stream>>>(
          static_cast<const A*>(t0), slices0, stride, w0, static_cast<const B*>(t1), slices1, stride, w1, term_eps, scale,
          post_w, post_eps, residual, pre_w, pre_eps, static_cast<O*>(out), y_out, C))));
  return launch_status();
}

extern "C" int distie_gated_decay_scan_max_dim() { return 256; }

extern "C" int distie_gated_decay_scan(const void* product, int dtype, int64_t ld, const float* logits, float* state,
                                       float* out, const int32_t* cu_q, const int32_t* state_slots, int B, int H, int D,
                                       int E, float q_scale, float tau, hipStream_t stream) {
  if (B <= 0) return 0;
  if (H < 1 || D < 1 || E < 1 || D > 256 || !(tau > 0.f) || ld < static_cast<int64_t>(H) * (2 * D + E))
    return DISTIE_BAD_ARGUMENT;
  const dim3 grid(B, H, (E + 63) / 64);
#define DISTIE_GSCAN(PARTS, ROWS)                                                                                     \
  DISTIE_DISPATCH(dtype, X, gated_decay_scan_kernel<X, PARTS, ROWS><<<grid, 64 * PARTS, 0, stream>>>(                \
      static_cast<const X*>(product), ld, logits, state, out, cu_q, state_slots, H, D, E, q_scale, tau))
  if (D <= 32) {
    DISTIE_GSCAN(4, 8);
  } else if (D <= 64) {
    DISTIE_GSCAN(4, 16);
  } else if (D <= 128) {
    DISTIE_GSCAN(4, 32);
  } else {
    DISTIE_GSCAN(8, 32);
  }
#undef DISTIE_GSCAN
  return launch_status();
}

extern "C" int distie_lru_gates(const void* u, int u_dtype, int64_t ldu, const void* ra, const float* ra_b, const void* ri,
                                const float* ri_b, int w_dtype, const float* lam, float rate, float* a_out, float* x_out,
                                int T, int R, int blocks, hipStream_t stream) {
  if (T <= 0) return 0;
  if (R < 1 || blocks < 1 || R % blocks || ldu < R) return DISTIE_BAD_ARGUMENT;
  const int n = R / blocks;
  const dim3 grid((T + LG_TOKENS - 1) / LG_TOKENS, blocks, (n + LG_OUT - 1) / LG_OUT);
  DISTIE_DISPATCH(u_dtype, X, DISTIE_DISPATCH(w_dtype, W,
      lru_gates_kernel<X, W><<<grid, 256, 0, stream>>>(
          static_cast<const X*>(u), ldu, static_cast<const W*>(ra), ra_b, static_cast<const W*>(ri), ri_b, lam, rate,
          a_out, x_out, T, R, n)));
  return launch_status();
}

extern "C" int distie_lru_scan(const float* a, const float* x, float* state, const void* mul, int mul_dtype, int64_t ldm,
                               int kind, void* out, int out_dtype, const int32_t* cu_q, const int32_t* state_slots, int B,
                               int R, hipStream_t stream) {
  if (B <= 0) return 0;
  if (R < 1 || kind < -1 || kind > 3 || (mul != nullptr && ldm < R)) return DISTIE_BAD_ARGUMENT;
  if (mul == nullptr) mul_dtype = DISTIE_F32;
  const int threads = R >= 256 ? 256 : (R >= 128 ? 128 : 64);
  const dim3 grid(B, (R + threads - 1) / threads);
  DISTIE_DISPATCH(mul_dtype, M, DISTIE_DISPATCH(out_dtype, O,
      lru_scan_kernel<M, O><<<grid, threads, 0, stream>>>(a, x, state, static_cast<const M*>(mul), ldm, kind,
                                                          static_cast<O*>(out), cu_q, state_slots, R)));
  return launch_status();
}

extern "C" int distie_route_topk(const void* x, int x_dtype, const void* weight, int w_dtype, const float* bias,
                                 int32_t* experts, float* gates, int T, int C, int E, int top, hipStream_t stream) {
  if (T <= 0) return 0;
  if (C < 1 || E < 1 || E > ROUTE_MAX_EXPERTS || top < 1 || top > E || top > ROUTE_MAX_TOP ||
      static_cast<size_t>(C) * sizeof(float) > 96 * 1024)
    return DISTIE_BAD_ARGUMENT;
  const size_t lds = static_cast<size_t>(C) * sizeof(float);
  DISTIE_DISPATCH(x_dtype, X, DISTIE_DISPATCH(w_dtype, W, {
    if (lds > 48 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(route_topk_kernel<X, W>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)) != hipSuccess)
      return DISTIE_BAD_ARGUMENT;
    route_topk_kernel<X, W><<<T, 256, lds, stream>>>(static_cast<const X*>(x), static_cast<const W*>(weight), bias,
                                                     experts, gates, C, E, top);
  }));
  return launch_status();
}

extern "C" int distie_route_scale(void* hidden, int dtype, int64_t ld, const int32_t* experts, const float* gates, int T,
                                  int top, int E, int F, hipStream_t stream) {
  if (T <= 0) return 0;
  if (top < 1 || E < 1 || F < 1 || ld < static_cast<int64_t>(E) * F) return DISTIE_BAD_ARGUMENT;
  const int width = E * F;
  const int per_row = (width + 255) / 256;
  const dim3 grid(T, per_row < 64 ? per_row : 64);
  DISTIE_DISPATCH(dtype, X, route_scale_kernel<X><<<grid, 256, 0, stream>>>(static_cast<X*>(hidden), ld, experts, gates,
                                                                            top, F, width));
  return launch_status();
}

extern "C" int distie_scale_f32(float* x, int64_t count, float scale, hipStream_t stream) {
  if (count <= 0) return 0;
  const int64_t blocks = (count + 255) / 256;
  if (blocks > 0x7fffffff) return DISTIE_BAD_ARGUMENT;
  scale_f32_kernel<<<static_cast<unsigned>(blocks), 256, 0, stream>>>(x, count, scale);
  return launch_status();
}

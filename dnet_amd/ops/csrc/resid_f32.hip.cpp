// fp32-residual layer plumbing (gfx950): kernels for model families that keep
// the residual stream, every norm statistic and every small per-channel
// parameter in 32-bit while activations are bf16 (or fp32).
//
//   rmsnorm_rows      y = x * rsqrt(mean(x^2) + eps) * w      (any in/out dtype)
//   ls_resid_rmsnorm  h += s1*a (+ s2*b);  y = rmsnorm(h) * wn (one pass per
//                     layer boundary: residual update fused with the next norm)
//   xielu             two-parameter squared / exponential activation
//   qknorm_append     RMS-normalize q and k (whole projection or per head),
//                     write q, append k and v to the KV cache at pos[b]+t
//
// One workgroup per token row; statistics are block-reduced in fp32. "short"
// stands for bf16 bits throughout.
#include "common.h"

namespace dnet {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<short>(const short* p) { return bits2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<short>(short* p, float v) { *p = f2bits(v); }

// W-wide element groups: W = 4 when every row length is a multiple of 4
// (16 B fp32 / 8 B bf16 accesses), else 1.
template <int W> struct vecf { float v[W]; };
template <int W, typename T>
__device__ __forceinline__ vecf<W> ldw(const T* p) {
  vecf<W> r;
  if constexpr (W == 1) {
    r.v[0] = ldf<T>(p);
  } else if constexpr (sizeof(T) == 4) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
  } else {
    const short4v t = *reinterpret_cast<const short4v*>(p);
#pragma unroll
    for (int j = 0; j < 4; ++j) r.v[j] = bits2f(t.x[j]);
  }
  return r;
}
template <int W, typename T>
__device__ __forceinline__ void stw(T* p, const vecf<W>& r) {
  if constexpr (W == 1) {
    stf<T>(p, r.v[0]);
  } else if constexpr (sizeof(T) == 4) {
    *reinterpret_cast<float4*>(p) = make_float4(r.v[0], r.v[1], r.v[2], r.v[3]);
  } else {
    short4v t;
#pragma unroll
    for (int j = 0; j < 4; ++j) t.x[j] = f2bits(r.v[j]);
    *reinterpret_cast<short4v*>(p) = t;
  }
}

template <typename TI, typename TO, int W>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(
    const TI* __restrict__ x, const float* __restrict__ w, TO* __restrict__ y,
    const int N, const float eps) {
  __shared__ float red[8];
  const int64_t row = blockIdx.x;
  const TI* xr = x + row * N;
  float ss = 0.f;
  for (int i = threadIdx.x * W; i < N; i += blockDim.x * W) {
    const vecf<W> v = ldw<W, TI>(xr + i);
#pragma unroll
    for (int j = 0; j < W; ++j) ss += v.v[j] * v.v[j];
  }
  ss = block_reduce_sum(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)N + eps);
  TO* yr = y + row * N;
  for (int i = threadIdx.x * W; i < N; i += blockDim.x * W) {
    vecf<W> v = ldw<W, TI>(xr + i);
    const vecf<W> g = ldw<W, float>(w + i);
#pragma unroll
    for (int j = 0; j < W; ++j) v.v[j] = v.v[j] * r * g.v[j];
    stw<W, TO>(yr + i, v);
  }
}

template <typename T, int W>
__global__ __launch_bounds__(256) void ls_resid_rmsnorm_kernel(
    float* __restrict__ h, const T* __restrict__ a, const float* __restrict__ s1,
    const T* __restrict__ b, const float* __restrict__ s2,
    const float* __restrict__ wn, T* __restrict__ y, const int N,
    const float eps) {
  __shared__ float red[8];
  const int64_t row = blockIdx.x;
  float* hr = h + row * N;
  const T* ar = a + row * N;
  const T* br = b ? b + row * N : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x * W; i < N; i += blockDim.x * W) {
    vecf<W> hv = ldw<W, float>(hr + i);
    const vecf<W> av = ldw<W, T>(ar + i), g1 = ldw<W, float>(s1 + i);
    vecf<W> d;
#pragma unroll
    for (int j = 0; j < W; ++j) d.v[j] = g1.v[j] * av.v[j];
    if (br) {
      const vecf<W> bv = ldw<W, T>(br + i), g2 = ldw<W, float>(s2 + i);
#pragma unroll
      for (int j = 0; j < W; ++j) d.v[j] += g2.v[j] * bv.v[j];
    }
#pragma unroll
    for (int j = 0; j < W; ++j) {
      hv.v[j] += d.v[j];
      ss += hv.v[j] * hv.v[j];
    }
    stw<W, float>(hr + i, hv);
  }
  if (!wn) return;                       // uniform: residual update only
  ss = block_reduce_sum(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)N + eps);
  T* yr = y + row * N;
  // each thread re-reads exactly the elements it wrote above
  for (int i = threadIdx.x * W; i < N; i += blockDim.x * W) {
    vecf<W> hv = ldw<W, float>(hr + i);
    const vecf<W> g = ldw<W, float>(wn + i);
#pragma unroll
    for (int j = 0; j < W; ++j) hv.v[j] = hv.v[j] * r * g.v[j];
    stw<W, T>(yr + i, hv);
  }
}

__device__ __forceinline__ float softplus_f(float t) {
  return t > 20.f ? t : log1pf(expf(t));
}

template <typename T, int W>
__global__ __launch_bounds__(256) void xielu_kernel(
    const T* __restrict__ z, const float* __restrict__ pq, T* __restrict__ y,
    const int64_t n) {
  const float ap = softplus_f(pq[0]);
  const float an = 0.5f + softplus_f(pq[1]);
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * W; i < n;
       i += (int64_t)gridDim.x * blockDim.x * W) {
    vecf<W> v = ldw<W, T>(z + i);
#pragma unroll
    for (int j = 0; j < W; ++j) {
      const float t = v.v[j];
      v.v[j] = t > 0.f ? ap * t * t + 0.5f * t
                       : an * (expm1f(t) - t) + 0.5f * t;
    }
    stw<W, T>(y + i, v);
  }
}

// qkv row layout: [q: nq*d | k: nkv*d | v: nkv*dv]. Token (b,t) = row b*T+t
// sits at position pos[b]+t of cache row slots[b] (default b); tokens with
// t >= lens[b] are padding: q is still written, the cache is not touched.
template <typename T, int W>
__global__ __launch_bounds__(256) void qknorm_append_kernel(
    const T* __restrict__ qkv, const float* __restrict__ qw,
    const float* __restrict__ kw, T* __restrict__ qout, T* __restrict__ kc,
    T* __restrict__ vc, const int* __restrict__ pos,
    const int* __restrict__ lens, const int* __restrict__ slots,
    const float eps, const int nq, const int nkv, const int d, const int dv,
    const int Tn, const int Bc, const int Hkv, const int Smax,
    const bool per_head) {
  __shared__ float red[8];
  const int64_t row = blockIdx.x;
  const int b = (int)(row / Tn);
  const int t = (int)(row % Tn);
  const int NQ = nq * d, NK = nkv * d, NV = nkv * dv;
  const T* src = qkv + row * (int64_t)(NQ + NK + NV);
  const int p = pos[b] + t;
  const int slot = slots ? slots[b] : b;
  const bool keep = (!lens || t < lens[b]) && p >= 0 && p < Smax &&
                    slot >= 0 && slot < Bc;
  T* qo = qout + row * (int64_t)NQ;
  const int64_t kbase = ((int64_t)slot * Hkv * Smax + p) * d;
  const int64_t vbase = ((int64_t)slot * Hkv * Smax + p) * dv;
  if (!per_head) {
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x * W; i < NQ; i += blockDim.x * W) {
      const vecf<W> v = ldw<W, T>(src + i);
#pragma unroll
      for (int j = 0; j < W; ++j) sq += v.v[j] * v.v[j];
    }
    for (int i = threadIdx.x * W; i < NK; i += blockDim.x * W) {
      const vecf<W> v = ldw<W, T>(src + NQ + i);
#pragma unroll
      for (int j = 0; j < W; ++j) sk += v.v[j] * v.v[j];
    }
    sq = block_reduce_sum(sq, red);
    sk = block_reduce_sum(sk, red);
    const float rq = 1.0f / sqrtf(sq / (float)NQ + eps);
    const float rk = 1.0f / sqrtf(sk / (float)NK + eps);
    for (int i = threadIdx.x * W; i < NQ; i += blockDim.x * W) {
      vecf<W> v = ldw<W, T>(src + i);
      const vecf<W> g = ldw<W, float>(qw + i);
#pragma unroll
      for (int j = 0; j < W; ++j) v.v[j] = v.v[j] * rq * g.v[j];
      stw<W, T>(qo + i, v);
    }
    if (keep)
      for (int i = threadIdx.x * W; i < NK; i += blockDim.x * W) {
        const int hk = i / d, e = i % d;       // d % W == 0: no straddling
        vecf<W> v = ldw<W, T>(src + NQ + i);
        const vecf<W> g = ldw<W, float>(kw + i);
#pragma unroll
        for (int j = 0; j < W; ++j) v.v[j] = v.v[j] * rk * g.v[j];
        stw<W, T>(kc + kbase + (int64_t)hk * Smax * d + e, v);
      }
  } else {
    // one wave per head; weights are per head-dim element
    const int wid = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
    const int nw = blockDim.x / kWave;
    for (int hh = wid; hh < nq + nkv; hh += nw) {
      const bool isq = hh < nq;
      const T* hs = isq ? src + hh * d : src + NQ + (hh - nq) * d;
      float ss = 0.f;
      for (int e = lane; e < d; e += kWave) {
        const float v = ldf<T>(hs + e);
        ss += v * v;
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
      const float r = 1.0f / sqrtf(ss / (float)d + eps);
      if (isq) {
        for (int e = lane; e < d; e += kWave)
          stf<T>(qo + hh * d + e, ldf<T>(hs + e) * r * qw[e]);
      } else if (keep) {
        for (int e = lane; e < d; e += kWave)
          stf<T>(kc + kbase + (int64_t)(hh - nq) * Smax * d + e,
                 ldf<T>(hs + e) * r * kw[e]);
      }
    }
  }
  if (keep)
    for (int i = threadIdx.x * W; i < NV; i += blockDim.x * W) {
      const int hk = i / dv, e = i % dv;
      stw<W, T>(vc + vbase + (int64_t)hk * Smax * dv + e,
                ldw<W, T>(src + NQ + NK + i));
    }
}

static bool is_bf16(const torch::Tensor& t) {
  return t.scalar_type() == torch::kBFloat16;
}
static bool is_f32(const torch::Tensor& t) {
  return t.scalar_type() == torch::kFloat32;
}
static const float* f32p(const c10::optional<torch::Tensor>& t) {
  if (!t.has_value()) return nullptr;
  DNET_CHECK(is_f32(*t) && t->is_contiguous(), "fp32 contiguous parameter");
  return t->data_ptr<float>();
}
static const int* i32p(const c10::optional<torch::Tensor>& t, int64_t n) {
  if (!t.has_value()) return nullptr;
  DNET_CHECK(t->scalar_type() == torch::kInt32 && t->is_contiguous() &&
                 t->numel() >= n, "int32 index tensor");
  return t->data_ptr<int>();
}

void rmsnorm_rows(torch::Tensor x, torch::Tensor w, torch::Tensor y,
                  double eps) {
  const int N = x.size(-1);
  const int64_t M = x.numel() / N;
  DNET_CHECK(x.is_contiguous() && y.is_contiguous() && y.numel() == x.numel(),
             "rmsnorm_rows: contiguous, same shape");
  DNET_CHECK(is_f32(w) && w.numel() == N && w.is_contiguous(), "w fp32 [N]");
  if (M == 0) return;
  auto st = current_stream();
  const float* wp = w.data_ptr<float>();
#define RN(TI, TO)                                                          \
  do {                                                                      \
    if (N % 4 == 0)                                                         \
      hipLaunchKernelGGL((rmsnorm_rows_kernel<TI, TO, 4>), dim3(M),         \
                         dim3(256), 0, st, (const TI*)x.data_ptr(), wp,     \
                         (TO*)y.data_ptr(), N, (float)eps);                 \
    else                                                                    \
      hipLaunchKernelGGL((rmsnorm_rows_kernel<TI, TO, 1>), dim3(M),         \
                         dim3(256), 0, st, (const TI*)x.data_ptr(), wp,     \
                         (TO*)y.data_ptr(), N, (float)eps);                 \
  } while (0)
  if (is_f32(x) && is_f32(y)) RN(float, float);
  else if (is_f32(x) && is_bf16(y)) RN(float, short);
  else if (is_bf16(x) && is_bf16(y)) RN(short, short);
  else if (is_bf16(x) && is_f32(y)) RN(short, float);
  else DNET_CHECK(false, "rmsnorm_rows: dtypes");
#undef RN
}

void ls_resid_rmsnorm(torch::Tensor h, torch::Tensor a, torch::Tensor s1,
                      c10::optional<torch::Tensor> b,
                      c10::optional<torch::Tensor> s2,
                      c10::optional<torch::Tensor> wn,
                      c10::optional<torch::Tensor> y, double eps) {
  const int N = h.size(-1);
  const int64_t M = h.numel() / N;
  DNET_CHECK(is_f32(h) && h.is_contiguous(), "h fp32 contiguous");
  DNET_CHECK(a.is_contiguous() && a.numel() == h.numel(), "a shape");
  DNET_CHECK(is_f32(s1) && s1.numel() == N, "s1 fp32 [N]");
  DNET_CHECK(b.has_value() == s2.has_value(), "b and s2 come together");
  if (b.has_value())
    DNET_CHECK(b->is_contiguous() && b->numel() == h.numel() &&
                   b->scalar_type() == a.scalar_type() && s2->numel() == N,
               "b shape/dtype");
  DNET_CHECK(wn.has_value() == y.has_value(), "wn and y come together");
  if (wn.has_value())
    DNET_CHECK(wn->numel() == N && y->is_contiguous() &&
                   y->numel() == h.numel() &&
                   y->scalar_type() == a.scalar_type(), "y shape/dtype");
  if (M == 0) return;
  auto st = current_stream();
#define LR(TT, WW)                                                          \
  hipLaunchKernelGGL((ls_resid_rmsnorm_kernel<TT, WW>), dim3(M), dim3(256), \
                     0, st, h.data_ptr<float>(), (const TT*)a.data_ptr(),   \
                     s1.data_ptr<float>(),                                  \
                     b.has_value() ? (const TT*)b->data_ptr() : nullptr,    \
                     f32p(s2), f32p(wn),                                    \
                     y.has_value() ? (TT*)y->data_ptr() : nullptr, N,       \
                     (float)eps)
  const bool v4 = N % 4 == 0;
  if (is_bf16(a)) { if (v4) LR(short, 4); else LR(short, 1); }
  else if (is_f32(a)) { if (v4) LR(float, 4); else LR(float, 1); }
  else DNET_CHECK(false, "ls_resid_rmsnorm: dtype");
#undef LR
}

void xielu(torch::Tensor z, torch::Tensor pq, torch::Tensor y) {
  DNET_CHECK(z.is_contiguous() && y.is_contiguous() &&
                 y.numel() == z.numel() && y.scalar_type() == z.scalar_type(),
             "xielu: shapes");
  DNET_CHECK(is_f32(pq) && pq.numel() == 2, "pq fp32 [2]");
  const int64_t n = z.numel();
  if (n == 0) return;
  const bool v4 = n % 4 == 0;
  const int64_t work = v4 ? n / 4 : n;
  const int blocks = (int)std::min<int64_t>((work + 255) / 256, 256 * 16);
  auto st = current_stream();
#define XI(TT, WW)                                                          \
  hipLaunchKernelGGL((xielu_kernel<TT, WW>), dim3(blocks), dim3(256), 0, st, \
                     (const TT*)z.data_ptr(), pq.data_ptr<float>(),         \
                     (TT*)y.data_ptr(), n)
  if (is_bf16(z)) { if (v4) XI(short, 4); else XI(short, 1); }
  else if (is_f32(z)) { if (v4) XI(float, 4); else XI(float, 1); }
  else DNET_CHECK(false, "xielu: dtype");
#undef XI
}

void qknorm_append(torch::Tensor qkv, torch::Tensor qw, torch::Tensor kw,
                   torch::Tensor qout, torch::Tensor kcache,
                   torch::Tensor vcache, torch::Tensor pos,
                   c10::optional<torch::Tensor> lens,
                   c10::optional<torch::Tensor> slots, double eps, int64_t nq,
                   int64_t nkv, int64_t d, int64_t dv, int64_t T,
                   bool per_head) {
  const int64_t M = qkv.size(0);
  DNET_CHECK(T > 0 && M % T == 0, "rows = B*T");
  const int64_t B = M / T;
  DNET_CHECK(qkv.is_contiguous() && qkv.size(1) == (nq + nkv) * d + nkv * dv,
             "qkv [M, nq*d + nkv*d + nkv*dv]");
  DNET_CHECK(qout.is_contiguous() && qout.size(0) == M &&
                 qout.size(1) == nq * d, "qout shape");
  DNET_CHECK(kcache.dim() == 4 && vcache.dim() == 4 &&
                 kcache.is_contiguous() && vcache.is_contiguous(), "cache");
  const int Bc = kcache.size(0), Hkv = kcache.size(1), Smax = kcache.size(2);
  DNET_CHECK(Hkv == nkv && kcache.size(3) == d && vcache.size(3) == dv &&
                 vcache.size(0) == Bc && vcache.size(1) == Hkv &&
                 vcache.size(2) == Smax, "cache dims");
  DNET_CHECK(qout.scalar_type() == qkv.scalar_type() &&
                 kcache.scalar_type() == qkv.scalar_type() &&
                 vcache.scalar_type() == qkv.scalar_type(), "dtypes");
  DNET_CHECK(is_f32(qw) && is_f32(kw) &&
                 qw.numel() == (per_head ? d : nq * d) &&
                 kw.numel() == (per_head ? d : nkv * d), "norm weights");
  if (!slots.has_value()) DNET_CHECK(B <= Bc, "more rows than cache slots");
  if (M == 0) return;
  auto st = current_stream();
#define QA(TT, WW)                                                           \
  hipLaunchKernelGGL((qknorm_append_kernel<TT, WW>), dim3(M), dim3(256), 0,  \
                     st,                                                     \
                     (const TT*)qkv.data_ptr(), qw.data_ptr<float>(),        \
                     kw.data_ptr<float>(), (TT*)qout.data_ptr(),             \
                     (TT*)kcache.data_ptr(), (TT*)vcache.data_ptr(),         \
                     i32p(pos, B), i32p(lens, B), i32p(slots, B), (float)eps, \
                     (int)nq, (int)nkv, (int)d, (int)dv, (int)T, Bc, Hkv,     \
                     Smax,                                                   \
                     per_head)
  const bool v4 = d % 4 == 0 && dv % 4 == 0;
  if (is_bf16(qkv)) { if (v4) QA(short, 4); else QA(short, 1); }
  else if (is_f32(qkv)) { if (v4) QA(float, 4); else QA(float, 1); }
  else DNET_CHECK(false, "qknorm_append: dtype");
#undef QA
}

}  // namespace dnet

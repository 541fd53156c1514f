// fp32-residual layer plumbing (gfx950): kernels for model families that keep
// the residual stream, every norm statistic and every small per-channel
// parameter in 32-bit while activations are bf16 (or fp32).
//
//   rmsnorm_rows      y = x * rsqrt(mean(x^2) + eps) * w      (any in/out dtype)
//   ls_resid_rmsnorm  h += s1*a (+ s2*b);  y = rmsnorm(h) * wn (one pass per
//                     layer boundary: residual update fused with the next norm)
//   xielu             two-parameter squared / exponential activation
//   qknorm_append     RMS-normalize q and k (whole projection or per head),
//                     optionally rotate interleaved channel pairs by position,
//                     write q, append k and v to the KV cache at pos[b]+t
//   resid_branches_rmsnorm  h += coef*(nrm(a) + nrm(b)) + f with optional
//                     RMS-normalized branches, next norm and a cast copy of h
//   gated_group_rmsnorm     grouped RMSNorm with a silu / sigmoid gate
//   act_slice, gelu_gather_mul, clamped_glu   small element-wise steps
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

// a channel pair (2i, 2i+1) as one 4 B (bf16) or 8 B (fp32) access
template <typename T>
__device__ __forceinline__ void ld_pair(const T* p, float& a, float& b);
template <> __device__ __forceinline__ void ld_pair<float>(const float* p, float& a, float& b) {
  const float2 t = *reinterpret_cast<const float2*>(p);
  a = t.x; b = t.y;
}
template <> __device__ __forceinline__ void ld_pair<short>(const short* p, float& a, float& b) {
  const unsigned t = *reinterpret_cast<const unsigned*>(p);
  union { unsigned u; float f; } lo, hi;
  lo.u = t << 16;
  hi.u = t & 0xffff0000u;
  a = lo.f; b = hi.f;
}
template <typename T>
__device__ __forceinline__ void st_pair(T* p, float a, float b);
template <> __device__ __forceinline__ void st_pair<float>(float* p, float a, float b) {
  *reinterpret_cast<float2*>(p) = make_float2(a, b);
}
template <> __device__ __forceinline__ void st_pair<short>(short* p, float a, float b) {
  *reinterpret_cast<unsigned*>(p) =
      (unsigned)(unsigned short)f2bits(a) | ((unsigned)(unsigned short)f2bits(b) << 16);
}

constexpr int kMaxRot = 128;   // rotated pairs per head (head size <= 256)

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
    const bool per_head, const float* __restrict__ rot_freq,
    const int nrot, const bool pairs) {
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
    // every head of the row turns by the same angles: one sincos per pair
    __shared__ float rot_c[kMaxRot], rot_s[kMaxRot];
    for (int i = threadIdx.x; i < nrot; i += blockDim.x)
      sincosf((float)p * rot_freq[i], &rot_s[i], &rot_c[i]);
    if (nrot > 0) __syncthreads();
    for (int hh = wid; hh < nq + nkv; hh += nw) {
      const bool isq = hh < nq;
      const T* hs = isq ? src + hh * d : src + NQ + (hh - nq) * d;
      if (!isq && !keep) continue;            // wave-uniform
      const float* wv = isq ? qw : kw;
      T* dst = isq ? qo + hh * d
                   : kc + kbase + (int64_t)(hh - nq) * Smax * d;
      if (d <= 4 * kWave) {
        // one read: a lane keeps channel pairs (2i, 2i+1), i = lane, lane+64
        float v0[2], v1[2];
        float ss = 0.f;
#pragma unroll
        for (int qd = 0; qd < 2; ++qd) {
          const int e0 = 2 * (lane + kWave * qd);
          v0[qd] = v1[qd] = 0.f;
          if (pairs) {                // d even, rows pair-aligned (uniform)
            if (e0 < d) ld_pair<T>(hs + e0, v0[qd], v1[qd]);
          } else {
            if (e0 < d) v0[qd] = ldf<T>(hs + e0);
            if (e0 + 1 < d) v1[qd] = ldf<T>(hs + e0 + 1);
          }
          ss += v0[qd] * v0[qd] + v1[qd] * v1[qd];
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
        const float r = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
        for (int qd = 0; qd < 2; ++qd) {
          const int pr = lane + kWave * qd;
          const int e0 = 2 * pr, e1 = e0 + 1;
          if (e0 >= d) continue;
          float a0 = v0[qd] * r * wv[e0];
          float a1 = e1 < d ? v1[qd] * r * wv[e1] : 0.f;
          if (pr < nrot && e1 < d) {
            // pairs i < nrot turn by position * rot_freq[i], in fp32
            const float sn = rot_s[pr], cs = rot_c[pr];
            const float u0 = a0 * cs - a1 * sn;
            a1 = a1 * cs + a0 * sn;
            a0 = u0;
          }
          if (pairs) {
            st_pair<T>(dst + e0, a0, a1);
          } else {
            stf<T>(dst + e0, a0);
            if (e1 < d) stf<T>(dst + e1, a1);
          }
        }
        continue;
      }
      float ss = 0.f;
      for (int e = lane; e < d; e += kWave) {
        const float v = ldf<T>(hs + e);
        ss += v * v;
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
      const float r = 1.0f / sqrtf(ss / (float)d + eps);
      for (int pr = lane; 2 * pr < d; pr += kWave) {
        const int e0 = 2 * pr, e1 = e0 + 1;
        float a0 = ldf<T>(hs + e0) * r * wv[e0];
        float a1 = e1 < d ? ldf<T>(hs + e1) * r * wv[e1] : 0.f;
        if (pr < nrot && e1 < d) {
          const float sn = rot_s[pr], cs = rot_c[pr];
          const float u0 = a0 * cs - a1 * sn;
          a1 = a1 * cs + a0 * sn;
          a0 = u0;
        }
        stf<T>(dst + e0, a0);
        if (e1 < d) stf<T>(dst + e1, a1);
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


// ---- branch sums, grouped gated norms, small element-wise steps ----------

template <typename T>
__device__ __forceinline__ float row_sumsq(const T* __restrict__ x, const int N,
                                           float* red) {
  float ss = 0.f;
  for (int i = threadIdx.x; i < N; i += blockDim.x) {
    const float v = ldf<T>(x + i);
    ss += v * v;
  }
  return block_reduce_sum(ss, red);
}

// h += coef * (nrm(a, wa) + nrm(b, wb)) + f;  nrm(x, w) = x * rsqrt(mean(x^2)
// + eps) * w, or x when w is null. Then y = rmsnorm(h) * wn (wn given) and
// xc = h in the activation dtype (xc given). f may be fp32 or T.
template <typename T, int W>
__global__ __launch_bounds__(256) void resid_branches_kernel(
    float* __restrict__ h, const T* __restrict__ a, const float* __restrict__ wa,
    const T* __restrict__ b, const float* __restrict__ wb, const float coef,
    const void* __restrict__ f, const bool f_f32, const float* __restrict__ wn,
    T* __restrict__ y, T* __restrict__ xc, const int N, const float eps) {
  __shared__ float red[8];
  const int64_t row = blockIdx.x;
  float* hr = h + row * N;
  const T* ar = a + row * N;
  const T* br = b ? b + row * N : nullptr;
  float ra = 1.f, rb = 1.f;
  if (wa) ra = 1.0f / sqrtf(row_sumsq<T>(ar, N, red) / (float)N + eps);
  if (br && wb) rb = 1.0f / sqrtf(row_sumsq<T>(br, N, red) / (float)N + eps);
  float ss = 0.f;
  for (int i = threadIdx.x * W; i < N; i += blockDim.x * W) {
    vecf<W> hv = ldw<W, float>(hr + i);
    vecf<W> d = ldw<W, T>(ar + i);
    if (wa) {
      const vecf<W> g = ldw<W, float>(wa + i);
#pragma unroll
      for (int j = 0; j < W; ++j) d.v[j] = d.v[j] * ra * g.v[j];
    }
    if (br) {
      vecf<W> e = ldw<W, T>(br + i);
      if (wb) {
        const vecf<W> g = ldw<W, float>(wb + i);
#pragma unroll
        for (int j = 0; j < W; ++j) e.v[j] = e.v[j] * rb * g.v[j];
      }
#pragma unroll
      for (int j = 0; j < W; ++j) d.v[j] += e.v[j];
    }
#pragma unroll
    for (int j = 0; j < W; ++j) d.v[j] *= coef;
    if (f) {
      const vecf<W> fv =
          f_f32 ? ldw<W, float>(reinterpret_cast<const float*>(f) + row * N + i)
                : ldw<W, T>(reinterpret_cast<const T*>(f) + row * N + i);
#pragma unroll
      for (int j = 0; j < W; ++j) d.v[j] += fv.v[j];
    }
#pragma unroll
    for (int j = 0; j < W; ++j) {
      hv.v[j] += d.v[j];
      ss += hv.v[j] * hv.v[j];
    }
    stw<W, float>(hr + i, hv);
    if (xc) stw<W, T>(xc + row * N + i, hv);
  }
  if (!wn) return;                       // uniform
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

__device__ __forceinline__ float sigmoid_f(float x) {
  return 1.0f / (1.0f + expf(-x));
}

// One wave per (row, group): out = rms_group(y [* gate]) * w [* gate], gate =
// silu or sigmoid of columns [gcol0, gcol0+N) of gate_src (row stride gld).
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void gated_group_rmsnorm_kernel(
    const float* __restrict__ y, const TG* __restrict__ gate_src,
    const int64_t gld, const int gcol0, const float* __restrict__ w,
    TO* __restrict__ out, const int N, const int groups, const float eps,
    const bool gate_silu, const bool gate_first) {
  const int wid = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int64_t row = blockIdx.y;
  const int grp = blockIdx.x * (blockDim.x / kWave) + wid;
  if (grp >= groups) return;             // wave-uniform
  const int gs = N / groups;
  const float* yr = y + row * N + (int64_t)grp * gs;
  const TG* gr = gate_src + row * gld + gcol0 + (int64_t)grp * gs;
  float ss = 0.f;
  for (int e = lane; e < gs; e += kWave) {
    float v = yr[e];
    if (gate_first) {
      const float g = ldf<TG>(gr + e);
      v *= gate_silu ? g * sigmoid_f(g) : sigmoid_f(g);
    }
    ss += v * v;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
  const float r = 1.0f / sqrtf(ss / (float)gs + eps);
  TO* orow = out + row * N + (int64_t)grp * gs;
  const float* wr = w + (int64_t)grp * gs;
  for (int e = lane; e < gs; e += kWave) {
    const float g = ldf<TG>(gr + e);
    const float gv = gate_silu ? g * sigmoid_f(g) : sigmoid_f(g);
    float v = yr[e];
    if (gate_first) v *= gv;
    v = v * r * wr[e];
    if (!gate_first) v *= gv;
    stf<TO>(orow + e, v);
  }
}

// Wide groups (>= 1024 channels): one workgroup per (row, group), 4-wide
// accesses when the group size and the gate's stride and offset allow.
template <typename TG, typename TO, int W>
__global__ __launch_bounds__(256) void gated_group_rmsnorm_wide_kernel(
    const float* __restrict__ y, const TG* __restrict__ gate_src,
    const int64_t gld, const int gcol0, const float* __restrict__ w,
    TO* __restrict__ out, const int N, const int groups, const float eps,
    const bool gate_silu, const bool gate_first) {
  __shared__ float red[8];
  const int64_t row = blockIdx.y;
  const int grp = blockIdx.x;
  const int gs = N / groups;
  const float* yr = y + row * N + (int64_t)grp * gs;
  const TG* gr = gate_src + row * gld + gcol0 + (int64_t)grp * gs;
  float ss = 0.f;
  for (int e = threadIdx.x * W; e < gs; e += blockDim.x * W) {
    vecf<W> v = ldw<W, float>(yr + e);
    if (gate_first) {
      const vecf<W> g = ldw<W, TG>(gr + e);
#pragma unroll
      for (int j = 0; j < W; ++j)
        v.v[j] *= gate_silu ? g.v[j] * sigmoid_f(g.v[j]) : sigmoid_f(g.v[j]);
    }
#pragma unroll
    for (int j = 0; j < W; ++j) ss += v.v[j] * v.v[j];
  }
  ss = block_reduce_sum(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)gs + eps);
  TO* orow = out + row * N + (int64_t)grp * gs;
  const float* wr = w + (int64_t)grp * gs;
  for (int e = threadIdx.x * W; e < gs; e += blockDim.x * W) {
    vecf<W> v = ldw<W, float>(yr + e);
    const vecf<W> g = ldw<W, TG>(gr + e), wv = ldw<W, float>(wr + e);
#pragma unroll
    for (int j = 0; j < W; ++j) {
      const float gv =
          gate_silu ? g.v[j] * sigmoid_f(g.v[j]) : sigmoid_f(g.v[j]);
      float t = v.v[j];
      if (gate_first) t *= gv;
      t = t * r * wv.v[j];
      if (!gate_first) t *= gv;
      v.v[j] = t;
    }
    stw<W, TO>(orow + e, v);
  }
}

// kind 0: max(z, 0)^2, kind 1: tanh(z); columns [col0, col0+n) of x (stride
// ld); W = 4 when ld, col0 and n are multiples of 4
template <typename T, int W>
__global__ __launch_bounds__(256) void act_slice_kernel(
    const T* __restrict__ x, const int64_t ld, const int col0,
    T* __restrict__ y, const int n, const int64_t total, const int kind) {
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * W;
       i < total; i += (int64_t)gridDim.x * blockDim.x * W) {
    const int64_t row = i / n;
    const int c = (int)(i % n);
    vecf<W> v = ldw<W, T>(x + row * ld + col0 + c);
#pragma unroll
    for (int j = 0; j < W; ++j) {
      if (kind == 0) {
        const float t = fmaxf(v.v[j], 0.f);
        v.v[j] = t * t;
      } else {
        v.v[j] = tanhf(v.v[j]);
      }
    }
    stw<W, T>(y + i, v);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_gather_mul_kernel(
    const T* __restrict__ z, const T* __restrict__ table, const int64_t tld,
    const int64_t V, const int64_t* __restrict__ tokens, const int col0,
    T* __restrict__ y, const int n, const int64_t total) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = i / n;
    const int c = (int)(i % n);
    int64_t tok = tokens[row];
    tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);
    const float v = ldf<T>(z + i);
    const float g =
        0.5f * v *
        (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    stf<T>(y + i, g * ldf<T>(table + tok * tld + col0 + c));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void clamped_glu_kernel(
    const T* __restrict__ gu, T* __restrict__ y, const int I,
    const int64_t total, const float alpha, const float limit) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = i / I;
    const int c = (int)(i % I);
    const float g = fminf(ldf<T>(gu + row * 2 * I + c), limit);
    const float u =
        fminf(fmaxf(ldf<T>(gu + row * 2 * I + I + c), -limit), limit);
    stf<T>(y + i, g * sigmoid_f(alpha * g) * (u + 1.0f));
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
                   bool per_head, c10::optional<torch::Tensor> rot_freq) {
  const int64_t M = qkv.size(0);
  int nrot = 0;
  if (rot_freq.has_value()) {
    DNET_CHECK(per_head, "rotation comes with the per-head norm");
    DNET_CHECK(is_f32(*rot_freq) && rot_freq->is_contiguous() &&
                   rot_freq->numel() * 2 <= d &&
                   rot_freq->numel() <= kMaxRot, "rot_freq fp32 [<= d/2]");
    nrot = (int)rot_freq->numel();
  }
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
                     per_head, nrot ? rot_freq->data_ptr<float>() : nullptr, \
                     nrot, pairs)
  const bool v4 = d % 4 == 0 && dv % 4 == 0;
  // per-head path: channel pairs as single accesses when every head starts
  // on a pair boundary in the projection row, in q and in the cache
  const bool pairs = d % 2 == 0 && qkv.size(1) % 2 == 0;
  if (is_bf16(qkv)) { if (v4) QA(short, 4); else QA(short, 1); }
  else if (is_f32(qkv)) { if (v4) QA(float, 4); else QA(float, 1); }
  else DNET_CHECK(false, "qknorm_append: dtype");
#undef QA
}

void resid_branches_rmsnorm(torch::Tensor h, torch::Tensor a,
                            c10::optional<torch::Tensor> wa,
                            c10::optional<torch::Tensor> b,
                            c10::optional<torch::Tensor> wb, double coef,
                            c10::optional<torch::Tensor> f,
                            c10::optional<torch::Tensor> wn,
                            c10::optional<torch::Tensor> y,
                            c10::optional<torch::Tensor> xc, double eps) {
  const int N = h.size(-1);
  const int64_t M = h.numel() / N;
  DNET_CHECK(is_f32(h) && h.is_contiguous(), "h fp32 contiguous");
  DNET_CHECK(a.is_contiguous() && a.numel() == h.numel() &&
                 (is_bf16(a) || is_f32(a)), "a shape/dtype");
  if (wa.has_value()) DNET_CHECK(wa->numel() == N, "wa fp32 [N]");
  if (b.has_value())
    DNET_CHECK(b->is_contiguous() && b->numel() == h.numel() &&
                   b->scalar_type() == a.scalar_type(), "b shape/dtype");
  if (wb.has_value()) DNET_CHECK(b.has_value() && wb->numel() == N, "wb");
  bool f_f32 = false;
  if (f.has_value()) {
    DNET_CHECK(f->is_contiguous() && f->numel() == h.numel() &&
                   (is_f32(*f) || f->scalar_type() == a.scalar_type()),
               "f shape/dtype");
    f_f32 = is_f32(*f);
  }
  DNET_CHECK(wn.has_value() == y.has_value(), "wn and y come together");
  if (wn.has_value())
    DNET_CHECK(wn->numel() == N && y->is_contiguous() &&
                   y->numel() == h.numel() &&
                   y->scalar_type() == a.scalar_type(), "y shape/dtype");
  if (xc.has_value())
    DNET_CHECK(xc->is_contiguous() && xc->numel() == h.numel() &&
                   xc->scalar_type() == a.scalar_type(), "xc shape/dtype");
  if (M == 0) return;
  auto st = current_stream();
#define RB(TT, WW)                                                           \
  hipLaunchKernelGGL((resid_branches_kernel<TT, WW>), dim3(M), dim3(256), 0, \
                     st, h.data_ptr<float>(), (const TT*)a.data_ptr(),       \
                     f32p(wa),                                               \
                     b.has_value() ? (const TT*)b->data_ptr() : nullptr,     \
                     f32p(wb), (float)coef,                                  \
                     f.has_value() ? (const void*)f->data_ptr() : nullptr,   \
                     f_f32, f32p(wn),                                        \
                     y.has_value() ? (TT*)y->data_ptr() : nullptr,           \
                     xc.has_value() ? (TT*)xc->data_ptr() : nullptr, N,      \
                     (float)eps)
  const bool v4 = N % 4 == 0;
  if (is_bf16(a)) { if (v4) RB(short, 4); else RB(short, 1); }
  else { if (v4) RB(float, 4); else RB(float, 1); }
#undef RB
}

void gated_group_rmsnorm(torch::Tensor y, torch::Tensor gate_src,
                         int64_t gate_col0, torch::Tensor w, torch::Tensor out,
                         int64_t groups, double eps, bool gate_silu,
                         bool gate_first) {
  DNET_CHECK(y.dim() == 2 && is_f32(y) && y.is_contiguous(), "y fp32 [M, N]");
  const int64_t M = y.size(0);
  const int N = y.size(1);
  DNET_CHECK(groups > 0 && N % groups == 0, "groups divide N");
  DNET_CHECK(gate_src.dim() == 2 && gate_src.is_contiguous() &&
                 gate_src.size(0) == M && gate_col0 >= 0 &&
                 gate_col0 + N <= gate_src.size(1), "gate columns");
  DNET_CHECK(is_f32(w) && w.is_contiguous() && w.numel() == N, "w fp32 [N]");
  DNET_CHECK(out.is_contiguous() && out.size(0) == M && out.size(1) == N,
             "out [M, N]");
  if (M == 0) return;
  auto st = current_stream();
  const int gs = N / (int)groups;
  const bool wide = gs >= 1024;
  const bool v4 = gs % 4 == 0 && gate_src.size(1) % 4 == 0 && gate_col0 % 4 == 0;
  const dim3 grid(wide ? (unsigned)groups : (unsigned)((groups + 3) / 4),
                  (unsigned)M);
#define GG_ARGS(TG, TO)                                                      \
  grid, dim3(256), 0, st, y.data_ptr<float>(),                               \
      (const TG*)gate_src.data_ptr(), gate_src.size(1), (int)gate_col0,      \
      w.data_ptr<float>(), (TO*)out.data_ptr(), N, (int)groups, (float)eps,  \
      gate_silu, gate_first
#define GG(TG, TO)                                                           \
  do {                                                                       \
    if (wide && v4)                                                          \
      hipLaunchKernelGGL((gated_group_rmsnorm_wide_kernel<TG, TO, 4>),       \
                         GG_ARGS(TG, TO));                                   \
    else if (wide)                                                           \
      hipLaunchKernelGGL((gated_group_rmsnorm_wide_kernel<TG, TO, 1>),       \
                         GG_ARGS(TG, TO));                                   \
    else                                                                     \
      hipLaunchKernelGGL((gated_group_rmsnorm_kernel<TG, TO>),               \
                         GG_ARGS(TG, TO));                                   \
  } while (0)
  if (is_bf16(gate_src) && is_bf16(out)) GG(short, short);
  else if (is_f32(gate_src) && is_f32(out)) GG(float, float);
  else if (is_bf16(gate_src) && is_f32(out)) GG(short, float);
  else if (is_f32(gate_src) && is_bf16(out)) GG(float, short);
  else DNET_CHECK(false, "gated_group_rmsnorm: dtypes");
#undef GG_ARGS
#undef GG
}

static int ew_blocks(int64_t total) {
  return (int)std::min<int64_t>((total + 255) / 256, 256 * 16);
}

void act_slice(torch::Tensor x, int64_t col0, torch::Tensor y, int64_t kind) {
  DNET_CHECK(x.dim() == 2 && x.is_contiguous() && y.dim() == 2 &&
                 y.is_contiguous() && y.size(0) == x.size(0) &&
                 y.scalar_type() == x.scalar_type(), "act_slice: shapes");
  const int n = y.size(1);
  DNET_CHECK(col0 >= 0 && col0 + n <= x.size(1), "act_slice: columns");
  DNET_CHECK(kind == 0 || kind == 1, "act_slice: kind");
  const int64_t total = y.numel();
  if (total == 0) return;
  auto st = current_stream();
  const bool v4 = x.size(1) % 4 == 0 && col0 % 4 == 0 && n % 4 == 0;
  const int blocks = ew_blocks(v4 ? total / 4 : total);
#define AS(TT, WW)                                                           \
  hipLaunchKernelGGL((act_slice_kernel<TT, WW>), dim3(blocks), dim3(256), 0, \
                     st, (const TT*)x.data_ptr(), x.size(1), (int)col0,      \
                     (TT*)y.data_ptr(), n, total, (int)kind)
  if (is_bf16(x)) { if (v4) AS(short, 4); else AS(short, 1); }
  else if (is_f32(x)) { if (v4) AS(float, 4); else AS(float, 1); }
  else DNET_CHECK(false, "act_slice: dtype");
#undef AS
}

void gelu_gather_mul(torch::Tensor z, torch::Tensor table,
                     torch::Tensor tokens, int64_t col0, torch::Tensor y) {
  DNET_CHECK(z.dim() == 2 && z.is_contiguous() && y.is_contiguous() &&
                 y.numel() == z.numel() &&
                 y.scalar_type() == z.scalar_type(), "gelu_gather_mul: z/y");
  DNET_CHECK(table.dim() == 2 && table.is_contiguous() &&
                 table.scalar_type() == z.scalar_type() && col0 >= 0 &&
                 col0 + z.size(1) <= table.size(1), "table columns");
  DNET_CHECK(tokens.scalar_type() == torch::kInt64 && tokens.is_contiguous() &&
                 tokens.numel() == z.size(0), "tokens int64 [M]");
  const int64_t total = z.numel();
  if (total == 0) return;
  auto st = current_stream();
  if (is_bf16(z))
    hipLaunchKernelGGL((gelu_gather_mul_kernel<short>),
                       dim3(ew_blocks(total)), dim3(256), 0, st,
                       (const short*)z.data_ptr(),
                       (const short*)table.data_ptr(), table.size(1),
                       table.size(0), tokens.data_ptr<int64_t>(), (int)col0,
                       (short*)y.data_ptr(), (int)z.size(1), total);
  else if (is_f32(z))
    hipLaunchKernelGGL((gelu_gather_mul_kernel<float>),
                       dim3(ew_blocks(total)), dim3(256), 0, st,
                       (const float*)z.data_ptr(),
                       (const float*)table.data_ptr(), table.size(1),
                       table.size(0), tokens.data_ptr<int64_t>(), (int)col0,
                       (float*)y.data_ptr(), (int)z.size(1), total);
  else DNET_CHECK(false, "gelu_gather_mul: dtype");
}

void clamped_glu(torch::Tensor gu, torch::Tensor y, double alpha,
                 double limit) {
  DNET_CHECK(gu.dim() == 2 && gu.is_contiguous() && gu.size(1) % 2 == 0 &&
                 y.is_contiguous() && y.size(0) == gu.size(0) &&
                 y.size(1) * 2 == gu.size(1) &&
                 y.scalar_type() == gu.scalar_type(), "clamped_glu: shapes");
  const int64_t total = y.numel();
  if (total == 0) return;
  auto st = current_stream();
  if (is_bf16(gu))
    hipLaunchKernelGGL((clamped_glu_kernel<short>), dim3(ew_blocks(total)),
                       dim3(256), 0, st, (const short*)gu.data_ptr(),
                       (short*)y.data_ptr(), (int)y.size(1), total,
                       (float)alpha, (float)limit);
  else if (is_f32(gu))
    hipLaunchKernelGGL((clamped_glu_kernel<float>), dim3(ew_blocks(total)),
                       dim3(256), 0, st, (const float*)gu.data_ptr(),
                       (float*)y.data_ptr(), (int)y.size(1), total,
                       (float)alpha, (float)limit);
  else DNET_CHECK(false, "clamped_glu: dtype");
}

}  // namespace dnet

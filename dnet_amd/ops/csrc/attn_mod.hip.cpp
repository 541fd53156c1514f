// Score-modified causal attention against the KV cache (gfx950), for decode
// (T = 1) and ragged batched prefill (T = padded length, lens = real ones)
// through one entry point, any head sizes (D != DV allowed), bf16 or fp32.
//
//   s_ij  = (q_i . k_j) * scale * temp[h]
//   s_ij  = cap * tanh(s_ij / cap)                    (cap > 0)
//   s_ij -= r1[h] * ln(1 + r2[h] * (i - j))           (r1/r2 given)
//   p_ij  = exp(s_ij) / (sum_{j<=i} exp(s_ij) + exp(sink[h]))
//
// Every score, weight and accumulator is fp32. Query (b,t) = row b*T+t sits
// at position pos[b]+t of cache row slots[b] and sees keys j <= i (and
// j > i - window when window > 0). The sequence geometry lives in device
// tensors, so a captured decode graph replays across steps.
//
// Two kernels:
//  * attn_mod_rows<T>: flash-decode layout. One workgroup per (q tile, kv
//    head, batch row): K/V chunks of 64 positions are staged through LDS once
//    and shared by up to 16 query rows (tokens x grouped heads); score phase =
//    one key per lane, accumulate phase = output dims across lanes with the
//    weight broadcast from a per-wave LDS slab. Used for decode, for fp32,
//    and for head sizes the MFMA kernel does not cover.
//  * attn_mod_mfma<DC,NV>: bf16 prefill on v_mfma_f32_16x16x32_bf16 — QK^T
//    and PV on the matrix cores, modifiers + online softmax in the fp32 C
//    fragments. Head sizes are zero-padded in LDS to DC*32 / NV*16.
#include "common.h"

namespace dnet {

using bf16x8 = __attribute__((ext_vector_type(8))) __bf16;
using bf16x2 = __attribute__((ext_vector_type(2))) __bf16;
using f32x4 = __attribute__((ext_vector_type(4))) float;

namespace {

template <typename T> __device__ __forceinline__ float ldv(const T* p);
template <> __device__ __forceinline__ float ldv<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldv<short>(const short* p) { return bits2f(*p); }
template <typename T> __device__ __forceinline__ void stv(T* p, float v);
template <> __device__ __forceinline__ void stv<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stv<short>(short* p, float v) { *p = f2bits(v); }

__device__ __forceinline__ float wave_all_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_all_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// dot of two LDS rows of n elements
__device__ __forceinline__ float dot_lds(const float* a, const float* b, int n) {
  float s = 0.f;
  for (int e = 0; e < n; ++e) s = fmaf(a[e], b[e], s);
  return s;
}
__device__ __forceinline__ float dot_lds(const short* a, const short* b, int n) {
  float s = 0.f;
  if ((n & 3) == 0) {      // rows are 8 B aligned (pitch is a multiple of 4)
    for (int e = 0; e < n; e += 4) {
      const short4v ka = *reinterpret_cast<const short4v*>(a + e);
      const short4v qb = *reinterpret_cast<const short4v*>(b + e);
      s = __builtin_amdgcn_fdot2_f32_bf16(
          *reinterpret_cast<const bf16x2*>(&ka.x[0]),
          *reinterpret_cast<const bf16x2*>(&qb.x[0]), s, false);
      s = __builtin_amdgcn_fdot2_f32_bf16(
          *reinterpret_cast<const bf16x2*>(&ka.x[2]),
          *reinterpret_cast<const bf16x2*>(&qb.x[2]), s, false);
    }
  } else {
    for (int e = 0; e < n; ++e) s = fmaf(bits2f(a[e]), bits2f(b[e]), s);
  }
  return s;
}

constexpr int kChunkR = 64;   // keys per staged chunk (one per lane)
constexpr int kRowsMax = 16;  // query rows per workgroup (4 per wave)

__host__ __device__ inline int pitch_of(int n, int elem) {
  // fp32: odd dword pitch; bf16: 8 B aligned rows with a 2-dword skew
  if (elem == 4) return n | 1;
  return ((n + 3) & ~3) + 4;
}

struct ModParams {
  const int* pos;
  const int* lens;
  const int* slots;
  const float* temp;
  const float* r1;
  const float* r2;
  const float* sinks;
  int T, Bc, Hq, Hkv, Smax, D, DV, QT, window;
  float scale, softcap;
};

template <typename T>
__global__ __launch_bounds__(256) void attn_mod_rows(
    const T* __restrict__ q, const T* __restrict__ kc,
    const T* __restrict__ vc, T* __restrict__ out, const ModParams P) {
  const int b = blockIdx.z;
  const int G = P.Hq / P.Hkv;
  const int GS = (G + kRowsMax - 1) / kRowsMax;     // head-group splits
  const int hkv = blockIdx.y / GS;
  const int g0 = (blockIdx.y % GS) * kRowsMax;
  const int Gb = min(kRowsMax, G - g0);
  const int t0 = blockIdx.x * P.QT;
  const int n = P.lens ? min(P.lens[b], P.T) : P.T;
  if (t0 >= n) return;
  const int slot = P.slots ? P.slots[b] : b;
  if (slot < 0 || slot >= P.Bc) return;
  const int p0 = P.pos[b];
  const int nt = min(P.QT, n - t0);
  const int rows = nt * Gb;
  const int D = P.D, DV = P.DV;
  const int PK = pitch_of(D, sizeof(T)), PV = pitch_of(DV, sizeof(T));
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* k_lds = reinterpret_cast<T*>(smem);                 // [64][PK]
  T* v_lds = k_lds + kChunkR * PK;                       // [64][PV]
  T* q_lds = v_lds + kChunkR * PV;                       // [16][PK]
  float* p_lds = reinterpret_cast<float*>(q_lds + kRowsMax * PK);  // [4][64]

  const int64_t qstride = (int64_t)P.Hq * D;
  for (int idx = threadIdx.x; idx < rows * D; idx += blockDim.x) {
    const int r = idx / D, e = idx % D;
    const int t = t0 + r / Gb, g = g0 + r % Gb;
    q_lds[r * PK + e] =
        q[((int64_t)b * P.T + t) * qstride + (int64_t)(hkv * G + g) * D + e];
  }

  // per-wave query rows r = wid + 4*rr
  float m[4], l[4], acc[4][4], tmp[4], r1[4], r2[4];
  int qi[4];
#pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    const int r = wid + 4 * rr;
    const int rc = min(r, rows - 1);
    const int h = hkv * G + g0 + rc % Gb;
    qi[rr] = (r < rows) ? p0 + t0 + rc / Gb : -1;
    tmp[rr] = P.scale * (P.temp ? P.temp[h] : 1.f);
    r1[rr] = P.r1 ? P.r1[h] : 0.f;
    r2[rr] = P.r1 ? P.r2[h] : 0.f;
    m[rr] = -1e30f;
    l[rr] = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[rr][j] = 0.f;
  }

  const int kv_end = min(p0 + t0 + nt, P.Smax);          // exclusive
  const int kv_begin =
      P.window > 0 ? max(0, p0 + t0 - P.window + 1) : 0;
  const int64_t kbase = ((int64_t)slot * P.Hkv + hkv) * P.Smax * D;
  const int64_t vbase = ((int64_t)slot * P.Hkv + hkv) * P.Smax * DV;

  for (int s0 = kv_begin & ~(kChunkR - 1); s0 < kv_end; s0 += kChunkR) {
    const int valid = min(kChunkR, kv_end - s0);
    __syncthreads();          // previous chunk consumed (and q staged)
    for (int idx = threadIdx.x; idx < kChunkR * D; idx += blockDim.x) {
      const int r = idx / D, e = idx % D;
      k_lds[r * PK + e] =
          r < valid ? kc[kbase + (int64_t)(s0 + r) * D + e] : (T)0;
    }
    for (int idx = threadIdx.x; idx < kChunkR * DV; idx += blockDim.x) {
      const int r = idx / DV, e = idx % DV;
      v_lds[r * PV + e] =
          r < valid ? vc[vbase + (int64_t)(s0 + r) * DV + e] : (T)0;
    }
    __syncthreads();
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const int i = qi[rr];
      if (i < s0) continue;                 // wave-uniform: nothing visible
      const int r = wid + 4 * rr;
      const int j = s0 + lane;
      bool live = lane < valid && j <= i;
      if (P.window > 0) live = live && (j > i - P.window);
      float s = dot_lds(&k_lds[lane * PK], &q_lds[r * PK], D) * tmp[rr];
      if (P.softcap > 0.f) s = P.softcap * tanhf(s / P.softcap);
      if (P.r1) s -= r1[rr] * log1pf(r2[rr] * (float)max(i - j, 0));
      if (!live) s = -INFINITY;
      const float mn = fmaxf(m[rr], wave_all_max(s));
      const float alpha = expf(m[rr] - mn);
      const float p = live ? expf(s - mn) : 0.f;
      l[rr] = l[rr] * alpha + wave_all_sum(p);
      m[rr] = mn;
      p_lds[wid * kChunkR + lane] = p;
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // wave-local slab
      const int vis = min(valid, i - s0 + 1);
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int dv = lane + 64 * jj;
        if (dv < DV) {
          float a = acc[rr][jj] * alpha;
          for (int s2 = 0; s2 < vis; ++s2)
            a = fmaf(p_lds[wid * kChunkR + s2], ldv<T>(&v_lds[s2 * PV + dv]),
                     a);
          acc[rr][jj] = a;
        }
      }
    }
  }

#pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    const int r = wid + 4 * rr;
    if (r >= rows) continue;
    const int t = t0 + r / Gb, h = hkv * G + g0 + r % Gb;
    float c = 1.f;
    if (P.sinks) {
      const float sk = P.sinks[h];
      const float m2 = fmaxf(m[rr], sk);
      c = expf(m[rr] - m2);
      l[rr] = l[rr] * c + expf(sk - m2);
    }
    const float inv = l[rr] > 0.f ? c / l[rr] : 0.f;
    T* op = out + ((int64_t)b * P.T + t) * P.Hq * DV + (int64_t)h * DV;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int dv = lane + 64 * jj;
      if (dv < DV) stv<T>(op + dv, acc[rr][jj] * inv);
    }
  }
}

}  // namespace

static const float* opt_f32(const c10::optional<torch::Tensor>& t, int64_t n,
                            const char* what) {
  if (!t.has_value()) return nullptr;
  DNET_CHECK(t->scalar_type() == torch::kFloat32 && t->is_contiguous() &&
                 t->numel() == n, what);
  return t->data_ptr<float>();
}
static const int* opt_i32(const c10::optional<torch::Tensor>& t, int64_t n,
                          const char* what) {
  if (!t.has_value()) return nullptr;
  DNET_CHECK(t->scalar_type() == torch::kInt32 && t->is_contiguous() &&
                 t->numel() >= n, what);
  return t->data_ptr<int>();
}

void attn_mod(torch::Tensor q, torch::Tensor kcache, torch::Tensor vcache,
              torch::Tensor pos, c10::optional<torch::Tensor> lens,
              c10::optional<torch::Tensor> slots, torch::Tensor out,
              int64_t T, double scale, c10::optional<torch::Tensor> temp,
              double softcap, c10::optional<torch::Tensor> dist_r1,
              c10::optional<torch::Tensor> dist_r2,
              c10::optional<torch::Tensor> sinks, int64_t window) {
  DNET_CHECK(kcache.dim() == 4 && vcache.dim() == 4 &&
                 kcache.is_contiguous() && vcache.is_contiguous(), "cache");
  const int Bc = kcache.size(0), Hkv = kcache.size(1), Smax = kcache.size(2);
  const int D = kcache.size(3), DV = vcache.size(3);
  DNET_CHECK(vcache.size(0) == Bc && vcache.size(1) == Hkv &&
                 vcache.size(2) == Smax, "k/v cache shapes differ");
  const int64_t M = q.size(0);
  DNET_CHECK(T > 0 && M % T == 0, "rows = B*T");
  const int64_t B = M / T;
  DNET_CHECK(q.dim() == 2 && q.is_contiguous() && q.size(1) % D == 0,
             "q [B*T, Hq*D]");
  const int Hq = q.size(1) / D;
  DNET_CHECK(Hq % Hkv == 0, "grouped heads");
  DNET_CHECK(out.is_contiguous() && out.size(0) == M &&
                 out.size(1) == (int64_t)Hq * DV, "out [B*T, Hq*DV]");
  DNET_CHECK(q.scalar_type() == kcache.scalar_type() &&
                 q.scalar_type() == vcache.scalar_type() &&
                 q.scalar_type() == out.scalar_type(), "dtypes");
  DNET_CHECK(D >= 1 && D <= 256 && DV >= 1 && DV <= 256, "head sizes <= 256");
  DNET_CHECK(dist_r1.has_value() == dist_r2.has_value(), "r1 and r2");
  if (!slots.has_value()) DNET_CHECK(B <= Bc, "more rows than cache slots");
  if (M == 0) return;
  ModParams P;
  P.pos = opt_i32(pos, B, "pos int32 [B]");
  P.lens = opt_i32(lens, B, "lens int32 [B]");
  P.slots = opt_i32(slots, B, "slots int32 [B]");
  P.temp = opt_f32(temp, Hq, "temp fp32 [Hq]");
  P.r1 = opt_f32(dist_r1, Hq, "r1 fp32 [Hq]");
  P.r2 = opt_f32(dist_r2, Hq, "r2 fp32 [Hq]");
  P.sinks = opt_f32(sinks, Hq, "sinks fp32 [Hq]");
  P.T = (int)T; P.Bc = Bc; P.Hq = Hq; P.Hkv = Hkv; P.Smax = Smax;
  P.D = D; P.DV = DV; P.window = (int)window;
  P.scale = (float)scale; P.softcap = (float)softcap;
  const int G = Hq / Hkv;
  const int GS = (G + kRowsMax - 1) / kRowsMax;
  P.QT = std::max(1, kRowsMax / std::min(G, kRowsMax));
  auto stream = current_stream();
  const bool f32 = q.scalar_type() == torch::kFloat32;
  DNET_CHECK(f32 || q.scalar_type() == torch::kBFloat16, "bf16 or fp32");
  const int es = f32 ? 4 : 2;
  const int PK = pitch_of(D, es), PV = pitch_of(DV, es);
  const size_t lds = (size_t)es * (kChunkR * PK + kChunkR * PV +
                                   kRowsMax * PK) + sizeof(float) * 4 * kChunkR;
  DNET_CHECK(lds <= 160 * 1024, "attn_mod: head sizes exceed LDS");
  const dim3 grid((unsigned)((T + P.QT - 1) / P.QT), (unsigned)(Hkv * GS),
                  (unsigned)B);
  if (f32) {
    if (lds > 64 * 1024)
      DNET_CHECK_HIP(hipFuncSetAttribute(
          (const void*)attn_mod_rows<float>,
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL((attn_mod_rows<float>), grid, dim3(256), lds, stream,
                       q.data_ptr<float>(), kcache.data_ptr<float>(),
                       vcache.data_ptr<float>(), out.data_ptr<float>(), P);
  } else {
    if (lds > 64 * 1024)
      DNET_CHECK_HIP(hipFuncSetAttribute(
          (const void*)attn_mod_rows<short>,
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL((attn_mod_rows<short>), grid, dim3(256), lds, stream,
                       (const short*)q.data_ptr(),
                       (const short*)kcache.data_ptr(),
                       (const short*)vcache.data_ptr(),
                       (short*)out.data_ptr(), P);
  }
}

}  // namespace dnet

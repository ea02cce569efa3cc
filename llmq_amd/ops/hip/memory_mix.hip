// Kernels around windowed attention beside a matrix memory (gfx950): the
// per-token step between the projections and the paged attention kernels
// (per-head norms, rotary positions, rotated unit-norm values, cache scatter),
// the turn-back of attended values, the gate walk and the read-out of an mLSTM,
// the average of two normed mixer outputs, and ungated activations.
//
// Numerics contract: activations arrive in the model dtype T (bf16 or fp32);
// norms, angles, gates, running maxima and denominators are fp32 with the
// accurate library functions and rounded to T once, on store.

#include "common.h"

// ------------------------------------------- q / k / v before the attention --
// One workgroup per token, one wave per head vector at a time. A head vector
// of n channels whose first rd are rotated in pairs (i, i + rd/2) is held by a
// wave as up to kRopePairs pairs and kRopeTail unrotated channels per lane, so
// norm and rotation need no exchange beyond the wave's sum of squares.
//   q [T, H, D] (rows strided): optional RMSNorm x weight, rotation, in place;
//   k [T, G, D]: the same, into the key cache; with v == null its raw values
//     go to the value cache (values = keys as projected);
//   v [T, G, DV]: optional division by the root mean square, rotation over
//     all DV channels with a table of its own, into the value cache.
// cos/sin of a token's angles (position * inv_freq[i], fp32, sincosf) are
// computed once per workgroup into LDS.
constexpr int kRopePairs = 4;    // 64 * 4 pairs: rotated widths up to 512
constexpr int kRopeTail = 8;     // 64 * 8 unrotated channels

template <typename T>
DEVINL void norm_rope_vector(const T* __restrict__ src, int n, int rd, const T* __restrict__ weight,
                             bool unit_norm, float eps, const float* __restrict__ cs, int lane,
                             T* __restrict__ dst, T* __restrict__ raw_dst) {
  const int half = rd / 2;
  float u[kRopePairs], v[kRopePairs], t[kRopeTail];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < kRopePairs; ++j) {
    const int i = lane + 64 * j;
    u[j] = v[j] = 0.f;
    if (i < half) {
      u[j] = to_f32(src[i]);
      v[j] = to_f32(src[i + half]);
      if (raw_dst) {
        raw_dst[i] = src[i];
        raw_dst[i + half] = src[i + half];
      }
    }
    ss += u[j] * u[j] + v[j] * v[j];
  }
#pragma unroll
  for (int j = 0; j < kRopeTail; ++j) {
    const int c = rd + lane + 64 * j;
    t[j] = 0.f;
    if (c < n) {
      t[j] = to_f32(src[c]);
      if (raw_dst) raw_dst[c] = src[c];
    }
    ss += t[j] * t[j];
  }
  float inv = 1.f;
  if (weight || unit_norm) {
    ss = wave_reduce_sum(ss);
    inv = 1.0f / sqrtf(ss / n + eps);
  }
#pragma unroll
  for (int j = 0; j < kRopePairs; ++j) {
    const int i = lane + 64 * j;
    if (i < half) {
      float a = u[j] * inv, b = v[j] * inv;
      if (weight) {
        a *= to_f32(weight[i]);
        b *= to_f32(weight[i + half]);
      }
      const float c = cs[2 * i], s = cs[2 * i + 1];
      dst[i] = from_f32<T>(a * c - b * s);
      dst[i + half] = from_f32<T>(b * c + a * s);
    }
  }
#pragma unroll
  for (int j = 0; j < kRopeTail; ++j) {
    const int c = rd + lane + 64 * j;
    if (c < n) {
      float a = t[j] * inv;
      if (weight) a *= to_f32(weight[c]);
      dst[c] = from_f32<T>(a);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void qkv_norm_rope_cache_kernel(
    T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride,
    const T* __restrict__ v, long v_stride,               // null: values = raw keys
    const T* __restrict__ q_w, const T* __restrict__ k_w, // [D] or null
    const float* __restrict__ inv_freq, int rot_dims,     // [rot_dims / 2] (rot_dims may be 0)
    const float* __restrict__ v_inv_freq,                 // [DV / 2] or null
    const long* __restrict__ positions, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const long* __restrict__ slots, int H, int G, int D, int DV, int block_size, float eps,
    int v_unit_norm) {
  extern __shared__ float cs_smem[];
  float* cs = cs_smem;                       // [rot_dims/2][cos, sin]
  float* vcs = cs + rot_dims;                // [DV/2][cos, sin]
  const long tok = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const float pos = (float)positions[tok];
  for (int i = tid; i < rot_dims / 2; i += 256) {
    float sn, c;
    sincosf(pos * inv_freq[i], &sn, &c);
    cs[2 * i] = c;
    cs[2 * i + 1] = sn;
  }
  if (v_inv_freq) {
    for (int i = tid; i < DV / 2; i += 256) {
      float sn, c;
      sincosf(pos * v_inv_freq[i], &sn, &c);
      vcs[2 * i] = c;
      vcs[2 * i + 1] = sn;
    }
  }
  __syncthreads();
  const long slot = slots[tok];
  const long blk = slot >= 0 ? slot / block_size : 0;
  const int off = slot >= 0 ? (int)(slot % block_size) : 0;
  const int items = H + G + (v ? G : 0);
  for (int it = w; it < items; it += 4) {
    if (it < H) {
      T* qh = q + tok * q_stride + (long)it * D;
      norm_rope_vector<T>(qh, D, rot_dims, q_w, false, eps, cs, lane, qh, nullptr);
    } else if (it < H + G) {
      if (slot < 0) continue;
      const int g = it - H;
      const long row = (blk * G + g) * block_size + off;
      norm_rope_vector<T>(k + tok * k_stride + (long)g * D, D, rot_dims, k_w, false, eps, cs,
                          lane, k_cache + row * D, v ? nullptr : v_cache + row * DV);
    } else {
      if (slot < 0) continue;
      const int g = it - H - G;
      const long row = (blk * G + g) * block_size + off;
      norm_rope_vector<T>(v + tok * v_stride + (long)g * DV, DV, v_inv_freq ? DV : 0, nullptr,
                          v_unit_norm != 0, eps, vcs, lane, v_cache + row * DV, nullptr);
    }
  }
}

// x [T, H, n] contiguous, in place: head vectors turned by sign * position over
// all n channels, pairs (i, i + n/2).
template <typename T>
__global__ __launch_bounds__(256) void rotate_heads_kernel(
    T* __restrict__ x, const long* __restrict__ positions, const float* __restrict__ inv_freq,
    int H, int n, float sign) {
  extern __shared__ float cs_smem[];
  const long tok = blockIdx.x;
  const int half = n / 2;
  const float pos = sign * (float)positions[tok];
  for (int i = threadIdx.x; i < half; i += 256) {
    float sn, c;
    sincosf(pos * inv_freq[i], &sn, &c);
    cs_smem[2 * i] = c;
    cs_smem[2 * i + 1] = sn;
  }
  __syncthreads();
  T* xt = x + tok * (long)H * n;
  for (int idx = threadIdx.x; idx < H * half; idx += 256) {
    const int h = idx / half, i = idx % half;
    T* xh = xt + (long)h * n;
    const float a = to_f32(xh[i]), b = to_f32(xh[i + half]);
    const float c = cs_smem[2 * i], s = cs_smem[2 * i + 1];
    xh[i] = from_f32<T>(a * c - b * s);
    xh[i + half] = from_f32<T>(b * c + a * s);
  }
}

// ------------------------------------------------------- mLSTM: gate walk ----
// gates fp32 [T, 2H] = input | forget pre-activations. Per (sequence, head):
//   i = cap tanh(g_i / cap),  f = logsigmoid(cap tanh(g_f / cap)),
//   m_t = max(f_t + m_(t-1), i_t),  m = 0 before a sequence's first token,
//   decay_t = e^(f_t + m_(t-1) - m_t), write_t = e^(i_t - m_t), floor_t = e^(-m_t).
// One workgroup per (sequence, head) walks chunks of 256 tokens: the gate
// functions and the three exponentials are computed by a thread per token,
// only the max/add chain in between is serial (one thread, LDS operands).
// out [3, T, H]; m_state [slots, H] holds the running maximum between steps.
__global__ __launch_bounds__(256) void mlstm_gates_kernel(
    float* __restrict__ out, const float* __restrict__ gates, float cap,
    float* __restrict__ m_state, const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ fresh, int H, long T) {
  __shared__ float fi[256], ff[256], ms[257];
  const int b = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int row0 = cu[b], n = cu[b + 1] - row0;
  if (n <= 0) return;
  float* mslot = m_state + (long)slots[b] * H + h;
  if (tid == 0) ms[0] = fresh[b] ? 0.f : *mslot;
  for (int t0 = 0; t0 < n; t0 += 256) {
    const int nt = min(256, n - t0);
    const long row = row0 + t0 + tid;
    float gi = 0.f, gf = 0.f;
    if (tid < nt) {
      gi = cap * tanhf(gates[row * 2 * H + h] / cap);
      const float z = cap * tanhf(gates[row * 2 * H + H + h] / cap);
      gf = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
      fi[tid] = gi;
      ff[tid] = gf;
    }
    __syncthreads();
    if (tid == 0) {
      float m = ms[0];
      for (int t = 0; t < nt; ++t) {
        m = fmaxf(ff[t] + m, fi[t]);
        ms[t + 1] = m;
      }
    }
    __syncthreads();
    if (tid < nt) {
      const float m_old = ms[tid], m_new = ms[tid + 1];
      out[row * H + h] = expf(gf + m_old - m_new);
      out[(T + row) * H + h] = expf(gi - m_new);
      out[(2 * T + row) * H + h] = expf(-m_new);
    }
    __syncthreads();
    if (tid == 0) ms[0] = ms[nt];
  }
  __syncthreads();
  if (tid == 0) *mslot = ms[0];
}

// ------------------------------------------------------- mLSTM: read-out -----
// o fp32 [T, H, DV + 1] (last column n . q), floor fp32 [T, H]. Per (token,
// head): y = o[:DV] / (max(|n . q|, floor) + 1e-6), divided by its root mean
// square, times weight [H * DV], times sigmoid(gate). One wave per head.
template <typename T>
__global__ __launch_bounds__(256) void mlstm_out_norm_gate_kernel(
    T* __restrict__ out, const float* __restrict__ o, const float* __restrict__ floor_,
    const T* __restrict__ weight, const T* __restrict__ gate, long g_stride, int H, int DV,
    float eps) {
  const long tok = blockIdx.x;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  for (int h = w; h < H; h += 4) {
    const float* oh = o + (tok * H + h) * (long)(DV + 1);
    const float den = fmaxf(fabsf(oh[DV]), floor_[tok * H + h]) + 1e-6f;
    float ss = 0.f;
    for (int c = lane; c < DV; c += 64) {
      const float y = oh[c] / den;
      ss += y * y;
    }
    ss = wave_reduce_sum(ss);
    const float inv = 1.0f / sqrtf(ss / DV + eps);
    for (int c = lane; c < DV; c += 64) {
      const float gt = to_f32(gate[tok * g_stride + (long)h * DV + c]);
      const float sg = 1.0f / (1.0f + expf(-gt));
      out[tok * (long)H * DV + (long)h * DV + c] =
          from_f32<T>(oh[c] / den * inv * to_f32(weight[(long)h * DV + c]) * sg);
    }
  }
}

// ------------------------------------------ average of two normed outputs ----
// out = (rmsnorm(a) * w_a + rmsnorm(b) * w_b) / 2, norms over the whole row.
template <typename T>
__global__ __launch_bounds__(256) void dual_norm_mean_kernel(
    T* __restrict__ out, const T* __restrict__ a, const T* __restrict__ w_a,
    const T* __restrict__ b, const T* __restrict__ w_b, int hidden, float eps) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const T* ar = a + row * hidden;
  const T* br = b + row * hidden;
  float sa = 0.f, sb = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    const float x = to_f32(ar[i]), y = to_f32(br[i]);
    sa += x * x;
    sb += y * y;
  }
  sa = block_reduce_sum(sa, red);
  __syncthreads();
  sb = block_reduce_sum(sb, red);
  const float ia = 1.0f / sqrtf(sa / hidden + eps), ib = 1.0f / sqrtf(sb / hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += 256)
    out[row * hidden + i] = from_f32<T>(0.5f * (to_f32(ar[i]) * ia * to_f32(w_a[i]) +
                                                 to_f32(br[i]) * ib * to_f32(w_b[i])));
}

// ------------------------------------------------------ ungated activations --
constexpr int kActRelu2 = 0;
constexpr int kActGeluErf = 1;

template <int ACT>
DEVINL float unary_act_f(float x) {
  if (ACT == kActRelu2) {
    const float r = fmaxf(x, 0.f);
    return r * r;
  }
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f));
}

// n8 granules of 16 bytes, then the scalar rest
template <typename T, int ACT>
__global__ void unary_act_kernel(T* __restrict__ out, const T* __restrict__ in, long n) {
  constexpr int VE = Vec8<T>::kElems;
  const long n8 = n / VE;
  const long stride = (long)gridDim.x * blockDim.x;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n8; i += stride) {
    const Vec8<T> v = load16(in + i * VE);
    Vec8<T> o;
#pragma unroll
    for (int j = 0; j < VE; ++j) o.data[j] = from_f32<T>(unary_act_f<ACT>(to_f32(v.data[j])));
    store16(out + i * VE, o);
  }
  for (long i = n8 * VE + blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = from_f32<T>(unary_act_f<ACT>(to_f32(in[i])));
}

// Kernels around windowed attention beside a matrix memory (gfx950): the
// per-token step between the projections and the paged attention kernels
// (per-head norms, rotary positions, rotated unit-norm values, cache scatter),
// the turn-back of attended values, the gate walk and the read-out of an mLSTM,
// the average of two normed mixer outputs, and ungated activations.
//
// Numerics shared by every kernel here: activations arrive in the model dtype T (bf16 or fp32);
// norms, angles, gates, running maxima and denominators are fp32 with the
// accurate library functions and rounded to T once, on store.

#include "common.h"

// ------------------------------------------- q / k / v before the attention --
// One workgroup per token. A head vector of n channels whose first rd are
// rotated in pairs (i, i + rd/2) belongs to a team of LG adjacent lanes (LG a
// power of two chosen by the host: the fewest lanes that hold the vector as up
// to kRopePairs pairs and kRopeTail unrotated channels each), so a wave works
// on 64 / LG heads at once and norm and rotation need no exchange beyond the
// team's sum of squares.
//   q [T, H, D] (rows strided): optional RMSNorm x weight, rotation, in place;
//   k [T, G, D]: the same, into the key cache; with v == null its raw values
//     go to the value cache (values = keys as projected);
//   v [T, G, DV]: optional division by the root mean square, rotation over
//     all DV channels with a table of its own, into the value cache.
// cos/sin of a token's angles (position * inv_freq[i], fp32, sincosf) are
// computed once per workgroup into LDS.
constexpr int kRopePairs = 4;
constexpr int kRopeTail = 8;

template <typename T>
DEVINL void norm_rope_vector(const T* __restrict__ src, int n, int rd, const T* __restrict__ weight,
                             bool unit_norm, float eps, const float* __restrict__ cs, int sub,
                             int LG, bool active, T* __restrict__ dst, T* __restrict__ raw_dst) {
  const int half = active ? rd / 2 : 0;
  if (!active) n = 0;
  float u[kRopePairs], v[kRopePairs], t[kRopeTail];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < kRopePairs; ++j) {
    const int i = sub + LG * j;
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
    const int c = rd + sub + LG * j;
    t[j] = 0.f;
    if (c < n) {
      t[j] = to_f32(src[c]);
      if (raw_dst) raw_dst[c] = src[c];
    }
    ss += t[j] * t[j];
  }
  float inv = 1.f;
  if (weight || unit_norm) {         // uniform over the wave: every lane takes part
    for (int off = LG >> 1; off > 0; off >>= 1) ss += __shfl_xor(ss, off, WAVE);
    inv = 1.0f / sqrtf(ss / max(n, 1) + eps);
  }
#pragma unroll
  for (int j = 0; j < kRopePairs; ++j) {
    const int i = sub + LG * j;
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
    const int c = rd + sub + LG * j;
    if (c < n) {
      float a = t[j] * inv;
      if (weight) a *= to_f32(weight[c]);
      dst[c] = from_f32<T>(a);
    }
  }
}

// The 16-byte form for bf16 vectors whose halves and unrotated rest are whole
// granules of 8: a lane holds at most one granule of each half (8 pairs) and
// one granule of the rest, so a team is as small as a vector has granule
// pairs and every access is one 16-byte load or store.
DEVINL void norm_rope_vec8(const __hip_bfloat16* __restrict__ src, int n, int rd,
                           const __hip_bfloat16* __restrict__ weight, bool unit_norm, float eps,
                           const float* __restrict__ cs, int sub, int LG, bool active,
                           __hip_bfloat16* __restrict__ dst, __hip_bfloat16* __restrict__ raw_dst) {
  using bf = __hip_bfloat16;
  const int half = rd / 2;
  const bool has_pair = active && sub * 8 < half;
  const bool has_tail = active && rd + sub * 8 < n;
  float u[8], v[8], t[8];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) u[e] = v[e] = t[e] = 0.f;
  if (has_pair) {
    const Vec8<bf> a = load16(src + sub * 8), b = load16(src + half + sub * 8);
    if (raw_dst) {
      store16(raw_dst + sub * 8, a);
      store16(raw_dst + half + sub * 8, b);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      u[e] = to_f32(a.data[e]);
      v[e] = to_f32(b.data[e]);
      ss += u[e] * u[e] + v[e] * v[e];
    }
  }
  if (has_tail) {
    const Vec8<bf> a = load16(src + rd + sub * 8);
    if (raw_dst) store16(raw_dst + rd + sub * 8, a);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      t[e] = to_f32(a.data[e]);
      ss += t[e] * t[e];
    }
  }
  float inv = 1.f;
  if (weight || unit_norm) {         // uniform over the wave: every lane takes part
    for (int off = LG >> 1; off > 0; off >>= 1) ss += __shfl_xor(ss, off, WAVE);
    inv = 1.0f / sqrtf(ss / max(active ? n : 1, 1) + eps);
  }
  if (has_pair) {
    Vec8<bf> wa, wb, oa, ob;
    if (weight) {
      wa = load16(weight + sub * 8);
      wb = load16(weight + half + sub * 8);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float a = u[e] * inv, b = v[e] * inv;
      if (weight) {
        a *= to_f32(wa.data[e]);
        b *= to_f32(wb.data[e]);
      }
      const float2 c_s = *reinterpret_cast<const float2*>(cs + 2 * (sub * 8 + e));
      oa.data[e] = __float2bfloat16(a * c_s.x - b * c_s.y);
      ob.data[e] = __float2bfloat16(b * c_s.x + a * c_s.y);
    }
    store16(dst + sub * 8, oa);
    store16(dst + half + sub * 8, ob);
  }
  if (has_tail) {
    Vec8<bf> wt, ot;
    if (weight) wt = load16(weight + rd + sub * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float a = t[e] * inv;
      if (weight) a *= to_f32(wt.data[e]);
      ot.data[e] = __float2bfloat16(a);
    }
    store16(dst + rd + sub * 8, ot);
  }
}

template <typename T, bool VEC>
DEVINL void norm_rope_any(const T* __restrict__ src, int n, int rd, const T* __restrict__ weight,
                          bool unit_norm, float eps, const float* __restrict__ cs, int sub, int LG,
                          bool active, T* __restrict__ dst, T* __restrict__ raw_dst) {
  if constexpr (VEC) norm_rope_vec8(src, n, rd, weight, unit_norm, eps, cs, sub, LG, active, dst, raw_dst);
  else norm_rope_vector<T>(src, n, rd, weight, unit_norm, eps, cs, sub, LG, active, dst, raw_dst);
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void qkv_norm_rope_cache_kernel(
    T* __restrict__ q, long q_stride, const T* __restrict__ k, long k_stride,
    const T* __restrict__ v, long v_stride,               // null: values = raw keys
    const T* __restrict__ q_w, const T* __restrict__ k_w, // [D] or null
    const float* __restrict__ inv_freq, int rot_dims,     // [rot_dims / 2] (rot_dims may be 0)
    const float* __restrict__ v_inv_freq,                 // [DV / 2] or null
    const long* __restrict__ positions, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const long* __restrict__ slots, int H, int G, int D, int DV, int block_size, float eps,
    int v_unit_norm, int LG) {
  extern __shared__ __align__(8) float cs_smem[];
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
  const int per_wave = 64 / LG, sub = lane % LG, team = lane / LG;
  // three passes, each uniform over the wave in what it norms: q, k, v
  for (int base = w * per_wave; base < H; base += 4 * per_wave) {
    const int h = base + team;
    T* qh = q + tok * q_stride + (long)min(h, H - 1) * D;
    norm_rope_any<T, VEC>(qh, D, rot_dims, q_w, false, eps, cs, sub, LG, h < H, qh, nullptr);
  }
  for (int base = w * per_wave; base < G; base += 4 * per_wave) {
    const int g = base + team;
    const bool act = g < G && slot >= 0;
    const long row = (blk * G + min(g, G - 1)) * block_size + off;
    norm_rope_any<T, VEC>(k + tok * k_stride + (long)min(g, G - 1) * D, D, rot_dims, k_w, false,
                          eps, cs, sub, LG, act, k_cache + row * D, v ? nullptr : v_cache + row * DV);
  }
  if (v) {
    for (int base = w * per_wave; base < G; base += 4 * per_wave) {
      const int g = base + team;
      const bool act = g < G && slot >= 0;
      const long row = (blk * G + min(g, G - 1)) * block_size + off;
      norm_rope_any<T, VEC>(v + tok * v_stride + (long)min(g, G - 1) * DV, DV, v_inv_freq ? DV : 0,
                            nullptr, v_unit_norm != 0, eps, vcs, sub, LG, act, v_cache + row * DV,
                            nullptr);
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

// The same for bf16 rows of up to CH * 2048 elements, a multiple of 8 wide:
// both rows stay in registers between the sums and the result, every access
// is 16 bytes.
template <int CH>
__global__ __launch_bounds__(256) void dual_norm_mean_vec_kernel(
    __hip_bfloat16* __restrict__ out, const __hip_bfloat16* __restrict__ a,
    const __hip_bfloat16* __restrict__ w_a, const __hip_bfloat16* __restrict__ b,
    const __hip_bfloat16* __restrict__ w_b, int hidden, float eps) {
  using bf = __hip_bfloat16;
  __shared__ float red[4];
  const long row = blockIdx.x;
  float av[CH][8], bv[CH][8];
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (c * 256 + threadIdx.x) * 8;
    if (i < hidden) {
      const Vec8<bf> x = load16(a + row * hidden + i), y = load16(b + row * hidden + i);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        av[c][j] = to_f32(x.data[j]);
        bv[c][j] = to_f32(y.data[j]);
        sa += av[c][j] * av[c][j];
        sb += bv[c][j] * bv[c][j];
      }
    }
  }
  sa = block_reduce_sum(sa, red);
  __syncthreads();
  sb = block_reduce_sum(sb, red);
  const float ia = 0.5f / sqrtf(sa / hidden + eps), ib = 0.5f / sqrtf(sb / hidden + eps);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (c * 256 + threadIdx.x) * 8;
    if (i < hidden) {
      const Vec8<bf> wa = load16(w_a + i), wb = load16(w_b + i);
      Vec8<bf> o;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        o.data[j] = __float2bfloat16(av[c][j] * ia * to_f32(wa.data[j]) +
                                     bv[c][j] * ib * to_f32(wb.data[j]));
      store16(out + row * hidden + i, o);
    }
  }
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

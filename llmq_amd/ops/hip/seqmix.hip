// Sequence-mixer kernels for hybrid decoders (gfx950): layers that keep the
// residual stream in fp32, attention over the paged KV cache under a
// block-local ("chunked") or a sliding-window / causal mask, with an optional
// learned per-distance bias and an optional per-head gate, and diagonal-decay
// recurrences (gated linear attention, HGRN2) over per-sequence fp32 state
// slots.
//
// Numerics contract shared by every kernel here: activations arrive in the
// model dtype T (bf16 or fp32); norms, scores, softmax weights, decays and
// recurrent state are fp32 in registers/LDS and rounded to T once, on store.

#include "common.h"

// ------------------------------------------------------------------ norms --
// Residual stream in fp32, sublayer I/O in T.

// out = rmsnorm(in) * (w + offset); TI/TO may differ (fp32 stream -> T).
// A row normed in `groups` equal consecutive parts is `groups` rows of
// `hidden` elements each to these kernels; part g reads the weights from
// g * hidden on.
template <typename TI, typename TO>
__global__ void rmsnorm_cast_kernel(TO* __restrict__ out, const TI* __restrict__ in,
                                    long in_stride, const TO* __restrict__ weight, int hidden,
                                    float eps, float offset, int groups) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const int part = (int)(row % groups);
  const TI* x = in + (row / groups) * in_stride + (long)part * hidden;
  TO* o = out + row * hidden;
  weight += (long)part * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float f = to_f32(x[i]);
    ss += f * f;
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x)
    o[i] = from_f32<TO>(to_f32(x[i]) * inv * (to_f32(weight[i]) + offset));
}

// Norm sandwich around an fp32 residual:
//   residual += rmsnorm(x) * (w_post + offset)        (fp32, in place)
//   x         = rmsnorm(residual) * (w_pre + offset)  (T, in place)
// One launch closes a sublayer and opens the next.
template <typename T>
__global__ void sandwich_norm_res32_kernel(T* __restrict__ x, float* __restrict__ residual,
                                           const T* __restrict__ w_post,
                                           const T* __restrict__ w_pre, int hidden,
                                           float eps, float offset, int groups) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  w_post += (row % groups) * hidden;
  w_pre += (row % groups) * hidden;
  T* xr = x + row * hidden;
  float* rr = residual + row * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float f = to_f32(xr[i]);
    ss += f * f;
  }
  ss = block_reduce_sum(ss, red);
  const float inv1 = 1.0f / sqrtf(ss / hidden + eps);
  float ss2 = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float r = rr[i] + to_f32(xr[i]) * inv1 * (to_f32(w_post[i]) + offset);
    rr[i] = r;
    ss2 += r * r;
  }
  ss2 = block_reduce_sum(ss2, red);
  const float inv2 = 1.0f / sqrtf(ss2 / hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x)
    xr[i] = from_f32<T>(rr[i] * inv2 * (to_f32(w_pre[i]) + offset));
}

// The same sandwich for bf16 rows of up to CH * 2048 elements, a multiple of
// 8 wide: every thread keeps its 8-element granules of the updated residual
// in registers, so x, the residual and the two weights cross memory exactly
// once, in 16-byte accesses. PER_WAVE: a row (or one part of a row normed in
// groups) of up to CH * 512 elements belongs to one wave, four rows to a
// workgroup, and the two sums are wave reductions without LDS or barriers.
template <int CH, bool PER_WAVE>
__global__ __launch_bounds__(256) void sandwich_norm_res32_vec_kernel(
    __hip_bfloat16* __restrict__ x, float* __restrict__ residual,
    const __hip_bfloat16* __restrict__ w_post, const __hip_bfloat16* __restrict__ w_pre,
    int hidden, float eps, float offset, int groups, long rows) {
  __shared__ float red[4];
  constexpr int TEAM = PER_WAVE ? 64 : 256;
  const int member = PER_WAVE ? (threadIdx.x & 63) : threadIdx.x;
  const long row = PER_WAVE ? blockIdx.x * 4L + (threadIdx.x >> 6) : blockIdx.x;
  if (PER_WAVE && row >= rows) return;
  w_post += (row % groups) * hidden;
  w_pre += (row % groups) * hidden;
  __hip_bfloat16* xr = x + row * hidden;
  float* rr = residual + row * hidden;
  float xv[CH][8], rv[CH][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (c * TEAM + member) * 8;
    if (i < hidden) {
      const Vec8<__hip_bfloat16> v = load16(xr + i);
      const float4 ra = *reinterpret_cast<const float4*>(rr + i);
      const float4 rb = *reinterpret_cast<const float4*>(rr + i + 4);
      rv[c][0] = ra.x; rv[c][1] = ra.y; rv[c][2] = ra.z; rv[c][3] = ra.w;
      rv[c][4] = rb.x; rv[c][5] = rb.y; rv[c][6] = rb.z; rv[c][7] = rb.w;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        xv[c][j] = to_f32(v.data[j]);
        ss += xv[c][j] * xv[c][j];
      }
    }
  }
  ss = PER_WAVE ? wave_reduce_sum(ss) : block_reduce_sum(ss, red);
  const float inv1 = 1.0f / sqrtf(ss / hidden + eps);
  float ss2 = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (c * TEAM + member) * 8;
    if (i < hidden) {
      const Vec8<__hip_bfloat16> wv = load16(w_post + i);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        rv[c][j] += xv[c][j] * inv1 * (to_f32(wv.data[j]) + offset);
        ss2 += rv[c][j] * rv[c][j];
      }
      *reinterpret_cast<float4*>(rr + i) = make_float4(rv[c][0], rv[c][1], rv[c][2], rv[c][3]);
      *reinterpret_cast<float4*>(rr + i + 4) = make_float4(rv[c][4], rv[c][5], rv[c][6], rv[c][7]);
    }
  }
  ss2 = PER_WAVE ? wave_reduce_sum(ss2) : block_reduce_sum(ss2, red);
  const float inv2 = 1.0f / sqrtf(ss2 / hidden + eps);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (c * TEAM + member) * 8;
    if (i < hidden) {
      const Vec8<__hip_bfloat16> wv = load16(w_pre + i);
      Vec8<__hip_bfloat16> ov;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        ov.data[j] = __float2bfloat16(rv[c][j] * inv2 * (to_f32(wv.data[j]) + offset));
      store16(xr + i, ov);
    }
  }
}

// ------------------------------------------------------------ activations --
// Scalar fallback of act_and_mul for widths that are not a multiple of the
// 16-byte vector (the vector kernel lives in elementwise.hip).
template <typename T, bool GELU>
__global__ void act_and_mul_scalar_kernel(T* __restrict__ out, const T* __restrict__ in,
                                          long rows, int d) {
  const long total = rows * d;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / d;
    const int col = (int)(idx % d);
    const float g = to_f32(in[row * 2 * d + col]);
    const float u = to_f32(in[row * 2 * d + d + col]);
    float act;
    if (GELU) {
      const float c = 0.7978845608028654f;
      act = 0.5f * g * (1.0f + tanhf(c * (g + 0.044715f * g * g * g)));
    } else {
      act = g / (1.0f + expf(-g));
    }
    out[idx] = from_f32<T>(act * u);
  }
}

// ------------------------------------------------- attention: projections --
// Per token: RMS-normalise the WHOLE q projection and the WHOLE k projection
// (all heads at once, plain weights), blend v with an earlier layer's values
// of the same token, and scatter k / v into the paged cache. q is normalised
// in place; k and v are only read (attention reads them back from the cache).
// Cache layouts: k [blocks, G, bs, D], v [blocks, G, bs, DV].
template <typename T>
__global__ void qknorm_vmix_cache_kernel(
    T* __restrict__ q, long q_stride, int nq,
    const T* __restrict__ k, long k_stride, int nk,
    const T* __restrict__ v, long v_stride, int nv,
    const T* __restrict__ q_w, const T* __restrict__ k_w,
    const T* __restrict__ v_first, long vf_stride, float lambda,
    T* __restrict__ k_cache, T* __restrict__ v_cache,
    const long* __restrict__ slots, int kv_heads, int dim, int vdim,
    int block_size, float eps) {
  __shared__ float red[4];
  const long tok = blockIdx.x;
  T* qr = q + tok * q_stride;
  const T* kr = k + tok * k_stride;
  const T* vr = v + tok * v_stride;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < nq; i += blockDim.x) {
    const float f = to_f32(qr[i]);
    sq += f * f;
  }
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const float f = to_f32(kr[i]);
    sk += f * f;
  }
  sq = block_reduce_sum(sq, red);
  sk = block_reduce_sum(sk, red);
  const float iq = 1.0f / sqrtf(sq / nq + eps);
  const float ik = 1.0f / sqrtf(sk / nk + eps);
  for (int i = threadIdx.x; i < nq; i += blockDim.x)
    qr[i] = from_f32<T>(to_f32(qr[i]) * iq * to_f32(q_w[i]));
  const long slot = slots[tok];
  if (slot < 0) return;  // padding row: nothing enters the cache
  const long blk = slot / block_size;
  const int off = (int)(slot % block_size);
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const int g = i / dim, d = i % dim;
    k_cache[((blk * kv_heads + g) * block_size + off) * dim + d] =
        from_f32<T>(to_f32(kr[i]) * ik * to_f32(k_w[i]));
  }
  const T* vf = v_first ? v_first + tok * vf_stride : nullptr;
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const int g = i / vdim, d = i % vdim;
    float val = to_f32(vr[i]);
    if (vf) val = (1.0f - lambda) * val + lambda * to_f32(vf[i]);
    v_cache[((blk * kv_heads + g) * block_size + off) * vdim + d] = from_f32<T>(val);
  }
}

// ---------------------------------------------- attention: prompt portions --
// Block-local causal attention with a per-distance bias, queries packed
// [Tq, H, D], keys/values read from the paged cache through the block table
// (the portion's own rows were scattered there first), so a prompt cut at
// any position sees exactly the keys a whole prompt would.
//
// Query i (absolute position) sees key j iff j <= i and j / block == i / block
// ("block" = the mask's span, counted from position 0). score = q.k * scale +
// bias[i - j, h]; softmax over the visible keys; the head's output is
// multiplied by sigmoid(gate[i, h]).
//
// Workgroup = 16 query rows x 1 head, 4 waves x 4 rows. Key tiles of 64 are
// staged in LDS as fp32; in the score phase a lane owns one key (4 rows
// register-blocked), in the PV phase a lane owns value channels.
constexpr int kAttnQT = 16;
constexpr int kAttnKT = 64;

// Masks of the paged attention kernels. Block-local: query i sees key j iff
// j <= i and both lie in the same span of `span` positions counted from 0.
// Window: j <= i and i - j < span (a span beyond every context = causal).
// Values sit in their own cache (row stride DV) or are the first DV channels
// of the key rows (v_row = D, latent caches); a null bias adds nothing.
constexpr int kMaskBlock = 0;
constexpr int kMaskWindow = 1;

DEVINL int mask_first_key(int pos, int span, int mode) {
  return mode == kMaskBlock ? (pos / span) * span : max(0, pos - span + 1);
}

// What a score gains for the distance d = i - j >= 0 of query and key.
// Table: bias[h, min(d, bias_len - 1)], a learned value per distance. Log:
// bias[h] = (r1, r2) and the score loses r1 * ln(1 + r2 * d).
constexpr int kBiasTable = 0;
constexpr int kBiasLog = 1;

// FAST (bf16 models): the hardware logarithm; fp32 models: log1pf.
template <bool FAST>
DEVINL float log_dist_bias(const float* __restrict__ r12, int d) {
  const float a = r12[1] * (float)d;
  return -r12[0] * (FAST ? __logf(1.0f + a) : log1pf(a));
}

template <bool FAST>
DEVINL float dist_bias(const float* __restrict__ bias, int bias_len, int mode, int h, int d) {
  if (mode == kBiasLog) return log_dist_bias<FAST>(bias + 2 * h, d);
  return bias[(long)h * bias_len + min(d, bias_len - 1)];
}

// Score cap: c * tanh(s / c), with 1 / c computed once per kernel. FAST (bf16
// models): through the hardware exponential and reciprocal,
// 1 - 2 / (e^(2x) + 1); fp32 models: tanhf.
template <bool FAST>
DEVINL float cap_score(float s, float cap, float inv_cap) {
  const float x = s * inv_cap;
  return cap * (FAST ? 1.0f - 2.0f * __builtin_amdgcn_rcpf(__expf(2.0f * x) + 1.0f) : tanhf(x));
}

// Kept first tokens (window mask only): besides its window a query sees every
// key j < keep_first. The keys below min(keep_first, first key of the window
// of the tile's first query) are walked as tiles of their own before the
// window's tiles, cut at that bound so no key is visited twice.
//
// Softmax sink: after the last key a head's denominator gains exp(sink[h]),
// a term without a key or a value.
DEVINL void add_sink(float& m, float& l, float& rescale, float sink) {
  const float m_new = fmaxf(m, sink);
  rescale = m > -INFINITY ? expf(m - m_new) : 0.f;
  l = l * rescale + expf(sink - m_new);
  m = m_new;
}

template <typename T, int NV>
__global__ __launch_bounds__(256) void chunk_bias_attn_prefill_kernel(
    T* __restrict__ out, long out_stride,
    const T* __restrict__ q, long q_stride,
    const T* __restrict__ gate, long g_stride,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const float* __restrict__ bias, int bias_len,   // [H, bias_len], bias_len = min(span, longest context)
    const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ cu_q,          // [B+1]
    const int* __restrict__ q_start,       // [B] position of a sequence's first query
    int H, int G, int D, int DV, int block_size, int span, float scale,
    int v_row, int mask_mode, int bias_mode, int keep_first, const float* __restrict__ sink,
    float softcap) {
  extern __shared__ float smem[];
  const int b = blockIdx.z, h = blockIdx.y;
  const int row0 = cu_q[b];
  const int nq = cu_q[b + 1] - row0;
  const int r0 = blockIdx.x * kAttnQT;
  if (r0 >= nq) return;
  const int rows = min(kAttnQT, nq - r0);
  const int pos0 = q_start[b] + r0;
  const int pos_last = pos0 + rows - 1;
  const int g = h / (H / G);
  const int DP = D + 1;
  // values that are the first channels of the key rows are read out of the
  // K tile: no V tile of their own
  const bool v_alias = v_cache == k_cache;
  const int VP = v_alias ? DP : DV;         // row stride of the V tile
  float* Ks = smem;                         // [KT][D+1]
  float* Vs = v_alias ? Ks : Ks + kAttnKT * DP;            // [KT][DV]
  float* Qs = Ks + kAttnKT * DP + (v_alias ? 0 : kAttnKT * DV);   // [QT][D]
  float* Ps = Qs + kAttnQT * D;             // [QT][KT]
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;

  for (int idx = tid; idx < kAttnQT * D; idx += 256) {
    const int r = idx / D, d = idx % D;
    Qs[idx] = r < rows
        ? to_f32(q[(long)(row0 + r0 + r) * q_stride + (long)h * D + d]) * scale
        : 0.f;
  }
  float m[4], l[4], acc[4][NV];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.f;
#pragma unroll
    for (int n = 0; n < NV; ++n) acc[r][n] = 0.f;
  }
  const int* bt = block_tables + (long)b * bt_stride;
  const int lo = mask_first_key(pos0, span, mask_mode);
  const int first_end = min(keep_first, lo);   // keys [0, first_end): kept, before every window
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;
  for (int kt = first_end > 0 ? 0 : lo; kt <= pos_last;) {
    const bool in_first = kt < first_end;
    const int kt_next = (in_first && kt + kAttnKT >= first_end) ? lo : kt + kAttnKT;
    const int nk = min(kAttnKT, (in_first ? first_end : pos_last + 1) - kt);
    __syncthreads();
    for (int idx = tid; idx < nk * D; idx += 256) {
      const int jj = idx / D, d = idx % D;
      const int key = kt + jj;
      const long base = (((long)bt[key / block_size] * G + g) * block_size +
                         key % block_size);
      Ks[jj * DP + d] = to_f32(k_cache[base * D + d]);
    }
    for (int idx = tid; idx < (v_alias ? 0 : nk * DV); idx += 256) {
      const int jj = idx / DV, d = idx % DV;
      const int key = kt + jj;
      const long base = (((long)bt[key / block_size] * G + g) * block_size +
                         key % block_size);
      Vs[jj * DV + d] = to_f32(v_cache[base * v_row + d]);
    }
    __syncthreads();
    // scores: lane = key, 4 rows at once
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    const int key = kt + lane;
    if (lane < nk) {
      const float* kr = Ks + lane * DP;
      const float* q0 = Qs + (w * 4) * D;
      for (int d = 0; d < D; ++d) {
        const float kd = kr[d];
        s[0] += q0[d] * kd;
        s[1] += q0[D + d] * kd;
        s[2] += q0[2 * D + d] * kd;
        s[3] += q0[3 * D + d] * kd;
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = pos0 + w * 4 + r;
      const bool vis = lane < nk && (w * 4 + r) < rows && key <= i &&
                       (key >= mask_first_key(i, span, mask_mode) || key < keep_first);
      const float sr = softcap > 0.f ? cap_score<sizeof(T) == 2>(s[r], softcap, inv_cap) : s[r];
      const float sc = !vis ? -INFINITY
          : bias ? sr + dist_bias<sizeof(T) == 2>(bias, bias_len, bias_mode, h, i - key) : sr;
      const float tmax = wave_reduce_max(sc);
      const float m_new = fmaxf(m[r], tmax);
      float p = 0.f, corr = 1.f;
      if (m_new > -INFINITY) {
        corr = expf(m[r] - m_new);  // m[r] = -inf -> 0
        p = vis ? expf(sc - m_new) : 0.f;
      }
      l[r] = l[r] * corr + wave_reduce_sum(p);
#pragma unroll
      for (int n = 0; n < NV; ++n) acc[r][n] *= corr;
      m[r] = m_new;
      Ps[(w * 4 + r) * kAttnKT + lane] = p;
    }
    __syncthreads();
    // PV: lane = value channel
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int c = lane + 64 * n;
      if (c < DV) {
        const float* p0 = Ps + (w * 4) * kAttnKT;
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
        for (int jj = 0; jj < nk; ++jj) {
          const float vv = Vs[jj * VP + c];
          a0 += p0[jj] * vv;
          a1 += p0[kAttnKT + jj] * vv;
          a2 += p0[2 * kAttnKT + jj] * vv;
          a3 += p0[3 * kAttnKT + jj] * vv;
        }
        acc[0][n] += a0;
        acc[1][n] += a1;
        acc[2][n] += a2;
        acc[3][n] += a3;
      }
    }
    kt = kt_next;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int rr = w * 4 + r;
    if (rr >= rows) continue;
    const long trow = row0 + r0 + rr;
    if (sink) {
      float rescale;
      add_sink(m[r], l[r], rescale, sink[h]);
#pragma unroll
      for (int n = 0; n < NV; ++n) acc[r][n] *= rescale;
    }
    float gs = 1.f;
    if (gate) gs = 1.0f / (1.0f + expf(-to_f32(gate[trow * g_stride + h])));
    const float inv = gs / l[r];
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int c = lane + 64 * n;
      if (c < DV) out[trow * out_stride + (long)h * DV + c] = from_f32<T>(acc[r][n] * inv);
    }
  }
}

// The bf16 form of the same kernel on the matrix cores.
//
// Workgroup = 64 query rows x 1 head, one wave per 16 rows. Per 64-key tile:
// K is staged row-major [key][D] and V transposed [channel][key] in LDS, so
// every MFMA operand is one 16-byte LDS read. When values are the first
// channels of the key rows (v_cache == k_cache) the V tile is filled from the
// K granules already in registers: nothing is fetched twice. S = Q K^T and O += P V run on
// v_mfma_f32_16x16x32_bf16 (A: row = lane%16, k = 8*(lane/16)..+7; C: rows
// 4*(lane/16)+reg, column lane%16), which puts a query row's scores and its
// output in the same registers of the same lanes: the online-softmax rescale
// needs no exchange. Scores, bias, mask and softmax stay fp32. The weights
// enter the second product as TWO bf16 planes (p = hi + lo, lo the rounding
// remainder of hi), so the product sees them to 16 mantissa bits instead of 8.
typedef __attribute__((ext_vector_type(8))) short sm_bf16x8;
typedef __attribute__((ext_vector_type(4))) float sm_f32x4;
constexpr int kMfmaQT = 64;
constexpr int kMfmaKT = 64;
constexpr int kMfmaKP = kMfmaKT + 8;   // padded key stride of the V^T and P tiles

template <int KS, int DT>
__global__ __launch_bounds__(256, 2) void chunk_bias_attn_prefill_mfma_kernel(
    __hip_bfloat16* __restrict__ out, long out_stride,
    const __hip_bfloat16* __restrict__ q, long q_stride,
    const __hip_bfloat16* __restrict__ gate, long g_stride,
    const __hip_bfloat16* __restrict__ k_cache, const __hip_bfloat16* __restrict__ v_cache,
    const float* __restrict__ bias, int bias_len,   // [H, bias_len]
    const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ cu_q, const int* __restrict__ q_start,
    int H, int G, int D, int DV, int block_size, int span, float scale,
    int v_row, int mask_mode, int ps, int n_split, float* __restrict__ part, int bias_mode,
    int keep_first, const float* __restrict__ sink, float softcap) {
  // n_split > 1: the grid's y dimension carries (key split, head); a
  // workgroup walks only its share of the key tiles and writes its
  // unnormalised output, running maximum and sum to `part`
  // [row, head, split, DV + 2] for attn_merge_splits_kernel.
  // ps = 1: row r of a sequence sits at position q_start + r (a prompt
  // portion). ps = 0: all rows of a sequence sit at q_start — the rows are the
  // query HEADS of one new token that share one kv head, laid out as rows of
  // a single head, so a decode step over a latent cache runs on the matrix
  // cores with every key tile staged once for all heads.
  extern __shared__ __align__(16) unsigned char smem_raw[];
  constexpr int VG = DT / 2;             // 32-channel groups of V per thread
  const int b = blockIdx.z, h = blockIdx.y % H, sp = blockIdx.y / H;
  const int row0 = cu_q[b];
  const int nq = cu_q[b + 1] - row0;
  const int r0 = blockIdx.x * kMfmaQT;
  if (r0 >= nq) return;
  const int rows = min(kMfmaQT, nq - r0);
  const int pos0 = q_start[b] + r0 * ps;
  const int pos_last = pos0 + (rows - 1) * ps;
  const int g = h / (H / G);
  const int ksn = (D + 31) / 32, dtn = (DV + 15) / 16;
  const bool v_alias = v_cache == k_cache;             // values = prefix of the key rows
  const int Dp = ksn * 32, DS = Dp + 8;
  short* Ks = reinterpret_cast<short*>(smem_raw);     // [KT][DS]
  short* Vt = Ks + kMfmaKT * DS;                      // [dtn*16][KP]
  short* Ps = Vt + dtn * 16 * kMfmaKP;                // [4 waves][hi, lo][16][KP]
  float* Bs = reinterpret_cast<float*>(Ps + 4 * 2 * 16 * kMfmaKP);  // [128] bias slice
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int col = lane & 15, kgrp = lane >> 4;

  sm_bf16x8 qf[KS];
  {
    const int r = w * 16 + col;
    const __hip_bfloat16* qr = q + (long)(row0 + r0 + r) * q_stride + (long)h * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d8 = ks * 32 + kgrp * 8;
      qf[ks] = (r < rows && d8 < D) ? *reinterpret_cast<const sm_bf16x8*>(qr + d8)
                                    : sm_bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  int irow[4], lorow[4];
  float m[4], l[4];
#pragma unroll
  for (int reg = 0; reg < 4; ++reg) {
    const int r = w * 16 + kgrp * 4 + reg;
    irow[reg] = r < rows ? pos0 + r * ps : -1;  // -1: no key satisfies key <= irow
    lorow[reg] = r < rows ? mask_first_key(pos0 + r * ps, span, mask_mode) : 0;
    m[reg] = -INFINITY;
    l[reg] = 0.f;
  }
  sm_f32x4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = sm_f32x4{0.f, 0.f, 0.f, 0.f};
  const int wave_first = pos0 + w * 16 * ps;
  const int wave_last = min(pos_last, wave_first + 15 * ps);
  const int wave_lo = mask_first_key(wave_first, span, mask_mode);
  const bool wave_rows = w * 16 < rows;
  const int* bt = block_tables + (long)b * bt_stride;
  const bool bias_log = bias_mode == kBiasLog;
  const float* bias_h = bias ? bias + (bias_log ? 2L * h : (long)h * bias_len) : nullptr;
  short* Pw = Ps + w * 2 * 16 * kMfmaKP;
  const bool v_vec = (DV % 8) == 0 && (v_row % 8) == 0;

  // Staging map: thread = (key = tid/4, sub = tid%4) moves the 16-byte
  // granules sub*8 + 32*i of its key's K row and V row. The next tile's
  // granules are fetched into registers before the current tile's math and
  // written to LDS after it, so HBM/L2 latency hides behind the MFMAs.
  const int skey = tid >> 2, sub = tid & 3;
  sm_bf16x8 kreg[KS], vreg[VG];
  const sm_bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  auto fetch = [&](int kt) {
    const int gkey = kt + skey;
    const bool live = gkey <= pos_last;
    long base = 0;
    if (live) base = ((long)bt[gkey / block_size] * G + g) * block_size + gkey % block_size;
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      const int d8 = sub * 8 + 32 * i;
      kreg[i] = (live && d8 < D) ? *reinterpret_cast<const sm_bf16x8*>(k_cache + base * D + d8)
                                 : zero8;
    }
#pragma unroll
    for (int i = 0; i < VG; ++i) {
      const int d8 = sub * 8 + 32 * i;
      sm_bf16x8 e = zero8;
      if (!v_alias && live && d8 < DV) {
        const __hip_bfloat16* vr = v_cache + base * v_row + d8;
        if (v_vec) {
          e = *reinterpret_cast<const sm_bf16x8*>(vr);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (d8 + j < DV) e[j] = __bfloat16_as_short(vr[j]);
        }
      }
      vreg[i] = e;
    }
  };
  int kt0 = mask_first_key(pos0, span, mask_mode);
  int key_end = pos_last;                // last key this workgroup visits
  if (n_split > 1) {
    const int tiles = (pos_last - kt0) / kMfmaKT + 1;
    const int chunk = (tiles + n_split - 1) / n_split;
    kt0 += sp * chunk * kMfmaKT;
    key_end = min(pos_last, kt0 + chunk * kMfmaKT - 1);
  }
  // kept first tokens (never together with key splits): their tiles come first
  const int win0 = kt0;
  const int first_end = min(keep_first, win0);
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;
  if (first_end > 0) kt0 = 0;
  if (kt0 <= key_end) fetch(kt0);
  for (int kt = kt0; kt <= key_end;) {
    const bool in_first = kt < first_end;
    const int kt_next = (in_first && kt + kMfmaKT >= first_end) ? win0 : kt + kMfmaKT;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      const int d8 = sub * 8 + 32 * i;
      if (d8 < Dp) *reinterpret_cast<sm_bf16x8*>(Ks + skey * DS + d8) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < VG; ++i) {
      const int d8 = sub * 8 + 32 * i;
      if (d8 < dtn * 16) {
        const sm_bf16x8 e = v_alias ? kreg[i] : vreg[i];
#pragma unroll
        for (int j = 0; j < 8; ++j) Vt[(d8 + j) * kMfmaKP + skey] = e[j];
      }
    }
    if (tid < 127) {
      // distances this tile can ask for: (pos0 + r) - (kt + c), r, c in [0, 64)
      const int d = pos0 - kt - 63 + tid;
      Bs[tid] = !bias_h || d < 0 ? 0.f
          : bias_log ? log_dist_bias<true>(bias_h, d)
          : d < bias_len ? bias_h[d] : 0.f;
    }
    __syncthreads();
    if (kt_next <= key_end) fetch(kt_next);
    const bool active = wave_rows && kt <= wave_last &&
                        (in_first || kt + kMfmaKT - 1 >= wave_lo);
    if (active) {
      sm_f32x4 s[4];
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        s[ct] = sm_f32x4{0.f, 0.f, 0.f, 0.f};
        const short* kr = Ks + (ct * 16 + col) * DS + kgrp * 8;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          if (ks < ksn) {
            const sm_bf16x8 bf = *reinterpret_cast<const sm_bf16x8*>(kr + ks * 32);
            s[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], bf, s[ct], 0, 0, 0);
          }
        }
      }
#pragma unroll
      for (int reg = 0; reg < 4; ++reg) {
        float sv[4], tmax = -INFINITY;
        const float* brow = Bs + (w * 16 + kgrp * 4 + reg) * ps + 63 - col;
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
          const int key = kt + ct * 16 + col;
          const bool vis = key <= irow[reg] &&
              (in_first ? key < first_end : (key >= lorow[reg] || key < keep_first));
          float sc = s[ct][reg] * scale;
          if (softcap > 0.f) sc = cap_score<true>(sc, softcap, inv_cap);
          sv[ct] = vis ? sc + brow[-ct * 16] : -INFINITY;
          tmax = fmaxf(tmax, sv[ct]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 1, WAVE));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 2, WAVE));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 4, WAVE));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 8, WAVE));
        const float m_new = fmaxf(m[reg], tmax);
        float alpha = 1.f, psum = 0.f;
        float pv[4] = {0.f, 0.f, 0.f, 0.f};
        if (m_new > -INFINITY) {
          alpha = __expf(m[reg] - m_new);
#pragma unroll
          for (int ct = 0; ct < 4; ++ct) {
            pv[ct] = sv[ct] > -INFINITY ? __expf(sv[ct] - m_new) : 0.f;
            psum += pv[ct];
          }
        }
        l[reg] = l[reg] * alpha + psum;   // per-lane partial; reduced at the end
        m[reg] = m_new;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[dt][reg] *= alpha;
        short* pr = Pw + (kgrp * 4 + reg) * kMfmaKP + col;
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
          const __hip_bfloat16 hi = __float2bfloat16(pv[ct]);
          const __hip_bfloat16 lo = __float2bfloat16(pv[ct] - __bfloat162float(hi));
          pr[ct * 16] = __bfloat16_as_short(hi);
          pr[16 * kMfmaKP + ct * 16] = __bfloat16_as_short(lo);
        }
      }
    }
    __syncthreads();
    if (active) {
#pragma unroll
      for (int k2 = 0; k2 < kMfmaKT / 32; ++k2) {
        const sm_bf16x8 a_hi = *reinterpret_cast<const sm_bf16x8*>(
            Pw + col * kMfmaKP + k2 * 32 + kgrp * 8);
        const sm_bf16x8 a_lo = *reinterpret_cast<const sm_bf16x8*>(
            Pw + (16 + col) * kMfmaKP + k2 * 32 + kgrp * 8);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          if (dt < dtn) {
            const sm_bf16x8 bf = *reinterpret_cast<const sm_bf16x8*>(
                Vt + (dt * 16 + col) * kMfmaKP + k2 * 32 + kgrp * 8);
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, bf, o[dt], 0, 0, 0);
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, bf, o[dt], 0, 0, 0);
          }
        }
      }
    }
    kt = kt_next;
  }
#pragma unroll
  for (int reg = 0; reg < 4; ++reg) {
    float ll = l[reg];
    ll += __shfl_xor(ll, 1, WAVE);
    ll += __shfl_xor(ll, 2, WAVE);
    ll += __shfl_xor(ll, 4, WAVE);
    ll += __shfl_xor(ll, 8, WAVE);
    const int r = w * 16 + kgrp * 4 + reg;
    if (r >= rows) continue;
    const long trow = row0 + r0 + r;
    if (sink && n_split == 1) {
      float rescale;
      add_sink(m[reg], ll, rescale, sink[h]);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[dt][reg] *= rescale;
    }
    if (n_split > 1) {
      float* pr = part + ((trow * H + h) * n_split + sp) * (long)(DV + 2);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const int c = dt * 16 + col;
        if (dt < dtn && c < DV) pr[c] = o[dt][reg];
      }
      if (col == 0) {
        pr[DV] = m[reg];
        pr[DV + 1] = ll;
      }
      continue;
    }
    float gs = 1.f;
    if (gate) gs = 1.0f / (1.0f + expf(-__bfloat162float(gate[trow * g_stride + h])));
    const float inv = gs / ll;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const int c = dt * 16 + col;
      if (dt < dtn && c < DV)
        out[trow * out_stride + (long)h * DV + c] = __float2bfloat16(o[dt][reg] * inv);
    }
  }
}

// Merge of key splits: out[row, head] = sum_s o_s e^(m_s - M) / sum_s l_s e^(m_s - M),
// M = max_s m_s; a split that saw no key has m = -inf and counts nothing.
// One wave per (row, head), lanes over value channels.
__global__ __launch_bounds__(256) void attn_merge_splits_kernel(
    __hip_bfloat16* __restrict__ out, long out_stride, const float* __restrict__ part,
    long pairs, int H, int DV, int n_split) {
  const long pair = blockIdx.x * 4L + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int lane = threadIdx.x & 63;
  const float* pp = part + pair * n_split * (long)(DV + 2);
  float M = -INFINITY;
  for (int sidx = 0; sidx < n_split; ++sidx) M = fmaxf(M, pp[sidx * (DV + 2) + DV]);
  float L = 0.f;
  for (int sidx = 0; sidx < n_split; ++sidx) {
    const float ms = pp[sidx * (DV + 2) + DV];
    if (ms > -INFINITY) L += pp[sidx * (DV + 2) + DV + 1] * expf(ms - M);
  }
  const long row = pair / H;
  const int h = (int)(pair % H);
  for (int c = lane; c < DV; c += 64) {
    float a = 0.f;
    for (int sidx = 0; sidx < n_split; ++sidx) {
      const float ms = pp[sidx * (DV + 2) + DV];
      if (ms > -INFINITY) a += pp[sidx * (DV + 2) + c] * expf(ms - M);
    }
    out[row * out_stride + (long)h * DV + c] = __float2bfloat16(a / L);
  }
}

// ------------------------------------------------ attention: single tokens --
// One workgroup per (sequence, group of HPW query heads that share a kv
// head); the query is the sequence's newest token (position ctx-1). Waves
// take key tiles of 64 round-robin, each with its own online softmax per
// head; partials merge through LDS. A lane owns one key of the tile: it reads
// that key's row once (16-byte loads when the row allows) and scores all HPW
// heads against it; in the PV phase a lane owns value channels and every
// value it reads feeds all HPW heads. With one kv head for all query heads
// (latent caches) the cache is read H / HPW times instead of H times. The
// workgroup has kDecWaves waves, so a context of 1024 keys is one tile per
// wave: the grid of a decode batch alone rarely fills the chip.
constexpr int kDecWaves = 16;

template <typename T, int NV, int HPW>
__global__ __launch_bounds__(64 * kDecWaves) void chunk_bias_attn_decode_kernel(
    T* __restrict__ out, long out_stride,
    const T* __restrict__ q, long q_stride,
    const T* __restrict__ gate, long g_stride,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const float* __restrict__ bias, int bias_len,
    const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ context_lens,
    int H, int G, int D, int DV, int block_size, int span, float scale,
    int v_row, int mask_mode, int bias_mode, int keep_first, const float* __restrict__ sink,
    float softcap) {
  extern __shared__ __align__(16) float smem[];
  const int h0 = blockIdx.x * HPW, b = blockIdx.y;
  const int g = h0 / (H / G);
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int Dq = (D + 3) & ~3;         // padded so float4 reads stay in a head's row
  float* Qs = smem;                    // [HPW][Dq]
  constexpr int NW = kDecWaves, NT = 64 * kDecWaves;
  float* Ms = Qs + HPW * Dq;           // [NW][HPW] max, [NW][HPW] sum
  float* As = Ms + 2 * NW * HPW;       // [NW][HPW][DV]
  for (int idx = tid; idx < HPW * Dq; idx += NT) {
    const int hh = idx / Dq, d = idx % Dq;
    Qs[idx] = d < D ? to_f32(q[(long)b * q_stride + (long)(h0 + hh) * D + d]) * scale : 0.f;
  }
  __syncthreads();
  const int i = context_lens[b] - 1;
  const int lo = mask_first_key(i, span, mask_mode);
  const int* bt = block_tables + (long)b * bt_stride;
  constexpr int VE = Vec8<T>::kElems;
  const bool k_vec = (D % VE) == 0;
  float m[HPW], l[HPW], acc[HPW][NV];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    m[hh] = -INFINITY;
    l[hh] = 0.f;
#pragma unroll
    for (int n = 0; n < NV; ++n) acc[hh][n] = 0.f;
  }
  // tiles: first the kept keys below the window, then the window's
  const int first_end = min(keep_first, lo);
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;
  const int n_first = (first_end + 63) / 64;
  const int n_tiles = n_first + (i - lo) / 64 + 1;
  for (int tile = w; tile < n_tiles; tile += NW) {
    const bool in_first = tile < n_first;
    const int kt = in_first ? tile * 64 : lo + (tile - n_first) * 64;
    const int nk = min(64, (in_first ? first_end : i + 1) - kt);
    const int key = kt + lane;
    long base = 0;
    float sc[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) sc[hh] = -INFINITY;
    if (lane < nk) {
      base = ((long)bt[key / block_size] * G + g) * block_size + key % block_size;
      const T* kr = k_cache + base * D;
      float s[HPW];
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) s[hh] = 0.f;
      if (k_vec) {
        for (int d = 0; d < D; d += VE) {
          const Vec8<T> kv = load16(kr + d);
          float kf[VE];
#pragma unroll
          for (int j = 0; j < VE; ++j) kf[j] = to_f32(kv.data[j]);
#pragma unroll
          for (int hh = 0; hh < HPW; ++hh) {
#pragma unroll
            for (int j = 0; j < VE; j += 4) {
              const float4 q4 = *reinterpret_cast<const float4*>(Qs + hh * Dq + d + j);
              s[hh] += q4.x * kf[j] + q4.y * kf[j + 1] + q4.z * kf[j + 2] + q4.w * kf[j + 3];
            }
          }
        }
      } else {
        for (int d = 0; d < D; ++d) {
          const float kd = to_f32(kr[d]);
#pragma unroll
          for (int hh = 0; hh < HPW; ++hh) s[hh] += Qs[hh * Dq + d] * kd;
        }
      }
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) {
        const float sr = softcap > 0.f ? cap_score<sizeof(T) == 2>(s[hh], softcap, inv_cap) : s[hh];
        sc[hh] = bias ? sr + dist_bias<sizeof(T) == 2>(bias, bias_len, bias_mode, h0 + hh, i - key)
                      : sr;
      }
    }
    float p[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      const float m_new = fmaxf(m[hh], wave_reduce_max(sc[hh]));  // nk >= 1: finite
      const float corr = expf(m[hh] - m_new);
      p[hh] = lane < nk ? expf(sc[hh] - m_new) : 0.f;
      l[hh] = l[hh] * corr + wave_reduce_sum(p[hh]);
      m[hh] = m_new;
#pragma unroll
      for (int n = 0; n < NV; ++n) acc[hh][n] *= corr;
    }
    for (int jj = 0; jj < nk; ++jj) {
      const long vb = __shfl(base, jj, WAVE);
      const T* vr = v_cache + vb * v_row;
      float vv[NV];
#pragma unroll
      for (int n = 0; n < NV; ++n) {
        const int c = lane + 64 * n;
        vv[n] = c < DV ? to_f32(vr[c]) : 0.f;
      }
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) {
        const float pj = __shfl(p[hh], jj, WAVE);
#pragma unroll
        for (int n = 0; n < NV; ++n) acc[hh][n] += pj * vv[n];
      }
    }
  }
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    if (lane == 0) {
      Ms[w * HPW + hh] = m[hh];
      Ms[(NW + w) * HPW + hh] = l[hh];
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int c = lane + 64 * n;
      if (c < DV) As[((long)w * HPW + hh) * DV + c] = acc[hh][n];
    }
  }
  __syncthreads();
  for (int idx = tid; idx < HPW * DV; idx += NT) {
    const int hh = idx / DV, c = idx % DV;
    float mm = -INFINITY;
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) mm = fmaxf(mm, Ms[ww * HPW + hh]);
    float a = 0.f, ll = 0.f;
    if (sink) {
      mm = fmaxf(mm, sink[h0 + hh]);
      ll = expf(sink[h0 + hh] - mm);
    }
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) {
      const float mw = Ms[ww * HPW + hh];
      const float f = mw > -INFINITY ? expf(mw - mm) : 0.f;
      ll += Ms[(NW + ww) * HPW + hh] * f;
      a += As[((long)ww * HPW + hh) * DV + c] * f;
    }
    float gs = 1.f;
    if (gate) gs = 1.0f / (1.0f + expf(-to_f32(gate[(long)b * g_stride + h0 + hh])));
    out[(long)b * out_stride + (long)(h0 + hh) * DV + c] = from_f32<T>(a * gs / ll);
  }
}

// ------------------------------------------- diagonal-decay recurrences ----
// Per head, per sequence: S_t = diag(a_t) S_{t-1} + w_t v_t^T, o_t = S_t^T q_t,
// state S in fp32 [D, DV] living in a per-sequence slot between steps. Two
// forms of the decay a_t and the write strength w_t per key channel:
//   gated linear attention (lower == null): a = sigmoid(z + z_bias)^(1/tau),
//     w = k;
//   HGRN2 (lower != null): a = l + (1 - l) * sigmoid(z + z_bias), w = 1 - a
//     (no key is read).
//   matrix memory (hdecay != null): per token and head ONE decay and one
//     write strength, computed beforehand (fp32 [T, H]): a = hdecay[t, h] on
//     every key channel, w = hwrite[t, h] * k; z is not read. With ones_col the
//     value gets one more column that is always 1, so the state's last column
//     accumulates the written keys alone (an mLSTM's normaliser vector) and
//     the output's last column is its product with q.
// q enters as q_scale * q, or q_scale * silu(q) with q_silu.
//
// Value columns evolve independently, so the grid splits DV: a workgroup owns
// 32 columns of one (sequence, head), two per thread. Its 256 threads are 16 column pairs x 16 key
// groups (4 per wave, one lane quad per column); a thread keeps DPL
// consecutive key channels of one column in registers, so a token costs it
// DPL multiply-adds per product. The partial o of a wave (quad reduce) goes to LDS and the four
// waves' partials are summed once per 16-token stage. Each stage's q, k and
// decay (computed once per stage, fp32: exp(log_sigmoid(z) / tau)) and v sit in LDS,
// zero-padded to 16*DPL channels. Sequential over tokens, parallel over
// (sequence, head, 32 columns). A sequence whose portion starts at position 0
// (fresh != 0) starts from a zero state without reading its slot, so reused
// slots need no clearing.
constexpr int kGlaTB = 16;
constexpr int kGlaCols = 32;   // value columns per workgroup (2 per thread)

template <typename T, int DPL>
__global__ __launch_bounds__(256) void gla_recurrence_kernel(
    float* __restrict__ o,                  // [T, H, DV] fp32
    const T* __restrict__ q, long q_stride,
    const T* __restrict__ k, long k_stride,
    const T* __restrict__ v, long v_stride,
    const T* __restrict__ z, long z_stride,
    const float* __restrict__ z_bias,       // [H*D]
    float* __restrict__ state,              // [slots, H, D, DV]
    const int* __restrict__ cu,             // [B+1] row offsets
    const int* __restrict__ slots,          // [B]
    const int* __restrict__ fresh,          // [B]
    int H, int D, int DV, float inv_tau, float q_scale,
    const float* __restrict__ lower,        // [H*D] or null
    int q_silu,
    const float* __restrict__ hdecay,       // [T, H] or null
    const float* __restrict__ hwrite,       // [T, H] (with hdecay)
    int ones_col) {                         // v has DV - 1 columns; column DV - 1 is 1
  constexpr int DP = 16 * DPL;          // padded key channels
  const int DVin = DV - (ones_col ? 1 : 0);
  __shared__ __align__(16) float qs[kGlaTB * DP];
  __shared__ __align__(16) float ks[kGlaTB * DP];
  __shared__ __align__(16) float as[kGlaTB * DP];
  __shared__ float vs[kGlaTB * kGlaCols];
  __shared__ float po[kGlaTB * 4 * kGlaCols];
  const int b = blockIdx.z, h = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  // a column's 4 key groups sit in one lane quad: their reduce is two DPP
  // quad permutes, no LDS traffic
  const int colw = lane >> 2, kg = lane & 3;
  const int c0 = blockIdx.x * kGlaCols + colw, c1 = c0 + 16;
  const int d0 = (w * 4 + kg) * DPL;
  const int row0 = cu[b];
  const int n = cu[b + 1] - row0;
  const long sbase = ((long)slots[b] * H + h) * D * (long)DV;
  float S0[DPL], S1[DPL];
  const bool use_old = fresh[b] == 0;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int d = d0 + i;
    S0[i] = (use_old && d < D && c0 < DV) ? state[sbase + (long)d * DV + c0] : 0.f;
    S1[i] = (use_old && d < D && c1 < DV) ? state[sbase + (long)d * DV + c1] : 0.f;
  }
  // A thread stages exactly DPL (token, channel) pairs per 16-token stage
  // (idx = tid + 256 j) and two values. The next stage's raw q, k, z and v
  // are fetched into registers before the current stage's token loop and
  // turned into LDS contents (scale, decay) after it.
  float rq[DPL], rk[DPL], rz[DPL], rv[2];
  auto fetch = [&](int t0) {
    const int nt = min(kGlaTB, n - t0);
#pragma unroll
    for (int j = 0; j < DPL; ++j) {
      const int idx = tid + 256 * j;
      const int tt = idx / DP, d = idx % DP;
      rq[j] = rk[j] = rz[j] = 0.f;
      if (tt < nt && d < D) {
        const long row = row0 + t0 + tt;
        rq[j] = to_f32(q[row * q_stride + (long)h * D + d]);
        if (k) rk[j] = to_f32(k[row * k_stride + (long)h * D + d]);
        if (hdecay) {
          rz[j] = hdecay[row * H + h];
          rk[j] *= hwrite[row * H + h];
        } else {
          rz[j] = to_f32(z[row * z_stride + (long)h * D + d]);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int idx = tid + 256 * j;
      const int tt = idx / kGlaCols, gc = blockIdx.x * kGlaCols + idx % kGlaCols;
      rv[j] = (tt < nt && gc < DVin)
          ? to_f32(v[(long)(row0 + t0 + tt) * v_stride + (long)h * DVin + gc])
          : (tt < nt && gc < DV) ? 1.f : 0.f;
    }
  };
  if (n > 0) fetch(0);
  for (int t0 = 0; t0 < n; t0 += kGlaTB) {
    const int nt = min(kGlaTB, n - t0);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < DPL; ++j) {
      const int idx = tid + 256 * j;
      const int d = idx % DP;
      float av = 0.f, kv = rk[j], qv = rq[j];
      if (q_silu) {
        if constexpr (std::is_same_v<T, float>) qv = qv / (1.0f + expf(-qv));
        else qv = qv / (1.0f + __expf(-qv));
      }
      if (hdecay) {
        av = rz[j];                     // 0 on padded rows and channels
      } else if (d < D && lower) {
        const float zz = rz[j] + z_bias[h * D + d];
        const float lo = lower[h * D + d];
        float sg;
        if constexpr (std::is_same_v<T, float>) sg = 1.0f / (1.0f + expf(-zz));
        else sg = 1.0f / (1.0f + __expf(-zz));
        av = lo + (1.0f - lo) * sg;
        kv = 1.0f - av;
      } else if (d < D) {
        const float zz = rz[j] + z_bias[h * D + d];
        // log sigmoid(zz) = min(zz, 0) - log1p(exp(-|zz|)); fp32 models take
        // the accurate library functions, bf16 models the hardware exp/log
        // (a few ulp of fp32, far below the rounding of their inputs)
        if constexpr (std::is_same_v<T, float>) {
          const float ls = fminf(zz, 0.f) - log1pf(expf(-fabsf(zz)));
          av = expf(ls * inv_tau);
        } else {
          const float ls = fminf(zz, 0.f) - __logf(1.0f + __expf(-fabsf(zz)));
          av = __expf(ls * inv_tau);
        }
      }
      qs[idx] = qv * q_scale;
      ks[idx] = kv;
      as[idx] = av;
    }
    vs[tid] = rv[0];
    vs[tid + 256] = rv[1];
    __syncthreads();
    if (t0 + kGlaTB < n) fetch(t0 + kGlaTB);
#pragma unroll 4
    for (int tt = 0; tt < nt; ++tt) {
      const float v0 = vs[tt * kGlaCols + colw];
      const float v1 = vs[tt * kGlaCols + 16 + colw];
      const float* qa = qs + tt * DP + d0;
      const float* ka = ks + tt * DP + d0;
      const float* aa = as + tt * DP + d0;
      float p0 = 0.f, p1 = 0.f;
      if constexpr (DPL % 4 == 0) {
#pragma unroll
        for (int i = 0; i < DPL; i += 4) {
          const float4 a4 = *reinterpret_cast<const float4*>(aa + i);
          const float4 k4 = *reinterpret_cast<const float4*>(ka + i);
          const float4 q4 = *reinterpret_cast<const float4*>(qa + i);
          S0[i] = a4.x * S0[i] + k4.x * v0;
          S0[i + 1] = a4.y * S0[i + 1] + k4.y * v0;
          S0[i + 2] = a4.z * S0[i + 2] + k4.z * v0;
          S0[i + 3] = a4.w * S0[i + 3] + k4.w * v0;
          p0 += S0[i] * q4.x + S0[i + 1] * q4.y + S0[i + 2] * q4.z + S0[i + 3] * q4.w;
          S1[i] = a4.x * S1[i] + k4.x * v1;
          S1[i + 1] = a4.y * S1[i + 1] + k4.y * v1;
          S1[i + 2] = a4.z * S1[i + 2] + k4.z * v1;
          S1[i + 3] = a4.w * S1[i + 3] + k4.w * v1;
          p1 += S1[i] * q4.x + S1[i + 1] * q4.y + S1[i + 2] * q4.z + S1[i + 3] * q4.w;
        }
      } else {
#pragma unroll
        for (int i = 0; i < DPL; ++i) {
          S0[i] = aa[i] * S0[i] + ka[i] * v0;
          p0 += S0[i] * qa[i];
          S1[i] = aa[i] * S1[i] + ka[i] * v1;
          p1 += S1[i] * qa[i];
        }
      }
      p0 += __shfl_xor(p0, 1, WAVE);
      p0 += __shfl_xor(p0, 2, WAVE);
      p1 += __shfl_xor(p1, 1, WAVE);
      p1 += __shfl_xor(p1, 2, WAVE);
      if (kg == 0) {
        po[(tt * 4 + w) * kGlaCols + colw] = p0;
        po[(tt * 4 + w) * kGlaCols + 16 + colw] = p1;
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int idx = tid + 256 * j;
      const int tt = idx / kGlaCols, cc = idx % kGlaCols;
      const int gc = blockIdx.x * kGlaCols + cc;
      if (tt < nt && gc < DV) {
        const float* pp = po + tt * 4 * kGlaCols + cc;
        o[((long)(row0 + t0 + tt) * H + h) * DV + gc] =
            (pp[0] + pp[kGlaCols]) + (pp[2 * kGlaCols] + pp[3 * kGlaCols]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int d = d0 + i;
    if (d < D && c0 < DV) state[sbase + (long)d * DV + c0] = S0[i];
    if (d < D && c1 < DV) state[sbase + (long)d * DV + c1] = S1[i];
  }
}

// Per (token, head): out = rmsnorm_DV(o) * w [* silu(gate)], rounded to T.
// One wave per head, lanes over value channels.
template <typename T>
__global__ __launch_bounds__(256) void gla_out_norm_gate_kernel(
    T* __restrict__ out, long out_stride, const float* __restrict__ o,
    const T* __restrict__ weight, const T* __restrict__ gate, long g_stride,
    int H, int DV, float eps) {
  const long tok = blockIdx.x;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  for (int h = w; h < H; h += 4) {
    const float* oh = o + (tok * H + h) * DV;
    float ss = 0.f;
    for (int c = lane; c < DV; c += 64) ss += oh[c] * oh[c];
    ss = wave_reduce_sum(ss);
    const float inv = 1.0f / sqrtf(ss / DV + eps);
    for (int c = lane; c < DV; c += 64) {
      float sg = 1.f;
      if (gate) {
        const float gt = to_f32(gate[tok * g_stride + (long)h * DV + c]);
        sg = gt / (1.0f + expf(-gt));
      }
      out[tok * out_stride + (long)h * DV + c] =
          from_f32<T>(oh[c] * inv * to_f32(weight[c]) * sg);
    }
  }
}

// Kernels of scan/attention hybrid decoders (gfx950): an embedding with a
// sinusoidal position vector, the scaled residual joins and the learned
// average over layer outputs on an fp32 stream, a plain paged K/V scatter,
// the minGRU recurrence, the short causal convolution and the selective scan
// of a Mamba mixer, a softmax top-k router and a clamped gated activation.
//
// Numerics as in seqmix.hip: activations arrive in the model dtype T (bf16
// or fp32); angles, norms, gates, step sizes, decays, router scores, recurrent
// state and the residual are fp32 in registers and rounded to T once, on
// store.

#include "common.h"

// ------------------------------------------------------------- embedding --
// out[t, :] = embedding[ids[t], :] + pe(positions[t]),  pe[2i] = sin(p f_i),
// pe[2i+1] = cos(p f_i); f is an fp32 table, the angle an fp32 product.
template <typename T>
__global__ void embed_sinusoid_kernel(float* __restrict__ out, const T* __restrict__ embedding,
                                      const long* __restrict__ ids,
                                      const long* __restrict__ positions,
                                      const float* __restrict__ inv_freq, int W, long vocab) {
  const long row = blockIdx.x;
  long id = ids[row];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const float p = (float)positions[row];
  const T* e = embedding + id * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float a = p * inv_freq[c >> 1];
    out[row * W + c] = to_f32(e[c]) + ((c & 1) ? cosf(a) : sinf(a));
  }
}

// ------------------------------------------------------- residual joins ----
// res (fp32, in place) += a1 * y [+ a2 * y2];  out = rmsnorm(res) * w.
// One workgroup per row.
template <typename T>
__global__ __launch_bounds__(256) void scaled_add_norm_kernel(
    T* __restrict__ out, float* __restrict__ res, const T* __restrict__ y,
    const T* __restrict__ y2, float a1, float a2, const T* __restrict__ w, int W, float eps) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  float* rr = res + row * W;
  const T* yr = y + row * W;
  const T* y2r = y2 ? y2 + row * W : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    float r = rr[i] + a1 * to_f32(yr[i]);
    if (y2r) r += a2 * to_f32(y2r[i]);
    rr[i] = r;
    ss += r * r;
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / W + eps);
  for (int i = threadIdx.x; i < W; i += 256)
    out[row * W + i] = from_f32<T>(rr[i] * inv * to_f32(w[i]));
}

// The same for bf16 rows of up to CH * 2048 elements, a multiple of 8 wide:
// the updated residual stays in registers between the two passes and every
// operand crosses memory once, in 16-byte accesses.
template <int CH>
__global__ __launch_bounds__(256) void scaled_add_norm_vec_kernel(
    __hip_bfloat16* __restrict__ out, float* __restrict__ res,
    const __hip_bfloat16* __restrict__ y, const __hip_bfloat16* __restrict__ y2, float a1,
    float a2, const __hip_bfloat16* __restrict__ w, int W, float eps) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  float* rr = res + row * W;
  float rv[CH][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (c * 256 + threadIdx.x) * 8;
    if (i < W) {
      const Vec8<__hip_bfloat16> v = load16(y + row * W + i);
      const float4 ra = *reinterpret_cast<const float4*>(rr + i);
      const float4 rb = *reinterpret_cast<const float4*>(rr + i + 4);
      rv[c][0] = ra.x; rv[c][1] = ra.y; rv[c][2] = ra.z; rv[c][3] = ra.w;
      rv[c][4] = rb.x; rv[c][5] = rb.y; rv[c][6] = rb.z; rv[c][7] = rb.w;
#pragma unroll
      for (int j = 0; j < 8; ++j) rv[c][j] += a1 * to_f32(v.data[j]);
      if (y2) {
        const Vec8<__hip_bfloat16> v2 = load16(y2 + row * W + i);
#pragma unroll
        for (int j = 0; j < 8; ++j) rv[c][j] += a2 * to_f32(v2.data[j]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += rv[c][j] * rv[c][j];
      *reinterpret_cast<float4*>(rr + i) = make_float4(rv[c][0], rv[c][1], rv[c][2], rv[c][3]);
      *reinterpret_cast<float4*>(rr + i + 4) = make_float4(rv[c][4], rv[c][5], rv[c][6], rv[c][7]);
    }
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / W + eps);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (c * 256 + threadIdx.x) * 8;
    if (i < W) {
      const Vec8<__hip_bfloat16> wv = load16(w + i);
      Vec8<__hip_bfloat16> ov;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        ov.data[j] = __float2bfloat16(rv[c][j] * inv * to_f32(wv.data[j]));
      store16(out + row * W + i, ov);
    }
  }
}

// The close of a layer under a learned average over layer outputs. stack is
// [>= n+1][rows][W] fp32 (ls = rows * W elements per entry); entries 0..n-1
// hold the embedding output and the layer results so far.
//   entry n-1 (in place) += a1 * y [+ a2 * y2]
//   entry n = sum_{j<n} coef[j] * entry j
//   out     = rmsnorm(entry n) * w
// One workgroup per row; VEC: 4 fp32 per thread and access.
template <typename T>
__global__ __launch_bounds__(256) void depth_mix_norm_kernel(
    T* __restrict__ out, float* __restrict__ stack, long ls, int n,
    const float* __restrict__ coef, const T* __restrict__ y, const T* __restrict__ y2, float a1,
    float a2, const T* __restrict__ w, int W, float eps) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  float* last = stack + (long)(n - 1) * ls + row * W;
  float* mix = stack + (long)n * ls + row * W;
  const T* yr = y + row * W;
  const T* y2r = y2 ? y2 + row * W : nullptr;
  const float c_last = coef[n - 1];
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    float r = last[i] + a1 * to_f32(yr[i]);
    if (y2r) r += a2 * to_f32(y2r[i]);
    last[i] = r;
    float m = 0.f;
    for (int j = 0; j < n - 1; ++j) m += coef[j] * stack[(long)j * ls + row * W + i];
    m += c_last * r;
    mix[i] = m;
    ss += m * m;
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / W + eps);
  for (int i = threadIdx.x; i < W; i += 256)
    out[row * W + i] = from_f32<T>(mix[i] * inv * to_f32(w[i]));
}

// bf16 rows of up to CH * 1024 elements, a multiple of 4 wide: the averaged
// row stays in registers for the norm; fp32 entries move in 16-byte accesses.
template <int CH>
__global__ __launch_bounds__(256) void depth_mix_norm_vec_kernel(
    __hip_bfloat16* __restrict__ out, float* __restrict__ stack, long ls, int n,
    const float* __restrict__ coef, const __hip_bfloat16* __restrict__ y,
    const __hip_bfloat16* __restrict__ y2, float a1, float a2,
    const __hip_bfloat16* __restrict__ w, int W, float eps) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  float* last = stack + (long)(n - 1) * ls + row * W;
  float* mix = stack + (long)n * ls + row * W;
  const float c_last = coef[n - 1];
  float mv[CH][4];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (c * 256 + threadIdx.x) * 4;
    if (i < W) {
      const float4 r4 = *reinterpret_cast<const float4*>(last + i);
      float r[4] = {r4.x, r4.y, r4.z, r4.w};
      const Vec4<__hip_bfloat16> v = load8(y + row * W + i);
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] += a1 * to_f32(v.data[j]);
      if (y2) {
        const Vec4<__hip_bfloat16> v2 = load8(y2 + row * W + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] += a2 * to_f32(v2.data[j]);
      }
      *reinterpret_cast<float4*>(last + i) = make_float4(r[0], r[1], r[2], r[3]);
      float m[4] = {0.f, 0.f, 0.f, 0.f};
      for (int jl = 0; jl < n - 1; ++jl) {
        const float cj = coef[jl];
        const float4 e = *reinterpret_cast<const float4*>(stack + (long)jl * ls + row * W + i);
        m[0] += cj * e.x; m[1] += cj * e.y; m[2] += cj * e.z; m[3] += cj * e.w;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        m[j] += c_last * r[j];
        mv[c][j] = m[j];
        ss += m[j] * m[j];
      }
      *reinterpret_cast<float4*>(mix + i) = make_float4(m[0], m[1], m[2], m[3]);
    }
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / W + eps);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (c * 256 + threadIdx.x) * 4;
    if (i < W) {
      const Vec4<__hip_bfloat16> wv = load8(w + i);
      Vec4<__hip_bfloat16> ov;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        ov.data[j] = __float2bfloat16(mv[c][j] * inv * to_f32(wv.data[j]));
      *reinterpret_cast<int2*>(out + row * W + i) = *reinterpret_cast<const int2*>(ov.data);
    }
  }
}

// ------------------------------------------------------- paged K/V scatter --
// k [T, G*D] and v [T, G*DV] (row-strided slices of a projection) into the
// paged cache [blocks, G, block_size, D | DV]; a negative slot writes nothing.
template <typename T>
__global__ void kv_scatter_kernel(const T* __restrict__ k, long k_stride, const T* __restrict__ v,
                                  long v_stride, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                  const long* __restrict__ slots, int G, int D, int DV,
                                  int block_size) {
  const long tok = blockIdx.x;
  const long slot = slots[tok];
  if (slot < 0) return;
  const long blk = slot / block_size, off = slot % block_size;
  const T* kr = k + tok * k_stride;
  const T* vr = v + tok * v_stride;
  for (int i = threadIdx.x; i < G * D; i += blockDim.x) {
    const int g = i / D, d = i % D;
    k_cache[((blk * G + g) * block_size + off) * D + d] = kr[i];
  }
  for (int i = threadIdx.x; i < G * DV; i += blockDim.x) {
    const int g = i / DV, d = i % DV;
    v_cache[((blk * G + g) * block_size + off) * DV + d] = vr[i];
  }
}

// ------------------------------------------------------------------ minGRU --
// Per sequence and channel:  S <- (1 - a) S + a c,  a = sigmoid(z + z_b),
// c = u' + 1/2 (u' >= 0) or sigmoid(u') with u' = u + u_b;  out = S * silu(g).
// z, u, g: row-strided slices of one projection output. state [slots, n]
// fp32, advanced in place; a fresh sequence starts from zero without reading
// its slot. A thread owns one channel of one sequence and walks its tokens;
// kGruPre tokens' operands are in flight at a time.
constexpr int kGruPre = 8;

DEVINL float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

template <typename T>
__global__ __launch_bounds__(256) void mingru_scan_kernel(
    T* __restrict__ out, const T* __restrict__ z, const T* __restrict__ u,
    const T* __restrict__ g, long in_stride, const float* __restrict__ z_b,
    const float* __restrict__ u_b, float* __restrict__ state, const int* __restrict__ cu,
    const int* __restrict__ slots, const int* __restrict__ fresh, int n) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= n) return;
  const int s = cu[b], e = cu[b + 1];
  if (e <= s) return;
  float* st = state + (long)slots[b] * n + c;
  float S = fresh[b] ? 0.f : *st;
  const float zb = z_b[c], ub = u_b[c];
  for (int t0 = s; t0 < e; t0 += kGruPre) {
    float zv[kGruPre], uv[kGruPre], gv[kGruPre];
#pragma unroll
    for (int i = 0; i < kGruPre; ++i) {
      const long r = (long)min(t0 + i, e - 1) * in_stride + c;
      zv[i] = to_f32(z[r]);
      uv[i] = to_f32(u[r]);
      gv[i] = to_f32(g[r]);
    }
#pragma unroll
    for (int i = 0; i < kGruPre; ++i) {
      if (t0 + i < e) {
        const float a = sigmoid_f(zv[i] + zb);
        const float uu = uv[i] + ub;
        const float cand = uu >= 0.f ? uu + 0.5f : sigmoid_f(uu);
        S = (1.0f - a) * S + a * cand;
        out[(long)(t0 + i) * n + c] = from_f32<T>(S * gv[i] * sigmoid_f(gv[i]));
      }
    }
  }
  *st = S;
}

// The same recurrence for long portions, parallel over time: a workgroup owns
// 64 channels of one sequence and NC contiguous chunks of its tokens, one
// wave per chunk. A linear recurrence S <- (1 - a) S + a c composes: a chunk
// is summarised by (P, E) = (product of its 1 - a, its end state from a zero
// start). Pass 1 computes every chunk's (P, E); a chunk's start state then
// follows from the sequence's start state and the summaries before it; pass 2
// walks the chunk again from that start and writes the outputs.
template <typename T, int NC>
__global__ __launch_bounds__(64 * NC) void mingru_scan_chunked_kernel(
    T* __restrict__ out, const T* __restrict__ z, const T* __restrict__ u,
    const T* __restrict__ g, long in_stride, const float* __restrict__ z_b,
    const float* __restrict__ u_b, float* __restrict__ state, const int* __restrict__ cu,
    const int* __restrict__ slots, const int* __restrict__ fresh, int n) {
  __shared__ float Ps[NC][64], Es[NC][64];
  constexpr bool FAST = sizeof(T) == 2;
  const int b = blockIdx.y;
  const int lane = threadIdx.x & 63, k = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  const int s = cu[b], e = cu[b + 1];
  if (e <= s) return;
  const bool live = c < n;
  const int cc = live ? c : 0;
  const int L = (e - s + NC - 1) / NC;
  const int t_lo = min(e, s + k * L), t_hi = min(e, t_lo + L);
  const float zb = z_b[cc], ub = u_b[cc];
  auto sig = [](float v) { return 1.0f / (1.0f + (FAST ? __expf(-v) : expf(-v))); };
  float P = 1.f, E = 0.f;
  for (int t0 = t_lo; t0 < t_hi; t0 += kGruPre) {
    float zv[kGruPre], uv[kGruPre];
#pragma unroll
    for (int i = 0; i < kGruPre; ++i) {
      const long r = (long)min(t0 + i, t_hi - 1) * in_stride + cc;
      zv[i] = to_f32(z[r]);
      uv[i] = to_f32(u[r]);
    }
#pragma unroll
    for (int i = 0; i < kGruPre; ++i) {
      if (t0 + i < t_hi) {
        const float a = sig(zv[i] + zb);
        const float uu = uv[i] + ub;
        const float cand = uu >= 0.f ? uu + 0.5f : sig(uu);
        E = (1.0f - a) * E + a * cand;
        P *= 1.0f - a;
      }
    }
  }
  Ps[k][lane] = P;
  Es[k][lane] = E;
  __syncthreads();
  float* st = state + (long)slots[b] * n + cc;
  float S = fresh[b] ? 0.f : *st;
  for (int kk = 0; kk < k; ++kk) S = Ps[kk][lane] * S + Es[kk][lane];
  for (int t0 = t_lo; t0 < t_hi; t0 += kGruPre) {
    float zv[kGruPre], uv[kGruPre], gv[kGruPre];
#pragma unroll
    for (int i = 0; i < kGruPre; ++i) {
      const long r = (long)min(t0 + i, t_hi - 1) * in_stride + cc;
      zv[i] = to_f32(z[r]);
      uv[i] = to_f32(u[r]);
      gv[i] = to_f32(g[r]);
    }
#pragma unroll
    for (int i = 0; i < kGruPre; ++i) {
      if (t0 + i < t_hi) {
        const float a = sig(zv[i] + zb);
        const float uu = uv[i] + ub;
        const float cand = uu >= 0.f ? uu + 0.5f : sig(uu);
        S = (1.0f - a) * S + a * cand;
        if (live) out[(long)(t0 + i) * n + c] = from_f32<T>(S * gv[i] * sig(gv[i]));
      }
    }
  }
  if (live && k == NC - 1) *st = S;   // the last chunk ends where the portion ends
}

// ------------------------------------------------ short causal convolution --
// out[t, c] = silu(b[c] + sum_k w[c, k] * V[j - (K-1) + k]) for row t = s + j
// of a sequence whose inputs are V[j >= 0] = x[s + j] and V[-(K-1) .. -1] =
// the K-1 inputs before this portion (tail[slot, k, c]; zeros for a fresh
// sequence). Not a recurrence: a thread owns one channel and kConvRows
// consecutive packed rows, wherever they fall in their sequences. The tail is
// advanced by a second kernel after every read of the old one has happened.
constexpr int kConvMaxTaps = 16;
constexpr int kConvGroup = 8;    // rows whose inputs a thread fetches together

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_silu_kernel(
    T* __restrict__ out, const T* __restrict__ x, long x_stride, const float* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ tail,
    const int* __restrict__ cu, const int* __restrict__ slots, const int* __restrict__ fresh,
    int B, int C, int K, int rows_per_thread, int silu) {
  // bias may be null; silu == 0 leaves the convolution's result as it is
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int total = cu[B];
  const int r0 = blockIdx.y * rows_per_thread;
  if (r0 >= total) return;
  const int r1 = min(total, r0 + rows_per_thread);
  float wk[kConvMaxTaps], win[kConvMaxTaps];
#pragma unroll
  for (int k = 0; k < kConvMaxTaps; ++k) wk[k] = k < K ? w[(long)c * K + k] : 0.f;
  const float bc = bias ? bias[c] : 0.f;
  int b = 0;
  while (cu[b + 1] <= r0) ++b;   // the sequence of row r0 (empty sequences skipped)
  bool load_window = true;
  for (int g0 = r0; g0 < r1; g0 += kConvGroup) {
    // the group's own inputs first: independent loads, all in flight at once
    float xg[kConvGroup];
#pragma unroll
    for (int i = 0; i < kConvGroup; ++i)
      xg[i] = to_f32(x[(long)min(g0 + i, r1 - 1) * x_stride + c]);
#pragma unroll
    for (int i = 0; i < kConvGroup; ++i) {
      const int r = g0 + i;
      if (r < r1) {
        while (cu[b + 1] <= r) {
          ++b;
          load_window = true;
        }
        if (load_window) {
          const int s = cu[b], j = r - s;
          const float* tl = tail + (long)slots[b] * (K - 1) * C + c;
          const bool fr = fresh[b] != 0;
          // win[k] = V[j - (K-1) + k], k < K-1
#pragma unroll
          for (int k = 0; k < kConvMaxTaps - 1; ++k) {
            if (k < K - 1) {
              const int jj = j - (K - 1) + k;
              win[k] = jj >= 0 ? to_f32(x[(long)(s + jj) * x_stride + c])
                               : (fr ? 0.f : tl[(long)(jj + K - 1) * C]);
            }
          }
          load_window = false;
        }
        const float xv = xg[i];
        float acc = bc;
#pragma unroll
        for (int k = 0; k < kConvMaxTaps - 1; ++k)
          if (k < K - 1) acc += wk[k] * win[k];
#pragma unroll
        for (int k = 0; k < kConvMaxTaps; ++k)
          if (k == K - 1) acc += wk[k] * xv;
        out[(long)r * C + c] = from_f32<T>(silu ? acc * sigmoid_f(acc) : acc);
#pragma unroll
        for (int k = 0; k < kConvMaxTaps - 2; ++k)
          if (k < K - 2) win[k] = win[k + 1];
#pragma unroll
        for (int k = 0; k < kConvMaxTaps - 1; ++k)
          if (k == K - 2) win[k] = xv;
      }
    }
  }
}

// tail[slot, k, c] <- V[n - (K-1) + k], n = the portion's length: its last
// K-1 inputs, reaching back into the old tail when the portion is shorter.
template <typename T>
__global__ __launch_bounds__(256) void conv_tail_update_kernel(
    const T* __restrict__ x, long x_stride, float* __restrict__ tail,
    const int* __restrict__ cu, const int* __restrict__ slots, const int* __restrict__ fresh,
    int C, int K) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int s = cu[b], n = cu[b + 1] - s;
  if (n <= 0) return;
  float* tl = tail + (long)slots[b] * (K - 1) * C + c;
  const bool fr = fresh[b] != 0;
  float nv[kConvMaxTaps];
#pragma unroll
  for (int k = 0; k < kConvMaxTaps - 1; ++k) {
    if (k < K - 1) {
      const int jj = n - (K - 1) + k;
      nv[k] = jj >= 0 ? to_f32(x[(long)(s + jj) * x_stride + c])
                      : (fr ? 0.f : tl[(long)(jj + K - 1) * C]);
    }
  }
#pragma unroll
  for (int k = 0; k < kConvMaxTaps - 1; ++k)
    if (k < K - 1) tl[(long)k * C] = nv[k];
}

// ---------------------------------------------------------- selective scan --
// Per sequence, channel c and state n:
//   step = softplus(dt[t, c] + dt_b[c])
//   S[c, n] <- exp(step * A[c, n]) * S[c, n] + step * x[t, c] * B[t, n]
//   y[t, c] = sum_n S[c, n] * C[t, n] + D[c] * x[t, c];  out = y * silu(z[t, c])
// state [slots, C, N] fp32, advanced in place; a fresh sequence starts from
// zero without reading its slot.
//
// A workgroup owns 64 / LPC channels of one sequence and NC contiguous chunks
// of its tokens, one wave per chunk: LPC adjacent lanes share a channel, each
// with NS of its states in registers (state index sub * NS + j). The
// recurrence is linear in S, so a chunk is summarised by the sum of its steps
// (its decay is exp(A * that sum)) and its end state from a zero start. Pass 1
// computes the summaries, a chunk's start state follows from the sequence's
// start state and the summaries before it, pass 2 walks the chunk again from
// there and writes the outputs. NC = 1 (single tokens, short portions) is the
// plain serial walk. B and C of kScanTT tokens per wave are staged in LDS as
// fp32 and read as broadcasts; a channel's x, dt and z of those tokens are
// fetched before the serial part. bf16 models use the hardware exp/log; fp32
// models the accurate functions.
constexpr int kScanTT = 8;

template <bool FAST>
DEVINL float scan_exp(float x) { return FAST ? __expf(x) : expf(x); }

template <bool FAST>
DEVINL float scan_softplus(float x) {
  if (x > 20.f) return x;
  return FAST ? __logf(1.0f + __expf(x)) : log1pf(expf(x));
}

template <typename T, int NS, int NC>
__global__ __launch_bounds__(64 * NC) void selective_scan_kernel(
    T* __restrict__ out, const T* __restrict__ x, long x_stride, const T* __restrict__ dt,
    long dt_stride, const float* __restrict__ dt_b, const float* __restrict__ A,
    const T* __restrict__ Bm, const T* __restrict__ Cm, long bc_stride,
    const float* __restrict__ Dp, const T* __restrict__ z, long z_stride,
    float* __restrict__ state, const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ fresh, int C, int N, int lpc) {
  // [NC][kScanTT][2][N] staged B and C rows, then (NC > 1) the chunk
  // summaries: [NC][64] step sums and [NC][NS][64] end states
  extern __shared__ float scan_smem[];
  constexpr bool FAST = sizeof(T) == 2;
  const int b = blockIdx.y;
  const int s = cu[b], e = cu[b + 1];
  if (e <= s) return;
  const int lane = threadIdx.x & 63, k = threadIdx.x >> 6;
  const int c = (blockIdx.x * 64 + lane) / lpc, sub = lane % lpc;
  const bool live = c < C;
  const int cc = live ? c : 0;
  const int n0 = sub * NS;
  float* bc = scan_smem + (long)k * kScanTT * 2 * N;
  float* sums = scan_smem + (long)NC * kScanTT * 2 * N;   // [NC][64]
  float* ends = sums + NC * 64;                            // [NC][NS][64]
  const int L = (e - s + NC - 1) / NC;                     // tokens per chunk
  const int t_lo = min(e, s + k * L), t_hi = min(e, t_lo + L);
  float S[NS], a[NS];
  float* st = state + ((long)slots[b] * C + cc) * N;
  const bool fr = fresh[b] != 0;
  if (NS % 4 == 0 && N % 4 == 0) {
#pragma unroll
    for (int j = 0; j < NS / 4 * 4; j += 4) {
      float4 av = make_float4(0.f, 0.f, 0.f, 0.f);
      if (live && n0 + j < N) av = *reinterpret_cast<const float4*>(A + (long)cc * N + n0 + j);
      a[j] = av.x;
      if (j + 1 < NS) a[j + 1] = av.y;
      if (j + 2 < NS) a[j + 2] = av.z;
      if (j + 3 < NS) a[j + 3] = av.w;
    }
  } else {
#pragma unroll
    for (int j = 0; j < NS; ++j) a[j] = (live && n0 + j < N) ? A[(long)cc * N + n0 + j] : 0.f;
  }
  const float db = dt_b[cc], dd = Dp[cc];

  // one pass over the chunk; OUT = false computes only the state
  auto walk = [&]<bool OUT>(float& step_sum) {
    for (int t0 = t_lo; t0 < t_lo + L; t0 += kScanTT) {   // same trip count in every wave
      const int nt = max(0, min(kScanTT, t_hi - t0));
      __syncthreads();
      for (int i = lane; i < nt * N; i += 64) {
        const int tt = i / N, n = i % N;
        bc[(tt * 2) * N + n] = to_f32(Bm[(long)(t0 + tt) * bc_stride + n]);
        if (OUT) bc[(tt * 2 + 1) * N + n] = to_f32(Cm[(long)(t0 + tt) * bc_stride + n]);
      }
      float xv[kScanTT], sp[kScanTT], zg[kScanTT];
#pragma unroll
      for (int tt = 0; tt < kScanTT; ++tt) {
        const long r = max(min(t0 + tt, t_hi - 1), s);
        xv[tt] = to_f32(x[r * x_stride + cc]);
        sp[tt] = scan_softplus<FAST>(to_f32(dt[r * dt_stride + cc]) + db);
        if (OUT) {
          const float zz = to_f32(z[r * z_stride + cc]);
          zg[tt] = zz / (1.0f + scan_exp<FAST>(-zz));
        }
      }
      __syncthreads();
#pragma unroll
      for (int tt = 0; tt < kScanTT; ++tt) {
        if (tt < nt) {
          const float step = sp[tt];
          const float xs = step * xv[tt];
          const float* bs = bc + (tt * 2) * N + n0;
          const float* cs = bs + N;
          step_sum += step;
          float acc = 0.f;
#pragma unroll
          for (int j = 0; j < NS; ++j) {
            if (n0 + j < N) {
              S[j] = scan_exp<FAST>(step * a[j]) * S[j] + xs * bs[j];
              if (OUT) acc += S[j] * cs[j];
            }
          }
          if (OUT) {
            for (int off = 1; off < lpc; off <<= 1) acc += __shfl_xor(acc, off, WAVE);
            if (live && sub == 0)
              out[(long)(t0 + tt) * C + c] = from_f32<T>((acc + dd * xv[tt]) * zg[tt]);
          }
        }
      }
    }
  };

  if constexpr (NC > 1) {
#pragma unroll
    for (int j = 0; j < NS; ++j) S[j] = 0.f;
    float step_sum = 0.f;
    walk.template operator()<false>(step_sum);
    sums[k * 64 + lane] = step_sum;
#pragma unroll
    for (int j = 0; j < NS; ++j) ends[(k * NS + j) * 64 + lane] = S[j];
    __syncthreads();
  }
  bool vec4 = false;   // a lane's states as 16-byte accesses
  if constexpr (NS % 4 == 0) {
    vec4 = N % 4 == 0;
    if (vec4) {
#pragma unroll
      for (int j = 0; j < NS; j += 4) {
        float4 sv = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live && !fr && n0 + j < N) sv = *reinterpret_cast<const float4*>(st + n0 + j);
        S[j] = sv.x; S[j + 1] = sv.y; S[j + 2] = sv.z; S[j + 3] = sv.w;
      }
    }
  }
  if (!vec4) {
#pragma unroll
    for (int j = 0; j < NS; ++j) S[j] = (live && !fr && n0 + j < N) ? st[n0 + j] : 0.f;
  }
  if constexpr (NC > 1) {
    for (int kk = 0; kk < k; ++kk) {
      const float ssum = sums[kk * 64 + lane];
#pragma unroll
      for (int j = 0; j < NS; ++j)
        S[j] = scan_exp<FAST>(ssum * a[j]) * S[j] + ends[(kk * NS + j) * 64 + lane];
    }
  }
  float unused = 0.f;
  walk.template operator()<true>(unused);
  if (live && k == NC - 1) {   // the last chunk ends where the portion ends
    if constexpr (NS % 4 == 0) {
      if (vec4) {
#pragma unroll
        for (int j = 0; j < NS; j += 4)
          if (n0 + j < N)
            *reinterpret_cast<float4*>(st + n0 + j) =
                make_float4(S[j], S[j + 1], S[j + 2], S[j + 3]);
      }
    }
    if (!vec4) {
#pragma unroll
      for (int j = 0; j < NS; ++j)
        if (n0 + j < N) st[n0 + j] = S[j];
    }
  }
}

// ------------------------------------------------------- softmax router ----
// Scores s = softmax(logits) over ALL experts in fp32; the `top` largest per
// token, largest first, ties to the lower expert index; weight = s * scale.
// One wave per token; a lane owns experts lane, lane + 64, ... (at most
// 64 * 32 experts).
__global__ __launch_bounds__(256) void softmax_topk_kernel(
    int* __restrict__ idx_out, float* __restrict__ w_out, const float* __restrict__ logits,
    long rows, int E, int top, float scale, const float* __restrict__ correction, int renorm) {
  // correction [E] (or null): the choice is made on s + correction, the
  // weights stay the plain scores. renorm: the chosen scores are divided by
  // their sum (+ 1e-20) before the scale.
  const int lane = threadIdx.x & 63;
  const long tok = blockIdx.x * 4L + (threadIdx.x >> 6);
  if (tok >= rows) return;
  const float* z = logits + tok * E;
  float mx = -INFINITY;
  for (int e = lane; e < E; e += 64) {
    const float v = z[e];
    if (v > mx) mx = v;
  }
  mx = wave_reduce_max(mx);
  float sum = 0.f;
  for (int e = lane; e < E; e += 64) {
    const float v = z[e];
    if (v == v) sum += expf(v - mx);
  }
  sum = wave_reduce_sum(sum);
  unsigned taken = 0u;   // bit n: expert lane + 64 n already chosen
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int best_e = 0x7fffffff;
    for (int e = lane, n = 0; e < E; e += 64, ++n) {
      if (taken & (1u << n)) continue;
      float v = z[e];
      if (correction) v = expf(v - mx) / sum + correction[e];
      if (!(v == v)) v = -3.0e38f;   // a NaN logit still yields a valid index
      if (v > best || best_e == 0x7fffffff) {   // ascending e: the first of equals stays
        best = v;
        best_e = e;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, WAVE);
      const int oe = __shfl_xor(best_e, off, WAVE);
      if (oe != 0x7fffffff && (best_e == 0x7fffffff || ob > best || (ob == best && oe < best_e))) {
        best = ob;
        best_e = oe;
      }
    }
    if ((best_e & 63) == lane) taken |= 1u << (best_e >> 6);
    if (lane == 0) {
      idx_out[tok * top + k] = best_e;
      w_out[tok * top + k] = expf((correction ? z[best_e] : best) - mx) / sum;
    }
  }
  if (lane == 0) {
    float total = 1.0f;
    if (renorm) {
      total = 1e-20f;
      for (int k = 0; k < top; ++k) total += w_out[tok * top + k];
    }
    for (int k = 0; k < top; ++k) w_out[tok * top + k] = w_out[tok * top + k] / total * scale;
  }
}

// ------------------------------------------------ clamped gated activation --
// in [rows, 2d] -> out [rows, d] = g * sigmoid(1.702 g) * (u + 1) with
// g = min(in[:, :d], limit), u = clamp(in[:, d:], -limit, limit).
DEVINL float clamp_swish(float g, float u, float limit) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
}

template <typename T>
__global__ void clamp_swish_mul_kernel(T* __restrict__ out, const T* __restrict__ in, long rows,
                                       int d, float limit) {
  const long total = rows * d;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / d;
    const int col = (int)(idx % d);
    const float g = to_f32(in[row * 2 * d + col]);
    const float u = to_f32(in[row * 2 * d + d + col]);
    out[idx] = from_f32<T>(clamp_swish(g, u, limit));
  }
}

// The same for bf16 rows a multiple of 8 wide: 16-byte accesses.
__global__ void clamp_swish_mul_vec_kernel(__hip_bfloat16* __restrict__ out,
                                           const __hip_bfloat16* __restrict__ in, long rows,
                                           int d, float limit) {
  const int per_row = d / 8;
  const long total = rows * per_row;
  for (long gi = blockIdx.x * (long)blockDim.x + threadIdx.x; gi < total;
       gi += (long)gridDim.x * blockDim.x) {
    const long row = gi / per_row;
    const int col = (int)(gi % per_row) * 8;
    const Vec8<__hip_bfloat16> gv = load16(in + row * 2 * d + col);
    const Vec8<__hip_bfloat16> uv = load16(in + row * 2 * d + d + col);
    Vec8<__hip_bfloat16> ov;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      ov.data[j] = __float2bfloat16(clamp_swish(to_f32(gv.data[j]), to_f32(uv.data[j]), limit));
    store16(out + row * d + col, ov);
  }
}

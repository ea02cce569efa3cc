// Kernels of looped hybrid decoders (gfx950) that sit between the vendor
// GEMMs: the rotary / norm / cache step of latent attention, the gated
// parallel residual join, the token-indexed side gate, the sigmoid top-k
// router and the matrix-vector form of an expert mixture.
//
// Numerics as in seqmix.hip: activations arrive in the model dtype T
// (bf16 or fp32); angles, norms, gates, router scores and the residual are
// fp32 in registers and rounded to T once, on store.

#include "common.h"

// ------------------------------------------------------ latent attention --
// Rotary positions on the first rot_dims channels of a vector x (n channels
// in all, the rest pass unchanged), channel j of the result. Pair i turns by
// angle pos * inv_freq[i]: (u, v) -> (u cos - v sin, v cos + u sin). Half
// layout: pair (i, i + rot_dims/2); interleaved: pair (2i, 2i + 1).
template <typename T>
DEVINL float rotary_channel(const T* __restrict__ x, int j, float pos,
                            const float* __restrict__ inv_freq, int rot_dims,
                            bool interleaved) {
  const float xj = to_f32(x[j]);
  if (j >= rot_dims) return xj;
  const int half = rot_dims >> 1;
  int i, partner;
  bool first;
  if (interleaved) {
    i = j >> 1;
    first = (j & 1) == 0;
    partner = first ? j + 1 : j - 1;
  } else {
    first = j < half;
    i = first ? j : j - half;
    partner = first ? j + half : j - half;
  }
  const float a = pos * inv_freq[i];
  const float c = cosf(a), s = sinf(a);
  const float xp = to_f32(x[partner]);
  return first ? xj * c - xp * s : xj * c + xp * s;
}

// Per token, between the projections and the attention kernel:
//   out[t, h, :R]  = q_lat[t, h, :]            (query mapped into the latent)
//   out[t, h, R:]  = rotary(q[t, h, dim:])     (rotated query part)
//   cache row      = rmsnorm(ckr[t, :R]) * c_w ‖ rotary(ckr[t, R:])
// The cache is [blocks, 1, block_size, R + DR]: one row per token, shared by
// all heads; a negative slot writes nothing (padding rows).
template <typename T>
__global__ __launch_bounds__(256) void latent_rope_pack_kernel(
    T* __restrict__ out,                       // [T, H, R+DR] contiguous
    const T* __restrict__ q, long q_s0, long q_s1,          // [T, H, dim+DR]
    const T* __restrict__ q_lat, long l_s0, long l_s1,      // [T, H, R]
    const T* __restrict__ ckr, long c_s0,                   // [T, R+DR]
    const T* __restrict__ c_w,                              // [R]
    const float* __restrict__ inv_freq,                     // [rot_dims/2]
    const long* __restrict__ positions, T* __restrict__ k_cache,
    const long* __restrict__ slots, int H, int dim, int DR, int R, int rot_dims,
    int interleaved, float eps) {
  __shared__ float red[4];
  const long tok = blockIdx.x;
  const float pos = (float)positions[tok];
  const int RW = R + DR;
  const T* cr = ckr + tok * c_s0;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const float f = to_f32(cr[i]);
    ss += f * f;
  }
  ss = block_reduce_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / R + eps);
  for (int idx = threadIdx.x; idx < H * RW; idx += blockDim.x) {
    const int h = idx / RW, c = idx % RW;
    float val;
    if (c < R) {
      val = to_f32(q_lat[tok * l_s0 + (long)h * l_s1 + c]);
    } else {
      val = rotary_channel(q + tok * q_s0 + (long)h * q_s1 + dim, c - R, pos, inv_freq,
                           rot_dims, interleaved != 0);
    }
    out[(tok * H + h) * RW + c] = from_f32<T>(val);
  }
  const long slot = slots[tok];
  if (slot < 0) return;
  T* row = k_cache + slot * RW;   // [blocks, 1, bs, RW]: slot = block * bs + offset
  for (int c = threadIdx.x; c < RW; c += blockDim.x) {
    float val;
    if (c < R) val = to_f32(cr[c]) * inv * to_f32(c_w[c]);
    else val = rotary_channel(cr + R, c - R, pos, inv_freq, rot_dims, interleaved != 0);
    row[c] = from_f32<T>(val);
  }
}

// ------------------------------------------------- gated parallel residual --
// res (fp32, in place) += sigmoid(g1 + b1) * y1 [+ sigmoid(g2 + b2) * y2];
// out = res rounded to T. y* are [rows, W] contiguous, g* row-strided slices
// of a wider projection output, b* fp32 [W].
template <typename T>
__global__ void gated_residual_add_kernel(
    T* __restrict__ out, float* __restrict__ res,
    const T* __restrict__ y1, const T* __restrict__ g1, long g1_stride,
    const float* __restrict__ b1,
    const T* __restrict__ y2, const T* __restrict__ g2, long g2_stride,
    const float* __restrict__ b2, long rows, int W) {
  const long total = rows * W;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / W;
    const int col = (int)(idx % W);
    const float z1 = to_f32(g1[row * g1_stride + col]) + b1[col];
    float add = to_f32(y1[idx]) / (1.0f + expf(-z1));
    if (y2) {
      const float z2 = to_f32(g2[row * g2_stride + col]) + b2[col];
      add += to_f32(y2[idx]) / (1.0f + expf(-z2));
    }
    const float r = res[idx] + add;
    res[idx] = r;
    out[idx] = from_f32<T>(r);
  }
}

// The same for bf16 rows a multiple of 8 wide with 16-byte-aligned gate
// slices: every operand crosses memory once, in 16-byte accesses.
__global__ void gated_residual_add_vec_kernel(
    __hip_bfloat16* __restrict__ out, float* __restrict__ res,
    const __hip_bfloat16* __restrict__ y1, const __hip_bfloat16* __restrict__ g1, long g1_stride,
    const float* __restrict__ b1,
    const __hip_bfloat16* __restrict__ y2, const __hip_bfloat16* __restrict__ g2, long g2_stride,
    const float* __restrict__ b2, long rows, int W) {
  const int per_row = W / 8;
  const long total = rows * per_row;
  for (long g = blockIdx.x * (long)blockDim.x + threadIdx.x; g < total;
       g += (long)gridDim.x * blockDim.x) {
    const long row = g / per_row;
    const int col = (int)(g % per_row) * 8;
    const long idx = row * W + col;
    const Vec8<__hip_bfloat16> yv = load16(y1 + idx);
    const Vec8<__hip_bfloat16> gv = load16(g1 + row * g1_stride + col);
    float r[8];
    const float4 ra = *reinterpret_cast<const float4*>(res + idx);
    const float4 rb = *reinterpret_cast<const float4*>(res + idx + 4);
    r[0] = ra.x; r[1] = ra.y; r[2] = ra.z; r[3] = ra.w;
    r[4] = rb.x; r[5] = rb.y; r[6] = rb.z; r[7] = rb.w;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float z = to_f32(gv.data[j]) + b1[col + j];
      r[j] += to_f32(yv.data[j]) / (1.0f + expf(-z));
    }
    if (y2) {
      const Vec8<__hip_bfloat16> yw = load16(y2 + idx);
      const Vec8<__hip_bfloat16> gw = load16(g2 + row * g2_stride + col);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float z = to_f32(gw.data[j]) + b2[col + j];
        r[j] += to_f32(yw.data[j]) / (1.0f + expf(-z));
      }
    }
    *reinterpret_cast<float4*>(res + idx) = make_float4(r[0], r[1], r[2], r[3]);
    *reinterpret_cast<float4*>(res + idx + 4) = make_float4(r[4], r[5], r[6], r[7]);
    Vec8<__hip_bfloat16> ov;
#pragma unroll
    for (int j = 0; j < 8; ++j) ov.data[j] = __float2bfloat16(r[j]);
    store16(out + idx, ov);
  }
}

// -------------------------------------------------------------- side gate --
// out[t, j] = gelu_tanh(a[t, j]) * table[tokens[t], offset + j]
template <typename T>
__global__ void side_gate_mul_kernel(T* __restrict__ out, const T* __restrict__ a,
                                     const T* __restrict__ table, long table_stride,
                                     const long* __restrict__ tokens, int offset, long rows,
                                     int d) {
  const long total = rows * d;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / d;
    const int col = (int)(idx % d);
    const float z = to_f32(a[idx]);
    const float c = 0.7978845608028654f;   // sqrt(2/pi)
    const float act = 0.5f * z * (1.0f + tanhf(c * (z + 0.044715f * z * z * z)));
    out[idx] = from_f32<T>(act * to_f32(table[tokens[row] * table_stride + offset + col]));
  }
}

// ----------------------------------------------------------------- router --
// Scores s = sigmoid(logits) in fp32; the `top` largest per token, largest
// first, ties to the lower expert index. One wave per token; a lane owns
// experts lane, lane + 64, ... (at most 64 * 32 experts).
__global__ __launch_bounds__(256) void sigmoid_topk_kernel(
    int* __restrict__ idx_out, float* __restrict__ w_out, const float* __restrict__ logits,
    long rows, int E, int top) {
  const int lane = threadIdx.x & 63;
  const long tok = blockIdx.x * 4L + (threadIdx.x >> 6);
  if (tok >= rows) return;
  const float* z = logits + tok * E;
  unsigned taken = 0u;   // bit n: expert lane + 64 n already chosen
  for (int k = 0; k < top; ++k) {
    float best = -1.f;
    int best_e = 0x7fffffff;
    for (int e = lane, n = 0; e < E; e += 64, ++n) {
      if (taken & (1u << n)) continue;
      float sc = 1.0f / (1.0f + expf(-z[e]));
      if (!(sc >= 0.f)) sc = -0.5f;   // a NaN logit still yields a valid index
      if (sc > best) {   // ascending e: the first of equal scores stays
        best = sc;
        best_e = e;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, WAVE);
      const int oe = __shfl_xor(best_e, off, WAVE);
      if (ob > best || (ob == best && oe < best_e)) {
        best = ob;
        best_e = oe;
      }
    }
    if ((best_e & 63) == lane) taken |= 1u << (best_e >> 6);
    if (lane == 0) {
      idx_out[tok * top + k] = best_e;
      w_out[tok * top + k] = best;
    }
  }
}

// --------------------------------------------- expert mixture, few rows ----
// Row r = (token t, choice k) uses expert e = idx[r] with input x = w[r] * h[t]
// rounded to T. Matrix-vector products read only the chosen experts'
// weights; accumulation is fp32, each product is rounded to T where a GEMM
// would round it.
//
// dot of a weight row with an fp32 vector in LDS, lanes striding the row in
// 16-byte granules when its length allows
template <typename T>
DEVINL float wave_dot(const T* __restrict__ wrow, const float* __restrict__ x, int n, int lane) {
  constexpr int VE = Vec8<T>::kElems;
  float acc = 0.f;
  if (n % VE == 0) {
    for (int i = lane * VE; i < n; i += 64 * VE) {
      const Vec8<T> v = load16(wrow + i);
#pragma unroll
      for (int j = 0; j < VE; ++j) acc += to_f32(v.data[j]) * x[i + j];
    }
  } else {
    for (int i = lane; i < n; i += 64) acc += to_f32(wrow[i]) * x[i];
  }
  return wave_reduce_sum(acc);
}

constexpr int kMoeRowsPerWave = 4;

// What an expert does between its two projections. Plain: silu(g) * u.
// Clamped: g = min(g, limit), u = clamp(u, +-limit), g * sigmoid(1.702 g) * (u + 1).
// Ungated experts (one projection, [E, F, W]): the exact GELU, or relu(.)^2.
constexpr int kMoeActSilu = 0;
constexpr int kMoeActClampSwish = 1;
constexpr int kMoeActGeluErf = 2;
constexpr int kMoeActRelu2 = 3;

DEVINL float moe_plain_act(float u, int act) {
  if (act == kMoeActRelu2) {
    const float r = fmaxf(u, 0.f);
    return r * r;
  }
  return 0.5f * u * (1.0f + erff(u * 0.70710678118654752f));
}

DEVINL float moe_gated_act(float g, float u, int act, float limit) {
  if (act == kMoeActClampSwish) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
  }
  return g / (1.0f + expf(-g)) * u;
}

// hmid[r, f] = act(gate_e[f] . x, up_e[f] . x);  gate_up [E, 2F, W]; a null w
// leaves the input unscaled (x = h[t]). Ungated activations: hmid[r, f] =
// act(up_e[f] . x) with gate_up [E, F, W].
template <typename T>
__global__ __launch_bounds__(256) void moe_gate_up_gemv_kernel(
    T* __restrict__ hmid, const T* __restrict__ h, const int* __restrict__ idx,
    const float* __restrict__ w, const T* __restrict__ gate_up, int top, int W, int F, int E,
    int act, float limit) {
  extern __shared__ float xs[];   // [W]
  const long r = blockIdx.y;
  const long t = r / top;
  const int e = min(max(idx[r], 0), E - 1);
  const float wr = w ? w[r] : 1.0f;
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    xs[i] = w ? to_f32(from_f32<T>(wr * to_f32(h[t * W + i]))) : to_f32(h[t * W + i]);
  __syncthreads();
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const bool gated = act < kMoeActGeluErf;
  const T* ge = gate_up + (long)e * (gated ? 2 : 1) * F * W;
  const int f0 = (blockIdx.x * 4 + wv) * kMoeRowsPerWave;
  for (int f = f0; f < min(F, f0 + kMoeRowsPerWave); ++f) {
    const float g = to_f32(from_f32<T>(wave_dot(ge + (long)f * W, xs, W, lane)));
    if (!gated) {
      if (lane == 0) hmid[r * F + f] = from_f32<T>(moe_plain_act(g, act));
      continue;
    }
    const float u = to_f32(from_f32<T>(wave_dot(ge + (long)(F + f) * W, xs, W, lane)));
    if (lane == 0) hmid[r * F + f] = from_f32<T>(moe_gated_act(g, u, act, limit));
  }
}

// y[t, c] = sum_k wo[t, k] * (down_{e(t,k)}[c] . hmid[t*top + k]);  down [E, W, F];
// a null wo weights every chosen expert's output with 1
template <typename T>
__global__ __launch_bounds__(256) void moe_down_gemv_kernel(
    T* __restrict__ y, const T* __restrict__ hmid, const int* __restrict__ idx,
    const T* __restrict__ down, int top, int W, int F, int E, const float* __restrict__ wo) {
  extern __shared__ float hs[];   // [top][F]
  const long t = blockIdx.y;
  for (int i = threadIdx.x; i < top * F; i += blockDim.x) hs[i] = to_f32(hmid[t * top * F + i]);
  __syncthreads();
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int c0 = (blockIdx.x * 4 + wv) * kMoeRowsPerWave;
  for (int c = c0; c < min(W, c0 + kMoeRowsPerWave); ++c) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const T* de = down + ((long)min(max(idx[t * top + k], 0), E - 1) * W + c) * F;
      const float dk = to_f32(from_f32<T>(wave_dot(de, hs + k * F, F, lane)));
      acc += wo ? wo[t * top + k] * dk : dk;
    }
    if (lane == 0) y[t * W + c] = from_f32<T>(acc);
  }
}

// --------------------------------- expert mixture, grouped by expert ------
// The sync-free form for decode batches: one workgroup per (expert, tile of
// output features) collects the rows routed to its expert from idx (in LDS,
// no host round trip, no sort) and runs them in chunks of kMoeTB rows, so a
// weight row is read once per chunk instead of once per row. Inputs of a
// chunk sit in LDS in the model dtype; accumulation is fp32.
//   GATE_UP: weight [E, 2F, K], x[r] = round(w[r] * h[r / top]) (h[r / top] when
//            w is null), out hmid[r, f] = act(gate_f . x, up_f . x)
//   else   : weight [E, N, K], x[r] = in[r], out[r, n] = weight_n . x
constexpr int kMoeTB = 8;        // rows per chunk
constexpr int kMoeFPW = 2;       // output features per wave and pass
constexpr int kMoeMaxRows = 2048;

template <typename T, bool GATE_UP>
__global__ __launch_bounds__(256) void moe_expert_gemv_kernel(
    T* __restrict__ out, const T* __restrict__ in, const int* __restrict__ idx,
    const float* __restrict__ w, const T* __restrict__ weight, int rows, int top, int K, int N,
    int act, float limit) {
  extern __shared__ __align__(16) unsigned char moe_smem[];
  __shared__ int count;
  int* list = reinterpret_cast<int*>(moe_smem);                 // [kMoeMaxRows]
  T* xs = reinterpret_cast<T*>(moe_smem + sizeof(int) * kMoeMaxRows);   // [kMoeTB][K]
  const int e = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  if (tid == 0) count = 0;
  __syncthreads();
  for (int r = tid; r < rows; r += 256)
    if (idx[r] == e) list[atomicAdd(&count, 1)] = r;
  __syncthreads();
  const int n = count;
  if (n == 0) return;
  constexpr int VE = Vec8<T>::kElems;
  const int n0 = (blockIdx.x * 4 + wv) * kMoeFPW;
  const T* we = weight + (long)e * (GATE_UP ? 2 : 1) * N * K;
  for (int c0 = 0; c0 < n; c0 += kMoeTB) {
    const int nt = min(kMoeTB, n - c0);
    __syncthreads();
    for (int i = tid; i < kMoeTB * K; i += 256) {
      const int tt = i / K, k = i % K;
      float v = 0.f;
      if (tt < nt) {
        const int r = list[c0 + tt];
        v = !GATE_UP ? to_f32(in[(long)r * K + k])
            : w ? to_f32(from_f32<T>(w[r] * to_f32(in[(long)(r / top) * K + k])))
                : to_f32(in[(long)(r / top) * K + k]);
      }
      xs[i] = from_f32<T>(v);
    }
    __syncthreads();
    for (int f = n0; f < min(N, n0 + kMoeFPW); ++f) {
      float a0[kMoeTB], a1[kMoeTB];
#pragma unroll
      for (int tt = 0; tt < kMoeTB; ++tt) a0[tt] = a1[tt] = 0.f;
      const T* r0 = we + (long)f * K;
      const T* r1 = we + (long)(N + f) * K;       // the up row (GATE_UP only)
      if (K % VE == 0) {
        for (int k = lane * VE; k < K; k += 64 * VE) {
          const Vec8<T> g8 = load16(r0 + k);
          Vec8<T> u8 = g8;
          if (GATE_UP) u8 = load16(r1 + k);
#pragma unroll
          for (int tt = 0; tt < kMoeTB; ++tt) {
            const Vec8<T> x8 = load16(xs + tt * K + k);
#pragma unroll
            for (int j = 0; j < VE; ++j) {
              const float xv = to_f32(x8.data[j]);
              a0[tt] += to_f32(g8.data[j]) * xv;
              if (GATE_UP) a1[tt] += to_f32(u8.data[j]) * xv;
            }
          }
        }
      } else {
        for (int k = lane; k < K; k += 64) {
          const float gv = to_f32(r0[k]);
          const float uv = GATE_UP ? to_f32(r1[k]) : 0.f;
#pragma unroll
          for (int tt = 0; tt < kMoeTB; ++tt) {
            const float xv = to_f32(xs[tt * K + k]);
            a0[tt] += gv * xv;
            if (GATE_UP) a1[tt] += uv * xv;
          }
        }
      }
#pragma unroll
      for (int tt = 0; tt < kMoeTB; ++tt) {
        a0[tt] = wave_reduce_sum(a0[tt]);
        if (GATE_UP) a1[tt] = wave_reduce_sum(a1[tt]);
      }
      if (lane < nt) {
        float g = 0.f, u = 0.f;
#pragma unroll
        for (int tt = 0; tt < kMoeTB; ++tt)
          if (tt == lane) {
            g = a0[tt];
            u = a1[tt];
          }
        const long r = list[c0 + lane];
        g = to_f32(from_f32<T>(g));
        if (GATE_UP) {
          u = to_f32(from_f32<T>(u));
          out[r * N + f] = from_f32<T>(moe_gated_act(g, u, act, limit));
        } else {
          out[r * N + f] = from_f32<T>(g);
        }
      }
    }
  }
}

// --------------------------------- expert mixture, every expert on every row --
// The join of the dense form (a batched GEMM pair that runs all E experts on
// all rows): y[t, :] = sum_e wd[t, e] * yk[e, t, :], fp32 accumulation. wd is
// the router's weights scattered into a dense [T, E] table, zero for experts
// a token did not choose; a null wd sums the experts' outputs as they are.
template <typename T>
__global__ void moe_combine_kernel(T* __restrict__ y, const T* __restrict__ yk,
                                   const float* __restrict__ wd, long rows, int W, int E) {
  const long total = rows * W;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long t = idx / W;
    float acc = 0.f;
    for (int e = 0; e < E; ++e) {
      const float v = to_f32(yk[(long)e * total + idx]);
      acc += wd ? wd[t * E + e] * v : v;
    }
    y[idx] = from_f32<T>(acc);
  }
}

// The join of the sorted form (rows grouped by expert, one GEMM pair per
// expert): y[t, :] = sum_k w[t, k] * ys[pos[t * top + k], :], where pos maps a
// (token, choice) pair to its row in the expert-sorted order; fp32
// accumulation; a null w sums the rows as they are.
template <typename T>
__global__ void moe_gather_combine_kernel(T* __restrict__ y, const T* __restrict__ ys,
                                          const long* __restrict__ pos,
                                          const float* __restrict__ w, long rows, int top, int W) {
  constexpr int VE = Vec8<T>::kElems;
  if (W % VE == 0) {
    const int per_row = W / VE;
    const long total = rows * per_row;
    for (long gi = blockIdx.x * (long)blockDim.x + threadIdx.x; gi < total;
         gi += (long)gridDim.x * blockDim.x) {
      const long t = gi / per_row;
      const int col = (int)(gi % per_row) * VE;
      float acc[VE];
#pragma unroll
      for (int j = 0; j < VE; ++j) acc[j] = 0.f;
      for (int k = 0; k < top; ++k) {
        const Vec8<T> v = load16(ys + pos[t * top + k] * W + col);
        const float wk = w ? w[t * top + k] : 1.0f;
#pragma unroll
        for (int j = 0; j < VE; ++j) acc[j] += wk * to_f32(v.data[j]);
      }
      Vec8<T> o;
#pragma unroll
      for (int j = 0; j < VE; ++j) o.data[j] = from_f32<T>(acc[j]);
      store16(y + t * W + col, o);
    }
    return;
  }
  const long total = rows * W;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long t = idx / W;
    const int col = (int)(idx % W);
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const float v = to_f32(ys[pos[t * top + k] * W + col]);
      acc += w ? w[t * top + k] * v : v;
    }
    y[idx] = from_f32<T>(acc);
  }
}

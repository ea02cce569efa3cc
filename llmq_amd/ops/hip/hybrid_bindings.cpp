// Torch bindings of the hybrid-decoder kernels: torch.ops.llmq_amd_hybrid.*
// Every launcher checks on the host that operand shapes match what the
// kernel and its grid assume before anything reaches the GPU.

#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>
#include <torch/library.h>

namespace {

#define HY_GPU(x) TORCH_CHECK(x.is_cuda(), #x " must be on GPU")
#define HY_INNER(x) TORCH_CHECK(x.stride(-1) == 1, #x ": innermost dim must be contiguous")
#define HY_I32(x) TORCH_CHECK(x.scalar_type() == at::kInt && x.is_contiguous(), #x " must be contiguous int32")

hipStream_t hy_stream() { return c10::hip::getCurrentHIPStream().stream(); }

template <typename F>
void hy_dispatch(const at::Tensor& t, const char* name, F&& f) {
  switch (t.scalar_type()) {
    case at::kBFloat16: f.template operator()<__hip_bfloat16>(); break;
    case at::kFloat: f.template operator()<float>(); break;
    default: TORCH_CHECK(false, name, ": unsupported dtype ", t.scalar_type());
  }
}

template <typename K>
void allow_lds(K kernel, size_t bytes) {
  TORCH_CHECK(bytes <= 160 * 1024, "kernel needs ", bytes, " B of LDS; the CU has 160 KB");
  if (bytes > 48 * 1024)
    C10_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
}

void rmsnorm_cast(at::Tensor out, at::Tensor in, at::Tensor weight, double eps, double offset,
                  int64_t groups_arg) {
  HY_GPU(in);
  // in: contiguous, or 2-D rows with a stride (a column slice of a wider matrix)
  TORCH_CHECK(out.is_contiguous() && weight.is_contiguous());
  TORCH_CHECK(in.is_contiguous() || (in.dim() == 2 && in.stride(1) == 1),
              "rmsnorm_cast: in must be contiguous or row-strided 2-D");
  const int width = in.size(-1);
  TORCH_CHECK(out.sizes() == in.sizes() && weight.numel() == width);
  TORCH_CHECK(weight.scalar_type() == out.scalar_type(), "weight dtype must equal out dtype");
  const int groups = (int)groups_arg;
  TORCH_CHECK(groups >= 1 && width % groups == 0, "groups must divide the row");
  // a row normed in groups is `groups` rows of width / groups to the kernel
  const int hidden = width / groups;
  const long rows = in.numel() / hidden;
  if (rows == 0) return;
  const long in_stride = in.is_contiguous() ? width : in.stride(0);
  hy_dispatch(out, "rmsnorm_cast", [&]<typename TO>() {
    if (in.scalar_type() == at::kFloat) {
      hipLaunchKernelGGL((rmsnorm_cast_kernel<float, TO>), dim3(rows), dim3(256), 0, hy_stream(),
                         reinterpret_cast<TO*>(out.data_ptr()), in.data_ptr<float>(), in_stride,
                         reinterpret_cast<const TO*>(weight.data_ptr()), hidden, (float)eps,
                         (float)offset, groups);
    } else {
      TORCH_CHECK(in.scalar_type() == out.scalar_type(), "rmsnorm_cast: in must be fp32 or out's dtype");
      hipLaunchKernelGGL((rmsnorm_cast_kernel<TO, TO>), dim3(rows), dim3(256), 0, hy_stream(),
                         reinterpret_cast<TO*>(out.data_ptr()),
                         reinterpret_cast<const TO*>(in.data_ptr()), in_stride,
                         reinterpret_cast<const TO*>(weight.data_ptr()), hidden, (float)eps,
                         (float)offset, groups);
    }
  });
}

void sandwich_norm_res32(at::Tensor x, at::Tensor residual, at::Tensor w_post, at::Tensor w_pre,
                         double eps, double offset, int64_t groups_arg) {
  HY_GPU(x);
  TORCH_CHECK(x.is_contiguous() && residual.is_contiguous());
  TORCH_CHECK(residual.scalar_type() == at::kFloat, "residual must be fp32");
  const int width = x.size(-1);
  TORCH_CHECK(residual.sizes() == x.sizes() && w_post.numel() == width && w_pre.numel() == width);
  TORCH_CHECK(w_post.scalar_type() == x.scalar_type() && w_pre.scalar_type() == x.scalar_type());
  TORCH_CHECK(w_post.is_contiguous() && w_pre.is_contiguous());
  const int groups = (int)groups_arg;
  TORCH_CHECK(groups >= 1 && width % groups == 0, "groups must divide the row");
  const int hidden = width / groups;
  const long rows = x.numel() / hidden;
  if (rows == 0) return;
  if (x.scalar_type() == at::kBFloat16 && hidden % 8 == 0 && hidden <= 4 * 2048) {
    using bf = __hip_bfloat16;
    auto launch = [&]<int CH, bool PER_WAVE>() {
      const long blocks = PER_WAVE ? (rows + 3) / 4 : rows;
      hipLaunchKernelGGL((sandwich_norm_res32_vec_kernel<CH, PER_WAVE>), dim3(blocks), dim3(256), 0,
                         hy_stream(), reinterpret_cast<bf*>(x.data_ptr()), residual.data_ptr<float>(),
                         reinterpret_cast<const bf*>(w_post.data_ptr()),
                         reinterpret_cast<const bf*>(w_pre.data_ptr()), hidden, (float)eps,
                         (float)offset, groups, rows);
    };
    // short rows (and the parts of rows normed in groups): a wave per row
    if (hidden <= 512) launch.template operator()<1, true>();
    else if (hidden <= 1024) launch.template operator()<2, true>();
    else if (hidden <= 2048) launch.template operator()<1, false>();
    else if (hidden <= 4096) launch.template operator()<2, false>();
    else launch.template operator()<4, false>();
    return;
  }
  hy_dispatch(x, "sandwich_norm_res32", [&]<typename T>() {
    hipLaunchKernelGGL(sandwich_norm_res32_kernel<T>, dim3(rows), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(x.data_ptr()), residual.data_ptr<float>(),
                       reinterpret_cast<const T*>(w_post.data_ptr()),
                       reinterpret_cast<const T*>(w_pre.data_ptr()), hidden, (float)eps,
                       (float)offset, groups);
  });
}

void act_and_mul(at::Tensor out, at::Tensor in, bool gelu) {
  HY_GPU(in);
  TORCH_CHECK(in.is_contiguous() && out.is_contiguous() && in.scalar_type() == out.scalar_type());
  const int d = out.size(-1);
  TORCH_CHECK(in.size(-1) == 2 * d, "in must be [..., 2*d]");
  const long rows = out.numel() / d;
  if (rows == 0) return;
  hy_dispatch(in, "act_and_mul", [&]<typename T>() {
    constexpr int VE = Vec8<T>::kElems;
    auto launch = [&]<bool G>() {
      if (d % VE == 0) {
        const long chunks = rows * (d / VE);
        const int grid = (int)std::min<long>((chunks + 255) / 256, 2048);
        hipLaunchKernelGGL((act_and_mul_kernel<T, G>), dim3(grid), dim3(256), 0, hy_stream(),
                           reinterpret_cast<T*>(out.data_ptr()),
                           reinterpret_cast<const T*>(in.data_ptr()), rows, d);
      } else {
        const int grid = (int)std::min<long>((rows * d + 255) / 256, 4096);
        hipLaunchKernelGGL((act_and_mul_scalar_kernel<T, G>), dim3(grid), dim3(256), 0,
                           hy_stream(), reinterpret_cast<T*>(out.data_ptr()),
                           reinterpret_cast<const T*>(in.data_ptr()), rows, d);
      }
    };
    if (gelu) launch.template operator()<true>();
    else launch.template operator()<false>();
  });
}

// q [T, nq], k [T, nk], v [T, nv]: row-strided views of one GEMM output.
void qknorm_vmix_cache(at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor q_w, at::Tensor k_w,
                       const std::optional<at::Tensor>& v_first, double lam, at::Tensor k_cache,
                       at::Tensor v_cache, at::Tensor slots, double eps) {
  HY_GPU(q);
  HY_INNER(q); HY_INNER(k); HY_INNER(v);
  TORCH_CHECK(q.dim() == 2 && k.dim() == 2 && v.dim() == 2);
  const long T_ = q.size(0);
  if (T_ == 0) return;
  TORCH_CHECK(k.size(0) == T_ && v.size(0) == T_ && slots.numel() == T_);
  TORCH_CHECK(slots.scalar_type() == at::kLong && slots.is_contiguous());
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.is_contiguous() && v_cache.is_contiguous());
  const int G = k_cache.size(1), bs = k_cache.size(2), D = k_cache.size(3), DV = v_cache.size(3);
  TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == G && v_cache.size(2) == bs);
  const int nq = q.size(1), nk = k.size(1), nv = v.size(1);
  TORCH_CHECK(nk == G * D && nv == G * DV, "k/v widths do not match the cache layout");
  TORCH_CHECK(q_w.numel() == nq && k_w.numel() == nk && q_w.is_contiguous() && k_w.is_contiguous());
  const auto dt = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == dt && v.scalar_type() == dt && q_w.scalar_type() == dt &&
              k_w.scalar_type() == dt && k_cache.scalar_type() == dt && v_cache.scalar_type() == dt,
              "qknorm_vmix_cache: one dtype for activations, weights and cache");
  const void* vf = nullptr;
  long vf_stride = 0;
  if (v_first.has_value()) {
    const at::Tensor& f = *v_first;
    TORCH_CHECK(f.dim() == 2 && f.size(0) == T_ && f.size(1) == nv && f.stride(1) == 1 &&
                f.scalar_type() == dt, "v_first must be [T, nv] of the same dtype");
    vf = f.data_ptr();
    vf_stride = f.stride(0);
  }
  hy_dispatch(q, "qknorm_vmix_cache", [&]<typename T>() {
    hipLaunchKernelGGL(qknorm_vmix_cache_kernel<T>, dim3(T_), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(q.data_ptr()), q.stride(0), nq,
                       reinterpret_cast<const T*>(k.data_ptr()), k.stride(0), nk,
                       reinterpret_cast<const T*>(v.data_ptr()), v.stride(0), nv,
                       reinterpret_cast<const T*>(q_w.data_ptr()),
                       reinterpret_cast<const T*>(k_w.data_ptr()),
                       reinterpret_cast<const T*>(vf), vf_stride, (float)lam,
                       reinterpret_cast<T*>(k_cache.data_ptr()),
                       reinterpret_cast<T*>(v_cache.data_ptr()), slots.data_ptr<long>(), G, D, DV,
                       bs, (float)eps);
  });
}

// v_row: value row stride in elements (DV for a value cache of its own, D
// when values are the first DV channels of the key rows); vptr: where they sit
struct AttnDims { int H, G, D, DV, bs, v_row; const void* vptr; const float* bias; int bias_len; };

AttnDims attn_check(const at::Tensor& out, const at::Tensor& q, const std::optional<at::Tensor>& gate,
                    const at::Tensor& k_cache, const std::optional<at::Tensor>& v_cache,
                    const std::optional<at::Tensor>& bias, const at::Tensor& block_tables,
                    long span, long mask_mode, long bias_mode) {
  HY_GPU(q);
  TORCH_CHECK(q.dim() == 3 && out.dim() == 3, "q [T, H, D], out [T, H, DV]");
  HY_INNER(q); HY_INNER(out);
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.is_contiguous());
  AttnDims a{(int)q.size(1), (int)k_cache.size(1), (int)q.size(2), (int)out.size(2),
             (int)k_cache.size(2), 0, nullptr, nullptr, 1};
  TORCH_CHECK(mask_mode == kMaskBlock || mask_mode == kMaskWindow, "unknown mask mode");
  TORCH_CHECK(q.stride(1) == a.D && out.stride(1) == a.DV, "heads must be packed");
  TORCH_CHECK(k_cache.size(3) == a.D, "query and key sizes differ");
  if (v_cache.has_value()) {
    TORCH_CHECK(v_cache->dim() == 4 && v_cache->is_contiguous() && v_cache->size(0) == k_cache.size(0) &&
                v_cache->size(1) == a.G && v_cache->size(2) == a.bs && v_cache->size(3) == a.DV &&
                v_cache->scalar_type() == q.scalar_type(), "value cache does not match");
    a.v_row = a.DV;
    a.vptr = v_cache->data_ptr();
  } else {
    TORCH_CHECK(a.DV <= a.D, "values read from key rows cannot be wider than the rows");
    a.v_row = a.D;
    a.vptr = k_cache.data_ptr();
  }
  TORCH_CHECK(out.size(0) == q.size(0) && out.size(1) == a.H);
  TORCH_CHECK(a.H % a.G == 0, "heads must be a multiple of kv heads");
  TORCH_CHECK(a.DV >= 1 && a.DV <= 512, "value size above 512 is not supported");
  TORCH_CHECK(span >= 1);
  TORCH_CHECK(bias_mode == kBiasTable || bias_mode == kBiasLog, "unknown bias mode");
  if (bias.has_value()) {
    TORCH_CHECK(bias->scalar_type() == at::kFloat && bias->is_contiguous() && bias->dim() == 2 &&
                bias->size(0) == a.H && bias->is_cuda(), "bias must be fp32 [H, n] on the GPU");
    TORCH_CHECK(bias_mode == kBiasLog ? bias->size(1) == 2
                                      : bias->size(1) >= 1 && bias->size(1) <= span,
                "bias is [H, 2] = (r1, r2) per head in log mode, else [H, n] with "
                "n = min(span, longest context the engine admits)");
    a.bias = bias->data_ptr<float>();
    a.bias_len = (int)bias->size(1);
  }
  TORCH_CHECK(q.scalar_type() == out.scalar_type() && q.scalar_type() == k_cache.scalar_type());
  HY_I32(block_tables);
  TORCH_CHECK(block_tables.dim() == 2);
  if (gate.has_value()) {
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == q.size(0) && gate->size(1) == a.H &&
                gate->stride(1) == 1 && gate->scalar_type() == q.scalar_type(), "gate must be [T, H]");
  }
  return a;
}

// the learned softmax term per query head: fp32 [H], or none
const float* sink_check(const std::optional<at::Tensor>& sink, const at::Tensor& q) {
  if (!sink.has_value()) return nullptr;
  TORCH_CHECK(sink->is_cuda() && sink->scalar_type() == at::kFloat && sink->is_contiguous() &&
              sink->numel() == q.size(1), "sink must be fp32 [H] on the GPU");
  return sink->data_ptr<float>();
}

template <typename F>
void dispatch_nv(int DV, F&& f) {
  if (DV <= 64) f.template operator()<1>();
  else if (DV <= 128) f.template operator()<2>();
  else if (DV <= 256) f.template operator()<4>();
  else f.template operator()<8>();
}

void paged_attn_prefill(at::Tensor out, at::Tensor q, const std::optional<at::Tensor>& gate,
                        at::Tensor k_cache, const std::optional<at::Tensor>& v_cache,
                        const std::optional<at::Tensor>& bias, at::Tensor block_tables,
                        at::Tensor cu_q, at::Tensor q_start, int64_t max_q, int64_t span,
                        double scale, int64_t mask_mode, int64_t pos_stride, int64_t bias_mode,
                        int64_t keep_first, const std::optional<at::Tensor>& sink, double softcap) {
  if (q.size(0) == 0) return;
  const float* sink_ptr = sink_check(sink, q);
  TORCH_CHECK(keep_first >= 0 && softcap >= 0.0);
  TORCH_CHECK(keep_first == 0 || mask_mode == kMaskWindow, "kept first tokens go with the window mask");
  TORCH_CHECK(pos_stride == 1 || (keep_first == 0 && !sink_ptr),
              "rows that share a position take no kept tokens and no sink");
  TORCH_CHECK(pos_stride == 0 || pos_stride == 1, "pos_stride is 0 (rows share a position) or 1");
  const AttnDims a = attn_check(out, q, gate, k_cache, v_cache, bias, block_tables, span, mask_mode,
                                bias_mode);
  HY_I32(cu_q); HY_I32(q_start);
  const int B = q_start.numel();
  TORCH_CHECK(cu_q.numel() == B + 1 && block_tables.size(0) == B && max_q >= 1);
  // bf16 with 16-byte-aligned q rows and key rows: the matrix-core kernel
  // (LLMQ_HYBRID_ATTN_VALU=1 keeps the fp32-ALU kernel, for A/B runs)
  static const bool force_valu = [] {
    const char* e = getenv("LLMQ_HYBRID_ATTN_VALU");
    return e && e[0] == '1';
  }();
  TORCH_CHECK(pos_stride == 1 || (q.scalar_type() == at::kBFloat16 && a.D % 8 == 0 && a.D <= 256 &&
                                  q.stride(0) % 8 == 0 && !gate.has_value()),
              "rows that share a position run on the matrix-core kernel only");
  if (q.scalar_type() == at::kBFloat16 && (!force_valu || pos_stride == 0) && a.D % 8 == 0 && a.D <= 256 &&
      a.DV <= 256 &&   // 16 channel tiles of 16 per wave; wider values run on the fp32 ALUs
      q.stride(0) % 8 == 0 && reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0) {
    const int ksn = (a.D + 31) / 32, dtn = (a.DV + 15) / 16;
    // rows that share a position (single tokens): a sequence is one
    // workgroup per 64 heads, so its keys are split over several until the
    // grid has about two workgroups per CU; the partials are merged below
    int n_split = 1;
    at::Tensor part;
    if (pos_stride == 0) {
      const long wgs = (long)((max_q + kMfmaQT - 1) / kMfmaQT) * a.H * B;
      const long max_tiles = std::max<long>(1, block_tables.size(1) * (long)a.bs / kMfmaKT);
      n_split = (int)std::min<long>(std::min<long>(8, max_tiles), std::max<long>(1, 512 / wgs));
      if (n_split > 1)
        part = at::empty({q.size(0), a.H, n_split, a.DV + 2}, q.options().dtype(at::kFloat));
    }
    const dim3 grid((max_q + kMfmaQT - 1) / kMfmaQT, a.H * n_split, B);
    using bf = __hip_bfloat16;
    auto launch = [&]<int KS, int DT>() {
      // K tile, V^T tile (the channel tiles in use), P hi/lo per wave, bias slice
      const size_t lds = sizeof(short) * ((size_t)kMfmaKT * (ksn * 32 + 8) +
                                          (size_t)dtn * 16 * kMfmaKP +
                                          (size_t)4 * 2 * 16 * kMfmaKP) + 128 * sizeof(float);
      auto kern = chunk_bias_attn_prefill_mfma_kernel<KS, DT>;
      allow_lds(kern, lds);
      hipLaunchKernelGGL(kern, grid, dim3(256), lds, hy_stream(),
                         reinterpret_cast<bf*>(out.data_ptr()), out.stride(0),
                         reinterpret_cast<const bf*>(q.data_ptr()), q.stride(0),
                         gate.has_value() ? reinterpret_cast<const bf*>(gate->data_ptr()) : nullptr,
                         gate.has_value() ? gate->stride(0) : 0L,
                         reinterpret_cast<const bf*>(k_cache.data_ptr()),
                         reinterpret_cast<const bf*>(a.vptr), a.bias, a.bias_len,
                         block_tables.data_ptr<int>(), (int)block_tables.stride(0),
                         cu_q.data_ptr<int>(), q_start.data_ptr<int>(), a.H, a.G, a.D, a.DV, a.bs,
                         (int)span, (float)scale, a.v_row, (int)mask_mode, (int)pos_stride,
                         n_split, n_split > 1 ? part.data_ptr<float>() : nullptr, (int)bias_mode,
                         (int)keep_first, sink_ptr, (float)softcap);
    };
    if (ksn <= 2 && dtn <= 4) launch.template operator()<2, 4>();
    else if (ksn <= 4 && dtn <= 8) launch.template operator()<4, 8>();
    else launch.template operator()<8, 16>();
    if (n_split > 1) {
      const long pairs = q.size(0) * (long)a.H;
      hipLaunchKernelGGL(attn_merge_splits_kernel, dim3((pairs + 3) / 4), dim3(256), 0, hy_stream(),
                         reinterpret_cast<bf*>(out.data_ptr()), out.stride(0),
                         part.data_ptr<float>(), pairs, a.H, a.DV, n_split);
    }
    return;
  }
  const bool alias = a.vptr == k_cache.data_ptr();
  const size_t lds = sizeof(float) * ((size_t)kAttnKT * (a.D + 1) +
                                      (alias ? 0 : (size_t)kAttnKT * a.DV) +
                                      (size_t)kAttnQT * a.D + (size_t)kAttnQT * kAttnKT);
  const dim3 grid((max_q + kAttnQT - 1) / kAttnQT, a.H, B);
  hy_dispatch(q, "chunk_bias_attn_prefill", [&]<typename T>() {
    dispatch_nv(a.DV, [&]<int NV>() {
      auto kern = chunk_bias_attn_prefill_kernel<T, NV>;
      allow_lds(kern, lds);
      hipLaunchKernelGGL(kern, grid, dim3(256), lds, hy_stream(),
                         reinterpret_cast<T*>(out.data_ptr()), out.stride(0),
                         reinterpret_cast<const T*>(q.data_ptr()), q.stride(0),
                         gate.has_value() ? reinterpret_cast<const T*>(gate->data_ptr()) : nullptr,
                         gate.has_value() ? gate->stride(0) : 0L,
                         reinterpret_cast<const T*>(k_cache.data_ptr()),
                         reinterpret_cast<const T*>(a.vptr), a.bias, a.bias_len,
                         block_tables.data_ptr<int>(), (int)block_tables.stride(0),
                         cu_q.data_ptr<int>(), q_start.data_ptr<int>(), a.H, a.G, a.D, a.DV, a.bs,
                         (int)span, (float)scale, a.v_row, (int)mask_mode, (int)bias_mode,
                         (int)keep_first, sink_ptr, (float)softcap);
    });
  });
}

void paged_attn_decode(at::Tensor out, at::Tensor q, const std::optional<at::Tensor>& gate,
                       at::Tensor k_cache, const std::optional<at::Tensor>& v_cache,
                       const std::optional<at::Tensor>& bias, at::Tensor block_tables,
                       at::Tensor context_lens, int64_t span, double scale, int64_t mask_mode,
                       int64_t bias_mode, int64_t keep_first, const std::optional<at::Tensor>& sink,
                       double softcap) {
  if (q.size(0) == 0) return;
  const float* sink_ptr = sink_check(sink, q);
  TORCH_CHECK(keep_first >= 0 && softcap >= 0.0);
  TORCH_CHECK(keep_first == 0 || mask_mode == kMaskWindow, "kept first tokens go with the window mask");
  const AttnDims a = attn_check(out, q, gate, k_cache, v_cache, bias, block_tables, span, mask_mode,
                                bias_mode);
  HY_I32(context_lens);
  const int B = q.size(0);
  TORCH_CHECK(context_lens.numel() == B && block_tables.size(0) == B);
  // query heads per workgroup: as many of one kv head's as divide evenly
  const int per_kv = a.H / a.G;
  int hpw = per_kv % 8 == 0 ? 8 : per_kv % 4 == 0 ? 4 : per_kv % 3 == 0 ? 3 : per_kv % 2 == 0 ? 2 : 1;
  auto lds_for = [&](int n) {
    return sizeof(float) * ((size_t)n * ((a.D + 3) & ~3) + 2 * kDecWaves * n +
                            (size_t)kDecWaves * n * a.DV);
  };
  while (hpw > 1 && lds_for(hpw) > 150 * 1024) hpw = hpw == 3 ? 1 : hpw / 2;   // wide heads: fewer per workgroup
  const size_t lds = lds_for(hpw);
  hy_dispatch(q, "paged_attn_decode", [&]<typename T>() {
    dispatch_nv(a.DV, [&]<int NV>() {
      auto launch = [&]<int HPW>() {
      auto kern = chunk_bias_attn_decode_kernel<T, NV, HPW>;
      allow_lds(kern, lds);
      hipLaunchKernelGGL(kern, dim3(a.H / HPW, B), dim3(64 * kDecWaves), lds, hy_stream(),
                         reinterpret_cast<T*>(out.data_ptr()), out.stride(0),
                         reinterpret_cast<const T*>(q.data_ptr()), q.stride(0),
                         gate.has_value() ? reinterpret_cast<const T*>(gate->data_ptr()) : nullptr,
                         gate.has_value() ? gate->stride(0) : 0L,
                         reinterpret_cast<const T*>(k_cache.data_ptr()),
                         reinterpret_cast<const T*>(a.vptr), a.bias, a.bias_len,
                         block_tables.data_ptr<int>(), (int)block_tables.stride(0),
                         context_lens.data_ptr<int>(), a.H, a.G, a.D, a.DV, a.bs, (int)span,
                         (float)scale, a.v_row, (int)mask_mode, (int)bias_mode, (int)keep_first,
                         sink_ptr, (float)softcap);
      };
      if (hpw == 8) launch.template operator()<8>();
      else if (hpw == 4) launch.template operator()<4>();
      else if (hpw == 3) launch.template operator()<3>();
      else if (hpw == 2) launch.template operator()<2>();
      else launch.template operator()<1>();
    });
  });
}

// q, k, z: [T, H, D]; v: [T, H, DV] (row-strided views); o: [T, H, DV] fp32;
// state: [slots, H, D, DV] fp32.
// lower given: the HGRN2 form (no key); q_silu: SiLU on q inside the kernel.
void gla_recurrence(at::Tensor o, at::Tensor q, const std::optional<at::Tensor>& k_opt,
                    at::Tensor v, at::Tensor z, at::Tensor z_bias, at::Tensor state, at::Tensor cu,
                    at::Tensor slots, at::Tensor fresh, double tau,
                    const std::optional<at::Tensor>& lower, bool q_silu, double q_scale_arg) {
  HY_GPU(q);
  const long T_ = q.size(0);
  if (T_ == 0) return;
  TORCH_CHECK(k_opt.has_value() != lower.has_value(),
              "a key (gated linear attention) or a lower bound (HGRN2), not both");
  const at::Tensor& k = k_opt.has_value() ? *k_opt : q;   // q stands in for shape checks
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3 && z.dim() == 3 && o.dim() == 3);
  HY_INNER(q); HY_INNER(k); HY_INNER(v); HY_INNER(z);
  const int H = q.size(1), D = q.size(2), DV = v.size(2);
  TORCH_CHECK(k.sizes() == q.sizes() && z.sizes() == q.sizes());
  TORCH_CHECK(v.size(0) == T_ && v.size(1) == H);
  TORCH_CHECK(q.stride(1) == D && k.stride(1) == D && z.stride(1) == D && v.stride(1) == DV,
              "heads must be packed");
  const float* lower_ptr = nullptr;
  if (lower.has_value()) {
    TORCH_CHECK(lower->scalar_type() == at::kFloat && lower->is_contiguous() &&
                lower->numel() == (long)H * D && lower->is_cuda(), "lower must be fp32 [H*D]");
    lower_ptr = lower->data_ptr<float>();
  }
  TORCH_CHECK(o.scalar_type() == at::kFloat && o.is_contiguous() && o.size(0) == T_ &&
              o.size(1) == H && o.size(2) == DV);
  TORCH_CHECK(state.scalar_type() == at::kFloat && state.is_contiguous() && state.dim() == 4 &&
              state.size(1) == H && state.size(2) == D && state.size(3) == DV, "state [slots, H, D, DV] fp32");
  TORCH_CHECK(z_bias.scalar_type() == at::kFloat && z_bias.is_contiguous() && z_bias.numel() == (long)H * D);
  HY_I32(cu); HY_I32(slots); HY_I32(fresh);
  const int B = slots.numel();
  TORCH_CHECK(cu.numel() == B + 1 && fresh.numel() == B);
  TORCH_CHECK(D <= 256, "key size above 256 is not supported");
  TORCH_CHECK(tau > 0);
  const auto dt = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == dt && v.scalar_type() == dt && z.scalar_type() == dt);
  const dim3 grid((DV + kGlaCols - 1) / kGlaCols, H, B);
  const float q_scale = (float)q_scale_arg;
  const bool has_k = k_opt.has_value();
  hy_dispatch(q, "gla_recurrence", [&]<typename T>() {
    auto launch = [&]<int DPL>() {
      hipLaunchKernelGGL((gla_recurrence_kernel<T, DPL>), grid, dim3(256), 0, hy_stream(),
                         o.data_ptr<float>(),
                         reinterpret_cast<const T*>(q.data_ptr()), q.stride(0),
                         has_k ? reinterpret_cast<const T*>(k.data_ptr()) : nullptr, k.stride(0),
                         reinterpret_cast<const T*>(v.data_ptr()), v.stride(0),
                         reinterpret_cast<const T*>(z.data_ptr()), z.stride(0),
                         z_bias.data_ptr<float>(), state.data_ptr<float>(), cu.data_ptr<int>(),
                         slots.data_ptr<int>(), fresh.data_ptr<int>(), H, D, DV,
                         (float)(1.0 / tau), q_scale, lower_ptr, (int)q_silu,
                         static_cast<const float*>(nullptr), static_cast<const float*>(nullptr), 0);
    };
    if (D <= 32) launch.template operator()<2>();
    else if (D <= 64) launch.template operator()<4>();
    else if (D <= 128) launch.template operator()<8>();
    else launch.template operator()<16>();
  });
}

void gla_out_norm_gate(at::Tensor out, at::Tensor o, at::Tensor weight,
                       const std::optional<at::Tensor>& gate_opt, double eps) {
  HY_GPU(o);
  TORCH_CHECK(o.dim() == 3 && o.scalar_type() == at::kFloat && o.is_contiguous());
  const long T_ = o.size(0);
  if (T_ == 0) return;
  const int H = o.size(1), DV = o.size(2);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T_ && out.size(1) == (long)H * DV && out.stride(1) == 1);
  const void* gate_ptr = nullptr;
  long gate_stride = 0;
  if (gate_opt.has_value()) {
    const at::Tensor& gate = *gate_opt;
    TORCH_CHECK(gate.dim() == 2 && gate.size(0) == T_ && gate.size(1) == (long)H * DV &&
                gate.stride(1) == 1 && gate.scalar_type() == out.scalar_type());
    gate_ptr = gate.data_ptr();
    gate_stride = gate.stride(0);
  }
  TORCH_CHECK(weight.numel() == DV && weight.is_contiguous());
  TORCH_CHECK(weight.scalar_type() == out.scalar_type());
  hy_dispatch(out, "gla_out_norm_gate", [&]<typename T>() {
    hipLaunchKernelGGL(gla_out_norm_gate_kernel<T>, dim3(T_), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(out.data_ptr()), out.stride(0), o.data_ptr<float>(),
                       reinterpret_cast<const T*>(weight.data_ptr()),
                       reinterpret_cast<const T*>(gate_ptr), gate_stride, H, DV, (float)eps);
  });
}

// ---- latent attention: rotary + latent norm + packed query + cache scatter
void latent_rope_pack(at::Tensor out, at::Tensor q, at::Tensor q_lat, at::Tensor ckr,
                      at::Tensor c_w, at::Tensor inv_freq, at::Tensor positions,
                      at::Tensor k_cache, at::Tensor slots, int64_t dim, int64_t rot_dims,
                      bool interleaved, double eps) {
  HY_GPU(q);
  const long T_ = q.size(0);
  if (T_ == 0) return;
  TORCH_CHECK(q.dim() == 3 && q_lat.dim() == 3 && ckr.dim() == 2 && out.dim() == 3);
  HY_INNER(q); HY_INNER(q_lat); HY_INNER(ckr);
  const int H = q.size(1), R = q_lat.size(2);
  const int DR = (int)q.size(2) - (int)dim;
  TORCH_CHECK(dim >= 0 && DR >= 1, "q must be [T, H, dim + rot part]");
  TORCH_CHECK(q_lat.size(0) == T_ && q_lat.size(1) == H && ckr.size(0) == T_ && ckr.size(1) == R + DR);
  TORCH_CHECK(out.is_contiguous() && out.size(0) == T_ && out.size(1) == H && out.size(2) == R + DR);
  TORCH_CHECK(rot_dims >= 2 && rot_dims % 2 == 0 && rot_dims <= DR, "rot_dims must be even, at most the rotated part");
  TORCH_CHECK(inv_freq.scalar_type() == at::kFloat && inv_freq.is_contiguous() &&
              inv_freq.numel() == rot_dims / 2 && inv_freq.is_cuda());
  TORCH_CHECK(c_w.numel() == R && c_w.is_contiguous());
  TORCH_CHECK(positions.scalar_type() == at::kLong && positions.is_contiguous() && positions.numel() == T_);
  TORCH_CHECK(slots.scalar_type() == at::kLong && slots.is_contiguous() && slots.numel() == T_);
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.is_contiguous() && k_cache.size(1) == 1 &&
              k_cache.size(3) == R + DR, "latent cache must be [blocks, 1, block, R + rot part]");
  const auto dt = q.scalar_type();
  TORCH_CHECK(q_lat.scalar_type() == dt && ckr.scalar_type() == dt && c_w.scalar_type() == dt &&
              out.scalar_type() == dt && k_cache.scalar_type() == dt,
              "latent_rope_pack: one dtype for activations, weights and cache");
  hy_dispatch(q, "latent_rope_pack", [&]<typename T>() {
    hipLaunchKernelGGL(latent_rope_pack_kernel<T>, dim3(T_), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(out.data_ptr()),
                       reinterpret_cast<const T*>(q.data_ptr()), q.stride(0), q.stride(1),
                       reinterpret_cast<const T*>(q_lat.data_ptr()), q_lat.stride(0), q_lat.stride(1),
                       reinterpret_cast<const T*>(ckr.data_ptr()), ckr.stride(0),
                       reinterpret_cast<const T*>(c_w.data_ptr()), inv_freq.data_ptr<float>(),
                       positions.data_ptr<long>(), reinterpret_cast<T*>(k_cache.data_ptr()),
                       slots.data_ptr<long>(), H, (int)dim, DR, R, (int)rot_dims,
                       (int)interleaved, (float)eps);
  });
}

// ---- gated parallel residual join
void gated_residual_add(at::Tensor out, at::Tensor res, at::Tensor y1, at::Tensor g1, at::Tensor b1,
                        const std::optional<at::Tensor>& y2, const std::optional<at::Tensor>& g2,
                        const std::optional<at::Tensor>& b2) {
  HY_GPU(res);
  TORCH_CHECK(res.dim() == 2 && res.is_contiguous() && res.scalar_type() == at::kFloat, "res must be fp32 [rows, W]");
  const long rows = res.size(0);
  const int W = res.size(1);
  if (rows == 0) return;
  auto check_pair = [&](const at::Tensor& y, const at::Tensor& g, const at::Tensor& b) {
    TORCH_CHECK(y.is_contiguous() && y.sizes() == res.sizes() && y.scalar_type() == out.scalar_type());
    TORCH_CHECK(g.dim() == 2 && g.size(0) == rows && g.size(1) == W && g.stride(1) == 1 &&
                g.scalar_type() == out.scalar_type());
    TORCH_CHECK(b.scalar_type() == at::kFloat && b.is_contiguous() && b.numel() == W && b.is_cuda());
  };
  TORCH_CHECK(out.is_contiguous() && out.sizes() == res.sizes());
  check_pair(y1, g1, b1);
  const bool two = y2.has_value();
  TORCH_CHECK(g2.has_value() == two && b2.has_value() == two, "second sublayer needs y, g and b");
  if (two) check_pair(*y2, *g2, *b2);
  const long g2s = two ? g2->stride(0) : 0;
  auto aligned = [](const at::Tensor& t) {
    return reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0 && t.stride(0) % 8 == 0;
  };
  if (out.scalar_type() == at::kBFloat16 && W % 8 == 0 && aligned(g1) && (!two || aligned(*g2))) {
    using bf = __hip_bfloat16;
    const int grid = (int)std::min<long>((rows * (W / 8) + 255) / 256, 4096);
    hipLaunchKernelGGL(gated_residual_add_vec_kernel, dim3(grid), dim3(256), 0, hy_stream(),
                       reinterpret_cast<bf*>(out.data_ptr()), res.data_ptr<float>(),
                       reinterpret_cast<const bf*>(y1.data_ptr()),
                       reinterpret_cast<const bf*>(g1.data_ptr()), g1.stride(0), b1.data_ptr<float>(),
                       two ? reinterpret_cast<const bf*>(y2->data_ptr()) : nullptr,
                       two ? reinterpret_cast<const bf*>(g2->data_ptr()) : nullptr, g2s,
                       two ? b2->data_ptr<float>() : nullptr, rows, W);
    return;
  }
  hy_dispatch(out, "gated_residual_add", [&]<typename T>() {
    const int grid = (int)std::min<long>((rows * W + 255) / 256, 4096);
    hipLaunchKernelGGL(gated_residual_add_kernel<T>, dim3(grid), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(out.data_ptr()), res.data_ptr<float>(),
                       reinterpret_cast<const T*>(y1.data_ptr()),
                       reinterpret_cast<const T*>(g1.data_ptr()), g1.stride(0), b1.data_ptr<float>(),
                       two ? reinterpret_cast<const T*>(y2->data_ptr()) : nullptr,
                       two ? reinterpret_cast<const T*>(g2->data_ptr()) : nullptr, g2s,
                       two ? b2->data_ptr<float>() : nullptr, rows, W);
  });
}

void side_gate_mul(at::Tensor out, at::Tensor a, at::Tensor table, at::Tensor tokens, int64_t offset) {
  HY_GPU(a);
  TORCH_CHECK(a.dim() == 2 && a.is_contiguous() && out.is_contiguous() && out.sizes() == a.sizes());
  const long rows = a.size(0);
  const int d = a.size(1);
  if (rows == 0) return;
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous() && offset >= 0 && offset + d <= table.size(1));
  TORCH_CHECK(tokens.scalar_type() == at::kLong && tokens.is_contiguous() && tokens.numel() == rows);
  TORCH_CHECK(table.scalar_type() == a.scalar_type() && out.scalar_type() == a.scalar_type());
  hy_dispatch(a, "side_gate_mul", [&]<typename T>() {
    const int grid = (int)std::min<long>((rows * d + 255) / 256, 4096);
    hipLaunchKernelGGL(side_gate_mul_kernel<T>, dim3(grid), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(out.data_ptr()), reinterpret_cast<const T*>(a.data_ptr()),
                       reinterpret_cast<const T*>(table.data_ptr()), table.stride(0),
                       tokens.data_ptr<long>(), (int)offset, rows, d);
  });
}

void sigmoid_topk(at::Tensor idx, at::Tensor w, at::Tensor logits, int64_t top) {
  HY_GPU(logits);
  TORCH_CHECK(logits.dim() == 2 && logits.is_contiguous() && logits.scalar_type() == at::kFloat,
              "router logits must be fp32 [T, E]");
  const long rows = logits.size(0);
  const int E = logits.size(1);
  if (rows == 0) return;
  TORCH_CHECK(top >= 1 && top <= E && E <= 64 * 32, "top must be within 1..E, E at most 2048");
  HY_I32(idx);
  TORCH_CHECK(idx.dim() == 2 && idx.size(0) == rows && idx.size(1) == top);
  TORCH_CHECK(w.scalar_type() == at::kFloat && w.is_contiguous() && w.sizes() == idx.sizes());
  hipLaunchKernelGGL(sigmoid_topk_kernel, dim3((rows + 3) / 4), dim3(256), 0, hy_stream(),
                     idx.data_ptr<int>(), w.data_ptr<float>(), logits.data_ptr<float>(), rows, E,
                     (int)top);
}

struct MoeDims { long T; int top, W, F, E; };

MoeDims moe_check(const at::Tensor& idx, int W, int F, int E) {
  HY_I32(idx);
  TORCH_CHECK(idx.dim() == 2 && idx.size(1) >= 1, "idx must be [T, top]");
  return MoeDims{idx.size(0), (int)idx.size(1), W, F, E};
}

void moe_gate_up_gemv(at::Tensor hmid, at::Tensor h, at::Tensor idx,
                      const std::optional<at::Tensor>& w, at::Tensor gate_up, int64_t act,
                      double limit) {
  HY_GPU(h);
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous() && gate_up.dim() == 3 && gate_up.is_contiguous());
  TORCH_CHECK(act >= kMoeActSilu && act <= kMoeActRelu2, "unknown expert activation");
  const bool gated = act < kMoeActGeluErf;      // ungated experts: gate_up is [E, F, W]
  TORCH_CHECK((!gated || gate_up.size(1) % 2 == 0) && gate_up.size(2) == h.size(1));
  const MoeDims m = moe_check(idx, h.size(1), gate_up.size(1) / (gated ? 2 : 1), gate_up.size(0));
  if (m.T == 0) return;
  TORCH_CHECK(idx.size(0) == h.size(0));
  const float* wp = nullptr;
  if (w.has_value()) {
    TORCH_CHECK(w->scalar_type() == at::kFloat && w->is_contiguous() && w->sizes() == idx.sizes() &&
                w->is_cuda());
    wp = w->data_ptr<float>();
  }
  TORCH_CHECK(hmid.is_contiguous() && hmid.dim() == 2 && hmid.size(0) == m.T * m.top && hmid.size(1) == m.F);
  TORCH_CHECK(hmid.scalar_type() == h.scalar_type() && gate_up.scalar_type() == h.scalar_type());
  const size_t lds = sizeof(float) * (size_t)m.W;
  const dim3 grid((m.F + 4 * kMoeRowsPerWave - 1) / (4 * kMoeRowsPerWave), m.T * m.top);
  hy_dispatch(h, "moe_gate_up_gemv", [&]<typename T>() {
    auto kern = moe_gate_up_gemv_kernel<T>;
    allow_lds(kern, lds);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, hy_stream(), reinterpret_cast<T*>(hmid.data_ptr()),
                       reinterpret_cast<const T*>(h.data_ptr()), idx.data_ptr<int>(),
                       wp, reinterpret_cast<const T*>(gate_up.data_ptr()), m.top,
                       m.W, m.F, m.E, (int)act, (float)limit);
  });
}

void moe_down_gemv(at::Tensor y, at::Tensor hmid, at::Tensor idx, at::Tensor down,
                   const std::optional<at::Tensor>& wo) {
  HY_GPU(hmid);
  TORCH_CHECK(down.dim() == 3 && down.is_contiguous() && hmid.dim() == 2 && hmid.is_contiguous());
  const MoeDims m = moe_check(idx, down.size(1), down.size(2), down.size(0));
  if (m.T == 0) return;
  TORCH_CHECK(hmid.size(0) == m.T * m.top && hmid.size(1) == m.F);
  TORCH_CHECK(y.is_contiguous() && y.dim() == 2 && y.size(0) == m.T && y.size(1) == m.W);
  TORCH_CHECK(y.scalar_type() == hmid.scalar_type() && down.scalar_type() == hmid.scalar_type());
  const float* wop = nullptr;
  if (wo.has_value()) {
    TORCH_CHECK(wo->scalar_type() == at::kFloat && wo->is_contiguous() && wo->sizes() == idx.sizes() &&
                wo->is_cuda());
    wop = wo->data_ptr<float>();
  }
  const size_t lds = sizeof(float) * (size_t)m.top * m.F;
  const dim3 grid((m.W + 4 * kMoeRowsPerWave - 1) / (4 * kMoeRowsPerWave), m.T);
  hy_dispatch(hmid, "moe_down_gemv", [&]<typename T>() {
    auto kern = moe_down_gemv_kernel<T>;
    allow_lds(kern, lds);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, hy_stream(), reinterpret_cast<T*>(y.data_ptr()),
                       reinterpret_cast<const T*>(hmid.data_ptr()), idx.data_ptr<int>(),
                       reinterpret_cast<const T*>(down.data_ptr()), m.top, m.W, m.F, m.E, wop);
  });
}

// Expert mixture grouped by expert, no host sync. gate_up: in = h [T, W],
// out = hmid [T*top, F]; else: in = hmid [T*top, F], out = yk [T*top, W].
void moe_expert_gemv(at::Tensor out, at::Tensor in, at::Tensor idx, const std::optional<at::Tensor>& w,
                     at::Tensor weight, bool gate_up, int64_t act, double limit) {
  HY_GPU(in);
  TORCH_CHECK(act == kMoeActSilu || act == kMoeActClampSwish, "unknown expert activation");
  HY_I32(idx);
  TORCH_CHECK(idx.dim() == 2 && idx.size(1) >= 1, "idx must be [T, top]");
  const long rows = idx.numel();
  const int top = idx.size(1);
  if (rows == 0) return;
  TORCH_CHECK(rows <= kMoeMaxRows, "grouped expert kernel handles at most ", kMoeMaxRows, " rows");
  TORCH_CHECK(weight.dim() == 3 && weight.is_contiguous() && in.dim() == 2 && in.is_contiguous() &&
              out.dim() == 2 && out.is_contiguous());
  const int E = weight.size(0), K = weight.size(2);
  const int N = gate_up ? weight.size(1) / 2 : weight.size(1);
  TORCH_CHECK(in.size(1) == K && out.size(0) == rows && out.size(1) == N);
  TORCH_CHECK(in.size(0) == (gate_up ? idx.size(0) : rows));
  TORCH_CHECK(in.scalar_type() == out.scalar_type() && weight.scalar_type() == out.scalar_type());
  const float* wp = nullptr;
  if (gate_up) TORCH_CHECK(weight.size(1) % 2 == 0);
  if (gate_up && w.has_value()) {
    TORCH_CHECK(w->scalar_type() == at::kFloat && w->is_contiguous() && w->numel() == rows &&
                w->is_cuda());
    wp = w->data_ptr<float>();
  }
  const dim3 grid((N + 4 * kMoeFPW - 1) / (4 * kMoeFPW), E);
  hy_dispatch(in, "moe_expert_gemv", [&]<typename T>() {
    const size_t lds = sizeof(int) * kMoeMaxRows + sizeof(T) * (size_t)kMoeTB * K;
    auto launch = [&]<bool GU>() {
      auto kern = moe_expert_gemv_kernel<T, GU>;
      allow_lds(kern, lds);
      hipLaunchKernelGGL(kern, grid, dim3(256), lds, hy_stream(), reinterpret_cast<T*>(out.data_ptr()),
                         reinterpret_cast<const T*>(in.data_ptr()), idx.data_ptr<int>(), wp,
                         reinterpret_cast<const T*>(weight.data_ptr()), (int)rows, top, K, N,
                         (int)act, (float)limit);
    };
    if (gate_up) launch.template operator()<true>();
    else launch.template operator()<false>();
  });
}


// yk [E, T, W] -> y [T, W] = sum_e wd[t, e] * yk[e, t] (wd null: plain sum)
void moe_combine(at::Tensor y, at::Tensor yk, const std::optional<at::Tensor>& wd) {
  HY_GPU(yk);
  TORCH_CHECK(yk.dim() == 3 && yk.is_contiguous() && y.dim() == 2 && y.is_contiguous());
  const int E = yk.size(0), W = yk.size(2);
  const long rows = yk.size(1);
  if (rows == 0) return;
  TORCH_CHECK(y.size(0) == rows && y.size(1) == W && y.scalar_type() == yk.scalar_type());
  const float* wp = nullptr;
  if (wd.has_value()) {
    TORCH_CHECK(wd->scalar_type() == at::kFloat && wd->is_contiguous() && wd->is_cuda() &&
                wd->dim() == 2 && wd->size(0) == rows && wd->size(1) == E, "wd must be fp32 [T, E]");
    wp = wd->data_ptr<float>();
  }
  const int grid = (int)std::min<long>((rows * W + 255) / 256, 4096);
  hy_dispatch(yk, "moe_combine", [&]<typename T>() {
    hipLaunchKernelGGL(moe_combine_kernel<T>, dim3(grid), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(y.data_ptr()), reinterpret_cast<const T*>(yk.data_ptr()),
                       wp, rows, W, E);
  });
}

// ys [T*top, W] (expert-sorted rows), pos [T*top] int64 -> y [T, W]
void moe_gather_combine(at::Tensor y, at::Tensor ys, at::Tensor pos,
                        const std::optional<at::Tensor>& w, int64_t top) {
  HY_GPU(ys);
  TORCH_CHECK(ys.dim() == 2 && ys.is_contiguous() && y.dim() == 2 && y.is_contiguous());
  const long rows = y.size(0);
  const int W = y.size(1);
  if (rows == 0) return;
  TORCH_CHECK(top >= 1 && ys.size(0) == rows * top && ys.size(1) == W &&
              y.scalar_type() == ys.scalar_type());
  TORCH_CHECK(pos.scalar_type() == at::kLong && pos.is_contiguous() && pos.is_cuda() &&
              pos.numel() == rows * top, "pos must be int64 [T * top]");
  const float* wp = nullptr;
  if (w.has_value()) {
    TORCH_CHECK(w->scalar_type() == at::kFloat && w->is_contiguous() && w->is_cuda() &&
                w->numel() == rows * top, "w must be fp32 [T, top]");
    wp = w->data_ptr<float>();
  }
  const int grid = (int)std::min<long>((rows * W / 4 + 255) / 256 + 1, 8192);
  hy_dispatch(ys, "moe_gather_combine", [&]<typename T>() {
    hipLaunchKernelGGL(moe_gather_combine_kernel<T>, dim3(grid), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(y.data_ptr()), reinterpret_cast<const T*>(ys.data_ptr()),
                       pos.data_ptr<long>(), wp, rows, (int)top, W);
  });
}

// ---- scan/attention hybrids ------------------------------------------------

#define HY_F32(x) TORCH_CHECK(x.scalar_type() == at::kFloat && x.is_contiguous() && x.is_cuda(), #x " must be contiguous fp32 on the GPU")

void embed_sinusoid(at::Tensor out, at::Tensor embedding, at::Tensor ids, at::Tensor positions,
                    at::Tensor inv_freq) {
  HY_GPU(embedding);
  TORCH_CHECK(embedding.dim() == 2 && embedding.is_contiguous());
  const long rows = ids.numel();
  const int W = embedding.size(1);
  if (rows == 0) return;
  TORCH_CHECK(ids.scalar_type() == at::kLong && ids.is_contiguous() && ids.is_cuda());
  TORCH_CHECK(positions.scalar_type() == at::kLong && positions.is_contiguous() &&
              positions.numel() == rows && positions.is_cuda());
  HY_F32(inv_freq); HY_F32(out);
  TORCH_CHECK(inv_freq.numel() == (W + 1) / 2, "inv_freq needs one entry per (sin, cos) pair");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == rows && out.size(1) == W);
  hy_dispatch(embedding, "embed_sinusoid", [&]<typename T>() {
    hipLaunchKernelGGL(embed_sinusoid_kernel<T>, dim3(rows), dim3(256), 0, hy_stream(),
                       out.data_ptr<float>(), reinterpret_cast<const T*>(embedding.data_ptr()),
                       ids.data_ptr<long>(), positions.data_ptr<long>(), inv_freq.data_ptr<float>(),
                       W, (long)embedding.size(0));
  });
}

void scaled_add_norm(at::Tensor out, at::Tensor res, at::Tensor y, const std::optional<at::Tensor>& y2,
                     double a1, double a2, at::Tensor weight, double eps) {
  HY_GPU(y);
  HY_F32(res);
  TORCH_CHECK(y.dim() == 2 && y.is_contiguous() && out.is_contiguous() && weight.is_contiguous());
  const long rows = y.size(0);
  const int W = y.size(1);
  if (rows == 0) return;
  TORCH_CHECK(res.sizes() == y.sizes() && out.sizes() == y.sizes() && weight.numel() == W);
  TORCH_CHECK(out.scalar_type() == y.scalar_type() && weight.scalar_type() == y.scalar_type());
  const void* y2p = nullptr;
  if (y2.has_value()) {
    TORCH_CHECK(y2->is_contiguous() && y2->sizes() == y.sizes() && y2->scalar_type() == y.scalar_type() &&
                y2->is_cuda());
    y2p = y2->data_ptr();
  }
  if (y.scalar_type() == at::kBFloat16 && W % 8 == 0 && W <= 4 * 2048) {
    using bf = __hip_bfloat16;
    auto launch = [&]<int CH>() {
      hipLaunchKernelGGL(scaled_add_norm_vec_kernel<CH>, dim3(rows), dim3(256), 0, hy_stream(),
                         reinterpret_cast<bf*>(out.data_ptr()), res.data_ptr<float>(),
                         reinterpret_cast<const bf*>(y.data_ptr()), reinterpret_cast<const bf*>(y2p),
                         (float)a1, (float)a2, reinterpret_cast<const bf*>(weight.data_ptr()), W,
                         (float)eps);
    };
    if (W <= 2048) launch.template operator()<1>();
    else if (W <= 4096) launch.template operator()<2>();
    else launch.template operator()<4>();
    return;
  }
  hy_dispatch(y, "scaled_add_norm", [&]<typename T>() {
    hipLaunchKernelGGL(scaled_add_norm_kernel<T>, dim3(rows), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(out.data_ptr()), res.data_ptr<float>(),
                       reinterpret_cast<const T*>(y.data_ptr()), reinterpret_cast<const T*>(y2p),
                       (float)a1, (float)a2, reinterpret_cast<const T*>(weight.data_ptr()), W,
                       (float)eps);
  });
}

void depth_mix_norm(at::Tensor out, at::Tensor stack, int64_t n, at::Tensor coef, at::Tensor y,
                    const std::optional<at::Tensor>& y2, double a1, double a2, at::Tensor weight,
                    double eps) {
  HY_GPU(y);
  HY_F32(stack); HY_F32(coef);
  TORCH_CHECK(y.dim() == 2 && y.is_contiguous() && out.is_contiguous() && weight.is_contiguous());
  const long rows = y.size(0);
  const int W = y.size(1);
  if (rows == 0) return;
  TORCH_CHECK(stack.dim() == 3 && stack.size(1) == rows && stack.size(2) == W);
  TORCH_CHECK(n >= 1 && n + 1 <= stack.size(0) && coef.numel() >= n,
              "the stack needs entries 0..n and one coefficient per entry below n");
  TORCH_CHECK(out.sizes() == y.sizes() && weight.numel() == W);
  TORCH_CHECK(out.scalar_type() == y.scalar_type() && weight.scalar_type() == y.scalar_type());
  const void* y2p = nullptr;
  if (y2.has_value()) {
    TORCH_CHECK(y2->is_contiguous() && y2->sizes() == y.sizes() && y2->scalar_type() == y.scalar_type() &&
                y2->is_cuda());
    y2p = y2->data_ptr();
  }
  const long ls = rows * (long)W;
  if (y.scalar_type() == at::kBFloat16 && W % 4 == 0 && W <= 8 * 1024) {
    using bf = __hip_bfloat16;
    auto launch = [&]<int CH>() {
      hipLaunchKernelGGL(depth_mix_norm_vec_kernel<CH>, dim3(rows), dim3(256), 0, hy_stream(),
                         reinterpret_cast<bf*>(out.data_ptr()), stack.data_ptr<float>(), ls, (int)n,
                         coef.data_ptr<float>(), reinterpret_cast<const bf*>(y.data_ptr()),
                         reinterpret_cast<const bf*>(y2p), (float)a1, (float)a2,
                         reinterpret_cast<const bf*>(weight.data_ptr()), W, (float)eps);
    };
    if (W <= 1024) launch.template operator()<1>();
    else if (W <= 2048) launch.template operator()<2>();
    else if (W <= 4096) launch.template operator()<4>();
    else launch.template operator()<8>();
    return;
  }
  hy_dispatch(y, "depth_mix_norm", [&]<typename T>() {
    hipLaunchKernelGGL(depth_mix_norm_kernel<T>, dim3(rows), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(out.data_ptr()), stack.data_ptr<float>(), ls, (int)n,
                       coef.data_ptr<float>(), reinterpret_cast<const T*>(y.data_ptr()),
                       reinterpret_cast<const T*>(y2p), (float)a1, (float)a2,
                       reinterpret_cast<const T*>(weight.data_ptr()), W, (float)eps);
  });
}

// k [T, G*D], v [T, G*DV]: row-strided views of one GEMM output.
void kv_scatter(at::Tensor k, at::Tensor v, at::Tensor k_cache, at::Tensor v_cache, at::Tensor slots) {
  HY_GPU(k);
  HY_INNER(k); HY_INNER(v);
  TORCH_CHECK(k.dim() == 2 && v.dim() == 2);
  const long T_ = k.size(0);
  if (T_ == 0) return;
  TORCH_CHECK(v.size(0) == T_ && slots.numel() == T_);
  TORCH_CHECK(slots.scalar_type() == at::kLong && slots.is_contiguous() && slots.is_cuda());
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.is_contiguous() && v_cache.is_contiguous());
  const int G = k_cache.size(1), bs = k_cache.size(2), D = k_cache.size(3), DV = v_cache.size(3);
  TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == G && v_cache.size(2) == bs);
  TORCH_CHECK(k.size(1) == G * D && v.size(1) == G * DV, "k/v widths do not match the cache layout");
  const auto dt = k.scalar_type();
  TORCH_CHECK(v.scalar_type() == dt && k_cache.scalar_type() == dt && v_cache.scalar_type() == dt,
              "kv_scatter: one dtype for activations and cache");
  hy_dispatch(k, "kv_scatter", [&]<typename T>() {
    hipLaunchKernelGGL(kv_scatter_kernel<T>, dim3(T_), dim3(256), 0, hy_stream(),
                       reinterpret_cast<const T*>(k.data_ptr()), k.stride(0),
                       reinterpret_cast<const T*>(v.data_ptr()), v.stride(0),
                       reinterpret_cast<T*>(k_cache.data_ptr()), reinterpret_cast<T*>(v_cache.data_ptr()),
                       slots.data_ptr<long>(), G, D, DV, bs);
  });
}

struct SeqDims { int B; };

SeqDims seq_check(const at::Tensor& cu, const at::Tensor& slots, const at::Tensor& fresh,
                  const at::Tensor& state) {
  HY_I32(cu); HY_I32(slots); HY_I32(fresh);
  TORCH_CHECK(cu.is_cuda() && slots.is_cuda() && fresh.is_cuda());
  const int B = slots.numel();
  TORCH_CHECK(cu.numel() == B + 1 && fresh.numel() == B);
  TORCH_CHECK(state.scalar_type() == at::kFloat && state.is_contiguous() && state.is_cuda(),
              "state must be contiguous fp32 on the GPU");
  return SeqDims{B};
}

// z, u, g [T, n]: row-strided slices of one projection output (same stride).
void mingru_scan(at::Tensor out, at::Tensor z, at::Tensor u, at::Tensor g, at::Tensor z_b,
                 at::Tensor u_b, at::Tensor state, at::Tensor cu, at::Tensor slots, at::Tensor fresh) {
  HY_GPU(z);
  HY_INNER(z); HY_INNER(u); HY_INNER(g);
  TORCH_CHECK(z.dim() == 2 && u.sizes() == z.sizes() && g.sizes() == z.sizes());
  const long T_ = z.size(0);
  const int n = z.size(1);
  if (T_ == 0) return;
  TORCH_CHECK(u.stride(0) == z.stride(0) && g.stride(0) == z.stride(0), "z, u, g must share a row stride");
  TORCH_CHECK(u.scalar_type() == z.scalar_type() && g.scalar_type() == z.scalar_type() &&
              out.scalar_type() == z.scalar_type());
  TORCH_CHECK(out.is_contiguous() && out.sizes() == z.sizes());
  HY_F32(z_b); HY_F32(u_b);
  TORCH_CHECK(z_b.numel() == n && u_b.numel() == n);
  const SeqDims d = seq_check(cu, slots, fresh, state);
  TORCH_CHECK(state.dim() == 2 && state.size(1) == n, "state [slots, n] fp32");
  // long portions run parallel over time: 16 (or 4) chunks per sequence
  const long avg = T_ / std::max(1, d.B);
  hy_dispatch(z, "mingru_scan", [&]<typename T>() {
    auto launch = [&]<int NC>() {
      if constexpr (NC == 1) {
        hipLaunchKernelGGL(mingru_scan_kernel<T>, dim3((n + 255) / 256, d.B), dim3(256), 0,
                           hy_stream(), reinterpret_cast<T*>(out.data_ptr()),
                           reinterpret_cast<const T*>(z.data_ptr()),
                           reinterpret_cast<const T*>(u.data_ptr()),
                           reinterpret_cast<const T*>(g.data_ptr()), z.stride(0),
                           z_b.data_ptr<float>(), u_b.data_ptr<float>(), state.data_ptr<float>(),
                           cu.data_ptr<int>(), slots.data_ptr<int>(), fresh.data_ptr<int>(), n);
      } else {
        hipLaunchKernelGGL((mingru_scan_chunked_kernel<T, NC>), dim3((n + 63) / 64, d.B),
                           dim3(64 * NC), 0, hy_stream(), reinterpret_cast<T*>(out.data_ptr()),
                           reinterpret_cast<const T*>(z.data_ptr()),
                           reinterpret_cast<const T*>(u.data_ptr()),
                           reinterpret_cast<const T*>(g.data_ptr()), z.stride(0),
                           z_b.data_ptr<float>(), u_b.data_ptr<float>(), state.data_ptr<float>(),
                           cu.data_ptr<int>(), slots.data_ptr<int>(), fresh.data_ptr<int>(), n);
      }
    };
    if (avg >= 128) launch.template operator()<16>();
    else if (avg >= 16) launch.template operator()<4>();
    else launch.template operator()<1>();
  });
}

// x [T, C] row-strided; weight [C, K] fp32; tail [slots, K-1, C] fp32.
void causal_conv_silu(at::Tensor out, at::Tensor x, at::Tensor weight,
                      const std::optional<at::Tensor>& bias_opt, at::Tensor tail, at::Tensor cu,
                      at::Tensor slots, at::Tensor fresh, bool silu) {
  HY_GPU(x);
  HY_INNER(x);
  TORCH_CHECK(x.dim() == 2);
  const long T_ = x.size(0);
  const int C = x.size(1);
  if (T_ == 0) return;
  HY_F32(weight);
  TORCH_CHECK(weight.dim() == 2 && weight.size(0) == C);
  const float* bias_ptr = nullptr;
  if (bias_opt.has_value()) {
    const at::Tensor& bias = *bias_opt;
    HY_F32(bias);
    TORCH_CHECK(bias.numel() == C);
    bias_ptr = bias.data_ptr<float>();
  }
  const int K = weight.size(1);
  TORCH_CHECK(K >= 1 && K <= kConvMaxTaps, "1 to ", kConvMaxTaps, " taps");
  TORCH_CHECK(out.is_contiguous() && out.sizes() == x.sizes() && out.scalar_type() == x.scalar_type());
  const SeqDims d = seq_check(cu, slots, fresh, tail);
  TORCH_CHECK(tail.dim() == 3 && tail.size(1) == K - 1 && tail.size(2) == C, "tail [slots, K-1, C] fp32");
  // few rows (single tokens): a thread per row; prompts: 32 rows per thread
  const int rpt = T_ <= 512 ? 1 : 32;
  const dim3 grid((C + 255) / 256, (T_ + rpt - 1) / rpt);
  hy_dispatch(x, "causal_conv_silu", [&]<typename T>() {
    hipLaunchKernelGGL(causal_conv_silu_kernel<T>, grid, dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(out.data_ptr()), reinterpret_cast<const T*>(x.data_ptr()),
                       x.stride(0), weight.data_ptr<float>(), bias_ptr,
                       tail.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(),
                       fresh.data_ptr<int>(), d.B, C, K, rpt, (int)silu);
    if (K > 1)
      hipLaunchKernelGGL(conv_tail_update_kernel<T>, dim3((C + 255) / 256, d.B), dim3(256), 0,
                         hy_stream(), reinterpret_cast<const T*>(x.data_ptr()), x.stride(0),
                         tail.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(),
                         fresh.data_ptr<int>(), C, K);
  });
}

// x [T, C] contiguous or row-strided, dt [T, C], z [T, C] row-strided, Bm / Cm
// [T, N] row-strided slices of one projection output; state [slots, C, N].
void selective_scan(at::Tensor out, at::Tensor x, at::Tensor dt, at::Tensor dt_b, at::Tensor A,
                    at::Tensor Bm, at::Tensor Cm, at::Tensor D, at::Tensor z, at::Tensor state,
                    at::Tensor cu, at::Tensor slots, at::Tensor fresh) {
  HY_GPU(x);
  HY_INNER(x); HY_INNER(dt); HY_INNER(z); HY_INNER(Bm); HY_INNER(Cm);
  TORCH_CHECK(x.dim() == 2 && dt.sizes() == x.sizes() && z.sizes() == x.sizes());
  const long T_ = x.size(0);
  const int C = x.size(1);
  if (T_ == 0) return;
  TORCH_CHECK(Bm.dim() == 2 && Bm.size(0) == T_ && Cm.sizes() == Bm.sizes() &&
              Bm.stride(0) == Cm.stride(0));
  const int N = Bm.size(1);
  HY_F32(dt_b); HY_F32(A); HY_F32(D);
  TORCH_CHECK(dt_b.numel() == C && D.numel() == C && A.dim() == 2 && A.size(0) == C && A.size(1) == N);
  const auto ty = x.scalar_type();
  TORCH_CHECK(dt.scalar_type() == ty && z.scalar_type() == ty && Bm.scalar_type() == ty &&
              Cm.scalar_type() == ty && out.scalar_type() == ty);
  TORCH_CHECK(out.is_contiguous() && out.sizes() == x.sizes());
  const SeqDims d = seq_check(cu, slots, fresh, state);
  TORCH_CHECK(state.dim() == 3 && state.size(1) == C && state.size(2) == N, "state [slots, C, N] fp32");
  TORCH_CHECK(N >= 1 && N <= 1024, "1 to 1024 states per channel");
  // NS states per lane, LPC lanes per channel (both powers of two)
  int ns = 1;
  while (ns < N && ns < 16) ns *= 2;
  int lpc = 1;
  while (ns * lpc < N) lpc *= 2;
  // long portions run parallel over time: 8 chunks per sequence
  const bool chunked = T_ / std::max(1, d.B) >= 64;
  const int nc = chunked ? 8 : 1;
  const dim3 grid(((long)C * lpc + 63) / 64, d.B);
  const size_t lds = sizeof(float) * ((size_t)nc * kScanTT * 2 * N +
                                      (chunked ? (size_t)nc * 64 * (1 + ns) : 0));
  hy_dispatch(x, "selective_scan", [&]<typename T>() {
    auto launch = [&]<int NS, int NC>() {
      auto kern = selective_scan_kernel<T, NS, NC>;
      allow_lds(kern, lds);
      hipLaunchKernelGGL(kern, grid, dim3(64 * NC), lds, hy_stream(),
                         reinterpret_cast<T*>(out.data_ptr()),
                         reinterpret_cast<const T*>(x.data_ptr()), x.stride(0),
                         reinterpret_cast<const T*>(dt.data_ptr()), dt.stride(0),
                         dt_b.data_ptr<float>(), A.data_ptr<float>(),
                         reinterpret_cast<const T*>(Bm.data_ptr()),
                         reinterpret_cast<const T*>(Cm.data_ptr()), Bm.stride(0),
                         D.data_ptr<float>(), reinterpret_cast<const T*>(z.data_ptr()), z.stride(0),
                         state.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(),
                         fresh.data_ptr<int>(), C, N, lpc);
    };
    auto by_ns = [&]<int NC>() {
      if (ns == 16) launch.template operator()<16, NC>();
      else if (ns == 8) launch.template operator()<8, NC>();
      else if (ns == 4) launch.template operator()<4, NC>();
      else if (ns == 2) launch.template operator()<2, NC>();
      else launch.template operator()<1, NC>();
    };
    if (chunked) by_ns.template operator()<8>();
    else by_ns.template operator()<1>();
  });
}

void softmax_topk(at::Tensor idx, at::Tensor w, at::Tensor logits, int64_t top, double scale,
                  const std::optional<at::Tensor>& correction, bool renorm) {
  HY_GPU(logits);
  TORCH_CHECK(logits.dim() == 2 && logits.is_contiguous() && logits.scalar_type() == at::kFloat,
              "router logits must be fp32 [T, E]");
  const long rows = logits.size(0);
  const int E = logits.size(1);
  if (rows == 0) return;
  TORCH_CHECK(top >= 1 && top <= E && E <= 64 * 32, "top must be within 1..E, E at most 2048");
  HY_I32(idx);
  TORCH_CHECK(idx.dim() == 2 && idx.size(0) == rows && idx.size(1) == top);
  TORCH_CHECK(w.scalar_type() == at::kFloat && w.is_contiguous() && w.sizes() == idx.sizes());
  const float* corr = nullptr;
  if (correction.has_value()) {
    TORCH_CHECK(correction->is_cuda() && correction->scalar_type() == at::kFloat &&
                correction->is_contiguous() && correction->numel() == E, "correction must be fp32 [E]");
    corr = correction->data_ptr<float>();
  }
  hipLaunchKernelGGL(softmax_topk_kernel, dim3((rows + 3) / 4), dim3(256), 0, hy_stream(),
                     idx.data_ptr<int>(), w.data_ptr<float>(), logits.data_ptr<float>(), rows, E,
                     (int)top, (float)scale, corr, (int)renorm);
}

void clamp_swish_mul(at::Tensor out, at::Tensor in, double limit) {
  HY_GPU(in);
  TORCH_CHECK(in.is_contiguous() && out.is_contiguous() && in.scalar_type() == out.scalar_type());
  const int d = out.size(-1);
  TORCH_CHECK(in.size(-1) == 2 * d, "in must be [..., 2*d]");
  const long rows = out.numel() / d;
  if (rows == 0) return;
  if (in.scalar_type() == at::kBFloat16 && d % 8 == 0) {
    using bf = __hip_bfloat16;
    const long chunks = rows * (d / 8);
    const int grid = (int)std::min<long>((chunks + 255) / 256, 4096);
    hipLaunchKernelGGL(clamp_swish_mul_vec_kernel, dim3(grid), dim3(256), 0, hy_stream(),
                       reinterpret_cast<bf*>(out.data_ptr()), reinterpret_cast<const bf*>(in.data_ptr()),
                       rows, d, (float)limit);
    return;
  }
  hy_dispatch(in, "clamp_swish_mul", [&]<typename T>() {
    const int grid = (int)std::min<long>((rows * d + 255) / 256, 4096);
    hipLaunchKernelGGL(clamp_swish_mul_kernel<T>, dim3(grid), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(out.data_ptr()), reinterpret_cast<const T*>(in.data_ptr()),
                       rows, d, (float)limit);
  });
}

// ---- windowed attention beside a matrix memory -------------------------------

// q [T, H, D], k [T, G, D], v [T, G, DV] or none: row-strided views with packed heads.
void qkv_norm_rope_cache(at::Tensor q, at::Tensor k, const std::optional<at::Tensor>& v_opt,
                         const std::optional<at::Tensor>& q_w, const std::optional<at::Tensor>& k_w,
                         const std::optional<at::Tensor>& inv_freq, int64_t rot_dims,
                         at::Tensor positions, at::Tensor k_cache, at::Tensor v_cache,
                         at::Tensor slots, double eps, bool v_unit_norm,
                         const std::optional<at::Tensor>& v_inv_freq) {
  HY_GPU(q);
  const long T_ = q.size(0);
  if (T_ == 0) return;
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && k.size(0) == T_ && k.size(2) == q.size(2));
  HY_INNER(q); HY_INNER(k);
  const int H = q.size(1), G = k.size(1), D = q.size(2);
  TORCH_CHECK(q.stride(1) == D && k.stride(1) == D, "heads must be packed");
  const auto dt = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == dt && k_cache.scalar_type() == dt && v_cache.scalar_type() == dt);
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.is_contiguous() && k_cache.size(1) == G &&
              k_cache.size(3) == D, "key cache must be [blocks, G, block, D]");
  const int bs = k_cache.size(2), DV = v_cache.size(3);
  TORCH_CHECK(v_cache.dim() == 4 && v_cache.is_contiguous() && v_cache.size(0) == k_cache.size(0) &&
              v_cache.size(1) == G && v_cache.size(2) == bs, "value cache must be [blocks, G, block, DV]");
  const void* v_ptr = nullptr;
  long v_stride = 0;
  if (v_opt.has_value()) {
    const at::Tensor& v = *v_opt;
    HY_INNER(v);
    TORCH_CHECK(v.dim() == 3 && v.size(0) == T_ && v.size(1) == G && v.size(2) == DV &&
                v.stride(1) == DV && v.scalar_type() == dt, "v must be [T, G, DV], heads packed");
    v_ptr = v.data_ptr();
    v_stride = v.stride(0);
  } else {
    TORCH_CHECK(DV == D && !v_unit_norm && !v_inv_freq.has_value(),
                "values that are the raw keys have the keys' size and pass unchanged");
  }
  auto weight_ptr = [&](const std::optional<at::Tensor>& w) -> const void* {
    if (!w.has_value()) return nullptr;
    TORCH_CHECK(w->is_cuda() && w->is_contiguous() && w->numel() == D && w->scalar_type() == dt,
                "a head norm weight must be [D] in the activations' dtype");
    return w->data_ptr();
  };
  const void* qw = weight_ptr(q_w);
  const void* kw = weight_ptr(k_w);
  auto table_ptr = [&](const std::optional<at::Tensor>& t, int dims) -> const float* {
    TORCH_CHECK(t.has_value() && t->is_cuda() && t->scalar_type() == at::kFloat &&
                t->is_contiguous() && t->numel() == dims / 2, "a rotary table must be fp32 [dims / 2]");
    return t->data_ptr<float>();
  };
  TORCH_CHECK(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= D, "rot_dims must be even, at most D");
  const float* table = rot_dims ? table_ptr(inv_freq, (int)rot_dims) : nullptr;
  const float* v_table = nullptr;
  if (v_inv_freq.has_value()) {
    TORCH_CHECK(DV % 2 == 0, "rotated values need an even size");
    v_table = table_ptr(v_inv_freq, DV);
  }
  // lanes per head vector: the fewest that hold its pairs and unrotated channels
  const int max_half = std::max<int>(rot_dims / 2, v_table ? DV / 2 : 0);
  const int max_tail = std::max<int>(D - rot_dims, (v_opt.has_value() && !v_table) ? DV : 0);
  // bf16 vectors made of whole 16-byte granules: a granule of each half and
  // one of the rest per lane
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = dt == at::kBFloat16 && D % 8 == 0 && DV % 8 == 0 && rot_dims % 16 == 0 &&
                   (!v_table || DV % 16 == 0) && q.stride(0) % 8 == 0 && k.stride(0) % 8 == 0 &&
                   v_stride % 8 == 0 && aligned(q.data_ptr()) && aligned(k.data_ptr()) &&
                   aligned(v_ptr) && aligned(qw) && aligned(kw);
  const int per_pair = vec ? 8 : kRopePairs, per_tail = vec ? 8 : kRopeTail;
  int LG = vec ? 1 : 8;
  while (LG < 64 && (max_half > LG * per_pair || max_tail > LG * per_tail)) LG *= 2;
  TORCH_CHECK(max_half <= LG * per_pair && max_tail <= LG * per_tail,
              "head size beyond what a wave holds in registers");
  TORCH_CHECK(positions.scalar_type() == at::kLong && positions.is_contiguous() &&
              positions.numel() == T_ && positions.is_cuda());
  TORCH_CHECK(slots.scalar_type() == at::kLong && slots.is_contiguous() && slots.numel() == T_ &&
              slots.is_cuda());
  const size_t lds = sizeof(float) * (size_t)(rot_dims + DV);
  auto launch = [&]<typename T, bool VEC>() {
    hipLaunchKernelGGL((qkv_norm_rope_cache_kernel<T, VEC>), dim3(T_), dim3(256), lds, hy_stream(),
                       reinterpret_cast<T*>(q.data_ptr()), q.stride(0),
                       reinterpret_cast<const T*>(k.data_ptr()), k.stride(0),
                       reinterpret_cast<const T*>(v_ptr), v_stride,
                       reinterpret_cast<const T*>(qw), reinterpret_cast<const T*>(kw), table,
                       (int)rot_dims, v_table, positions.data_ptr<long>(),
                       reinterpret_cast<T*>(k_cache.data_ptr()),
                       reinterpret_cast<T*>(v_cache.data_ptr()), slots.data_ptr<long>(), H, G, D, DV,
                       bs, (float)eps, (int)v_unit_norm, LG);
  };
  if (vec) launch.template operator()<__hip_bfloat16, true>();
  else hy_dispatch(q, "qkv_norm_rope_cache", [&]<typename T>() { launch.template operator()<T, false>(); });
}

void rotate_heads(at::Tensor x, at::Tensor positions, at::Tensor inv_freq, bool inverse) {
  HY_GPU(x);
  const long T_ = x.size(0);
  if (T_ == 0) return;
  TORCH_CHECK(x.dim() == 3 && x.is_contiguous() && x.size(2) % 2 == 0, "x must be contiguous [T, H, n], n even");
  const int H = x.size(1), n = x.size(2);
  HY_F32(inv_freq);
  TORCH_CHECK(inv_freq.numel() == n / 2);
  TORCH_CHECK(positions.scalar_type() == at::kLong && positions.is_contiguous() &&
              positions.numel() == T_ && positions.is_cuda());
  hy_dispatch(x, "rotate_heads", [&]<typename T>() {
    hipLaunchKernelGGL(rotate_heads_kernel<T>, dim3(T_), dim3(256), sizeof(float) * n, hy_stream(),
                       reinterpret_cast<T*>(x.data_ptr()), positions.data_ptr<long>(),
                       inv_freq.data_ptr<float>(), H, n, inverse ? -1.0f : 1.0f);
  });
}

// out fp32 [3, T, H]; gates fp32 [T, 2H]; m_state fp32 [slots, H]
void mlstm_gates(at::Tensor out, at::Tensor gates, double cap, at::Tensor m_state, at::Tensor cu,
                 at::Tensor slots, at::Tensor fresh) {
  HY_F32(gates);
  const long T_ = gates.size(0);
  if (T_ == 0) return;
  TORCH_CHECK(gates.dim() == 2 && gates.size(1) % 2 == 0);
  const int H = gates.size(1) / 2;
  HY_F32(out);
  TORCH_CHECK(out.dim() == 3 && out.size(0) == 3 && out.size(1) == T_ && out.size(2) == H);
  const SeqDims d = seq_check(cu, slots, fresh, m_state);
  TORCH_CHECK(m_state.dim() == 2 && m_state.size(1) == H && cap > 0.0, "m_state [slots, H] fp32");
  hipLaunchKernelGGL(mlstm_gates_kernel, dim3(d.B, H), dim3(256), 0, hy_stream(),
                     out.data_ptr<float>(), gates.data_ptr<float>(), (float)cap,
                     m_state.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(),
                     fresh.data_ptr<int>(), H, T_);
}

// The recurrence kernel in its scalar-gate mode: q, k [T, H, D], v [T, H, DV]
// (row-strided views, heads packed); decay, write fp32 [T, H]; o fp32
// [T, H, DV + 1]; state fp32 [slots, H, D, DV + 1].
void matrix_memory(at::Tensor o, at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor decay,
                   at::Tensor write, at::Tensor state, at::Tensor cu, at::Tensor slots,
                   at::Tensor fresh, double q_scale) {
  HY_GPU(q);
  const long T_ = q.size(0);
  if (T_ == 0) return;
  TORCH_CHECK(q.dim() == 3 && k.sizes() == q.sizes() && v.dim() == 3);
  HY_INNER(q); HY_INNER(k); HY_INNER(v);
  const int H = q.size(1), D = q.size(2), DVin = v.size(2), DV = DVin + 1;
  TORCH_CHECK(v.size(0) == T_ && v.size(1) == H);
  TORCH_CHECK(q.stride(1) == D && k.stride(1) == D && v.stride(1) == DVin, "heads must be packed");
  HY_F32(decay); HY_F32(write);
  TORCH_CHECK(decay.dim() == 2 && decay.size(0) == T_ && decay.size(1) == H &&
              write.sizes() == decay.sizes(), "decay and write must be fp32 [T, H]");
  TORCH_CHECK(o.scalar_type() == at::kFloat && o.is_contiguous() && o.dim() == 3 &&
              o.size(0) == T_ && o.size(1) == H && o.size(2) == DV);
  const SeqDims sd = seq_check(cu, slots, fresh, state);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D && state.size(3) == DV,
              "state [slots, H, D, DV + 1] fp32");
  TORCH_CHECK(D <= 256, "key size above 256 is not supported");
  const auto dt = q.scalar_type();
  TORCH_CHECK(k.scalar_type() == dt && v.scalar_type() == dt);
  const dim3 grid((DV + kGlaCols - 1) / kGlaCols, H, sd.B);
  hy_dispatch(q, "matrix_memory", [&]<typename T>() {
    auto launch = [&]<int DPL>() {
      hipLaunchKernelGGL((gla_recurrence_kernel<T, DPL>), grid, dim3(256), 0, hy_stream(),
                         o.data_ptr<float>(),
                         reinterpret_cast<const T*>(q.data_ptr()), q.stride(0),
                         reinterpret_cast<const T*>(k.data_ptr()), k.stride(0),
                         reinterpret_cast<const T*>(v.data_ptr()), v.stride(0),
                         static_cast<const T*>(nullptr), 0L, static_cast<const float*>(nullptr),
                         state.data_ptr<float>(), cu.data_ptr<int>(), slots.data_ptr<int>(),
                         fresh.data_ptr<int>(), H, D, DV, 1.0f, (float)q_scale,
                         static_cast<const float*>(nullptr), 0, decay.data_ptr<float>(),
                         write.data_ptr<float>(), 1);
    };
    if (D <= 32) launch.template operator()<2>();
    else if (D <= 64) launch.template operator()<4>();
    else if (D <= 128) launch.template operator()<8>();
    else launch.template operator()<16>();
  });
}

void mlstm_out_norm_gate(at::Tensor out, at::Tensor o, at::Tensor floor_, at::Tensor weight,
                         at::Tensor gate, double eps) {
  HY_GPU(o);
  TORCH_CHECK(o.dim() == 3 && o.scalar_type() == at::kFloat && o.is_contiguous() && o.size(2) >= 2);
  const long T_ = o.size(0);
  if (T_ == 0) return;
  const int H = o.size(1), DV = o.size(2) - 1;
  HY_F32(floor_);
  TORCH_CHECK(floor_.numel() == T_ * H);
  TORCH_CHECK(out.dim() == 2 && out.is_contiguous() && out.size(0) == T_ && out.size(1) == (long)H * DV);
  TORCH_CHECK(gate.dim() == 2 && gate.size(0) == T_ && gate.size(1) == (long)H * DV &&
              gate.stride(1) == 1 && gate.scalar_type() == out.scalar_type());
  TORCH_CHECK(weight.numel() == (long)H * DV && weight.is_contiguous() &&
              weight.scalar_type() == out.scalar_type());
  hy_dispatch(out, "mlstm_out_norm_gate", [&]<typename T>() {
    hipLaunchKernelGGL(mlstm_out_norm_gate_kernel<T>, dim3(T_), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(out.data_ptr()), o.data_ptr<float>(),
                       floor_.data_ptr<float>(), reinterpret_cast<const T*>(weight.data_ptr()),
                       reinterpret_cast<const T*>(gate.data_ptr()), gate.stride(0), H, DV, (float)eps);
  });
}

void dual_norm_mean(at::Tensor out, at::Tensor a, at::Tensor w_a, at::Tensor b, at::Tensor w_b,
                    double eps) {
  HY_GPU(a);
  TORCH_CHECK(a.dim() == 2 && a.is_contiguous() && b.is_contiguous() && out.is_contiguous() &&
              b.sizes() == a.sizes() && out.sizes() == a.sizes());
  const long rows = a.size(0);
  const int W = a.size(1);
  if (rows == 0) return;
  const auto dt = a.scalar_type();
  TORCH_CHECK(b.scalar_type() == dt && out.scalar_type() == dt && w_a.scalar_type() == dt &&
              w_b.scalar_type() == dt && w_a.is_contiguous() && w_b.is_contiguous() &&
              w_a.numel() == W && w_b.numel() == W);
  if (dt == at::kBFloat16 && W % 8 == 0 && W <= 4 * 2048) {
    using bf = __hip_bfloat16;
    auto launch = [&]<int CH>() {
      hipLaunchKernelGGL(dual_norm_mean_vec_kernel<CH>, dim3(rows), dim3(256), 0, hy_stream(),
                         reinterpret_cast<bf*>(out.data_ptr()), reinterpret_cast<const bf*>(a.data_ptr()),
                         reinterpret_cast<const bf*>(w_a.data_ptr()),
                         reinterpret_cast<const bf*>(b.data_ptr()),
                         reinterpret_cast<const bf*>(w_b.data_ptr()), W, (float)eps);
    };
    if (W <= 2048) launch.template operator()<1>();
    else if (W <= 4096) launch.template operator()<2>();
    else launch.template operator()<4>();
    return;
  }
  hy_dispatch(a, "dual_norm_mean", [&]<typename T>() {
    hipLaunchKernelGGL(dual_norm_mean_kernel<T>, dim3(rows), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(out.data_ptr()), reinterpret_cast<const T*>(a.data_ptr()),
                       reinterpret_cast<const T*>(w_a.data_ptr()),
                       reinterpret_cast<const T*>(b.data_ptr()),
                       reinterpret_cast<const T*>(w_b.data_ptr()), W, (float)eps);
  });
}

void unary_act(at::Tensor out, at::Tensor in, int64_t act) {
  HY_GPU(in);
  TORCH_CHECK(in.is_contiguous() && out.is_contiguous() && out.sizes() == in.sizes() &&
              out.scalar_type() == in.scalar_type());
  TORCH_CHECK(act == kActRelu2 || act == kActGeluErf, "unknown activation");
  const long n = in.numel();
  if (n == 0) return;
  TORCH_CHECK(reinterpret_cast<uintptr_t>(in.data_ptr()) % 16 == 0 &&
              reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0, "unary_act: 16-byte aligned tensors");
  const int grid = (int)std::min<long>((n / 8 + 255) / 256 + 1, 8192);
  hy_dispatch(in, "unary_act", [&]<typename T>() {
    auto launch = [&]<int ACT>() {
      hipLaunchKernelGGL((unary_act_kernel<T, ACT>), dim3(grid), dim3(256), 0, hy_stream(),
                         reinterpret_cast<T*>(out.data_ptr()), reinterpret_cast<const T*>(in.data_ptr()), n);
    };
    if (act == kActRelu2) launch.template operator()<kActRelu2>();
    else launch.template operator()<kActGeluErf>();
  });
}

}  // namespace


TORCH_LIBRARY(llmq_amd_hybrid, m) {
  m.def("rmsnorm_cast(Tensor(a!) out, Tensor input, Tensor weight, float eps, float offset, int groups=1) -> ()");
  m.def("sandwich_norm_res32(Tensor(a!) x, Tensor(b!) residual, Tensor w_post, Tensor w_pre, float eps, float offset, int groups=1) -> ()");
  m.def("act_and_mul(Tensor(a!) out, Tensor input, bool gelu) -> ()");
  m.def("qknorm_vmix_cache(Tensor(a!) q, Tensor k, Tensor v, Tensor q_w, Tensor k_w, Tensor? v_first, float lam, Tensor(b!) k_cache, Tensor(c!) v_cache, Tensor slots, float eps) -> ()");
  m.def("paged_attn_prefill(Tensor(a!) out, Tensor q, Tensor? gate, Tensor k_cache, Tensor? v_cache, Tensor? bias, Tensor block_tables, Tensor cu_q, Tensor q_start, int max_q, int span, float scale, int mask_mode, int pos_stride, int bias_mode, int keep_first=0, Tensor? sink=None, float softcap=0.0) -> ()");
  m.def("paged_attn_decode(Tensor(a!) out, Tensor q, Tensor? gate, Tensor k_cache, Tensor? v_cache, Tensor? bias, Tensor block_tables, Tensor context_lens, int span, float scale, int mask_mode, int bias_mode, int keep_first=0, Tensor? sink=None, float softcap=0.0) -> ()");
  m.def("gla_recurrence(Tensor(a!) o, Tensor q, Tensor? k, Tensor v, Tensor z, Tensor z_bias, Tensor(b!) state, Tensor cu, Tensor slots, Tensor fresh, float tau, Tensor? lower, bool q_silu, float q_scale) -> ()");
  m.def("gla_out_norm_gate(Tensor(a!) out, Tensor o, Tensor weight, Tensor? gate, float eps) -> ()");
  m.def("latent_rope_pack(Tensor(a!) out, Tensor q, Tensor q_lat, Tensor ckr, Tensor c_w, Tensor inv_freq, Tensor positions, Tensor(b!) k_cache, Tensor slots, int dim, int rot_dims, bool interleaved, float eps) -> ()");
  m.def("gated_residual_add(Tensor(a!) out, Tensor(b!) res, Tensor y1, Tensor g1, Tensor b1, Tensor? y2, Tensor? g2, Tensor? b2) -> ()");
  m.def("side_gate_mul(Tensor(a!) out, Tensor a, Tensor table, Tensor tokens, int offset) -> ()");
  m.def("sigmoid_topk(Tensor(a!) idx, Tensor(b!) w, Tensor logits, int top) -> ()");
  m.def("moe_gate_up_gemv(Tensor(a!) hmid, Tensor h, Tensor idx, Tensor? w, Tensor gate_up, int act, float limit) -> ()");
  m.def("moe_down_gemv(Tensor(a!) y, Tensor hmid, Tensor idx, Tensor down, Tensor? wo) -> ()");
  m.def("moe_expert_gemv(Tensor(a!) out, Tensor input, Tensor idx, Tensor? w, Tensor weight, bool gate_up, int act, float limit) -> ()");
  m.def("moe_combine(Tensor(a!) y, Tensor yk, Tensor? wd) -> ()");
  m.def("moe_gather_combine(Tensor(a!) y, Tensor ys, Tensor pos, Tensor? w, int top) -> ()");
  m.def("embed_sinusoid(Tensor(a!) out, Tensor embedding, Tensor ids, Tensor positions, Tensor inv_freq) -> ()");
  m.def("scaled_add_norm(Tensor(a!) out, Tensor(b!) res, Tensor y, Tensor? y2, float a1, float a2, Tensor weight, float eps) -> ()");
  m.def("depth_mix_norm(Tensor(a!) out, Tensor(b!) stack, int n, Tensor coef, Tensor y, Tensor? y2, float a1, float a2, Tensor weight, float eps) -> ()");
  m.def("kv_scatter(Tensor k, Tensor v, Tensor(a!) k_cache, Tensor(b!) v_cache, Tensor slots) -> ()");
  m.def("mingru_scan(Tensor(a!) out, Tensor z, Tensor u, Tensor g, Tensor z_b, Tensor u_b, Tensor(b!) state, Tensor cu, Tensor slots, Tensor fresh) -> ()");
  m.def("causal_conv_silu(Tensor(a!) out, Tensor x, Tensor weight, Tensor? bias, Tensor(b!) tail, Tensor cu, Tensor slots, Tensor fresh, bool silu=True) -> ()");
  m.def("selective_scan(Tensor(a!) out, Tensor x, Tensor dt, Tensor dt_b, Tensor A, Tensor Bm, Tensor Cm, Tensor D, Tensor z, Tensor(b!) state, Tensor cu, Tensor slots, Tensor fresh) -> ()");
  m.def("softmax_topk(Tensor(a!) idx, Tensor(b!) w, Tensor logits, int top, float scale, Tensor? correction=None, bool renorm=False) -> ()");
  m.def("clamp_swish_mul(Tensor(a!) out, Tensor input, float limit) -> ()");
  m.def("qkv_norm_rope_cache(Tensor(a!) q, Tensor k, Tensor? v, Tensor? q_w, Tensor? k_w, Tensor? inv_freq, int rot_dims, Tensor positions, Tensor(b!) k_cache, Tensor(c!) v_cache, Tensor slots, float eps, bool v_unit_norm, Tensor? v_inv_freq) -> ()");
  m.def("rotate_heads(Tensor(a!) x, Tensor positions, Tensor inv_freq, bool inverse) -> ()");
  m.def("mlstm_gates(Tensor(a!) out, Tensor gates, float cap, Tensor(b!) m_state, Tensor cu, Tensor slots, Tensor fresh) -> ()");
  m.def("matrix_memory(Tensor(a!) o, Tensor q, Tensor k, Tensor v, Tensor decay, Tensor write, Tensor(b!) state, Tensor cu, Tensor slots, Tensor fresh, float q_scale) -> ()");
  m.def("mlstm_out_norm_gate(Tensor(a!) out, Tensor o, Tensor floor, Tensor weight, Tensor gate, float eps) -> ()");
  m.def("dual_norm_mean(Tensor(a!) out, Tensor a, Tensor w_a, Tensor b, Tensor w_b, float eps) -> ()");
  m.def("unary_act(Tensor(a!) out, Tensor input, int act) -> ()");
}

TORCH_LIBRARY_IMPL(llmq_amd_hybrid, CUDA, m) {
  m.impl("rmsnorm_cast", &rmsnorm_cast);
  m.impl("sandwich_norm_res32", &sandwich_norm_res32);
  m.impl("act_and_mul", &act_and_mul);
  m.impl("qknorm_vmix_cache", &qknorm_vmix_cache);
  m.impl("paged_attn_prefill", &paged_attn_prefill);
  m.impl("paged_attn_decode", &paged_attn_decode);
  m.impl("latent_rope_pack", &latent_rope_pack);
  m.impl("gated_residual_add", &gated_residual_add);
  m.impl("side_gate_mul", &side_gate_mul);
  m.impl("sigmoid_topk", &sigmoid_topk);
  m.impl("moe_gate_up_gemv", &moe_gate_up_gemv);
  m.impl("moe_down_gemv", &moe_down_gemv);
  m.impl("moe_expert_gemv", &moe_expert_gemv);
  m.impl("gla_recurrence", &gla_recurrence);
  m.impl("gla_out_norm_gate", &gla_out_norm_gate);
  m.impl("moe_combine", &moe_combine);
  m.impl("moe_gather_combine", &moe_gather_combine);
  m.impl("embed_sinusoid", &embed_sinusoid);
  m.impl("scaled_add_norm", &scaled_add_norm);
  m.impl("depth_mix_norm", &depth_mix_norm);
  m.impl("kv_scatter", &kv_scatter);
  m.impl("mingru_scan", &mingru_scan);
  m.impl("causal_conv_silu", &causal_conv_silu);
  m.impl("selective_scan", &selective_scan);
  m.impl("softmax_topk", &softmax_topk);
  m.impl("clamp_swish_mul", &clamp_swish_mul);
  m.impl("qkv_norm_rope_cache", &qkv_norm_rope_cache);
  m.impl("rotate_heads", &rotate_heads);
  m.impl("mlstm_gates", &mlstm_gates);
  m.impl("matrix_memory", &matrix_memory);
  m.impl("mlstm_out_norm_gate", &mlstm_out_norm_gate);
  m.impl("dual_norm_mean", &dual_norm_mean);
  m.impl("unary_act", &unary_act);
}

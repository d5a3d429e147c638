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

void rmsnorm_cast(at::Tensor out, at::Tensor in, at::Tensor weight, double eps, double offset) {
  HY_GPU(in);
  TORCH_CHECK(in.is_contiguous() && out.is_contiguous() && weight.is_contiguous());
  const int hidden = in.size(-1);
  TORCH_CHECK(out.sizes() == in.sizes() && weight.numel() == hidden);
  TORCH_CHECK(weight.scalar_type() == out.scalar_type(), "weight dtype must equal out dtype");
  const long rows = in.numel() / hidden;
  if (rows == 0) return;
  hy_dispatch(out, "rmsnorm_cast", [&]<typename TO>() {
    if (in.scalar_type() == at::kFloat) {
      hipLaunchKernelGGL((rmsnorm_cast_kernel<float, TO>), dim3(rows), dim3(256), 0, hy_stream(),
                         reinterpret_cast<TO*>(out.data_ptr()), in.data_ptr<float>(),
                         reinterpret_cast<const TO*>(weight.data_ptr()), hidden, (float)eps,
                         (float)offset);
    } else {
      TORCH_CHECK(in.scalar_type() == out.scalar_type(), "rmsnorm_cast: in must be fp32 or out's dtype");
      hipLaunchKernelGGL((rmsnorm_cast_kernel<TO, TO>), dim3(rows), dim3(256), 0, hy_stream(),
                         reinterpret_cast<TO*>(out.data_ptr()),
                         reinterpret_cast<const TO*>(in.data_ptr()),
                         reinterpret_cast<const TO*>(weight.data_ptr()), hidden, (float)eps,
                         (float)offset);
    }
  });
}

void sandwich_norm_res32(at::Tensor x, at::Tensor residual, at::Tensor w_post, at::Tensor w_pre,
                         double eps, double offset) {
  HY_GPU(x);
  TORCH_CHECK(x.is_contiguous() && residual.is_contiguous());
  TORCH_CHECK(residual.scalar_type() == at::kFloat, "residual must be fp32");
  const int hidden = x.size(-1);
  TORCH_CHECK(residual.sizes() == x.sizes() && w_post.numel() == hidden && w_pre.numel() == hidden);
  TORCH_CHECK(w_post.scalar_type() == x.scalar_type() && w_pre.scalar_type() == x.scalar_type());
  const long rows = x.numel() / hidden;
  if (rows == 0) return;
  if (x.scalar_type() == at::kBFloat16 && hidden % 8 == 0 && hidden <= 4 * 2048) {
    using bf = __hip_bfloat16;
    auto launch = [&]<int CH>() {
      hipLaunchKernelGGL(sandwich_norm_res32_vec_kernel<CH>, dim3(rows), dim3(256), 0, hy_stream(),
                         reinterpret_cast<bf*>(x.data_ptr()), residual.data_ptr<float>(),
                         reinterpret_cast<const bf*>(w_post.data_ptr()),
                         reinterpret_cast<const bf*>(w_pre.data_ptr()), hidden, (float)eps,
                         (float)offset);
    };
    if (hidden <= 2048) launch.template operator()<1>();
    else if (hidden <= 4096) launch.template operator()<2>();
    else launch.template operator()<4>();
    return;
  }
  hy_dispatch(x, "sandwich_norm_res32", [&]<typename T>() {
    hipLaunchKernelGGL(sandwich_norm_res32_kernel<T>, dim3(rows), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(x.data_ptr()), residual.data_ptr<float>(),
                       reinterpret_cast<const T*>(w_post.data_ptr()),
                       reinterpret_cast<const T*>(w_pre.data_ptr()), hidden, (float)eps,
                       (float)offset);
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

struct AttnDims { int H, G, D, DV, bs; };

AttnDims attn_check(const at::Tensor& out, const at::Tensor& q, const std::optional<at::Tensor>& gate,
                    const at::Tensor& k_cache, const at::Tensor& v_cache, const at::Tensor& bias,
                    const at::Tensor& block_tables, long span) {
  HY_GPU(q);
  TORCH_CHECK(q.dim() == 3 && out.dim() == 3, "q [T, H, D], out [T, H, DV]");
  HY_INNER(q); HY_INNER(out);
  AttnDims a{(int)q.size(1), (int)k_cache.size(1), (int)q.size(2), (int)v_cache.size(3),
             (int)k_cache.size(2)};
  TORCH_CHECK(q.stride(1) == a.D && out.stride(1) == a.DV, "heads must be packed");
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous());
  TORCH_CHECK(k_cache.size(3) == a.D && v_cache.size(1) == a.G && v_cache.size(2) == a.bs);
  TORCH_CHECK(out.size(0) == q.size(0) && out.size(1) == a.H && out.size(2) == a.DV);
  TORCH_CHECK(a.H % a.G == 0, "heads must be a multiple of kv heads");
  TORCH_CHECK(a.DV <= 256, "value size above 256 is not supported");
  TORCH_CHECK(span >= 1 && bias.scalar_type() == at::kFloat && bias.is_contiguous() &&
              bias.dim() == 2 && bias.size(0) == a.H && bias.size(1) >= 1 && bias.size(1) <= span,
              "bias must be fp32 [H, n], n = min(span, longest context the engine admits)");
  TORCH_CHECK(q.scalar_type() == out.scalar_type() && q.scalar_type() == k_cache.scalar_type() &&
              q.scalar_type() == v_cache.scalar_type());
  HY_I32(block_tables);
  TORCH_CHECK(block_tables.dim() == 2);
  if (gate.has_value()) {
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == q.size(0) && gate->size(1) == a.H &&
                gate->stride(1) == 1 && gate->scalar_type() == q.scalar_type(), "gate must be [T, H]");
  }
  return a;
}

template <typename F>
void dispatch_nv(int DV, F&& f) {
  if (DV <= 64) f.template operator()<1>();
  else if (DV <= 128) f.template operator()<2>();
  else f.template operator()<4>();
}

void chunk_bias_attn_prefill(at::Tensor out, at::Tensor q, const std::optional<at::Tensor>& gate,
                             at::Tensor k_cache, at::Tensor v_cache, at::Tensor bias,
                             at::Tensor block_tables, at::Tensor cu_q, at::Tensor q_start,
                             int64_t max_q, int64_t span, double scale) {
  if (q.size(0) == 0) return;
  const AttnDims a = attn_check(out, q, gate, k_cache, v_cache, bias, block_tables, span);
  HY_I32(cu_q); HY_I32(q_start);
  const int B = q_start.numel();
  TORCH_CHECK(cu_q.numel() == B + 1 && block_tables.size(0) == B && max_q >= 1);
  // bf16 with 16-byte-aligned q rows and key rows: the matrix-core kernel
  // (LLMQ_HYBRID_ATTN_VALU=1 keeps the fp32-ALU kernel, for A/B runs)
  static const bool force_valu = [] {
    const char* e = getenv("LLMQ_HYBRID_ATTN_VALU");
    return e && e[0] == '1';
  }();
  if (q.scalar_type() == at::kBFloat16 && !force_valu && a.D % 8 == 0 && a.D <= 256 &&
      q.stride(0) % 8 == 0 && reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0) {
    const int ksn = (a.D + 31) / 32, dtn = (a.DV + 15) / 16;
    const dim3 grid((max_q + kMfmaQT - 1) / kMfmaQT, a.H, B);
    using bf = __hip_bfloat16;
    auto launch = [&]<int KS, int DT>() {
      // K tile, V^T tile (all DT*16 channel rows), P hi/lo per wave, bias slice
      const size_t lds = sizeof(short) * ((size_t)kMfmaKT * (ksn * 32 + 8) +
                                          (size_t)DT * 16 * kMfmaKP +
                                          (size_t)4 * 2 * 16 * kMfmaKP) + 128 * sizeof(float);
      auto kern = chunk_bias_attn_prefill_mfma_kernel<KS, DT>;
      allow_lds(kern, lds);
      hipLaunchKernelGGL(kern, grid, dim3(256), lds, hy_stream(),
                         reinterpret_cast<bf*>(out.data_ptr()), out.stride(0),
                         reinterpret_cast<const bf*>(q.data_ptr()), q.stride(0),
                         gate.has_value() ? reinterpret_cast<const bf*>(gate->data_ptr()) : nullptr,
                         gate.has_value() ? gate->stride(0) : 0L,
                         reinterpret_cast<const bf*>(k_cache.data_ptr()),
                         reinterpret_cast<const bf*>(v_cache.data_ptr()), bias.data_ptr<float>(),
                         (int)bias.size(1),
                         block_tables.data_ptr<int>(), (int)block_tables.stride(0),
                         cu_q.data_ptr<int>(), q_start.data_ptr<int>(), a.H, a.G, a.D, a.DV, a.bs,
                         (int)span, (float)scale);
    };
    if (ksn <= 2 && dtn <= 4) launch.template operator()<2, 4>();
    else if (ksn <= 4 && dtn <= 8) launch.template operator()<4, 8>();
    else launch.template operator()<8, 16>();
    return;
  }
  const size_t lds = sizeof(float) * ((size_t)kAttnKT * (a.D + 1) + (size_t)kAttnKT * a.DV +
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
                         reinterpret_cast<const T*>(v_cache.data_ptr()), bias.data_ptr<float>(),
                         (int)bias.size(1),
                         block_tables.data_ptr<int>(), (int)block_tables.stride(0),
                         cu_q.data_ptr<int>(), q_start.data_ptr<int>(), a.H, a.G, a.D, a.DV, a.bs,
                         (int)span, (float)scale);
    });
  });
}

void chunk_bias_attn_decode(at::Tensor out, at::Tensor q, const std::optional<at::Tensor>& gate,
                            at::Tensor k_cache, at::Tensor v_cache, at::Tensor bias,
                            at::Tensor block_tables, at::Tensor context_lens, int64_t span,
                            double scale) {
  if (q.size(0) == 0) return;
  const AttnDims a = attn_check(out, q, gate, k_cache, v_cache, bias, block_tables, span);
  HY_I32(context_lens);
  const int B = q.size(0);
  TORCH_CHECK(context_lens.numel() == B && block_tables.size(0) == B);
  const size_t lds = sizeof(float) * ((size_t)a.D + 4 * 64 + 8 + 4 * (size_t)a.DV);
  hy_dispatch(q, "chunk_bias_attn_decode", [&]<typename T>() {
    dispatch_nv(a.DV, [&]<int NV>() {
      auto kern = chunk_bias_attn_decode_kernel<T, NV>;
      allow_lds(kern, lds);
      hipLaunchKernelGGL(kern, dim3(a.H, B), dim3(256), lds, hy_stream(),
                         reinterpret_cast<T*>(out.data_ptr()), out.stride(0),
                         reinterpret_cast<const T*>(q.data_ptr()), q.stride(0),
                         gate.has_value() ? reinterpret_cast<const T*>(gate->data_ptr()) : nullptr,
                         gate.has_value() ? gate->stride(0) : 0L,
                         reinterpret_cast<const T*>(k_cache.data_ptr()),
                         reinterpret_cast<const T*>(v_cache.data_ptr()), bias.data_ptr<float>(),
                         (int)bias.size(1),
                         block_tables.data_ptr<int>(), (int)block_tables.stride(0),
                         context_lens.data_ptr<int>(), a.H, a.G, a.D, a.DV, a.bs, (int)span,
                         (float)scale);
    });
  });
}

// q, k, z: [T, H, D]; v: [T, H, DV] (row-strided views); o: [T, H, DV] fp32;
// state: [slots, H, D, DV] fp32.
void gla_recurrence(at::Tensor o, at::Tensor q, at::Tensor k, at::Tensor v, at::Tensor z,
                    at::Tensor z_bias, at::Tensor state, at::Tensor cu, at::Tensor slots,
                    at::Tensor fresh, double tau) {
  HY_GPU(q);
  const long T_ = q.size(0);
  if (T_ == 0) return;
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3 && z.dim() == 3 && o.dim() == 3);
  HY_INNER(q); HY_INNER(k); HY_INNER(v); HY_INNER(z);
  const int H = q.size(1), D = q.size(2), DV = v.size(2);
  TORCH_CHECK(k.sizes() == q.sizes() && z.sizes() == q.sizes());
  TORCH_CHECK(v.size(0) == T_ && v.size(1) == H);
  TORCH_CHECK(q.stride(1) == D && k.stride(1) == D && z.stride(1) == D && v.stride(1) == DV,
              "heads must be packed");
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
  const float q_scale = 1.0f / sqrtf((float)D);
  hy_dispatch(q, "gla_recurrence", [&]<typename T>() {
    auto launch = [&]<int DPL>() {
      hipLaunchKernelGGL((gla_recurrence_kernel<T, DPL>), grid, dim3(256), 0, hy_stream(),
                         o.data_ptr<float>(),
                         reinterpret_cast<const T*>(q.data_ptr()), q.stride(0),
                         reinterpret_cast<const T*>(k.data_ptr()), k.stride(0),
                         reinterpret_cast<const T*>(v.data_ptr()), v.stride(0),
                         reinterpret_cast<const T*>(z.data_ptr()), z.stride(0),
                         z_bias.data_ptr<float>(), state.data_ptr<float>(), cu.data_ptr<int>(),
                         slots.data_ptr<int>(), fresh.data_ptr<int>(), H, D, DV,
                         (float)(1.0 / tau), q_scale);
    };
    if (D <= 32) launch.template operator()<2>();
    else if (D <= 64) launch.template operator()<4>();
    else if (D <= 128) launch.template operator()<8>();
    else launch.template operator()<16>();
  });
}

void gla_out_norm_gate(at::Tensor out, at::Tensor o, at::Tensor weight, at::Tensor gate, double eps) {
  HY_GPU(o);
  TORCH_CHECK(o.dim() == 3 && o.scalar_type() == at::kFloat && o.is_contiguous());
  const long T_ = o.size(0);
  if (T_ == 0) return;
  const int H = o.size(1), DV = o.size(2);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T_ && out.size(1) == (long)H * DV && out.stride(1) == 1);
  TORCH_CHECK(gate.dim() == 2 && gate.size(0) == T_ && gate.size(1) == (long)H * DV && gate.stride(1) == 1);
  TORCH_CHECK(weight.numel() == DV && weight.is_contiguous());
  TORCH_CHECK(gate.scalar_type() == out.scalar_type() && weight.scalar_type() == out.scalar_type());
  hy_dispatch(out, "gla_out_norm_gate", [&]<typename T>() {
    hipLaunchKernelGGL(gla_out_norm_gate_kernel<T>, dim3(T_), dim3(256), 0, hy_stream(),
                       reinterpret_cast<T*>(out.data_ptr()), out.stride(0), o.data_ptr<float>(),
                       reinterpret_cast<const T*>(weight.data_ptr()),
                       reinterpret_cast<const T*>(gate.data_ptr()), gate.stride(0), H, DV,
                       (float)eps);
  });
}

}  // namespace

TORCH_LIBRARY(llmq_amd_hybrid, m) {
  m.def("rmsnorm_cast(Tensor(a!) out, Tensor input, Tensor weight, float eps, float offset) -> ()");
  m.def("sandwich_norm_res32(Tensor(a!) x, Tensor(b!) residual, Tensor w_post, Tensor w_pre, float eps, float offset) -> ()");
  m.def("act_and_mul(Tensor(a!) out, Tensor input, bool gelu) -> ()");
  m.def("qknorm_vmix_cache(Tensor(a!) q, Tensor k, Tensor v, Tensor q_w, Tensor k_w, Tensor? v_first, float lam, Tensor(b!) k_cache, Tensor(c!) v_cache, Tensor slots, float eps) -> ()");
  m.def("chunk_bias_attn_prefill(Tensor(a!) out, Tensor q, Tensor? gate, Tensor k_cache, Tensor v_cache, Tensor bias, Tensor block_tables, Tensor cu_q, Tensor q_start, int max_q, int span, float scale) -> ()");
  m.def("chunk_bias_attn_decode(Tensor(a!) out, Tensor q, Tensor? gate, Tensor k_cache, Tensor v_cache, Tensor bias, Tensor block_tables, Tensor context_lens, int span, float scale) -> ()");
  m.def("gla_recurrence(Tensor(a!) o, Tensor q, Tensor k, Tensor v, Tensor z, Tensor z_bias, Tensor(b!) state, Tensor cu, Tensor slots, Tensor fresh, float tau) -> ()");
  m.def("gla_out_norm_gate(Tensor(a!) out, Tensor o, Tensor weight, Tensor gate, float eps) -> ()");
}

TORCH_LIBRARY_IMPL(llmq_amd_hybrid, CUDA, m) {
  m.impl("rmsnorm_cast", &rmsnorm_cast);
  m.impl("sandwich_norm_res32", &sandwich_norm_res32);
  m.impl("act_and_mul", &act_and_mul);
  m.impl("qknorm_vmix_cache", &qknorm_vmix_cache);
  m.impl("chunk_bias_attn_prefill", &chunk_bias_attn_prefill);
  m.impl("chunk_bias_attn_decode", &chunk_bias_attn_decode);
  m.impl("gla_recurrence", &gla_recurrence);
  m.impl("gla_out_norm_gate", &gla_out_norm_gate);
}

// C ABI of the MFMA GEMM family: argument checks, epilogue selection and the static scratch buffer.
// The kernels, epilogues and launch heuristics live in gemm_impl.h.
#include <cstring>

#include "gemm_impl.h"
#include "gemm_w4.h"

namespace ttmi {

// ------------------------------------------------------------ static scratch buffer -----
// Partial tiles of ttmi_gemm_bias_layer_norm_static: device memory that exists from module load to
// process end on every GPU the library runs on, so that entry point never allocates.  In host code
// the array's name is only a handle: the device address is asked for once per device, with that
// device current, and kept; kernels and fills get that pointer.
constexpr size_t kStaticScratchBytes = TTMI_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static int static_scratch(float** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static float* ptrs[kMaxDevices] = {};
  int dev = 0;
  TTMI_HIP(hipGetDevice(&dev));
  TTMI_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal out of range");
  std::lock_guard<std::mutex> lock(mu);
  if (ptrs[dev] == nullptr) {
    void* p = nullptr;
    TTMI_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    TTMI_REQUIRE(p != nullptr, "the static scratch buffer has no device address");
    ptrs[dev] = static_cast<float*>(p);
  }
  *out = ptrs[dev];
  return 0;
}

static int gemm_bias_layer_norm_impl(const void* a, const void* w, void* out, const void* residual, const float* residual_f32,
                              const void* bias, const void* gamma, const void* beta, float* out_f32, int64_t m, int64_t n,
                              int64_t k, float eps, int dtype, void* stream) {
  TTMI_REQUIRE(a && w && out && bias && gamma && beta, "null tensor");
  TTMI_REQUIRE((residual_f32 != nullptr) == (out_f32 != nullptr), "residual_f32 and out_f32 go together");
  TTMI_REQUIRE(residual != nullptr || residual_f32 != nullptr, "a residual is required");
  // Large problems write the bare product to `out` before the residual is read.
  TTMI_REQUIRE(out != residual && out != a, "out must not alias residual or a");
  TTMI_REQUIRE(m >= 0 && n >= 0 && m < (1ll << 31) && n < (1ll << 31) && k < (1ll << 31), "dimension out of range");
  if (m == 0 || n == 0) return 0;
  TTMI_REQUIRE(k > 0, "K must be positive");
  hipStream_t s = (hipStream_t)stream;
  TTMI_DISPATCH_FLOAT(dtype, T, {
    constexpr int KPC = 16 / sizeof(T);
    const bool aligned = aligned16(a) && aligned16(w) && k % KPC == 0;
    auto aligned_rows = [&](const void* p, size_t elem) { return (reinterpret_cast<uintptr_t>(p) % (4 * elem)) == 0; };
    const bool rows_ok = n % 4 == 0 && n <= 4096 && aligned_rows(out, sizeof(T)) && aligned_rows(bias, sizeof(T)) &&
                         aligned_rows(gamma, sizeof(T)) && aligned_rows(beta, sizeof(T)) &&
                         (residual_f32 != nullptr ? aligned16(residual_f32) && aligned16(out_f32) : aligned_rows(residual, sizeof(T)));
    const SplitPlan plan = rows_ok ? plan_split<T>(m, n, k, 1, aligned) : SplitPlan{SplitKind::kNone, 1};
    GemmArgs g{};
    g.a = (const char*)a;
    g.b = (const char*)w;
    g.m = (int)m; g.n = (int)n; g.k = (int)k;
    g.lda = k; g.ldb = k;
    g.inner = 1;
    int large_tile_slices = 0;
    if constexpr (sizeof(T) == 2) {
      if (rows_ok) large_tile_slices = w4_splitk_slices<T>(g, aligned);
      // These slices are an optimisation of a product that also runs whole.  Where the caller has fixed the
      // workspace (the static entry point) and the partial products do not fit it, the product runs whole instead of
      // being refused.
      if (large_tile_slices > 1 && tl_fixed_workspace.ptr != nullptr &&
          (size_t)large_tile_slices * (size_t)m * (size_t)n * sizeof(float) > tl_fixed_workspace.bytes)
        large_tile_slices = 0;
    }
    if (plan.kind != SplitKind::kNone || large_tile_slices > 1) {
      auto reduce = [&](const float* ws, int slices, bool, hipStream_t st) {
        auto launch = [&](auto iters) {
          hipLaunchKernelGGL((splitk_reduce_layer_norm_kernel<T, decltype(iters)::value>), dim3((unsigned)m), dim3(256), 0, st, ws,
                             slices, (int)m, (int)n, (const T*)bias, (const T*)residual, residual_f32, (const T*)gamma,
                             (const T*)beta, (T*)out, out_f32, eps);
        };
        if (n <= 1024) launch(std::integral_constant<int, 1>{});
        else if (n <= 2048) launch(std::integral_constant<int, 2>{});
        else launch(std::integral_constant<int, 4>{});
      };
      constexpr int BK = kRowBytes / sizeof(T);
      if constexpr (sizeof(T) == 2) {
        if (large_tile_slices > 1) return (launch_w4_splitk<T>(g, large_tile_slices, s, reduce));
      }
      if (plan.kind == SplitKind::kDmaTiles) return (launch_fast_splitk<T>(g, plan.splits, k / BK, BK, s, reduce));
      return (launch_splitk<T>(g, plan.splits, k / BK, BK, s, reduce));
    }
  });
  // Large problems: the GEMM kernel's own tiles cover the chip; LayerNorm follows as its own pass.
  // With an fp32 residual stream and room for it, the product stays in fp32 too: the GEMM stores its accumulators to
  // out_f32 and the LayerNorm pass reads them there, so that (as in the K-sliced path above) nothing is rounded
  // between the matrix pipe and the normalisation.
  if (residual_f32 != nullptr && out_f32 != residual_f32 && dtype != TTMI_F32) {
    ttmi_epilogue_args f32_args{};
    const int rc = ttmi_gemm_fused(a, w, out_f32, m, n, k, k, k, n, TTMI_EPI_F32_OUT, &f32_args, dtype, stream);
    if (rc != 0) return rc;
    return ttmi_add_bias_layer_norm_product32(out, residual_f32, bias, gamma, beta, out_f32, m, n, eps, dtype, stream);
  }
  const int rc = ttmi_gemm(a, w, out, m, n, k, k, k, n, 1, 1.f, 0.f, dtype, stream);
  if (rc != 0) return rc;
  if (residual_f32 != nullptr)
    return ttmi_add_bias_layer_norm_residual32(out, residual_f32, bias, gamma, beta, out_f32, m, n, eps, dtype, stream);
  return ttmi_add_bias_layer_norm(out, residual, bias, gamma, beta, m, n, eps, dtype, stream);
}

}  // namespace ttmi

using namespace ttmi;

extern "C" {

int ttmi_gemm(const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
              int64_t ldc, int trans_b, float alpha, float beta, int dtype, void* stream) {
  TTMI_REQUIRE(a && b && c, "null matrix");
  TTMI_REQUIRE(lda >= k && ldc >= n && ldb >= (trans_b ? k : n), "leading dimension too small");
  TTMI_DISPATCH_FLOAT(dtype, T, return gemm_alpha_beta<T>(a, b, c, m, n, k, lda, ldb, ldc, 1, 0, 0, 0, 0, 0, 0, 1,
                                                          trans_b, alpha, beta, (hipStream_t)stream));
  return 0;
}

int ttmi_gemm_strided_batched(const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k, int64_t lda,
                              int64_t ldb, int64_t ldc, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                              int64_t batch_count, int trans_b, float alpha, float beta, int dtype, void* stream) {
  TTMI_REQUIRE(a && b && c, "null matrix");
  TTMI_REQUIRE(lda >= k && ldc >= n && ldb >= (trans_b ? k : n), "leading dimension too small");
  TTMI_REQUIRE(batch_count >= 0 && batch_count < 65536, "batch_count out of range");
  TTMI_DISPATCH_FLOAT(dtype, T, return gemm_alpha_beta<T>(a, b, c, m, n, k, lda, ldb, ldc, 1, stride_a, 0, stride_b,
                                                          0, stride_c, 0, batch_count, trans_b, alpha, beta,
                                                          (hipStream_t)stream));
  return 0;
}

int ttmi_gemm_batched_heads(const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k, int64_t lda,
                            int64_t ldb, int64_t ldc, int64_t heads, int64_t a_batch, int64_t a_head,
                            int64_t b_batch, int64_t b_head, int64_t c_batch, int64_t c_head, int64_t batch,
                            int trans_b, float alpha, float beta, int dtype, void* stream) {
  TTMI_REQUIRE(a && b && c, "null matrix");
  TTMI_REQUIRE(heads > 0 && batch >= 0 && batch * heads < 65536, "batch*heads out of range");
  TTMI_DISPATCH_FLOAT(dtype, T, return gemm_alpha_beta<T>(a, b, c, m, n, k, lda, ldb, ldc, (int)heads, a_batch,
                                                          a_head, b_batch, b_head, c_batch, c_head, batch * heads,
                                                          trans_b, alpha, beta, (hipStream_t)stream));
  return 0;
}

int ttmi_gemm_fused(const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k, int64_t lda,
                    int64_t ldb, int64_t ldc, int epilogue, const ttmi_epilogue_args* args, int dtype,
                    void* stream) {
  TTMI_REQUIRE(a && b && args, "null argument");
  TTMI_REQUIRE(m < (1ll << 31) && n < (1ll << 31) && k < (1ll << 31), "dimension too large");
  TTMI_REQUIRE(lda >= k && ldb >= k, "leading dimension too small");
  hipStream_t s = (hipStream_t)stream;
  GemmArgs g{};
  g.a = (const char*)a;
  g.b = (const char*)b;
  g.m = (int)m; g.n = (int)n; g.k = (int)k;
  g.lda = lda; g.ldb = ldb;
  g.inner = 1;
  TTMI_DISPATCH_FLOAT(dtype, T, {
    constexpr int KPC = 16 / sizeof(T);
    const bool aligned = aligned16(a) && aligned16(b) && lda % KPC == 0 && ldb % KPC == 0 && k % KPC == 0;
    const bool c_vec = aligned16(c) && ldc % KPC == 0 && aligned16(args->bias) && aligned16(args->residual);
    const bool qkv_vec = aligned16(args->q) && aligned16(args->k) && aligned16(args->v) && aligned16(args->bias) &&
                         args->head_dim % 8 == 0;
    switch (epilogue) {
      case TTMI_EPI_BIAS: {
        TTMI_REQUIRE(c && args->bias && ldc >= n, "BIAS epilogue needs c and bias");
        EpiBias<T, 0, false, false> epi{(T*)c, (const T*)args->bias, nullptr, ldc, c_vec};
        return (launch_gemm<T, false>(g, epi, 1, aligned, s));
      }
      case TTMI_EPI_BIAS_ACT: {
        TTMI_REQUIRE(c && args->bias && ldc >= n, "BIAS_ACT epilogue needs c and bias");
        if (args->act == TTMI_ACT_GELU) {
          EpiBias<T, TTMI_ACT_GELU, true, false> epi{(T*)c, (const T*)args->bias, nullptr, ldc, c_vec};
          return (launch_gemm<T, false>(g, epi, 1, aligned, s));
        } else if (args->act == TTMI_ACT_TANH) {
          EpiBias<T, TTMI_ACT_TANH, true, false> epi{(T*)c, (const T*)args->bias, nullptr, ldc, c_vec};
          return (launch_gemm<T, false>(g, epi, 1, aligned, s));
        } else if (args->act == TTMI_ACT_RELU) {
          EpiBias<T, TTMI_ACT_RELU, true, false> epi{(T*)c, (const T*)args->bias, nullptr, ldc, c_vec};
          return (launch_gemm<T, false>(g, epi, 1, aligned, s));
        }
        return fail(TTMI_EINVAL, "unknown activation");
      }
      case TTMI_EPI_F32_OUT: {
        TTMI_REQUIRE(c && ldc >= n, "F32_OUT epilogue needs c");
        EpiF32<T> epi{(float*)c, (const T*)args->bias, ldc, aligned16(c) && ldc % 4 == 0 && aligned16(args->bias)};
        return (launch_gemm<T, false>(g, epi, 1, aligned, s));
      }
      case TTMI_EPI_BIAS_RESIDUAL: {
        TTMI_REQUIRE(c && args->bias && args->residual && ldc >= n, "BIAS_RESIDUAL epilogue needs c, bias, residual");
        EpiBias<T, 0, false, true> epi{(T*)c, (const T*)args->bias, (const T*)args->residual, ldc, c_vec};
        return (launch_gemm<T, false>(g, epi, 1, aligned, s));
      }
      case TTMI_EPI_QKV_SPLIT:
      case TTMI_EPI_QKV_SPLIT_PAD: {
        const bool pad = epilogue == TTMI_EPI_QKV_SPLIT_PAD;
        TTMI_REQUIRE(args->seq > 0 && args->heads > 0 && args->head_dim > 0, "QKV epilogue needs seq/heads/head_dim");
        const bool single = n == args->heads * args->head_dim;  // one projection: only q is written
        TTMI_REQUIRE(single || n == 3 * args->heads * args->head_dim, "N must be heads*head_dim or 3*heads*head_dim");
        TTMI_REQUIRE(args->q && args->bias && (single || (args->k && args->v)), "QKV epilogue needs q, k, v, bias");
        TTMI_REQUIRE(!single || args->v_seq_pitch == 0, "v_seq_pitch needs the three-way split");
        if (pad) TTMI_REQUIRE(args->token_rows != nullptr && args->batch > 0, "padded QKV epilogue needs token_rows and batch");
        else TTMI_REQUIRE(m % args->seq == 0, "M must be a multiple of seq");
        const int hidden = (int)(args->heads * args->head_dim);
        const int64_t vp = args->v_seq_pitch;
        TTMI_REQUIRE(vp == 0 || (vp >= args->seq && vp % 8 == 0 && vp < (1ll << 31) && hidden % 8 == 0),
                     "v_seq_pitch must be 0 or a multiple of 8 that is >= seq (hidden a multiple of 8)");
        if (pad) {
          EpiQkvSplit<T, true> epi{(T*)args->q, (T*)args->k, (T*)args->v, (const T*)args->bias, args->token_rows,
                                   (int)args->seq, (int)args->heads, (int)args->head_dim, hidden,
                                   FastDiv((uint32_t)args->seq), FastDiv((uint32_t)hidden), FastDiv((uint32_t)args->head_dim), qkv_vec, (int)vp};
          return (launch_gemm<T, false>(g, epi, 1, aligned, s));
        }
        EpiQkvSplit<T, false> epi{(T*)args->q, (T*)args->k, (T*)args->v, (const T*)args->bias, nullptr,
                                  (int)args->seq, (int)args->heads, (int)args->head_dim, hidden,
                                  FastDiv((uint32_t)args->seq), FastDiv((uint32_t)hidden), FastDiv((uint32_t)args->head_dim), qkv_vec, (int)vp};
        return (launch_gemm<T, false>(g, epi, 1, aligned, s));
      }
      default:
        return fail(TTMI_EINVAL, "unknown epilogue");
    }
  });
  return 0;
}

int ttmi_gemm_describe(int64_t m, int64_t n, int64_t k, int epilogue, const ttmi_epilogue_args* args, int dtype, char* out,
                       size_t capacity) {
  TTMI_REQUIRE(out != nullptr && capacity > 0, "no room for the answer");
  // operands that pass every alignment test; nothing dereferences them in a dry run
  void* fake = reinterpret_cast<void*>((uintptr_t)1 << 20);
  ttmi_epilogue_args filled{};
  if (args != nullptr) filled = *args;
  filled.bias = fake;
  filled.residual = fake;
  filled.q = filled.k = filled.v = fake;
  if (epilogue == TTMI_EPI_QKV_SPLIT_PAD) filled.token_rows = static_cast<const int32_t*>(fake);
  std::string name;
  struct Install {
    explicit Install(std::string* p) { tl_describe = p; }
    ~Install() { tl_describe = nullptr; }
  } install(&name);
  const int rc = epilogue == TTMI_EPI_NONE ? ttmi_gemm(fake, fake, fake, m, n, k, k, k, n, 1, 1.f, 0.f, dtype, nullptr)
                                           : ttmi_gemm_fused(fake, fake, fake, m, n, k, k, k, n, epilogue, &filled, dtype, nullptr);
  if (rc != 0) return rc;
  TTMI_REQUIRE(name.size() < capacity, "the answer does not fit");
  std::memcpy(out, name.c_str(), name.size() + 1);
  return 0;
}

int ttmi_gemm_bias_layer_norm(const void* a, const void* w, void* out, const void* residual, const float* residual_f32,
                              const void* bias, const void* gamma, const void* beta, float* out_f32, int64_t m, int64_t n,
                              int64_t k, float eps, int dtype, void* stream) {
  return gemm_bias_layer_norm_impl(a, w, out, residual, residual_f32, bias, gamma, beta, out_f32, m, n, k, eps, dtype, stream);
}

int ttmi_gemm_bias_layer_norm_static(const void* a, const void* w, void* out, const void* residual,
                                     const float* residual_f32, const void* bias, const void* gamma, const void* beta,
                                     float* out_f32, int64_t m, int64_t n, int64_t k, float eps, int dtype, void* stream) {
  float* ws = nullptr;
  {
    const int rc = static_scratch(&ws);
    if (rc != 0) return rc;
  }
  // Every split-K launch below this call takes its partial tiles from the static buffer, or is refused.  (The
  // switch lowers the size that is admitted, so that tests reach the refusal with problems of ordinary size.)
  size_t capacity = kStaticScratchBytes;
  const int limit = kernel_switch(kSwitchStaticScratchLimit);
  if (limit >= 0) capacity = std::min(capacity, (size_t)limit);
  struct Install {
    Install(float* p, size_t bytes) { tl_fixed_workspace = FixedWorkspace{p, bytes}; }
    ~Install() { tl_fixed_workspace = FixedWorkspace{}; }
  } install(ws, capacity);
  return gemm_bias_layer_norm_impl(a, w, out, residual, residual_f32, bias, gamma, beta, out_f32, m, n, k, eps, dtype, stream);
}

int ttmi_gemm_i8(const int8_t* a, const int8_t* b, int32_t* c, int64_t m, int64_t n, int64_t k, int64_t lda,
                 int64_t ldb, int64_t ldc, void* stream) {
  TTMI_REQUIRE(a && b && c, "null matrix");
  TTMI_REQUIRE(m < (1ll << 31) && n < (1ll << 31) && k < (1ll << 31), "dimension too large");
  TTMI_REQUIRE(lda >= k && ldb >= k && ldc >= n, "leading dimension too small");
  GemmArgs g{};
  g.a = (const char*)a;
  g.b = (const char*)b;
  g.m = (int)m; g.n = (int)n; g.k = (int)k;
  g.lda = lda; g.ldb = ldb;
  g.inner = 1;
  EpiInt32 epi{c, ldc, aligned16(c) && ldc % 4 == 0};
  const bool aligned = aligned16(a) && aligned16(b) && lda % 16 == 0 && ldb % 16 == 0 && k % 16 == 0;
  return launch_gemm<int8_t, false>(g, epi, 1, aligned, (hipStream_t)stream);
}

static int gemm_i8_dequant_impl(const int8_t* a, const int8_t* b, float* c, const float* act_scale_dev, const float* w_scale,
                                const float* bias, int act, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                                int64_t ldc, float* absmax_slots, void* stream) {
  TTMI_REQUIRE(a && b && c && act_scale_dev && w_scale, "null tensor");
  TTMI_REQUIRE(act >= TTMI_ACT_NONE && act <= TTMI_ACT_RELU, "unknown activation");
  TTMI_REQUIRE(m < (1ll << 31) && n < (1ll << 31) && k < (1ll << 31), "dimension too large");
  TTMI_REQUIRE(lda >= k && ldb >= k && ldc >= n, "leading dimension too small");
  GemmArgs g{};
  g.a = (const char*)a;
  g.b = (const char*)b;
  g.m = (int)m; g.n = (int)n; g.k = (int)k;
  g.lda = lda; g.ldb = ldb;
  g.inner = 1;
  EpiDequant epi{c, act_scale_dev, w_scale, bias, ldc, aligned16(c) && ldc % 4 == 0, act, absmax_slots};
  const bool aligned = aligned16(a) && aligned16(b) && lda % 16 == 0 && ldb % 16 == 0 && k % 16 == 0;
  return launch_gemm<int8_t, false>(g, epi, 1, aligned, (hipStream_t)stream);
}

int ttmi_gemm_i8_dequant(const int8_t* a, const int8_t* b, float* c, const float* act_scale_dev, const float* w_scale,
                         const float* bias, int act, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb, int64_t ldc,
                         void* stream) {
  return gemm_i8_dequant_impl(a, b, c, act_scale_dev, w_scale, bias, act, m, n, k, lda, ldb, ldc, nullptr, stream);
}

int ttmi_gemm_i8_dequant_absmax(const int8_t* a, const int8_t* b, float* c, const float* act_scale_dev, const float* w_scale,
                                const float* bias, int act, int64_t m, int64_t n, int64_t k, int64_t lda, int64_t ldb,
                                int64_t ldc, float* absmax_slots, int* slots_written, void* stream) {
  TTMI_REQUIRE(absmax_slots && slots_written, "null absmax arguments");
  static_assert(kAbsmaxSlots == TTMI_ABSMAX_SLOTS, "slot count of the C ABI");
  tl_absmax_written = 0;
  *slots_written = 0;
  if (m <= 0 || n <= 0) return 0;
  const int rc = gemm_i8_dequant_impl(a, b, c, act_scale_dev, w_scale, bias, act, m, n, k, lda, ldb, ldc, absmax_slots, stream);
  *slots_written = rc == 0 ? tl_absmax_written : 0;
  return rc;
}

int ttmi_gemm_i8_dequant_qkv_split(const int8_t* a, const int8_t* b, const float* act_scale_dev, const float* w_scale,
                                   const float* bias, float* q, float* k_out, float* v, int64_t m, int64_t n, int64_t k,
                                   int64_t lda, int64_t ldb, int64_t seq, int64_t heads, int64_t head_dim, void* stream) {
  TTMI_REQUIRE(a && b && act_scale_dev && w_scale && bias && q && k_out && v, "null tensor");
  TTMI_REQUIRE(m < (1ll << 31) && n < (1ll << 31) && k < (1ll << 31), "dimension too large");
  TTMI_REQUIRE(lda >= k && ldb >= k, "leading dimension too small");
  TTMI_REQUIRE(seq > 0 && heads > 0 && head_dim > 0 && n == 3 * heads * head_dim, "N must be 3*heads*head_dim");
  TTMI_REQUIRE(m % seq == 0, "M must be a multiple of seq");
  GemmArgs g{};
  g.a = (const char*)a;
  g.b = (const char*)b;
  g.m = (int)m; g.n = (int)n; g.k = (int)k;
  g.lda = lda; g.ldb = ldb;
  g.inner = 1;
  const int hidden = (int)(heads * head_dim);
  const bool vec = aligned16(q) && aligned16(k_out) && aligned16(v) && head_dim % 8 == 0;
  EpiDequantQkvSplit epi{{q, k_out, v, bias, nullptr, (int)seq, (int)heads, (int)head_dim, hidden, FastDiv((uint32_t)seq),
                          FastDiv((uint32_t)hidden), FastDiv((uint32_t)head_dim), vec, 0},
                         act_scale_dev, w_scale};
  const bool aligned = aligned16(a) && aligned16(b) && lda % 16 == 0 && ldb % 16 == 0 && k % 16 == 0;
  return launch_gemm<int8_t, false>(g, epi, 1, aligned, (hipStream_t)stream);
}

}  // extern "C"

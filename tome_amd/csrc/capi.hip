// extern "C" surface of libtome_logprob.so (declared in include/tome_logprob.h): argument
// checks on the host, then the kernel launchers.  Nothing here allocates device memory.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "../../include/tome_logprob.h"

namespace tome {
hipError_t row_logprob_launch(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                              const int32_t* targets, const int32_t* row_valid, float temperature,
                              float* out_lp, float* out_lse, float* out_entropy, int32_t* out_argmax,
                              void* workspace, hipStream_t stream);
hipError_t row_logprob_launch_rows(const void* logits, int dtype, int64_t n_rows, const int32_t* row_index, int64_t rows,
                                   int64_t V, int64_t row_stride, const int32_t* targets, const int32_t* row_valid,
                                   float temperature, float* out_lp, float* out_lse, float* out_entropy,
                                   int32_t* out_argmax, void* workspace, hipStream_t stream);
int row_splits_for(int64_t rows, int64_t V, int vec);
size_t row_scratch_set_limit(size_t bytes);
hipError_t row_logprob_noalloc_launch(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                                      const int32_t* targets, const int32_t* row_valid, float temperature,
                                      float* out_lp, float* out_lse, float* out_entropy, int32_t* out_argmax,
                                      bool* too_big, hipStream_t stream);
hipError_t row_lse_partials_launch(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                                   float temperature, float* out_lse, void* workspace, int* splits, hipStream_t stream);
hipError_t full_log_softmax_launch(const void* in, void* out, int dtype, int64_t rows, int64_t V,
                                   int64_t in_stride, int64_t out_stride, float temperature,
                                   float* row_lse, const void* partials, int splits, hipStream_t stream);
bool full_log_softmax_one_pass(const void* in, const void* out, int dtype, int64_t rows, int64_t V, int64_t in_stride, int64_t out_stride);
hipError_t full_log_softmax_onepass_launch(const void* in, void* out, int64_t rows, int64_t V, int64_t in_stride,
                                           int64_t out_stride, float temperature, float* row_lse, hipStream_t stream);
hipError_t row_sample_launch(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                             const float* uniforms, const int32_t* row_valid, float temperature, int top_k,
                             int32_t* out_token, float* out_lp, float* out_lse, int32_t* out_argmax,
                             int32_t* out_topk_idx, float* out_topk_logit, void* workspace, hipStream_t stream);
size_t row_sample_workspace_bytes(int64_t rows, int64_t V, int dtype_vec, int top_k);
size_t fused_workspace_bytes(int64_t n_tokens, int64_t H, int64_t V, int n_weights, bool with_norm);
bool fused_needs_32bit_extents(int64_t n_tokens, int64_t H, int64_t V);
void fused_force_kernel(int kind);
hipError_t fused_lmhead_launch(const void* hidden, const void* norm_weight, float norm_eps, const void* w0,
                               const void* w1, int64_t n_tokens, int64_t H, int64_t V, int64_t hidden_stride,
                               int64_t weight_stride, const int32_t* targets,
                               const int32_t* row_valid, float temperature, float* out_lp, float* out_lse,
                               float* out_entropy, int32_t* out_argmax, float* out_ref_lp, float* out_k3,
                               void* workspace, hipStream_t stream);
hipError_t fused_pair_launch(const void* hidden, const void* hidden_ref, const void* norm_weight, float norm_eps,
                             const void* w0, const void* w1, int64_t n_tokens, int64_t H, int64_t V,
                             int64_t hidden_stride, int64_t weight_stride, const int32_t* targets,
                             const int32_t* row_valid, float temperature, float* out_lp, float* out_entropy,
                             float* out_ref_lp, float* out_k3, void* workspace, hipStream_t stream);
hipError_t mfma_probe_launch(const void* operands, int n_workgroups, int steps, int flags, float* sink, hipStream_t stream);
struct LoraJobHost;
hipError_t lora_merge_launch(const LoraJobHost* jobs, int n_jobs, void* workspace, hipStream_t stream);
size_t lora_workspace_bytes(const LoraJobHost* jobs, int n_jobs);
}  // namespace tome

namespace {
thread_local int g_last_hip_error = 0;

int hip_result(hipError_t e) {
  if (e == hipSuccess) return TOME_OK;
  g_last_hip_error = (int)e;
  return TOME_E_HIP;
}

bool bad_temperature(float t) { return !(t > 0.f) || !isfinite(t); }

// rows * V elements must be addressable and the flat workgroup index must fit a 32-bit grid.
bool bad_matrix(int64_t rows, int64_t V, int64_t stride) {
  if (rows < 0 || V <= 0 || stride < V) return true;
  if (V > (int64_t)0x7fffffff) return true;             // unit indices are 32-bit
  if (rows > ((int64_t)1 << 31) / 64) return true;      // rows * splits (<= 64) must fit the grid
  if (rows > 0 && stride > INT64_MAX / 4 / rows) return true;
  return false;
}

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }
}  // namespace

extern "C" {

int tome_abi_version(void) { return TOME_ABI_VERSION; }

int tome_last_hip_error(void) { return g_last_hip_error; }

const char* tome_strerror(int code) {
  switch (code) {
    case TOME_OK: return "ok";
    case TOME_E_NULL: return "a required pointer is NULL";
    case TOME_E_DTYPE: return "unsupported dtype code";
    case TOME_E_SHAPE: return "bad shape or stride";
    case TOME_E_WORKSPACE: return "workspace too small";
    case TOME_E_TEMPERATURE: return "temperature must be finite and > 0";
    case TOME_E_ALIGN: return "pointer or stride not aligned as the kernel requires";
    case TOME_E_HIP: return "HIP runtime error (see tome_last_hip_error)";
    case TOME_E_SCRATCH: return "the call needs more scratch than the allocation-free entry point's fixed buffer holds";
    default: return "unknown error code";
  }
}

size_t tome_row_logprob_workspace(int64_t rows, int64_t V) {
  if (rows <= 0 || V <= 0) return 0;
  // Worst case over the vector and the element-wise path; 16 bytes per (row, split).
  const int s_vec = tome::row_splits_for(rows, V, 8), s_one = tome::row_splits_for(rows, V, 1);
  const int s4 = tome::row_splits_for(rows, V, 4);
  int s = s_vec > s_one ? s_vec : s_one;
  if (s4 > s) s = s4;
  return s <= 1 ? 0 : align256((size_t)rows * (size_t)s * 16);
}

int tome_row_logprob(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                     const int32_t* targets, const int32_t* row_valid, float temperature, float* out_lp,
                     float* out_lse, float* out_entropy, int32_t* out_argmax, void* workspace,
                     size_t workspace_bytes, void* stream) {
  if (dtype != TOME_F32 && dtype != TOME_BF16) return TOME_E_DTYPE;
  if (bad_matrix(rows, V, row_stride)) return TOME_E_SHAPE;
  if (bad_temperature(temperature)) return TOME_E_TEMPERATURE;
  if (rows == 0) return TOME_OK;
  if (!logits) return TOME_E_NULL;
  if (out_lp && !targets) return TOME_E_NULL;
  if (!out_lp && !out_lse && !out_entropy && !out_argmax) return TOME_E_NULL;
  const size_t need = tome_row_logprob_workspace(rows, V);
  if (need > 0 && (!workspace || workspace_bytes < need)) return TOME_E_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(logits) % (dtype == TOME_F32 ? 4 : 2) != 0) return TOME_E_ALIGN;
  return hip_result(tome::row_logprob_launch(logits, dtype, rows, V, row_stride, targets, row_valid, temperature,
                                             out_lp, out_lse, out_entropy, out_argmax, workspace,
                                             static_cast<hipStream_t>(stream)));
}

int tome_row_logprob_rows(const void* logits, int dtype, int64_t n_rows, int64_t V, int64_t row_stride,
                          const int32_t* row_index, int64_t n_index, const int32_t* targets, float temperature,
                          float* out_lp, float* out_lse, float* out_entropy, int32_t* out_argmax, void* workspace,
                          size_t workspace_bytes, void* stream) {
  if (dtype != TOME_F32 && dtype != TOME_BF16) return TOME_E_DTYPE;
  if (bad_matrix(n_rows, V, row_stride) || bad_matrix(n_index, V, row_stride)) return TOME_E_SHAPE;
  if (bad_temperature(temperature)) return TOME_E_TEMPERATURE;
  if (n_index == 0) return TOME_OK;
  if (!logits || !row_index) return TOME_E_NULL;
  if (out_lp && !targets) return TOME_E_NULL;
  if (!out_lp && !out_lse && !out_entropy && !out_argmax) return TOME_E_NULL;
  const size_t need = tome_row_logprob_workspace(n_index, V);
  if (need > 0 && (!workspace || workspace_bytes < need)) return TOME_E_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(logits) % (dtype == TOME_F32 ? 4 : 2) != 0) return TOME_E_ALIGN;
  return hip_result(tome::row_logprob_launch_rows(logits, dtype, n_rows, row_index, n_index, V, row_stride, targets,
                                                  nullptr, temperature, out_lp, out_lse, out_entropy, out_argmax,
                                                  workspace, static_cast<hipStream_t>(stream)));
}

int tome_row_logprob_noalloc(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                             const int32_t* targets, const int32_t* row_valid, float temperature, float* out_lp,
                             float* out_lse, float* out_entropy, int32_t* out_argmax, void* stream) {
  if (dtype != TOME_F32 && dtype != TOME_BF16) return TOME_E_DTYPE;
  if (bad_matrix(rows, V, row_stride)) return TOME_E_SHAPE;
  if (bad_temperature(temperature)) return TOME_E_TEMPERATURE;
  if (rows == 0) return TOME_OK;
  if (!logits) return TOME_E_NULL;
  if (out_lp && !targets) return TOME_E_NULL;
  if (!out_lp && !out_lse && !out_entropy && !out_argmax) return TOME_E_NULL;
  if (reinterpret_cast<uintptr_t>(logits) % (dtype == TOME_F32 ? 4 : 2) != 0) return TOME_E_ALIGN;
  bool too_big = false;
  const hipError_t e = tome::row_logprob_noalloc_launch(logits, dtype, rows, V, row_stride, targets, row_valid,
                                                        temperature, out_lp, out_lse, out_entropy, out_argmax,
                                                        &too_big, static_cast<hipStream_t>(stream));
  if (too_big) return TOME_E_SCRATCH;
  return hip_result(e);
}

size_t tome_row_logprob_noalloc_limit(size_t bytes) { return tome::row_scratch_set_limit(bytes); }

size_t tome_row_sample_workspace(int dtype, int64_t rows, int64_t V, int top_k) {
  if (rows <= 0 || V <= 0 || top_k < 1 || top_k > 32) return 0;
  return tome::row_sample_workspace_bytes(rows, V, dtype == TOME_F32 ? 4 : 8, top_k);
}

int tome_row_sample(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                    const float* uniforms, const int32_t* row_valid, float temperature, int top_k,
                    int32_t* out_token, float* out_lp, float* out_lse, int32_t* out_argmax,
                    int32_t* out_topk_idx, float* out_topk_logit, void* workspace, size_t workspace_bytes,
                    void* stream) {
  if (dtype != TOME_F32 && dtype != TOME_BF16) return TOME_E_DTYPE;
  if (bad_matrix(rows, V, row_stride) || top_k < 1 || top_k > 32) return TOME_E_SHAPE;
  if (bad_temperature(temperature)) return TOME_E_TEMPERATURE;
  if (rows == 0) return TOME_OK;
  if (!logits || !out_token) return TOME_E_NULL;
  const size_t need = tome_row_sample_workspace(dtype, rows, V, top_k);
  if (need > 0 && (!workspace || workspace_bytes < need)) return TOME_E_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(logits) % (dtype == TOME_F32 ? 4 : 2) != 0) return TOME_E_ALIGN;
  return hip_result(tome::row_sample_launch(logits, dtype, rows, V, row_stride, uniforms, row_valid, temperature,
                                            top_k, out_token, out_lp, out_lse, out_argmax, out_topk_idx,
                                            out_topk_logit, workspace, static_cast<hipStream_t>(stream)));
}

int tome_full_log_softmax(const void* logits, void* out, int dtype, int64_t rows, int64_t V,
                          int64_t in_row_stride, int64_t out_row_stride, float temperature, float* row_lse,
                          void* workspace, size_t workspace_bytes, void* stream) {
  if (dtype != TOME_F32 && dtype != TOME_BF16) return TOME_E_DTYPE;
  if (bad_matrix(rows, V, in_row_stride) || out_row_stride < V) return TOME_E_SHAPE;
  if (bad_temperature(temperature)) return TOME_E_TEMPERATURE;
  if (rows == 0) return TOME_OK;
  if (!logits || !out || !row_lse) return TOME_E_NULL;
  const size_t need = tome_row_logprob_workspace(rows, V);
  if (need > 0 && (!workspace || workspace_bytes < need)) return TOME_E_WORKSPACE;
  const int esize = dtype == TOME_F32 ? 4 : 2;
  if (reinterpret_cast<uintptr_t>(logits) % esize != 0 || reinterpret_cast<uintptr_t>(out) % esize != 0) return TOME_E_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // bf16 rows that fit one workgroup's registers: read once, written once
  if (tome::full_log_softmax_one_pass(logits, out, dtype, rows, V, in_row_stride, out_row_stride))
    return hip_result(tome::full_log_softmax_onepass_launch(logits, out, rows, V, in_row_stride, out_row_stride, temperature,
                                                            row_lse, s));
  // otherwise two passes: the rows' logsumexp (split rows leave their partials in the workspace), then the matrix
  int splits = 1;
  const hipError_t e = tome::row_lse_partials_launch(logits, dtype, rows, V, in_row_stride, temperature, row_lse, workspace,
                                                     &splits, s);
  if (e != hipSuccess) return hip_result(e);
  return hip_result(tome::full_log_softmax_launch(logits, out, dtype, rows, V, in_row_stride, out_row_stride, temperature,
                                                  row_lse, workspace, splits, s));
}

static int check_fused(const void* hidden, const void* w, int64_t n_tokens, int64_t H, int64_t V,
                       int64_t hidden_stride, int64_t weight_stride, const int32_t* targets, float temperature) {
  if (n_tokens < 0 || H <= 0 || V <= 0 || hidden_stride < H || weight_stride < H) return TOME_E_SHAPE;
  if (V > (int64_t)0x7fffffff || n_tokens > (int64_t)0x7fffffff || H > (int64_t)1 << 20) return TOME_E_SHAPE;
  // Row strides travel as 32-bit byte counts (checked before anything is multiplied by them).
  if (hidden_stride > (int64_t)0x7fffffff || weight_stride > (int64_t)0x7fffffff) return TOME_E_SHAPE;
  // The generic kernel (H % 64 != 0) also addresses both matrices with 32-bit byte offsets: each must stay
  // below 4 GiB there.  The other kernels use 64-bit addresses.
  if (tome::fused_needs_32bit_extents(n_tokens, H, V) &&
      (n_tokens * hidden_stride * 2 >= ((int64_t)1 << 32) || V * weight_stride * 2 >= ((int64_t)1 << 32)))
    return TOME_E_SHAPE;
  if (bad_temperature(temperature)) return TOME_E_TEMPERATURE;
  if (n_tokens == 0) return TOME_OK;
  if (!hidden || !w || !targets) return TOME_E_NULL;
  if (H % 8 != 0 || hidden_stride % 8 != 0 || weight_stride % 8 != 0 ||
      reinterpret_cast<uintptr_t>(hidden) % 16 != 0 || reinterpret_cast<uintptr_t>(w) % 16 != 0)
    return TOME_E_ALIGN;
  return TOME_OK;
}

void tome_select_fused_kernel(int kind) {
  tome::fused_force_kernel(kind == 0 || kind == 1 || (kind >= 3 && kind <= 5) ? kind : -1);
}

size_t tome_fused_lmhead_logprob_workspace(int64_t n_tokens, int64_t H, int64_t V) {
  if (n_tokens <= 0 || H <= 0 || V <= 0) return 0;
  return align256(tome::fused_workspace_bytes(n_tokens, H, V, 1, false));
}

int tome_fused_lmhead_logprob(const void* hidden, const void* weight, int64_t n_tokens, int64_t H, int64_t V,
                              int64_t hidden_stride, int64_t weight_stride, const int32_t* targets,
                              const int32_t* row_valid, float temperature, float* out_lp, float* out_lse,
                              float* out_entropy, int32_t* out_argmax, void* workspace, size_t workspace_bytes,
                              void* stream) {
  const int rc = check_fused(hidden, weight, n_tokens, H, V, hidden_stride, weight_stride, targets, temperature);
  if (rc != TOME_OK || n_tokens == 0) return rc;
  if (!out_lp) return TOME_E_NULL;
  const size_t need = tome_fused_lmhead_logprob_workspace(n_tokens, H, V);
  if (!workspace || workspace_bytes < need) return TOME_E_WORKSPACE;
  return hip_result(tome::fused_lmhead_launch(hidden, nullptr, 0.f, weight, nullptr, n_tokens, H, V, hidden_stride, weight_stride,
                                              targets, row_valid, temperature, out_lp, out_lse, out_entropy,
                                              out_argmax, nullptr, nullptr, workspace,
                                              static_cast<hipStream_t>(stream)));
}

size_t tome_norm_lmhead_logprob_workspace(int64_t n_tokens, int64_t H, int64_t V) {
  if (n_tokens <= 0 || H <= 0 || V <= 0) return 0;
  return align256(tome::fused_workspace_bytes(n_tokens, H, V, 1, true));
}

int tome_norm_lmhead_logprob(const void* hidden, const void* norm_weight, float norm_eps, const void* weight,
                             int64_t n_tokens, int64_t H, int64_t V, int64_t hidden_stride, int64_t weight_stride,
                             const int32_t* targets, const int32_t* row_valid, float temperature, float* out_lp,
                             float* out_lse, float* out_entropy, int32_t* out_argmax, void* workspace,
                             size_t workspace_bytes, void* stream) {
  const int rc = check_fused(hidden, weight, n_tokens, H, V, hidden_stride, weight_stride, targets, temperature);
  if (rc != TOME_OK || n_tokens == 0) return rc;
  if (!out_lp || !norm_weight) return TOME_E_NULL;
  if (reinterpret_cast<uintptr_t>(norm_weight) % 16 != 0) return TOME_E_ALIGN;
  if (!(norm_eps >= 0.f) || !isfinite(norm_eps)) return TOME_E_SHAPE;
  const size_t need = tome_norm_lmhead_logprob_workspace(n_tokens, H, V);
  if (!workspace || workspace_bytes < need) return TOME_E_WORKSPACE;
  return hip_result(tome::fused_lmhead_launch(hidden, norm_weight, norm_eps, weight, nullptr, n_tokens, H, V,
                                              hidden_stride, weight_stride, targets, row_valid, temperature, out_lp,
                                              out_lse, out_entropy, out_argmax, nullptr, nullptr, workspace,
                                              static_cast<hipStream_t>(stream)));
}

size_t tome_grpo_dual_workspace(int64_t n_tokens, int64_t H, int64_t V) {
  if (n_tokens <= 0 || H <= 0 || V <= 0) return 0;
  return align256(tome::fused_workspace_bytes(n_tokens, H, V, 2, false));
}

int tome_grpo_dual(const void* hidden, const void* w_policy, const void* w_ref, int64_t n_tokens, int64_t H,
                   int64_t V, int64_t hidden_stride, int64_t weight_stride, const int32_t* targets,
                   const int32_t* row_valid, float temperature, float* out_lp, float* out_ref_lp, float* out_k3,
                   float* out_entropy, void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = check_fused(hidden, w_policy, n_tokens, H, V, hidden_stride, weight_stride, targets, temperature);
  if (rc != TOME_OK || n_tokens == 0) return rc;
  if (!w_ref || !out_lp || !out_ref_lp) return TOME_E_NULL;
  if (reinterpret_cast<uintptr_t>(w_ref) % 16 != 0) return TOME_E_ALIGN;
  const size_t need = tome_grpo_dual_workspace(n_tokens, H, V);
  if (!workspace || workspace_bytes < need) return TOME_E_WORKSPACE;
  return hip_result(tome::fused_lmhead_launch(hidden, nullptr, 0.f, w_policy, w_ref, n_tokens, H, V, hidden_stride, weight_stride,
                                              targets, row_valid, temperature, out_lp, nullptr, out_entropy,
                                              nullptr, out_ref_lp, out_k3, workspace,
                                              static_cast<hipStream_t>(stream)));
}

size_t tome_grpo_pair_workspace(int64_t n_tokens, int64_t H, int64_t V, int with_norm) {
  if (n_tokens <= 0 || H <= 0 || V <= 0) return 0;
  // two partial sets; with a norm weight, one normalised copy per hidden-state matrix
  return align256(tome::fused_workspace_bytes(n_tokens, H, V, 2, with_norm != 0) +
                  (with_norm ? align256((size_t)n_tokens * H * 2) : 0));
}

int tome_grpo_pair(const void* hidden_policy, const void* hidden_ref, const void* norm_weight, float norm_eps,
                   const void* w_policy, const void* w_ref, int64_t n_tokens, int64_t H, int64_t V,
                   int64_t hidden_stride, int64_t weight_stride, const int32_t* targets, const int32_t* row_valid,
                   float temperature, float* out_lp, float* out_ref_lp, float* out_k3, float* out_entropy,
                   void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = check_fused(hidden_policy, w_policy, n_tokens, H, V, hidden_stride, weight_stride, targets, temperature);
  if (rc != TOME_OK || n_tokens == 0) return rc;
  if (!hidden_ref || !w_ref || !out_lp || !out_ref_lp) return TOME_E_NULL;
  if (reinterpret_cast<uintptr_t>(w_ref) % 16 != 0 || reinterpret_cast<uintptr_t>(hidden_ref) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(norm_weight) % 16 != 0)
    return TOME_E_ALIGN;
  if (norm_weight && (!(norm_eps >= 0.f) || !isfinite(norm_eps))) return TOME_E_SHAPE;
  const size_t need = tome_grpo_pair_workspace(n_tokens, H, V, norm_weight != nullptr);
  if (!workspace || workspace_bytes < need) return TOME_E_WORKSPACE;
  return hip_result(tome::fused_pair_launch(hidden_policy, hidden_ref, norm_weight, norm_eps, w_policy, w_ref, n_tokens,
                                            H, V, hidden_stride, weight_stride, targets, row_valid, temperature,
                                            out_lp, out_entropy, out_ref_lp, out_k3, workspace,
                                            static_cast<hipStream_t>(stream)));
}

int tome_probe_mfma_ceiling(const void* operands, size_t operand_bytes, int n_workgroups, int steps, int flags,
                            float* sink, size_t sink_bytes, void* stream) {
  if (!operands || !sink) return TOME_E_NULL;
  // Bounded so that one call cannot occupy the GPU for long: 4096 workgroups x 65536 slabs is a few hundred ms.
  if (n_workgroups <= 0 || n_workgroups > 4096 || steps <= 0 || steps > (1 << 16) || flags < 0 || flags > 7)
    return TOME_E_SHAPE;
  if (operand_bytes < (size_t)64 * 1024 || sink_bytes < (size_t)n_workgroups * 512 * sizeof(float)) return TOME_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(operands) % 16 != 0) return TOME_E_ALIGN;
  return hip_result(tome::mfma_probe_launch(operands, n_workgroups, steps, flags, sink, static_cast<hipStream_t>(stream)));
}

static int check_lora_jobs(const TomeLoraJob* jobs, int64_t n_jobs) {
  if (n_jobs < 0 || n_jobs > 65536) return TOME_E_SHAPE;
  if (n_jobs == 0) return TOME_OK;
  if (!jobs) return TOME_E_NULL;
  int64_t units = 0;
  for (int64_t i = 0; i < n_jobs; ++i) {
    const TomeLoraJob& j = jobs[i];
    if (!j.base || !j.out) return TOME_E_NULL;
    if ((j.lora_a == nullptr) != (j.lora_b == nullptr)) return TOME_E_NULL;
    if (j.rows < 0 || j.cols <= 0 || j.rows > 0x7fffffff - 16 || j.cols > 0x7fffffff - 512) return TOME_E_SHAPE;
    if (j.base_stride < j.cols || j.out_stride < j.cols || j.base_stride > 0x7fffffff || j.out_stride > 0x7fffffff)
      return TOME_E_SHAPE;
    if (j.lora_a && (j.rank < 8 || j.rank > 128)) return TOME_E_SHAPE;
    if (!isfinite(j.scale)) return TOME_E_SHAPE;
    if (j.cols % 8 != 0 || j.base_stride % 8 != 0 || j.out_stride % 8 != 0 || (j.lora_a && j.rank % 8 != 0) ||
        reinterpret_cast<uintptr_t>(j.base) % 16 != 0 || reinterpret_cast<uintptr_t>(j.out) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(j.lora_b) % 16 != 0 || reinterpret_cast<uintptr_t>(j.lora_a) % 2 != 0)
      return TOME_E_ALIGN;
    units += ((j.rows + 15) / 16) * ((j.cols + 511) / 512);
    if (units > 0x7fffffff) return TOME_E_SHAPE;  // one workgroup per unit at most: must fit the grid
  }
  return TOME_OK;
}

size_t tome_lora_merge_workspace(const TomeLoraJob* jobs, int64_t n_jobs) {
  if (check_lora_jobs(jobs, n_jobs) != TOME_OK || n_jobs == 0) return 0;
  return tome::lora_workspace_bytes(reinterpret_cast<const tome::LoraJobHost*>(jobs), (int)n_jobs);
}

int tome_lora_merge(const TomeLoraJob* jobs, int64_t n_jobs, void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = check_lora_jobs(jobs, n_jobs);
  if (rc != TOME_OK || n_jobs == 0) return rc;
  const size_t need = tome::lora_workspace_bytes(reinterpret_cast<const tome::LoraJobHost*>(jobs), (int)n_jobs);
  if (!workspace || workspace_bytes < need) return TOME_E_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return TOME_E_ALIGN;
  return hip_result(tome::lora_merge_launch(reinterpret_cast<const tome::LoraJobHost*>(jobs), (int)n_jobs, workspace,
                                            static_cast<hipStream_t>(stream)));
}

}  // extern "C"

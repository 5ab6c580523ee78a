// The reference's own launcher names, exported with their exact float32 signatures so that the ctypes
// loader of Src/Main_Scripts/core/cuda_opt_wrapper.py:50-79 binds this library unchanged:
//   rms_norm_launcher, rope_precompute_launcher, rope_apply_launcher, swiglu_launcher, swiglu_fused_launcher
//   (Src/Main_Scripts/core/transformer_ops.cu:331-434; call sites cuda_opt_wrapper.py:98-108, 156-169,
//   219-228, 337-344).
// Each is a thin alias of the ats_* entry point beside it.  They return void like the originals; where the
// originals print and exit() on a failed launch (transformer_ops.cu:321-329) these never terminate the
// process: the failure text stays readable through ats_last_error_string(), and ats_legacy_last_status()
// returns the status code of the calling thread's last legacy call.
#include <vector>

#include "ats_common.hpp"

namespace ats {
static thread_local int g_legacy_status = ATS_OK;
}

extern "C" int ats_legacy_last_status(void) { return ats::g_legacy_status; }

// y = x * rsqrt(mean(x^2) + eps) * w over [batch_seq, hidden_size] float32 rows.
extern "C" void rms_norm_launcher(const float* input, const float* weight, float* output, int batch_seq,
                                  int hidden_size, float eps, ats_stream_t stream) {
    ats::g_legacy_status =
        ats_rmsnorm_fwd(input, weight, output, batch_seq, hidden_size, eps, ATS_F32, ATS_F32, stream);
}

// cos/sin caches [max_seq_len, head_dim / 2] float32, angle = pos * theta^(-2d / head_dim), evaluated in
// float64 and rounded once (the original evaluates them with the fast float32 intrinsics).
extern "C" void rope_precompute_launcher(float* cos_cache, float* sin_cache, int max_seq_len, int head_dim,
                                         float theta, ats_stream_t stream) {
    ats::g_legacy_status =
        ats_rope_table(cos_cache, sin_cache, max_seq_len, head_dim, head_dim / 2, (double)theta, 1.0, stream);
}

// In-place rotation of q and k, both [batch_size, num_heads, seq_len, head_dim] float32 and contiguous, by the
// rows position_offset .. position_offset + seq_len - 1 of the half-width caches.  The signature carries no
// cache length, so, as in the original, the caller guarantees position_offset + seq_len <= max_seq_len.
extern "C" void rope_apply_launcher(float* q, float* k, const float* cos, const float* sin, int batch_size,
                                    int num_heads, int seq_len, int head_dim, int position_offset,
                                    ats_stream_t stream) {
    if (position_offset < 0 || seq_len < 0) {
        ats::set_error("rope_apply_launcher: position_offset=%d seq_len=%d", position_offset, seq_len);
        ats::g_legacy_status = ATS_ERR_INVALID_ARG;
        return;
    }
    const int64_t sl = head_dim, sh = (int64_t)seq_len * head_dim, sb = sh * num_heads;
    ats::g_legacy_status =
        ats_rope_fwd(q, k, q, k, cos, sin, head_dim / 2, position_offset + seq_len, batch_size, num_heads,
                     k ? num_heads : 0, seq_len, head_dim, position_offset, sb, sh, sl, sb, sh, sl, ATS_F32, stream);
}

// output = gate * silu(up), elementwise over [total_tokens, intermediate_size] float32.
extern "C" void swiglu_launcher(const float* gate, const float* up, float* output, int total_tokens,
                                int intermediate_size, ats_stream_t stream) {
    if (total_tokens < 0 || intermediate_size < 0) {
        ats::set_error("swiglu_launcher: total_tokens=%d intermediate_size=%d", total_tokens, intermediate_size);
        ats::g_legacy_status = ATS_ERR_INVALID_ARG;
        return;
    }
    ats::g_legacy_status =
        ats_swiglu_mul(gate, up, output, (int64_t)total_tokens * intermediate_size, ATS_F32, stream);
}

namespace ats {
// Tables of the two products below, written on the device so that the launcher neither copies from host
// memory nor waits: one group of total_tokens rows, multiplied by the gate weight and by the up weight.
__global__ void legacy_swiglu_tables_kernel(const float* gate_weight, const float* up_weight, int total_tokens,
                                            const void** b_ptrs, int32_t* row_start, int32_t* row_count) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        b_ptrs[0] = gate_weight;
        b_ptrs[1] = up_weight;
        row_start[0] = 0;
        row_count[0] = total_tokens;
    }
}
}  // namespace ats

// output[t, j] = (x[t] . gate_weight[j]) * silu(x[t] . up_weight[j]) over [total_tokens, intermediate_size],
// float32, weights [intermediate_size, hidden_size] (Src/Main_Scripts/core/transformer_ops.cu:268-313, 411-434;
// no call site in the reference's Python).  As in the original the biases are accepted and not applied
// (transformer_ops.cu:427-431 passes neither to its kernel).  Two float32 products on the matrix cores into
// a stream-ordered scratch buffer, then the elementwise activation; hidden_size and intermediate_size must be
// multiples of 4 (16-byte rows, which the original's float4 loads assume as well).
extern "C" void swiglu_fused_launcher(const float* input, const float* gate_weight, const float* up_weight,
                                      const float* gate_bias, const float* up_bias, float* output, int total_tokens,
                                      int hidden_size, int intermediate_size, bool use_bias, ats_stream_t stream) {
    using namespace ats;
    (void)gate_bias;
    (void)up_bias;
    (void)use_bias;
    const char* who = "swiglu_fused_launcher";
    if (total_tokens < 0 || hidden_size <= 0 || intermediate_size <= 0 ||
        (total_tokens > 0 && (!input || !gate_weight || !up_weight || !output))) {
        set_error("%s: total_tokens=%d hidden_size=%d intermediate_size=%d or a null pointer", who, total_tokens,
                  hidden_size, intermediate_size);
        g_legacy_status = ATS_ERR_INVALID_ARG;
        return;
    }
    if (total_tokens == 0) {
        g_legacy_status = ATS_OK;
        return;
    }
    hipStream_t s = as_stream(stream);
    const size_t n_out = (size_t)total_tokens * (size_t)intermediate_size;
    const size_t off_tables = 2 * n_out * sizeof(float);
    const size_t bytes = off_tables + 32;
    unsigned char* dev = nullptr;
    hipError_t e = hipMallocAsync(reinterpret_cast<void**>(&dev), bytes, s);
    if (e != hipSuccess) {
        set_error("%s: scratch allocation of %zu bytes failed: %s", who, bytes, hipGetErrorString(e));
        g_legacy_status = ATS_ERR_LAUNCH;
        return;
    }
    float* gu = reinterpret_cast<float*>(dev);
    const void** b_ptrs = reinterpret_cast<const void**>(dev + off_tables);
    int32_t* row_start = reinterpret_cast<int32_t*>(dev + off_tables + 16);
    int32_t* row_count = reinterpret_cast<int32_t*>(dev + off_tables + 24);
    hipLaunchKernelGGL(legacy_swiglu_tables_kernel, dim3(1), dim3(64), 0, s, gate_weight, up_weight, total_tokens, b_ptrs,
                       row_start, row_count);
    int rc = hipGetLastError() == hipSuccess ? ATS_OK : ATS_ERR_LAUNCH;
    if (rc != ATS_OK) set_error("%s: launch failed", who);
    for (int half = 0; half < 2 && rc == ATS_OK; ++half)
        rc = ats_grouped_gemm_nt(input, nullptr, hidden_size, total_tokens, nullptr, 1,
                                 reinterpret_cast<const void* const*>(b_ptrs + half), hidden_size, intermediate_size,
                                 gu + half * n_out, intermediate_size, row_start, row_count, nullptr, 1, total_tokens,
                                 intermediate_size, hidden_size, ATS_F32, ATS_F32, stream);
    if (rc == ATS_OK) rc = ats_swiglu_mul(gu, gu + n_out, output, (int64_t)n_out, ATS_F32, stream);
    (void)hipFreeAsync(dev, s);
    g_legacy_status = rc;
}

// ---- training-step launchers (Src/Main_Scripts/training/fused_loss.cu:183-214, fused_grad_clip.cu:117-175;
// call sites Src/Main_Scripts/training/cuda_kernels.py:154-164, 340-346).  The originals own their scratch
// memory; so do these (stream-ordered allocations), which makes them the only entry points of the library
// that allocate.
namespace ats {
__global__ void legacy_loss_outputs_kernel(const float* __restrict__ sums, float* __restrict__ loss_out,
                                           float* __restrict__ accuracy_out, long long* __restrict__ valid_out) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        loss_out[0] = sums[2];                    // sum of the token losses over valid tokens
        accuracy_out[0] = sums[3];                // number of correct arg-max predictions, as a float
        valid_out[0] = (long long)sums[4];        // valid tokens
    }
}
}  // namespace ats

// loss_out = sum of -log softmax(logits)[label] over the valid tokens, accuracy_out = number of tokens whose
// arg-max equals the label (float), valid_tokens_out = their count; the caller divides (cuda_kernels.py:168-175).
// The original accumulates with float atomics in arrival order; the sums here are formed in a fixed order.
extern "C" void fused_cross_entropy_accuracy_launcher(const float* logits, const int64_t* labels, int64_t pad_token_id,
                                                      float* loss_out, float* accuracy_out, int64_t* valid_tokens_out,
                                                      int total_tokens, int vocab_size, ats_stream_t stream) {
    using namespace ats;
    const char* who = "fused_cross_entropy_accuracy_launcher";
    if (total_tokens < 0 || vocab_size <= 0 || !loss_out || !accuracy_out || !valid_tokens_out ||
        (total_tokens > 0 && (!logits || !labels))) {
        set_error("%s: total_tokens=%d vocab_size=%d or a null pointer", who, total_tokens, vocab_size);
        g_legacy_status = ATS_ERR_INVALID_ARG;
        return;
    }
    hipStream_t s = as_stream(stream);
    float* scratch = nullptr;
    const size_t n = (size_t)4 * (size_t)total_tokens + 8;
    hipError_t e = hipMallocAsync(reinterpret_cast<void**>(&scratch), n * sizeof(float), s);
    if (e != hipSuccess) {
        set_error("%s: scratch allocation of %zu bytes failed: %s", who, n * sizeof(float), hipGetErrorString(e));
        g_legacy_status = ATS_ERR_LAUNCH;
        return;
    }
    float* sums = scratch + (size_t)4 * total_tokens;
    const size_t T = (size_t)total_tokens;
    g_legacy_status = ats_cross_entropy_fwd(logits, labels, pad_token_id, nullptr, scratch, scratch + T, scratch + 2 * T,
                                            scratch + 3 * T, sums, total_tokens, vocab_size, ATS_F32, stream);
    if (g_legacy_status == ATS_OK) {
        hipLaunchKernelGGL(legacy_loss_outputs_kernel, dim3(1), dim3(64), 0, s, sums, loss_out, accuracy_out,
                           reinterpret_cast<long long*>(valid_tokens_out));
        if (hipGetLastError() != hipSuccess) {
            set_error("%s: launch failed", who);
            g_legacy_status = ATS_ERR_LAUNCH;
        }
    }
    (void)hipFreeAsync(scratch, s);
}

// Total L2 norm of num_tensors float32 gradients (device arrays of pointers and int32 element counts), then
// grads *= max_norm / (norm + 1e-6) if that factor is below 1.  Returns the norm, which, as in the original,
// costs a synchronisation of the stream; the element counts are fetched first to lay out the chunked
// reduction (fixed summation order instead of the original's float atomics).
extern "C" float fused_grad_clip_launcher(float** grad_ptrs_device, int* grad_sizes_device, int num_tensors, float max_norm,
                                          ats_stream_t stream) {
    using namespace ats;
    const char* who = "fused_grad_clip_launcher";
    if (num_tensors < 0 || (num_tensors > 0 && (!grad_ptrs_device || !grad_sizes_device))) {
        set_error("%s: num_tensors=%d or a null pointer", who, num_tensors);
        g_legacy_status = ATS_ERR_INVALID_ARG;
        return 0.f;
    }
    if (num_tensors == 0) {
        g_legacy_status = ATS_OK;
        return 0.f;
    }
    hipStream_t s = as_stream(stream);
    std::vector<int> sizes32((size_t)num_tensors);
    hipError_t e = hipMemcpyAsync(sizes32.data(), grad_sizes_device, sizeof(int) * (size_t)num_tensors, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) {
        set_error("%s: reading the element counts failed: %s", who, hipGetErrorString(e));
        g_legacy_status = ATS_ERR_LAUNCH;
        return 0.f;
    }
    const int chunk = ats_grad_clip_chunk_elems();
    std::vector<int64_t> sizes64((size_t)num_tensors);
    std::vector<int32_t> chunk_start((size_t)num_tensors + 1);
    int64_t chunks = 0;
    for (int i = 0; i < num_tensors; ++i) {
        if (sizes32[i] < 0) {
            set_error("%s: tensor %d has %d elements", who, i, sizes32[i]);
            g_legacy_status = ATS_ERR_INVALID_ARG;
            return 0.f;
        }
        sizes64[i] = sizes32[i];
        chunk_start[i] = (int32_t)chunks;
        chunks += (sizes32[i] + chunk - 1) / chunk;
    }
    chunk_start[num_tensors] = (int32_t)chunks;
    if (chunks > 0x7fffffff) {
        set_error("%s: %lld chunks", who, (long long)chunks);
        g_legacy_status = ATS_ERR_UNSUPPORTED;
        return 0.f;
    }
    // one device block: sizes (int64), chunk starts (int32), partial sums and the two norm outputs (float)
    const size_t off_cs = sizeof(int64_t) * (size_t)num_tensors;
    const size_t off_part = (off_cs + sizeof(int32_t) * ((size_t)num_tensors + 1) + 15) / 16 * 16;
    const size_t off_norm = off_part + sizeof(float) * (size_t)(chunks > 0 ? chunks : 1);
    const size_t bytes = off_norm + 2 * sizeof(float);
    unsigned char* dev = nullptr;
    e = hipMallocAsync(reinterpret_cast<void**>(&dev), bytes, s);
    if (e != hipSuccess) {
        set_error("%s: scratch allocation of %zu bytes failed: %s", who, bytes, hipGetErrorString(e));
        g_legacy_status = ATS_ERR_LAUNCH;
        return 0.f;
    }
    float norm_host[2] = {0.f, 0.f};
    e = hipMemcpyAsync(dev, sizes64.data(), off_cs, hipMemcpyHostToDevice, s);
    if (e == hipSuccess)
        e = hipMemcpyAsync(dev + off_cs, chunk_start.data(), sizeof(int32_t) * ((size_t)num_tensors + 1), hipMemcpyHostToDevice, s);
    int rc = e == hipSuccess ? ATS_OK : ATS_ERR_LAUNCH;
    if (rc == ATS_OK)
        rc = ats_grad_norm_clip(reinterpret_cast<void* const*>(grad_ptrs_device), reinterpret_cast<const int64_t*>(dev),
                                reinterpret_cast<const int32_t*>(dev + off_cs), num_tensors, (int)chunks, ATS_F32, nullptr,
                                reinterpret_cast<float*>(dev + off_part), reinterpret_cast<float*>(dev + off_norm), max_norm, 1,
                                stream);
    if (rc == ATS_OK) {
        e = hipMemcpyAsync(norm_host, dev + off_norm, sizeof(norm_host), hipMemcpyDeviceToHost, s);
        if (e == hipSuccess) e = hipStreamSynchronize(s);     // the host vectors above stay alive until here
        if (e != hipSuccess) {
            set_error("%s: reading the norm failed: %s", who, hipGetErrorString(e));
            rc = ATS_ERR_LAUNCH;
        }
    } else {
        (void)hipStreamSynchronize(s);
    }
    (void)hipFreeAsync(dev, s);
    g_legacy_status = rc;
    return rc == ATS_OK ? norm_host[0] : 0.f;
}

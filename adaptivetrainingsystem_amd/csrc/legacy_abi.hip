// The reference's own launcher names, exported with their exact float32 signatures so that the ctypes
// loader of Src/Main_Scripts/core/cuda_opt_wrapper.py:50-79 binds this library unchanged:
//   rms_norm_launcher, rope_precompute_launcher, rope_apply_launcher, swiglu_launcher
//   (Src/Main_Scripts/core/transformer_ops.cu:331-409; call sites cuda_opt_wrapper.py:98-108, 156-169,
//   219-228, 337-344).
// Each is a thin alias of the ats_* entry point beside it.  They return void like the originals; where the
// originals print and exit() on a failed launch (transformer_ops.cu:321-329) these never terminate the
// process: the failure text stays readable through ats_last_error_string(), and ats_legacy_last_status()
// returns the status code of the calling thread's last legacy call.
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

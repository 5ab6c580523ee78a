/* CPU oracle, integer side of the capacity dispatch, in plain C.
 *
 * TEST INFRASTRUCTURE ONLY: loaded by the tests, the smoke check and the
 * CPU-baseline leg of the benchmark; never by the product path.
 *
 * Literal restatement of the reference's first-come-first-served loop
 * (Src/Main_Scripts/core/moe_cuda_wrapper.py:316-324, second copy at
 * Src/Main_Scripts/cuda_debug_script.py:101-109): assignments are visited in
 * (token, choice) order, each takes the next free slot of its expert, and is
 * dropped when the expert already holds `capacity` rows.
 *
 * Pinned by: the Python literal loop and the stable-counting-sort closed form
 * in sparse_layer_oracle.py (three independent formulations must agree).
 */
#include <stdint.h>

/* idx: [T*k] expert ids.  token_map: [E*C], filled with -1 for empty slots.
 * slot: [T*k], slot inside the expert or -1 when dropped.  hist: [E]
 * pre-capacity counts.  kept: [E] = min(hist, C).  Returns the number of
 * dropped assignments, or -1 on an out-of-range expert id. */
int64_t oracle_fcfs_dispatch(const int32_t* idx, int64_t T, int32_t k, int32_t E, int32_t C,
                             int32_t* token_map, int32_t* slot, int32_t* hist, int32_t* kept) {
    int64_t dropped = 0;
    for (int64_t i = 0; i < (int64_t)E * C; ++i) token_map[i] = -1;
    for (int32_t e = 0; e < E; ++e) { hist[e] = 0; kept[e] = 0; }
    for (int64_t t = 0; t < T; ++t) {
        for (int32_t j = 0; j < k; ++j) {
            int64_t a = t * k + j;
            int32_t e = idx[a];
            if (e < 0 || e >= E) return -1;
            hist[e] += 1;
            int32_t pos = kept[e];
            if (pos < C) {
                token_map[(int64_t)e * C + pos] = (int32_t)a;
                slot[a] = pos;
                kept[e] = pos + 1;
            } else {
                slot[a] = -1;
                dropped += 1;
            }
        }
    }
    return dropped;
}

/* Literal restatement of the combine loop (moe_cuda_wrapper.py:343-357) in
 * float32: ascending expert, ascending slot, out[t] += w[t,j] * y[e,pos]
 * with a separately rounded product and sum (compiled without contraction). */
void oracle_combine_f32(const float* expert_out, const int32_t* token_map, const float* w,
                        int64_t T, int32_t k, int32_t E, int32_t C, int32_t H, float* out) {
    for (int64_t i = 0; i < T * H; ++i) out[i] = 0.0f;
    for (int32_t e = 0; e < E; ++e) {
        for (int32_t pos = 0; pos < C; ++pos) {
            int32_t m = token_map[(int64_t)e * C + pos];
            if (m < 0) continue;
            int64_t t = m / k;
            if (t >= T) continue;
            float wt = w[m];
            const float* y = expert_out + ((int64_t)e * C + pos) * H;
            float* o = out + t * H;
            for (int32_t h = 0; h < H; ++h) {
                volatile float p = wt * y[h];
                o[h] = o[h] + p;
            }
        }
    }
}

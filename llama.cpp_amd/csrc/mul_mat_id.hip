// MUL_MAT_ID host entry: quantize the nb1*T rows of b once, then route every
// (token, expert slot) pair to its expert's weights on the device: per-slot GEMV for a few slots,
// slots sorted by expert and one tile launch over all experts for many.
#include "common.hpp"
#include "qdot.hpp"

using namespace mi355;

extern "C" {

// Above this many (token, expert slot) pairs the slots are sorted by expert and run through the tile kernel,
// which reads every expert's matrix once; below it each slot streams its expert's matrix through the GEMV.
static constexpr int64_t ROUTED_MIN_SLOTS = 32;   // measured cross-over on 8 experts of 14336 x 4096

static bool use_routed_tiles(int type, const void *as, int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t T) {
    if (T * n_used < ROUTED_MIN_SLOTS || n_expert > 256 || K % QKK != 0 ||
        (type != MI355_Q4_K && type != MI355_Q5_K && type != MI355_Q6_K && type != MI355_IQ4_XS))
        return false;
    const row_layout L = make_row_layout(type, K);
    return layout_aligned(as, L) && (N * L.row_bytes) % 16 == 0;
}

size_t mi355_mul_mat_id_ws_bytes(int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T) {
    const size_t act = (mi355_act_bytes(K, nb1 * T) + 255) & ~(size_t)255;   // the per-super-block format is the smaller one
    return act + mi355_mul_mat_id_q8k_route_bytes(n_expert, n_used, T);
}

int mi355_mul_mat_id(void *stream, int type, const void *as, const float *b, const int32_t *ids, int64_t ids_stride,
                     float *dst, int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T,
                     void *ws, size_t ws_bytes) {
    MI355_REQUIRE(is_weight_type(type), "mul_mat_id: unsupported weight type %d", type);
    MI355_REQUIRE(N > 0 && K > 0 && n_expert > 0 && n_used > 0 && nb1 > 0 && T > 0, "mul_mat_id: bad shape");
    MI355_REQUIRE(K % type_block_elems(type) == 0, "mul_mat_id: K=%lld is not a multiple of the block size", (long long)K);
    MI355_REQUIRE(ids_stride >= n_used, "mul_mat_id: ids_stride < n_used");
    if (ws == nullptr || ws_bytes < mi355_mul_mat_id_ws_bytes(K, n_expert, n_used, nb1, T)) {
        set_error("mul_mat_id: workspace of %zu bytes, need %zu", ws_bytes, mi355_mul_mat_id_ws_bytes(K, n_expert, n_used, nb1, T));
        return MI355_ERR_WORKSPACE;
    }
    if (use_routed_tiles(type, as, N, K, n_expert, n_used, T)) {
        int rc = mi355_quantize_act_q8k(stream, b, ws, K, nb1 * T, K);
        if (rc != MI355_OK) return rc;
        const size_t act = (mi355_act_bytes(K, nb1 * T) + 255) & ~(size_t)255;
        return mi355_mul_mat_id_q8k(stream, type, as, ws, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T, (uint8_t *)ws + act,
                                    ws_bytes - act);
    }
    int rc = mi355_quantize_act(stream, b, ws, K, nb1 * T, K);
    if (rc != MI355_OK) return rc;
    if (T * n_used >= ROUTED_MIN_SLOTS && mi355_mul_mat_id_q_supported(type, as, N, K, n_expert)) {   // per-32-block types: the routed form of their tile kernel
        const size_t act = (mi355_act_bytes(K, nb1 * T) + 255) & ~(size_t)255;
        return mi355_mul_mat_id_q(stream, type, as, ws, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T, (uint8_t *)ws + act, ws_bytes - act);
    }
    return mi355_mul_mat_id_vec(stream, type, as, ws, ids, ids_stride, dst, N, K, n_expert, n_used, nb1, T);
}

}  // extern "C"

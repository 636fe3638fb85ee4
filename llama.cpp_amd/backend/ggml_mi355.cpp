// ggml backend plug-in for one AMD Instinct MI355X (gfx950).
//
// This file is the drop-in boundary: it fills the five vtables of
// ggml/src/ggml-backend-impl.h:17-207 (buffer type, buffer, backend, device, reg) and
// exports ggml_backend_init / ggml_backend_score, the two symbols the registry dlsym()s
// (ggml/src/ggml-backend-reg.cpp:229-245).  It is loaded through GGML_BACKEND_PATH or by
// sitting next to the executable as libggml-<name>.so, so test-backend-ops, llama-bench and
// llama-cli run on it unmodified.  All arithmetic lives behind the C ABI of
// include/mi355_kernels.h; this file only routes ggml tensors to it.
//
// Conventions kept from the reference's backends:
//  * work is declined in supports_op, never inside graph_compute;
//  * tensor->data is a device address: get_base() + allocator offset, views included;
//  * buffer set/get_tensor synchronise the device first, because the scheduler may read a
//    result right after an asynchronous graph_compute (ggml/src/ggml-backend.cpp:243-252).
//
// Quantized tensors of type Q4_0 / Q4_1 / Q5_0 / Q5_1 / IQ4_NL / IQ4_XS / Q8_0 / Q6_K live in HBM in the 16-byte-aligned row layout
// described in mi355_kernels.h; set_tensor applies that byte permutation and get_tensor
// undoes it, so every caller sees the reference's bytes.

#include "ggml-backend-impl.h"
#include "ggml-impl.h"
#include "ggml.h"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "mi355_kernels.h"

#define MI355_HIP_OK(expr)                                                                                      \
    do {                                                                                                        \
        hipError_t e_ = (expr);                                                                                 \
        if (e_ != hipSuccess) GGML_ABORT("MI355: %s failed: %s", #expr, hipGetErrorString(e_));                 \
    } while (0)

#define MI355_K_OK(expr)                                                                                        \
    do {                                                                                                        \
        int rc_ = (expr);                                                                                       \
        if (rc_ != MI355_OK) GGML_ABORT("MI355: %s failed (%d): %s", #expr, rc_, mi355_last_error());           \
    } while (0)

namespace {

// ------------------------------------------------------------------------------- helpers
bool is_repacked_type(ggml_type t) {
    return t == GGML_TYPE_Q4_0 || t == GGML_TYPE_Q8_0 || t == GGML_TYPE_Q6_K || t == GGML_TYPE_Q4_1 || t == GGML_TYPE_Q5_0 || t == GGML_TYPE_Q5_1 ||
           t == GGML_TYPE_IQ4_NL || t == GGML_TYPE_IQ4_XS;
}
bool is_weight_type(ggml_type t) { return is_repacked_type(t) || t == GGML_TYPE_Q4_K || t == GGML_TYPE_Q5_K; }
// types whose matrices can get tile images for the wide-tile GEMM (mi355_kq_unpack_tiles)
bool has_tile_images(ggml_type t) { return t == GGML_TYPE_Q4_K || t == GGML_TYPE_Q5_K || t == GGML_TYPE_Q6_K || t == GGML_TYPE_IQ4_XS; }
// ... and those among them with no super-block tile kernel on packed rows: without images they take the per-32-block kernels
bool tiles_or_generic(ggml_type t) { return t == GGML_TYPE_Q5_K || t == GGML_TYPE_IQ4_XS; }
// rows of K elements are 16-byte multiples in the device layout when K is a multiple of this (256 for the other types)
int64_t aligned_row_elems(ggml_type t) { return t == GGML_TYPE_Q6_K ? 2048 : t == GGML_TYPE_IQ4_XS ? 512 : 256; }

int to_mi355_type(ggml_type t) {
    switch (t) {
        case GGML_TYPE_F32: return MI355_F32;
        case GGML_TYPE_F16: return MI355_F16;
        case GGML_TYPE_I32: return MI355_I32;
        case GGML_TYPE_Q4_0: return MI355_Q4_0;
        case GGML_TYPE_Q4_1: return MI355_Q4_1;
        case GGML_TYPE_Q5_0: return MI355_Q5_0;
        case GGML_TYPE_Q5_1: return MI355_Q5_1;
        case GGML_TYPE_IQ4_NL: return MI355_IQ4_NL;
        case GGML_TYPE_IQ4_XS: return MI355_IQ4_XS;
        case GGML_TYPE_Q8_0: return MI355_Q8_0;
        case GGML_TYPE_Q4_K: return MI355_Q4_K;
        case GGML_TYPE_Q5_K: return MI355_Q5_K;
        case GGML_TYPE_Q6_K: return MI355_Q6_K;
        default: return -1;
    }
}

mi355_tensor desc(const ggml_tensor * t) {
    mi355_tensor d;
    d.data = t->data;
    d.type = to_mi355_type(t->type);
    for (int i = 0; i < 4; i++) {
        d.ne[i] = t->ne[i];
        d.nb[i] = t->nb[i];
    }
    return d;
}

bool strides_mult16(const ggml_tensor * t) { return t->nb[1] % 16 == 0 && t->nb[2] % 16 == 0 && t->nb[3] % 16 == 0; }

// A Q8_0 / Q4_0 tensor that is read or written block by block (a quantized KV cache).  Its memory belongs to `root` (the tensor
// itself or the one it is a view of), which set_tensor keeps in the device row layout: blocks are addressed through the root's
// rows, whatever shape the view has.
struct kv_operand {
    const void * p = nullptr;      // first byte in plain ggml addressing
    const void * base = nullptr;   // data of the owning tensor
    int64_t row_blocks = 0;        // blocks per row of the owning tensor
    bool ok = false;
};
kv_operand kv_operand_of(const ggml_tensor * t) {
    kv_operand o;
    o.p = t->data;
    if (t->type == GGML_TYPE_F16) {
        o.ok = true;
        return o;
    }
    if (t->type != GGML_TYPE_Q8_0 && t->type != GGML_TYPE_Q4_0) return o;
    const ggml_tensor * root = t->view_src ? t->view_src : t;
    const size_t bb = ggml_type_size(t->type);
    if (root->type != t->type || !ggml_is_contiguous(root) || root->ne[0] % 32 != 0 || t->ne[0] % 32 != 0 || t->nb[0] != bb) return o;
    if (t->nb[1] % bb != 0 || t->nb[2] % bb != 0 || t->nb[3] % bb != 0 || (t->view_src && t->view_offs % bb != 0)) return o;
    o.base = root->data;
    o.row_blocks = root->ne[0] / 32;
    o.ok = true;
    return o;
}

// ------------------------------------------------------------------------------- device state
struct device_ctx {
    int device = 0;
    std::string name;
    std::string description;
};

// Quantized form of an f32 activation tensor, kept while consecutive MUL_MAT nodes consume the same src1
struct act_cache {
    const void * src = nullptr;   // data pointer of the f32 tensor this was quantized from (B rows of K, contiguous)
    int64_t K = 0, B = 0;
    int format = 0;               // ACT_Q8_1 (32-element blocks, GEMV), ACT_Q8K (256-element super-blocks, tile GEMM) or ACT_Q8KT (the same as tile images)
    bool valid = false;
    void * ptr = nullptr;         // where the quantized form lives (one of the two slots of backend_ctx::act)
};
enum { ACT_Q8_1 = 1, ACT_Q8K = 2, ACT_Q8KT = 3 };

constexpr int IOTA_N = 16384;

struct backend_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    void * ws = nullptr;   // scratch for quantized activations / attention partials
    size_t ws_size = 0;
    void * act = nullptr;  // quantized activation shared by consecutive matrix products (see act_cache)
    size_t act_size = 0;
    act_cache cache;
    bool fuse = true;      // MI355_NO_FUSION=1 executes the graph node for node
    int32_t * iota = nullptr;   // device {0, 1, 2, ... IOTA_N - 1}: token t of a batch goes to row t of a KV-cache view
    // {cos, sin} per (token, pair) of a prompt batch's rotations, written once per graph for the Q/K/V launches of all its layers
    float * rope_tab = nullptr;
    size_t rope_tab_floats = 0;
    uint64_t graph_serial = 0, rope_tab_serial = 0;   // the table is that of graph rope_tab_serial ...
    const void * rope_tab_pos = nullptr, * rope_tab_ff = nullptr;   // ... for these positions, frequency factors and parameters
    int32_t rope_tab_params[11] = {0};
    int64_t rope_tab_D = 0, rope_tab_T = 0;
    // products whose result is written somewhere else than into their own tensor (see match_prefill_qkv)
    const ggml_tensor * redirect_node[2] = {nullptr, nullptr};
    void * redirect_to[2] = {nullptr, nullptr};
    int n_redirect = 0;
    void * out_ptr(const ggml_tensor * t) const {
        for (int k = 0; k < n_redirect; k++)
            if (redirect_node[k] == t) return redirect_to[k];
        return t->data;
    }
    unsigned * tickets = nullptr;   // zeroed arrival counters of the gate/up launch (one per 32 output rows)
    size_t n_tickets = 0;
    long async_uploads = 0, events_recorded = 0;   // reported with MI355_GRAPH_STATS=1
    // Host-to-device hand-over of split inputs (backend_cpy_tensor_async): the bytes are copied into one of these pinned slots
    // at the call and uploaded from there, so the upload never reads the caller's memory after the call returns.
    static constexpr int STAGE_SLOTS = 8;
    static constexpr size_t STAGE_BYTES = (size_t) 1 << 20;
    void * stage = nullptr;                 // STAGE_SLOTS x STAGE_BYTES of pinned host memory, allocated at the first use
    hipEvent_t stage_done[STAGE_SLOTS] = {};   // recorded after the upload that reads slot i
    int stage_next = 0;
    const ggml_tensor * done_ahead = nullptr;      // a product that went out with an earlier node's launch (see tiled_multi)

    // ---- replay of decode graphs as HIP graphs (see backend_graph_compute)
    struct replay_state {
        bool enabled = true;          // MI355_NO_GRAPH=1 turns replay off
        uint64_t seen_sig = 0;        // signature of the last graph that ran launch by launch ...
        uint64_t seen_gen = 0;        // ... and the scratch-buffer generation it ran with
        uint64_t bad_sig = 0;         // a graph whose capture did not work out: not tried again
        uint64_t exec_sig = 0, exec_gen = 0;
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        long replays = 0, captures = 0;
        double host_us = 0.0;         // host time spent in graph_compute calls that ended in a replay
    } replay;
    uint64_t alloc_gen = 1;           // bumped whenever a scratch buffer moves: captured launches hold the old addresses
    bool capturing = false, capture_broken = false;
    int32_t * cells = nullptr;        // device {head, head + 1, ...}: cache cell of token t of this graph's batch
    int64_t cells_head = -1;          // what `cells` holds
    int64_t kv_head = -1;             // first cache cell this graph stores to, or -1 when its stores do not agree on one
    int kv_redirected = 0;            // cache stores of this graph that went through `cells`

    // a scratch buffer has to move: impossible while launches are being recorded (they would keep the old address and
    // nothing may synchronize); the recording is thrown away afterwards and the graph runs launch by launch
    bool may_allocate() {
        if (capturing) {
            capture_broken = true;
            return false;
        }
        alloc_gen++;
        return true;
    }

    unsigned * ticket_buffer(size_t n) {
        if (n > n_tickets && may_allocate()) {
            if (tickets) {
                MI355_HIP_OK(hipStreamSynchronize(stream));
                MI355_HIP_OK(hipFree(tickets));
            }
            n_tickets = (n + 1023) & ~(size_t) 1023;
            MI355_HIP_OK(hipMalloc((void **) &tickets, n_tickets * sizeof(unsigned)));
            MI355_HIP_OK(hipMemset(tickets, 0, n_tickets * sizeof(unsigned)));   // every launch leaves them zero again
        }
        return tickets;
    }
    std::string name;

    // a node is about to write [p, p + bytes): the cached activation dies if that touches the tensor it came from
    void note_write(const void * p, size_t bytes) {
        if (!cache.valid) return;
        const char * a0 = (const char *) cache.src, * a1 = a0 + (size_t) cache.K * (size_t) cache.B * sizeof(float);
        const char * b0 = (const char *) p, * b1 = b0 + bytes;
        if (a0 < b1 && b0 < a1) cache.valid = false;
    }

    // two slots, so that a launch can read one quantized activation while it writes the next one
    void act_reserve(size_t need) {
        if (need > act_size && may_allocate()) {
            if (act) {
                MI355_HIP_OK(hipStreamSynchronize(stream));
                MI355_HIP_OK(hipFree(act));
            }
            act_size = (need + (size_t(4) << 20)) & ~((size_t(1) << 20) - 1);
            MI355_HIP_OK(hipMalloc(&act, 2 * act_size));
            cache.valid = false;
        }
    }
    void * act_slot(size_t need, bool keep_cached = false) {   // keep_cached: pick the slot the valid cache does not occupy
        act_reserve(need);
        char * s0 = (char *) act, * s1 = s0 + act_size;
        if (keep_cached && cache.valid && cache.ptr == s0) return s1;
        return s0;
    }
    bool cached(const void * src, int64_t K, int64_t B, int format) const {
        return cache.valid && cache.src == src && cache.K == K && cache.B == B && cache.format == format;
    }

    void * workspace(size_t need) {
        if (need > ws_size && may_allocate()) {
            if (ws) {
                MI355_HIP_OK(hipStreamSynchronize(stream));   // kernels in flight may still read the old one
                MI355_HIP_OK(hipFree(ws));
            }
            ws_size = (need + (size_t(32) << 20)) & ~((size_t(1) << 20) - 1);
            MI355_HIP_OK(hipMalloc(&ws, ws_size));
        }
        return ws;
    }
};

struct buffer_ctx {
    int device = 0;
    void * base = nullptr;
    size_t size = 0;
};

ggml_backend_buffer_type_t mi355_buffer_type(int device);
ggml_guid_t mi355_guid() {
    static ggml_guid guid = { 0x4d, 0x49, 0x33, 0x35, 0x35, 0x58, 0x2d, 0x67, 0x66, 0x78, 0x39, 0x35, 0x30, 0x2d, 0x30, 0x31 };
    return &guid;
}

// one staging buffer for layout-permuted uploads / read-backs (guarded: the model loader and the
// compute thread may both call into buffers)
struct staging {
    std::mutex mu;
    void * ptr = nullptr;
    size_t size = 0;
    void * get(size_t need) {
        if (need > size) {
            if (ptr) MI355_HIP_OK(hipFree(ptr));
            size = (need + (size_t(1) << 20)) & ~((size_t(1) << 20) - 1);
            MI355_HIP_OK(hipMalloc(&ptr, size));
        }
        return ptr;
    }
};
staging & stage() {
    static staging s;
    return s;
}

// Unpacked int8 planes of Q6_K weight matrices for the tile GEMM (mi355_kq_unpack_planes), built the first time a matrix in a
// weights buffer meets a batch above 8 and kept until that buffer is freed or the tensor is written again.  Keyed by the
// tensor's data address.  MI355_NO_PLANES=1 keeps the packed rows only (2 bytes per Q6_K weight less device memory).
// launches spent on one-time copies of weights (planes, tile images): reported apart from a graph's own launches
std::atomic<uint64_t> g_prep_launches{0};

struct plane_store {
    std::mutex mu;
    struct entry { void * planes; int64_t rows, K; };
    std::unordered_map<const void *, entry> map;
    bool enabled = getenv("MI355_NO_PLANES") == nullptr;

    const void * get(hipStream_t s, const ggml_tensor * w) {
        if (!enabled || w->type != GGML_TYPE_Q6_K || w->buffer == nullptr || w->buffer->usage != GGML_BACKEND_BUFFER_USAGE_WEIGHTS) return nullptr;
        std::lock_guard<std::mutex> lock(mu);
        auto it = map.find(w->data);
        if (it != map.end()) return it->second.rows == w->ne[1] && it->second.K == w->ne[0] ? it->second.planes : nullptr;
        if (!ggml_is_contiguous(w)) return nullptr;
        void * planes = nullptr;
        if (hipMalloc(&planes, mi355_kq_planes_bytes(w->ne[1], w->ne[0]) + 256) != hipSuccess) {   // out of memory: stay with the packed rows
            (void) hipGetLastError();
            enabled = false;
            return nullptr;
        }
        const uint64_t before = mi355_launch_count();
        MI355_K_OK(mi355_kq_unpack_planes(s, to_mi355_type(w->type), w->data, planes, w->ne[1], w->ne[0]));
        g_prep_launches += mi355_launch_count() - before;
        map.emplace(w->data, entry{planes, w->ne[1], w->ne[0]});
        return planes;
    }
    // whether a tensor whose data lies in [base, base + size) has an entry
    bool any(const void * base, size_t size) {
        std::lock_guard<std::mutex> lock(mu);
        for (const auto & kv : map)
            if ((const char *) kv.first >= (const char *) base && (const char *) kv.first < (const char *) base + size) return true;
        return false;
    }
    // forget (and free) the planes of tensors whose data lies in [base, base + size); the caller has synchronized the device
    void drop(const void * base, size_t size) {
        std::lock_guard<std::mutex> lock(mu);
        for (auto it = map.begin(); it != map.end();) {
            if ((const char *) it->first >= (const char *) base && (const char *) it->first < (const char *) base + size) {
                MI355_HIP_OK(hipFree(it->second.planes));
                it = map.erase(it);
            } else {
                ++it;
            }
        }
    }
};
plane_store & planes() {
    static plane_store p;
    return p;
}

// Tile images of K-quant weight matrices for the wide-tile GEMM (mi355_kq_unpack_tiles: both int8 planes cut into 1 KiB tiles plus
// per-super-block scales, 2 bytes per weight), built the first time a matrix in a weights buffer meets a batch of TILE_MIN_BATCH
// rows or more and kept until that buffer is freed or the tensor is written again.  Keyed by the tensor's data address.
// MI355_NO_TILES=1 keeps the packed rows only.  Below TILE_MIN_BATCH rows the second copy's 2 bytes per weight make the product
// HBM-bound and the kernels that unpack the packed rows are quicker.  (Q6_K matrices on their images from 33 rows on, measured
// with llama-bench on the 8B Q4_K_M file: pp64 +1..4 %, pp96 and pp128 within 1.5 %, pp160 -4.5 %.)
constexpr int64_t TILE_MIN_BATCH = 192;
// Q5_K has no tile kernel on packed rows and no matrix-core kernel for few rows: its images serve every batch above the GEMV's
constexpr int64_t TILE_MIN_BATCH_Q5_K = 33;
inline int64_t tile_min_batch(ggml_type t) { return t == GGML_TYPE_Q5_K ? TILE_MIN_BATCH_Q5_K : TILE_MIN_BATCH; }
struct tile_store {
    std::mutex mu;
    struct entry { void * tiles; int64_t rows, K; };
    std::unordered_map<const void *, entry> map;
    bool enabled = getenv("MI355_NO_TILES") == nullptr;

    const void * get(hipStream_t s, const ggml_tensor * w) {
        if (!enabled || !has_tile_images(w->type) || w->buffer == nullptr ||
            w->buffer->usage != GGML_BACKEND_BUFFER_USAGE_WEIGHTS)
            return nullptr;
        std::lock_guard<std::mutex> lock(mu);
        auto it = map.find(w->data);
        if (it != map.end()) return it->second.rows == w->ne[1] && it->second.K == w->ne[0] ? it->second.tiles : nullptr;
        if (!ggml_is_contiguous(w)) return nullptr;
        void * tiles = nullptr;
        if (hipMalloc(&tiles, mi355_kq_tiles_bytes(to_mi355_type(w->type), w->ne[1], w->ne[0]) + 256) != hipSuccess) {   // out of memory: stay with the packed rows
            (void) hipGetLastError();
            enabled = false;
            return nullptr;
        }
        const uint64_t before = mi355_launch_count();
        MI355_K_OK(mi355_kq_unpack_tiles(s, to_mi355_type(w->type), w->data, tiles, w->ne[1], w->ne[0]));
        g_prep_launches += mi355_launch_count() - before;
        map.emplace(w->data, entry{tiles, w->ne[1], w->ne[0]});
        return tiles;
    }
    // whether a tensor whose data lies in [base, base + size) has an entry
    bool any(const void * base, size_t size) {
        std::lock_guard<std::mutex> lock(mu);
        for (const auto & kv : map)
            if ((const char *) kv.first >= (const char *) base && (const char *) kv.first < (const char *) base + size) return true;
        return false;
    }
    // forget (and free) the images of tensors whose data lies in [base, base + size); the caller has synchronized the device
    void drop(const void * base, size_t size) {
        std::lock_guard<std::mutex> lock(mu);
        for (auto it = map.begin(); it != map.end();) {
            if ((const char *) it->first >= (const char *) base && (const char *) it->first < (const char *) base + size) {
                MI355_HIP_OK(hipFree(it->second.tiles));
                it = map.erase(it);
            } else {
                ++it;
            }
        }
    }
};
tile_store & tiles() {
    static tile_store t;
    return t;
}

// ------------------------------------------------------------------------------- buffer
void buffer_free(ggml_backend_buffer_t buffer) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    MI355_HIP_OK(hipSetDevice(ctx->device));
    MI355_HIP_OK(hipDeviceSynchronize());
    planes().drop(ctx->base, ctx->size);
    tiles().drop(ctx->base, ctx->size);
    if (ctx->base) MI355_HIP_OK(hipFree(ctx->base));
    delete ctx;
}

void * buffer_get_base(ggml_backend_buffer_t buffer) { return ((buffer_ctx *) buffer->context)->base; }

// number of rows / elements per row of a tensor whose rows are contiguous blocks
int64_t tensor_nrows(const ggml_tensor * t) { return t->ne[1] * t->ne[2] * t->ne[3]; }

// Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, IQ4_XS, Q8_0 and Q6_K tensors live in the device row layout, which is defined by the rows of the tensor that owns the memory: a
// view (a slice of experts, a permuted or 1-D view of a cache) addresses bytes of that tensor, so transfers through a view go
// through the owner's layout at the view's byte offset.
struct repack_target {
    bool yes = false;
    void * base = nullptr;   // the owner's data
    int64_t k = 0, nrows = 0;
    size_t off = 0;          // byte offset of the tensor inside the owner
};
repack_target repack_of(const ggml_tensor * t) {
    repack_target r;
    const ggml_tensor * owner = t->view_src ? t->view_src : t;
    if (!is_repacked_type(owner->type) || owner->type != t->type || !ggml_is_contiguous(owner) || owner->data == nullptr) return r;
    r.yes = true;
    r.base = owner->data;
    r.k = owner->ne[0];
    r.nrows = tensor_nrows(owner);
    r.off = (size_t) ((const char *) t->data - (const char *) owner->data);
    return r;
}

// Copies through the null stream are ordered against every backend stream of the device (those are created blocking), in both
// directions, so plain uploads and read-backs need no device-wide synchronization of their own; the paths that reuse the shared
// staging buffer or free memory keep it.
void buffer_set_tensor(ggml_backend_buffer_t buffer, ggml_tensor * tensor, const void * data, size_t offset, size_t size) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    MI355_HIP_OK(hipSetDevice(ctx->device));
    if (size == 0) return;
    if (has_tile_images(tensor->type)) {
        MI355_HIP_OK(hipDeviceSynchronize());
        planes().drop(tensor->data, ggml_nbytes(tensor));   // rebuilt from the new contents on next use
        tiles().drop(tensor->data, ggml_nbytes(tensor));
    }
    if (const repack_target rt = repack_of(tensor); rt.yes) {
        MI355_HIP_OK(hipDeviceSynchronize());
        std::lock_guard<std::mutex> lock(stage().mu);
        void * tmp = stage().get(size);
        MI355_HIP_OK(hipMemcpy(tmp, data, size, hipMemcpyHostToDevice));
        MI355_K_OK(mi355_weights_scatter(nullptr, to_mi355_type(tensor->type), tmp, rt.base, rt.k, rt.nrows, rt.off + offset, size));
        MI355_HIP_OK(hipDeviceSynchronize());
    } else {
        MI355_HIP_OK(hipMemcpy((char *) tensor->data + offset, data, size, hipMemcpyHostToDevice));
    }
}

void buffer_get_tensor(ggml_backend_buffer_t buffer, const ggml_tensor * tensor, void * data, size_t offset, size_t size) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    MI355_HIP_OK(hipSetDevice(ctx->device));
    if (size == 0) return;
    if (const repack_target rt = repack_of(tensor); rt.yes) {
        MI355_HIP_OK(hipDeviceSynchronize());
        std::lock_guard<std::mutex> lock(stage().mu);
        void * tmp = stage().get(size);
        MI355_K_OK(mi355_weights_gather(nullptr, to_mi355_type(tensor->type), rt.base, tmp, rt.k, rt.nrows, rt.off + offset, size));
        MI355_HIP_OK(hipMemcpy(data, tmp, size, hipMemcpyDeviceToHost));
    } else {
        MI355_HIP_OK(hipMemcpy(data, (const char *) tensor->data + offset, size, hipMemcpyDeviceToHost));
    }
}

void buffer_memset_tensor(ggml_backend_buffer_t buffer, ggml_tensor * tensor, uint8_t value, size_t offset, size_t size) {
    if (size == 0) return;
    if (repack_of(tensor).yes) {
        std::vector<uint8_t> host(size, value);   // rare path: route through the layout permutation
        buffer_set_tensor(buffer, tensor, host.data(), offset, size);
        return;
    }
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    MI355_HIP_OK(hipSetDevice(ctx->device));
    MI355_HIP_OK(hipDeviceSynchronize());
    MI355_HIP_OK(hipMemset((char *) tensor->data + offset, value, size));
    MI355_HIP_OK(hipDeviceSynchronize());
}

bool buffer_cpy_tensor(ggml_backend_buffer_t buffer, const ggml_tensor * src, ggml_tensor * dst) {
    // same buffer type on both sides: identical layouts (device layout included), plain device copy
    if (src->buffer == nullptr || src->buffer->buft != buffer->buft) return false;
    // views of tensors in the device row layout may belong to owners with different rows: leave those to get + set
    if (is_repacked_type(src->type) && (src->view_src || dst->view_src)) return false;
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    MI355_HIP_OK(hipSetDevice(ctx->device));
    MI355_HIP_OK(hipDeviceSynchronize());
    if (dst->type == GGML_TYPE_Q6_K) planes().drop(dst->data, ggml_nbytes(dst));
    if (has_tile_images(dst->type)) tiles().drop(dst->data, ggml_nbytes(dst));
    MI355_HIP_OK(hipMemcpy(dst->data, src->data, ggml_nbytes(src), hipMemcpyDeviceToDevice));
    MI355_HIP_OK(hipDeviceSynchronize());
    return true;
}

void buffer_clear(ggml_backend_buffer_t buffer, uint8_t value) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    MI355_HIP_OK(hipSetDevice(ctx->device));
    MI355_HIP_OK(hipDeviceSynchronize());
    planes().drop(ctx->base, ctx->size);
    tiles().drop(ctx->base, ctx->size);
    MI355_HIP_OK(hipMemset(ctx->base, value, ctx->size));
    MI355_HIP_OK(hipDeviceSynchronize());
}

const ggml_backend_buffer_i buffer_iface = {
    /* .free_buffer   = */ buffer_free,
    /* .get_base      = */ buffer_get_base,
    /* .init_tensor   = */ nullptr,
    /* .memset_tensor = */ buffer_memset_tensor,
    /* .set_tensor    = */ buffer_set_tensor,
    /* .get_tensor    = */ buffer_get_tensor,
    /* .cpy_tensor    = */ buffer_cpy_tensor,
    /* .clear         = */ buffer_clear,
    /* .reset         = */ nullptr,
};

// ------------------------------------------------------------------------------- buffer type
const char * buft_get_name(ggml_backend_buffer_type_t buft) { return ((device_ctx *) buft->device->context)->name.c_str(); }

ggml_backend_buffer_t buft_alloc_buffer(ggml_backend_buffer_type_t buft, size_t size) {
    device_ctx * dctx = (device_ctx *) buft->device->context;
    if (hipSetDevice(dctx->device) != hipSuccess) return nullptr;
    buffer_ctx * ctx = new buffer_ctx;
    ctx->device = dctx->device;
    ctx->size = size;
    // a little slack so 16-byte loads at the very end of the last tensor stay inside the allocation
    hipError_t err = hipMalloc(&ctx->base, size + 256);
    if (err != hipSuccess) {
        (void) hipGetLastError();
        GGML_LOG_ERROR("MI355: allocating %.2f MiB on device %d failed: %s\n", size / 1024.0 / 1024.0, dctx->device, hipGetErrorString(err));
        delete ctx;
        return nullptr;
    }
    return ggml_backend_buffer_init(buft, buffer_iface, ctx, size);
}

size_t buft_get_alignment(ggml_backend_buffer_type_t) { return 256; }

size_t buft_get_max_size(ggml_backend_buffer_type_t buft) {
    device_ctx * dctx = (device_ctx *) buft->device->context;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dctx->device) != hipSuccess) return SIZE_MAX;
    return prop.totalGlobalMem;
}

const ggml_backend_buffer_type_i buft_iface = {
    /* .get_name       = */ buft_get_name,
    /* .alloc_buffer   = */ buft_alloc_buffer,
    /* .get_alignment  = */ buft_get_alignment,
    /* .get_max_size   = */ buft_get_max_size,
    /* .get_alloc_size = */ nullptr,   // ggml_nbytes: the device layout keeps every tensor's footprint
    /* .is_host        = */ nullptr,
};

// ------------------------------------------------------------------------------- pinned host buffer type
// Host memory the device reaches by DMA without staging (hipHostMalloc): llama.cpp places the logits it reads back and the
// intermediate tensors its CPU backend hands to the device there (ggml_backend_dev_host_buffer_type, src/llama.cpp:8577,
// :9468), which makes those copies one DMA each and lets them be asynchronous.  To the CPU it is an ordinary CPU buffer.
const char * host_buft_get_name(ggml_backend_buffer_type_t) { return "MI355X_Host"; }

void host_buffer_free(ggml_backend_buffer_t buffer) { (void) hipHostFree(buffer->context); }

ggml_backend_buffer_t host_buft_alloc_buffer(ggml_backend_buffer_type_t buft, size_t size) {
    void * ptr = nullptr;
    if (getenv("MI355_NO_PINNED") != nullptr || hipHostMalloc(&ptr, size, hipHostMallocDefault) != hipSuccess) {
        (void) hipGetLastError();
        return ggml_backend_buft_alloc_buffer(ggml_backend_cpu_buffer_type(), size);   // pageable memory works too, only slower
    }
    ggml_backend_buffer_t buffer = ggml_backend_cpu_buffer_from_ptr(ptr, size);
    buffer->buft = buft;
    buffer->iface.free_buffer = host_buffer_free;
    return buffer;
}

ggml_backend_buffer_type_t mi355_host_buffer_type(ggml_backend_dev_t dev) {
    static ggml_backend_buffer_type host = {
        /* .iface   = */ {
            /* .get_name       = */ host_buft_get_name,
            /* .alloc_buffer   = */ host_buft_alloc_buffer,
            /* .get_alignment  = */ ggml_backend_cpu_buffer_type()->iface.get_alignment,
            /* .get_max_size   = */ nullptr,
            /* .get_alloc_size = */ ggml_backend_cpu_buffer_type()->iface.get_alloc_size,
            /* .is_host        = */ ggml_backend_cpu_buffer_type()->iface.is_host,
        },
        /* .device  = */ dev,
        /* .context = */ nullptr,
    };
    return &host;
}

// ------------------------------------------------------------------------------- op support
bool f32_rows(const ggml_tensor * t) { return t->type == GGML_TYPE_F32 && t->nb[0] == sizeof(float); }

// Buffers are 256-byte aligned and the allocator places tensors on that alignment, so a tensor's address is 16-byte aligned
// unless it is a view at an odd byte offset into its source (view_offs is relative to the tensor that owns the memory).
// The kernels that read with 128-bit loads need this; a view that fails it is left to another backend.
bool base_aligned16(const ggml_tensor * t) { return t->view_src == nullptr || t->view_offs % 16 == 0; }

bool supports_mul_mat(const ggml_tensor * op) {
    const ggml_tensor * a = op->src[0];
    const ggml_tensor * b = op->src[1];
    if (op->type != GGML_TYPE_F32 || !ggml_is_contiguous(op)) return false;
    if (b->type != GGML_TYPE_F32) return false;
    if (is_weight_type(a->type)) {
        // quantized weights: whole contiguous matrices; activations as 16-byte aligned f32 rows
        if (!ggml_is_contiguous(a)) return false;
        if (b->nb[0] != sizeof(float) || !strides_mult16(b) || !base_aligned16(b)) return false;
        if (b->ne[2] % a->ne[2] != 0 || b->ne[3] % a->ne[3] != 0) return false;
        return b->ne[1] <= 65535;
    }
    if (a->type == GGML_TYPE_F32 || a->type == GGML_TYPE_F16) {
        // dense weights (MoE router and other small matrices): any strides
        if (b->ne[2] % a->ne[2] != 0 || b->ne[3] % a->ne[3] != 0) return false;
        return op->ne[1] <= 65535 && op->ne[2] * op->ne[3] <= 65535;
    }
    return false;
}

bool supports_mul_mat_id(const ggml_tensor * op) {
    const ggml_tensor * as = op->src[0];
    const ggml_tensor * b = op->src[1];
    const ggml_tensor * ids = op->src[2];
    if (!is_weight_type(as->type) || !ggml_is_contiguous(as)) return false;
    if (b->type != GGML_TYPE_F32 || !ggml_is_contiguous(b)) return false;
    if (ids->type != GGML_TYPE_I32 || ids->nb[0] != sizeof(int32_t) || ids->nb[1] % sizeof(int32_t) != 0) return false;
    if (op->type != GGML_TYPE_F32 || !ggml_is_contiguous(op)) return false;
    if (as->ne[3] != 1 || b->ne[3] != 1 || ids->ne[2] != 1 || ids->ne[3] != 1) return false;
    if (as->ne[0] % 4 != 0) return false;
    return ids->ne[0] * ids->ne[1] <= 65535;
}

bool supports_flash_attn(const ggml_tensor * op) {
    const ggml_tensor * q = op->src[0];
    const ggml_tensor * k = op->src[1];
    const ggml_tensor * v = op->src[2];
    const ggml_tensor * mask = op->src[3];
    if (q->type != GGML_TYPE_F32 || q->nb[0] != 4) return false;
    const int64_t D = q->ne[0];
    if (!(D == 64 || D == 80 || D == 96 || D == 112 || D == 128 || D == 256) || k->ne[0] != D || v->ne[0] != D) return false;
    if (!strides_mult16(q) || !base_aligned16(q)) return false;
    for (const ggml_tensor * t : {k, v}) {
        if (t->type == GGML_TYPE_F16) {
            if (t->nb[0] != 2 || !strides_mult16(t) || !base_aligned16(t)) return false;
        } else if (!kv_operand_of(t).ok || D % 32 != 0 || q->ne[3] != 1) {   // Q8_0 / Q4_0 cache rows
            return false;
        }
    }
    if (q->ne[2] % k->ne[2] != 0 || k->ne[2] != v->ne[2] || k->ne[1] != v->ne[1]) return false;
    if (q->ne[3] != k->ne[3] || q->ne[3] != v->ne[3]) return false;
    if (mask && (mask->type != GGML_TYPE_F16 || !ggml_is_contiguous(mask) || mask->ne[0] != k->ne[1])) return false;
    if (!ggml_is_contiguous(op)) return false;
    return q->ne[1] <= 65535 && q->ne[2] <= 65535;
}

bool device_supports_op(ggml_backend_dev_t, const ggml_tensor * op) {
    switch (op->op) {
        case GGML_OP_NONE:
        case GGML_OP_RESHAPE:
        case GGML_OP_VIEW:
        case GGML_OP_PERMUTE:
        case GGML_OP_TRANSPOSE:
            return true;
        case GGML_OP_MUL_MAT:
            return supports_mul_mat(op);
        case GGML_OP_MUL_MAT_ID:
            return supports_mul_mat_id(op);
        case GGML_OP_FLASH_ATTN_EXT:
            return supports_flash_attn(op);
        case GGML_OP_RMS_NORM:
            return f32_rows(op->src[0]) && f32_rows(op);
        case GGML_OP_ADD:
        case GGML_OP_SUB:
        case GGML_OP_MUL:
        case GGML_OP_DIV:
            return op->src[0]->type == GGML_TYPE_F32 && op->src[1]->type == GGML_TYPE_F32 && op->type == GGML_TYPE_F32;
        case GGML_OP_UNARY:
            if (op->src[0]->type != GGML_TYPE_F32 || op->type != GGML_TYPE_F32) return false;
            switch (ggml_get_unary_op(op)) {
                case GGML_UNARY_OP_ABS: case GGML_UNARY_OP_SGN: case GGML_UNARY_OP_NEG: case GGML_UNARY_OP_STEP:
                case GGML_UNARY_OP_TANH: case GGML_UNARY_OP_ELU: case GGML_UNARY_OP_RELU: case GGML_UNARY_OP_SIGMOID:
                case GGML_UNARY_OP_GELU: case GGML_UNARY_OP_GELU_QUICK: case GGML_UNARY_OP_SILU:
                case GGML_UNARY_OP_HARDSWISH: case GGML_UNARY_OP_HARDSIGMOID: case GGML_UNARY_OP_EXP:
                    return true;
                default:
                    return false;
            }
        case GGML_OP_SCALE:
            return op->src[0]->type == GGML_TYPE_F32 && op->type == GGML_TYPE_F32;
        case GGML_OP_CPY:
        case GGML_OP_DUP:
        case GGML_OP_CONT: {
            const ggml_type st = op->src[0]->type;
            const ggml_type dt = op->op == GGML_OP_CPY ? op->src[1]->type : op->type;
            const bool sf = st == GGML_TYPE_F32 || st == GGML_TYPE_F16, df = dt == GGML_TYPE_F32 || dt == GGML_TYPE_F16;
            if (op->op == GGML_OP_CPY && st == GGML_TYPE_F32 && (dt == GGML_TYPE_Q8_0 || dt == GGML_TYPE_Q4_0)) {
                // the store into a quantized KV cache (contiguous f32 rows into consecutive blocks) and the copy back after a K-shift
                // (contiguous f32 rows into a view whose rows start on block boundaries)
                const ggml_tensor * a = op->src[0], * d = op->src[1];
                if (!ggml_is_contiguous(a) || a->ne[0] % 32 != 0 || !kv_operand_of(d).ok || !base_aligned16(a)) return false;
                return ggml_is_contiguous(d) ? ggml_nelements(a) == ggml_nelements(d) && d->ne[0] % 32 == 0 : ggml_are_same_shape(a, d);
            }
            if (op->op == GGML_OP_CPY && dt == GGML_TYPE_F32 && (st == GGML_TYPE_Q8_0 || st == GGML_TYPE_Q4_0)) {
                // ggml_cast of a quantized cache view to f32 (the first step of its K-shift)
                const ggml_tensor * a = op->src[0], * d = op->src[1];
                return ggml_is_contiguous(d) && ggml_are_same_shape(a, d) && a->ne[0] % 32 == 0 && kv_operand_of(a).ok && base_aligned16(d);
            }
            if (op->op == GGML_OP_CPY && st == dt && (st == GGML_TYPE_Q8_0 || st == GGML_TYPE_Q4_0)) {
                // consecutive blocks of a quantized tensor to consecutive blocks of another (the row copies of a cache defragmentation)
                const ggml_tensor * a = op->src[0], * d = op->src[1];
                return ggml_is_contiguous(a) && ggml_is_contiguous(d) && ggml_nelements(a) == ggml_nelements(d) && a->ne[0] % 32 == 0 && d->ne[0] % 32 == 0 &&
                       kv_operand_of(a).ok && kv_operand_of(d).ok;
            }
            return (sf && df) || (st == GGML_TYPE_I32 && dt == GGML_TYPE_I32);
        }
        case GGML_OP_GET_ROWS: {
            const ggml_tensor * a = op->src[0];
            if (op->src[1]->type != GGML_TYPE_I32 || op->type != GGML_TYPE_F32 || op->src[1]->ne[3] != 1) return false;
            if (a->type == GGML_TYPE_F32 || a->type == GGML_TYPE_F16) return true;
            // quantized rows: whole rows in the device layout (views over rows and batches are fine)
            return is_weight_type(a->type) && a->nb[0] == ggml_type_size(a->type) && a->nb[1] == ggml_row_size(a->type, a->ne[0]);
        }
        case GGML_OP_SOFT_MAX: {
            const ggml_tensor * mask = op->src[1];
            if (!f32_rows(op->src[0]) || !ggml_is_contiguous(op)) return false;
            if (mask && ((mask->type != GGML_TYPE_F32 && mask->type != GGML_TYPE_F16) || !ggml_is_contiguous(mask))) return false;
            return true;
        }
        case GGML_OP_ROPE: {
            const int mode = ((const int32_t *) op->op_params)[2];
            if (mode != 0 && mode != GGML_ROPE_TYPE_NEOX) return false;   // no mrope / vision
            // f32, or f16 onto f16 (the in-place rotation of an f16 K cache when the context is shifted)
            const bool f16 = op->src[0]->type == GGML_TYPE_F16 && op->type == GGML_TYPE_F16 && op->src[0]->nb[0] == sizeof(ggml_fp16_t) &&
                             op->nb[0] == sizeof(ggml_fp16_t);
            if (!(f16 || (f32_rows(op->src[0]) && f32_rows(op))) || op->src[1]->type != GGML_TYPE_I32) return false;
            if (op->src[2] && op->src[2]->type != GGML_TYPE_F32) return false;
            return op->src[0]->ne[0] % 2 == 0;
        }
        case GGML_OP_SUM_ROWS:
            return f32_rows(op->src[0]) && op->type == GGML_TYPE_F32;
        case GGML_OP_ARGSORT:
            return f32_rows(op->src[0]) && op->src[0]->ne[0] <= 1024 && ggml_is_contiguous(op);
        default:
            return false;
    }
}

// ------------------------------------------------------------------------------- op execution
void compute_mul_mat(backend_ctx * ctx, ggml_tensor * dst) {
    const ggml_tensor * a = dst->src[0];
    const ggml_tensor * b = dst->src[1];
    if (!is_weight_type(a->type)) {
        mi355_tensor da = desc(a), db = desc(b), dd = desc(dst);
        MI355_K_OK(mi355_mul_mat_f(ctx->stream, &da, &db, &dd));
        return;
    }
    const int64_t K = a->ne[0], N = a->ne[1], B = b->ne[1];
    const int64_t r2 = b->ne[2] / a->ne[2], r3 = b->ne[3] / a->ne[3];
    // the quantized activation, and behind it room for the slices of a product that is split along K
    const size_t split_q = mi355_mul_mat_q_ws_bytes(N, K, B), split_k = mi355_mul_mat_q8k_ws_bytes(N, K, B);
    const size_t ws_bytes = mi355_mul_mat_ws_bytes(K, B) + (split_q > split_k ? split_q : split_k);
    void * ws = ctx->workspace(ws_bytes);
    for (int64_t i3 = 0; i3 < b->ne[3]; i3++) {
        for (int64_t i2 = 0; i2 < b->ne[2]; i2++) {
            const char * W = (const char *) a->data + (i2 / r2) * a->nb[2] + (i3 / r3) * a->nb[3];
            const float * x = (const float *) ((const char *) b->data + i2 * b->nb[2] + i3 * b->nb[3]);
            float * y = (float *) ((char *) ctx->out_ptr(dst) + i2 * dst->nb[2] + i3 * dst->nb[3]);
            MI355_K_OK(mi355_mul_mat(ctx->stream, to_mi355_type(a->type), W, x, y, N, K, B, (int64_t) (b->nb[1] / sizeof(float)),
                                     (int64_t) (dst->nb[1] / sizeof(float)), ws, ws_bytes));
        }
    }
}

void compute_mul_mat_id(backend_ctx * ctx, ggml_tensor * dst) {
    const ggml_tensor * as = dst->src[0];
    const ggml_tensor * b = dst->src[1];
    const ggml_tensor * ids = dst->src[2];
    const int64_t K = as->ne[0], N = as->ne[1], n_expert = as->ne[2];
    const int64_t nb1 = b->ne[1], T = b->ne[2], n_used = ids->ne[0];
    const size_t ws_bytes = mi355_mul_mat_id_ws_bytes(K, n_expert, n_used, nb1, T);
    void * ws = ctx->workspace(ws_bytes);
    MI355_K_OK(mi355_mul_mat_id(ctx->stream, to_mi355_type(as->type), as->data, (const float *) b->data, (const int32_t *) ids->data,
                                (int64_t) (ids->nb[1] / sizeof(int32_t)), (float *) dst->data, N, K, n_expert, n_used, nb1, T, ws, ws_bytes));
}

void compute_flash_attn(backend_ctx * ctx, ggml_tensor * dst) {
    const ggml_tensor * q = dst->src[0];
    const ggml_tensor * k = dst->src[1];
    const ggml_tensor * v = dst->src[2];
    const ggml_tensor * mask = dst->src[3];
    float scale, max_bias, softcap;
    memcpy(&scale, (const float *) dst->op_params + 0, sizeof(float));
    memcpy(&max_bias, (const float *) dst->op_params + 1, sizeof(float));
    memcpy(&softcap, (const float *) dst->op_params + 2, sizeof(float));
    const int64_t D = q->ne[0], Nq = q->ne[1], Hq = q->ne[2], Nkv = k->ne[1], Hkv = k->ne[2];
    if (k->type != GGML_TYPE_F16 || v->type != GGML_TYPE_F16) {   // quantized cache (one batch: supports_op)
        const kv_operand ko = kv_operand_of(k), vo = kv_operand_of(v);
        GGML_ASSERT(ko.ok && vo.ok);
        const size_t ws_bytes = mi355_flash_attn_kv_ws_bytes(D, Nq, Nkv, Hq, Hkv, to_mi355_type(k->type), to_mi355_type(v->type));
        void * ws = ctx->workspace(ws_bytes);
        MI355_K_OK(mi355_flash_attn_ext_kv(ctx->stream, (const float *) q->data, ko.p, to_mi355_type(k->type), ko.base, ko.row_blocks, vo.p,
                                           to_mi355_type(v->type), vo.base, vo.row_blocks, mask ? mask->data : nullptr, (float *) dst->data, D, Nq, Nkv,
                                           Hq, Hkv, q->nb[1], q->nb[2], k->nb[1], k->nb[2], v->nb[1], v->nb[2], mask ? mask->nb[1] : 0, scale, max_bias,
                                           softcap, ws, ws_bytes, nullptr));
        return;
    }
    const size_t ws_bytes = mi355_flash_attn_ws_bytes(D, Nq, Nkv, Hq) < (size_t(256) << 20) ? mi355_flash_attn_ws_bytes(D, Nq, Nkv, Hq) : (size_t(256) << 20);
    void * ws = ctx->workspace(ws_bytes);
    for (int64_t i3 = 0; i3 < q->ne[3]; i3++) {
        MI355_K_OK(mi355_flash_attn_ext(ctx->stream, (const float *) ((const char *) q->data + i3 * q->nb[3]), (const char *) k->data + i3 * k->nb[3],
                                        (const char *) v->data + i3 * v->nb[3], mask ? mask->data : nullptr,
                                        (float *) ((char *) dst->data + i3 * dst->nb[3]), D, Nq, Nkv, Hq, Hkv, q->nb[1], q->nb[2], k->nb[1], k->nb[2],
                                        v->nb[1], v->nb[2], mask ? mask->nb[1] : 0, scale, max_bias, softcap, ws, ws_bytes));
    }
}

void compute_node(backend_ctx * ctx, ggml_tensor * node) {
    hipStream_t s = ctx->stream;
    switch (node->op) {
        case GGML_OP_MUL_MAT: compute_mul_mat(ctx, node); break;
        case GGML_OP_MUL_MAT_ID: compute_mul_mat_id(ctx, node); break;
        case GGML_OP_FLASH_ATTN_EXT: compute_flash_attn(ctx, node); break;
        case GGML_OP_RMS_NORM: {
            float eps;
            memcpy(&eps, node->op_params, sizeof(float));
            mi355_tensor a = desc(node->src[0]), d = desc(node);
            MI355_K_OK(mi355_rms_norm(s, &a, &d, eps));
        } break;
        case GGML_OP_ADD: case GGML_OP_SUB: case GGML_OP_MUL: case GGML_OP_DIV: {
            const int op = node->op == GGML_OP_ADD ? 0 : node->op == GGML_OP_SUB ? 1 : node->op == GGML_OP_MUL ? 2 : 3;
            mi355_tensor a = desc(node->src[0]), b = desc(node->src[1]), d = desc(node);
            MI355_K_OK(mi355_bin_bcast(s, op, &a, &b, &d));
        } break;
        case GGML_OP_UNARY: {
            mi355_tensor a = desc(node->src[0]), d = desc(node);
            MI355_K_OK(mi355_unary(s, (int) ggml_get_unary_op(node), &a, &d));
        } break;
        case GGML_OP_SCALE: {
            float f;
            memcpy(&f, node->op_params, sizeof(float));
            mi355_tensor a = desc(node->src[0]), d = desc(node);
            MI355_K_OK(mi355_scale(s, &a, &d, f));
        } break;
        case GGML_OP_CPY: {
            const ggml_tensor * dt = node->src[1];
            const ggml_tensor * st = node->src[0];
            if (st->type == dt->type && (st->type == GGML_TYPE_Q8_0 || st->type == GGML_TYPE_Q4_0)) {   // block ranges, each side in its owner's layout
                const kv_operand a = kv_operand_of(st), d = kv_operand_of(dt);
                GGML_ASSERT(a.ok && d.ok);
                const ptrdiff_t bb = (ptrdiff_t) ggml_type_size(st->type);
                MI355_K_OK(mi355_cpy_quant_blocks(s, to_mi355_type(st->type), a.base, (int64_t) (((const char *) a.p - (const char *) a.base) / bb), a.row_blocks,
                                                  (void *) d.base, (int64_t) (((const char *) d.p - (const char *) d.base) / bb), d.row_blocks,
                                                  ggml_nelements(dt) / 32));
                break;
            }
            const bool to_quant = dt->type == GGML_TYPE_Q8_0 || dt->type == GGML_TYPE_Q4_0;
            const bool from_quant = st->type == GGML_TYPE_Q8_0 || st->type == GGML_TYPE_Q4_0;
            if (to_quant || from_quant) {
                const ggml_tensor * qt = to_quant ? dt : st, * ft = to_quant ? st : dt;
                const kv_operand o = kv_operand_of(qt);
                GGML_ASSERT(o.ok);
                const int64_t bb = (int64_t) ggml_type_size(qt->type);
                const int64_t first = (int64_t) (((const char *) o.p - (const char *) o.base) / (ptrdiff_t) bb);
                if (to_quant && ggml_is_contiguous(qt)) {   // consecutive blocks, whatever the two shapes are
                    MI355_K_OK(mi355_cpy_f32_quant(s, to_mi355_type(qt->type), (const float *) ft->data, (void *) o.base, first, o.row_blocks, ggml_nelements(qt)));
                } else {
                    const int64_t strides[3] = {(int64_t) qt->nb[1] / bb, (int64_t) qt->nb[2] / bb, (int64_t) qt->nb[3] / bb};
                    MI355_K_OK(mi355_cpy_quant_view(s, to_mi355_type(qt->type), from_quant ? 1 : 0, (float *) ft->data, (void *) o.base, first, o.row_blocks,
                                                    qt->ne, strides));
                }
                break;
            }
            mi355_tensor a = desc(node->src[0]), d = desc(node->src[1]);
            MI355_K_OK(mi355_cpy(s, &a, &d));
        } break;
        case GGML_OP_DUP: case GGML_OP_CONT: {
            mi355_tensor a = desc(node->src[0]), d = desc(node);
            MI355_K_OK(mi355_cpy(s, &a, &d));
        } break;
        case GGML_OP_GET_ROWS: {
            mi355_tensor a = desc(node->src[0]), i = desc(node->src[1]), d = desc(node);
            MI355_K_OK(mi355_get_rows(s, &a, &i, &d));
        } break;
        case GGML_OP_SOFT_MAX: {
            float scale, max_bias;
            memcpy(&scale, (const float *) node->op_params + 0, sizeof(float));
            memcpy(&max_bias, (const float *) node->op_params + 1, sizeof(float));
            mi355_tensor a = desc(node->src[0]), d = desc(node), m;
            if (node->src[1]) m = desc(node->src[1]);
            MI355_K_OK(mi355_soft_max(s, &a, node->src[1] ? &m : nullptr, &d, scale, max_bias));
        } break;
        case GGML_OP_ROPE: {
            const int32_t * p = (const int32_t *) node->op_params;
            float freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow;
            memcpy(&freq_base, p + 5, sizeof(float));
            memcpy(&freq_scale, p + 6, sizeof(float));
            memcpy(&ext_factor, p + 7, sizeof(float));
            memcpy(&attn_factor, p + 8, sizeof(float));
            memcpy(&beta_fast, p + 9, sizeof(float));
            memcpy(&beta_slow, p + 10, sizeof(float));
            mi355_tensor a = desc(node->src[0]), d = desc(node);
            MI355_K_OK(mi355_rope(s, &a, (const int32_t *) node->src[1]->data, node->src[2] ? (const float *) node->src[2]->data : nullptr, &d,
                                  p[1], p[2], p[4], freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow));
        } break;
        case GGML_OP_SUM_ROWS: {
            mi355_tensor a = desc(node->src[0]), d = desc(node);
            MI355_K_OK(mi355_sum_rows(s, &a, &d));
        } break;
        case GGML_OP_ARGSORT: {
            mi355_tensor a = desc(node->src[0]), d = desc(node);
            MI355_K_OK(mi355_argsort(s, &a, &d, ((const int32_t *) node->op_params)[0] == GGML_SORT_ORDER_DESC ? 1 : 0));
        } break;
        default:
            GGML_ABORT("MI355: op %s reached graph_compute but is not supported (supports_op should have declined it)", ggml_op_name(node->op));
    }
}

// ------------------------------------------------------------------------------- backend (stream)
const char * backend_get_name(ggml_backend_t backend) { return ((backend_ctx *) backend->context)->name.c_str(); }

void backend_free(ggml_backend_t backend) {
    backend_ctx * ctx = (backend_ctx *) backend->context;
    (void) hipSetDevice(ctx->device);
    (void) hipStreamSynchronize(ctx->stream);
    if (ctx->ws) (void) hipFree(ctx->ws);
    if (ctx->act) (void) hipFree(ctx->act);
    if (ctx->iota) (void) hipFree(ctx->iota);
    if (ctx->rope_tab) (void) hipFree(ctx->rope_tab);
    if (ctx->cells) (void) hipFree(ctx->cells);
    if (ctx->tickets) (void) hipFree(ctx->tickets);
    if (ctx->stage) (void) hipHostFree(ctx->stage);
    for (hipEvent_t e : ctx->stage_done)
        if (e) (void) hipEventDestroy(e);
    if (ctx->replay.exec) (void) hipGraphExecDestroy(ctx->replay.exec);
    if (ctx->replay.graph) (void) hipGraphDestroy(ctx->replay.graph);
    if (getenv("MI355_GRAPH_STATS"))
        fprintf(stderr, "MI355 graph replay: %ld captures, %ld replays, %.1f us of host time per replay\n", ctx->replay.captures, ctx->replay.replays,
                ctx->replay.replays ? ctx->replay.host_us / (double) ctx->replay.replays : 0.0);
    if (getenv("MI355_GRAPH_STATS") && (ctx->async_uploads || ctx->events_recorded))
        fprintf(stderr, "MI355 transfers: %ld uploads on the backend stream, %ld events recorded\n", ctx->async_uploads, ctx->events_recorded);
    if (ctx->stream) (void) hipStreamDestroy(ctx->stream);
    delete ctx;
    delete backend;
}

// Asynchronous uploads and read-backs on the backend's own stream (ggml_backend_tensor_set_async / _get_async,
// ggml/src/ggml-backend.cpp:238-262): ordered with the graphs of this backend, complete after synchronize().  Tensors kept in
// the device row layout go through the synchronous path, which applies the permutation.
void backend_set_tensor_async(ggml_backend_t backend, ggml_tensor * tensor, const void * data, size_t offset, size_t size) {
    backend_ctx * ctx = (backend_ctx *) backend->context;
    ggml_backend_buffer_t buf = tensor->view_src ? tensor->view_src->buffer : tensor->buffer;
    // the layout permutation goes through the staging buffer; a K-quant matrix may have int8 planes or tile images to forget
    const bool has_images = (tensor->type == GGML_TYPE_Q4_K || tensor->type == GGML_TYPE_Q5_K) &&
                            (planes().any(tensor->data, ggml_nbytes(tensor)) || tiles().any(tensor->data, ggml_nbytes(tensor)));
    if (repack_of(tensor).yes || has_images || size == 0) {
        MI355_HIP_OK(hipStreamSynchronize(ctx->stream));
        buf->iface.set_tensor(buf, tensor, data, offset, size);
        return;
    }
    MI355_HIP_OK(hipSetDevice(ctx->device));
    MI355_HIP_OK(hipMemcpyAsync((char *) tensor->data + offset, data, size, hipMemcpyHostToDevice, ctx->stream));
    ctx->async_uploads++;
}

void backend_get_tensor_async(ggml_backend_t backend, const ggml_tensor * tensor, void * data, size_t offset, size_t size) {
    backend_ctx * ctx = (backend_ctx *) backend->context;
    ggml_backend_buffer_t buf = tensor->view_src ? tensor->view_src->buffer : tensor->buffer;
    if (repack_of(tensor).yes || size == 0) {
        MI355_HIP_OK(hipStreamSynchronize(ctx->stream));
        buf->iface.get_tensor(buf, tensor, data, offset, size);
        return;
    }
    MI355_HIP_OK(hipSetDevice(ctx->device));
    MI355_HIP_OK(hipMemcpyAsync(data, (const char *) tensor->data + offset, size, hipMemcpyDeviceToHost, ctx->stream));
}

// Copies a tensor into one of this backend's tensors on its stream (ggml_backend_tensor_copy_async, ggml-backend.cpp:380-409; the
// scheduler hands split inputs over this way, :1384).  Served: a source of this same backend, and a source in host memory
// produced by a backend that computes synchronously (the CPU backend: its result is complete when the scheduler gets here) of
// up to STAGE_BYTES.  A host source is copied into a pinned slot of this backend before the call returns and uploaded from the
// slot: the scheduler keeps the source alive only until the consuming split starts, and a later CPU split may reuse that
// memory while an upload that read it directly (a true DMA when the source is pinned) would still be in flight.
// Anything else returns false and the caller synchronizes and copies.
bool backend_cpy_tensor_async(ggml_backend_t backend_src, ggml_backend_t backend_dst, const ggml_tensor * src, ggml_tensor * dst) {
    backend_ctx * ctx = (backend_ctx *) backend_dst->context;
    ggml_backend_buffer_t dbuf = dst->view_src ? dst->view_src->buffer : dst->buffer;
    ggml_backend_buffer_t sbuf = src->view_src ? src->view_src->buffer : src->buffer;
    if (!dbuf || !sbuf || dbuf->buft->iface.get_name != buft_get_name || dbuf->buft->device != backend_dst->device) return false;
    if (!ggml_is_contiguous(src) || !ggml_is_contiguous(dst) || src->type != dst->type || ggml_nbytes(src) != ggml_nbytes(dst)) return false;
    if (repack_of(dst).yes || is_repacked_type(src->type)) return false;   // layout permutations take the synchronous path
    const size_t n = ggml_nbytes(src);
    if (ggml_backend_buffer_is_host(sbuf)) {
        ggml_backend_dev_t sdev = ggml_backend_get_device(backend_src);
        if (!sdev || ggml_backend_dev_type(sdev) != GGML_BACKEND_DEVICE_TYPE_CPU) return false;
        if (n > backend_ctx::STAGE_BYTES) return false;
        MI355_HIP_OK(hipSetDevice(ctx->device));
        if (!ctx->stage) {
            if (hipHostMalloc(&ctx->stage, backend_ctx::STAGE_SLOTS * backend_ctx::STAGE_BYTES, hipHostMallocDefault) != hipSuccess) {
                (void) hipGetLastError();
                ctx->stage = nullptr;
                return false;
            }
            for (hipEvent_t & e : ctx->stage_done) MI355_HIP_OK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
        }
        const int slot = ctx->stage_next;
        ctx->stage_next = (slot + 1) % backend_ctx::STAGE_SLOTS;
        MI355_HIP_OK(hipEventSynchronize(ctx->stage_done[slot]));   // the upload that last read this slot (never recorded: returns at once)
        void * at = (char *) ctx->stage + (size_t) slot * backend_ctx::STAGE_BYTES;
        memcpy(at, src->data, n);
        MI355_HIP_OK(hipMemcpyAsync(dst->data, at, n, hipMemcpyHostToDevice, ctx->stream));
        MI355_HIP_OK(hipEventRecord(ctx->stage_done[slot], ctx->stream));
    } else if (backend_src == backend_dst && sbuf->buft == dbuf->buft) {
        MI355_HIP_OK(hipSetDevice(ctx->device));
        MI355_HIP_OK(hipMemcpyAsync(dst->data, src->data, n, hipMemcpyDeviceToDevice, ctx->stream));
    } else {
        return false;
    }
    ctx->cache.valid = false;
    return true;
}

void backend_synchronize(ggml_backend_t backend) {
    backend_ctx * ctx = (backend_ctx *) backend->context;
    MI355_HIP_OK(hipStreamSynchronize(ctx->stream));
}

// Events (ggml_backend_event_*, ggml/src/ggml-backend.cpp:413-445): a HIP event without timing.  The model loader records one
// after each chunk it uploads from a pinned buffer and waits for it before refilling that buffer
// (src/llama-model-loader.cpp:1040-1046); the scheduler uses them between the copies of a pipelined graph (:1370-1438).
void backend_event_record(ggml_backend_t backend, ggml_backend_event_t event) {
    backend_ctx * ctx = (backend_ctx *) backend->context;
    MI355_HIP_OK(hipSetDevice(ctx->device));
    MI355_HIP_OK(hipEventRecord((hipEvent_t) event->context, ctx->stream));
    ctx->events_recorded++;
}

void backend_event_wait(ggml_backend_t backend, ggml_backend_event_t event) {
    backend_ctx * ctx = (backend_ctx *) backend->context;
    MI355_HIP_OK(hipSetDevice(ctx->device));
    MI355_HIP_OK(hipStreamWaitEvent(ctx->stream, (hipEvent_t) event->context, 0));
}

// ------------------------------------------------------------------------------- graph execution with local fusion
// The graph llama.cpp builds for a token is ~25 small nodes per layer.  The executor looks a few nodes ahead and
// replaces the sequences below by the fused entry points of the kernel library (each is tested bit-identical to the
// separate launches).  A pattern only matches when the skipped intermediate has exactly one consumer in this graph
// and is not a graph output, so nothing observable changes:
//   RMS_NORM -> MUL(weight)                      one launch, and the Q8_1 form of the result when a quantized MUL_MAT follows
//   UNARY(SILU) -> MUL                           one launch, same
//   FLASH_ATTN_EXT (few rows) -> MUL_MAT         attention also writes the Q8_1 form of its output
//   MUL_MAT, MUL_MAT, ... on the same src1       activation quantized once; up to 4 matrices per GEMV launch
//   MUL_MAT -> ADD(residual)                     residual added in the GEMV / tile GEMM epilogue
bool is_noop(const ggml_tensor * t) {
    switch (t->op) {
        case GGML_OP_NONE: case GGML_OP_RESHAPE: case GGML_OP_VIEW: case GGML_OP_PERMUTE: case GGML_OP_TRANSPOSE: return true;
        default: return ggml_is_empty(t);
    }
}

struct graph_walk {
    ggml_cgraph * g;
    int n;
    std::vector<int> uses;   // per node index: how many nodes of this graph read it
    std::vector<const ggml_tensor *> nodes;

    explicit graph_walk(ggml_cgraph * cg) : g(cg), n(ggml_graph_n_nodes(cg)), uses(n, 0), nodes(n) {
        std::unordered_map<const ggml_tensor *, int> index;
        index.reserve((size_t) n * 2);
        for (int i = 0; i < n; i++) {
            nodes[i] = ggml_graph_node(g, i);
            index[nodes[i]] = i;
        }
        auto count = [&](const ggml_tensor * t) {
            if (!t) return;
            auto it = index.find(t);
            if (it != index.end()) uses[it->second]++;
        };
        for (int i = 0; i < n; i++) {   // each distinct tensor a node reads counts once
            const ggml_tensor * seen[GGML_MAX_SRC + 1];
            int n_seen = 0;
            auto once = [&](const ggml_tensor * t) {
                if (!t) return;
                for (int k = 0; k < n_seen; k++)
                    if (seen[k] == t) return;
                seen[n_seen++] = t;
                count(t);
            };
            for (int s = 0; s < GGML_MAX_SRC; s++) once(nodes[i]->src[s]);
            once(nodes[i]->view_src);
        }
    }
    int next(int i) const {   // next node that launches work, or n
        for (i = i + 1; i < n; i++)
            if (!is_noop(nodes[i])) return i;
        return n;
    }
    bool sole_use(int i) const { return uses[i] == 1 && !(nodes[i]->flags & GGML_TENSOR_FLAG_OUTPUT); }
};

bool is_quant_gemv_candidate(const ggml_tensor * mm) {
    // quantized weights in 16-byte aligned rows, one 2-D activation matrix of at most 32 contiguous rows (up to 4: the batch-1
    // kernels; from there to 32: the weight-streaming matrix-core kernel)
    const ggml_tensor * a = mm->src[0];
    const ggml_tensor * b = mm->src[1];
    if (mm->op != GGML_OP_MUL_MAT || !is_weight_type(a->type)) return false;
    if (a->ne[2] != 1 || a->ne[3] != 1 || b->ne[2] != 1 || b->ne[3] != 1) return false;
    if (b->ne[1] > 32 || b->nb[1] != b->ne[0] * sizeof(float)) return false;
    const int64_t K = a->ne[0];
    if (K % 256 != 0 || K % aligned_row_elems(a->type) != 0) return false;   // rows that are 16-byte multiples (Q6_K: 210-byte, IQ4_XS: 136-byte blocks)
    return ((uintptr_t) a->data & 15) == 0 && ((uintptr_t) b->data & 15) == 0;
}

bool is_q8k_tile_candidate(const ggml_tensor * mm) {
    const ggml_tensor * a = mm->src[0];
    const ggml_tensor * b = mm->src[1];
    if (mm->op != GGML_OP_MUL_MAT || !has_tile_images(a->type)) return false;
    if (a->ne[2] != 1 || a->ne[3] != 1 || b->ne[2] != 1 || b->ne[3] != 1) return false;
    if (b->ne[1] <= 32 || b->nb[1] % 16 != 0) return false;
    const int64_t K = a->ne[0];
    if (K % aligned_row_elems(a->type) != 0) return false;
    return ((uintptr_t) a->data & 15) == 0 && ((uintptr_t) b->data & 15) == 0;
}

// does the node after `i` (skipping views) multiply a quantized matrix by the tensor whose data starts at `data`?
bool feeds_quant_gemv(const graph_walk & w, int i, const void * data, int64_t K, int64_t B) {
    const int j = w.next(i);
    if (j >= w.n) return false;
    const ggml_tensor * mm = w.nodes[j];
    return is_quant_gemv_candidate(mm) && mm->src[1]->data == data && mm->src[0]->ne[0] == K && mm->src[1]->ne[1] == B;
}

// does the node after `i` (skipping views) run the K-quant tile GEMM on the tensor whose data starts at `data`?
bool feeds_q8k_tiles(const graph_walk & w, int i, const void * data, int64_t K, int64_t B) {
    const int j = w.next(i);
    if (j >= w.n || K % 256 != 0 || B > 65535) return false;
    const ggml_tensor * mm = w.nodes[j];
    return is_q8k_tile_candidate(mm) && mm->src[1]->data == data && mm->src[0]->ne[0] == K && mm->src[1]->ne[1] == B &&
           mm->src[1]->nb[1] == (size_t) K * sizeof(float);
}

// 33 to 128 activation rows on Q4_K: the weight-streaming matrix-core kernel on the packed rows (mi355_mul_mat_mid), which takes
// the activations as tile images
bool takes_mid_kernel(const ggml_tensor * mm) {
    const int64_t B = mm->src[1]->ne[1];
    return mm->src[0]->type == GGML_TYPE_Q4_K && B > 32 && B <= 128 &&
           mi355_mul_mat_mid_supported(MI355_Q4_K, mm->src[0]->data, mm->src[0]->ne[0], B) && (size_t) ggml_nbytes(mm->src[0]) < ((size_t) 1 << 32);
}

// activation format of a K-quant tile product: tile images when the batch is large and the weights have (or can get) theirs
int q8k_format_for(hipStream_t s, const ggml_tensor * mm) {
    if (takes_mid_kernel(mm)) return ACT_Q8KT;
    return mm->src[1]->ne[1] >= tile_min_batch(mm->src[0]->type) && tiles().get(s, mm->src[0]) != nullptr ? ACT_Q8KT : ACT_Q8K;
}

// A MUL_MAT_ID with few (token, expert slot) pairs streams each slot's expert through the GEMV on Q8_1 activations; with many
// slots and K-quant experts it sorts the slots by expert and uses the tile kernel on per-super-block activations.
bool mmid_uses_tiles(const ggml_tensor * op) {
    const ggml_tensor * as = op->src[0];
    const int64_t K = as->ne[0], slots = op->src[2]->ne[0] * op->src[1]->ne[2];
    if (slots < 32 || as->ne[2] > 256 || K % 256 != 0 || ((uintptr_t) as->data & 15) != 0) return false;
    return has_tile_images(as->type) && K % aligned_row_elems(as->type) == 0;   // the types of the routed super-block tile kernel
}

// does the node after `i` (skipping views) route the rows of the tensor at `data` through quantized experts by GEMV?
bool feeds_quant_mmid(const graph_walk & w, int i, const void * data, int64_t K, int64_t rows) {
    const int j = w.next(i);
    if (j >= w.n) return false;
    const ggml_tensor * op = w.nodes[j];
    if (op->op != GGML_OP_MUL_MAT_ID || mmid_uses_tiles(op)) return false;
    const ggml_tensor * b = op->src[1];
    return b->data == data && b->ne[0] == K && b->ne[1] * b->ne[2] == rows && K % 32 == 0;
}

// Is the tensor at `data` first read by an f32 MUL_MAT (the router of a mixture-of-experts layer) and, a few nodes later, by a
// MUL_MAT_ID that takes its rows quantized to Q8_1?  Nothing in between may take the activation slots: only the router's own chain
// (SOFT_MAX, ARGSORT, GET_ROWS, SUM_ROWS, DIV and views) is accepted there.
bool router_then_quant_mmid(const graph_walk & w, int i, const void * data, int64_t K, int64_t rows) {
    int j = w.next(i);
    if (j >= w.n || w.nodes[j]->op != GGML_OP_MUL_MAT || w.nodes[j]->src[0]->type != GGML_TYPE_F32 || w.nodes[j]->src[1]->data != data) return false;
    for (int k = 0; k < 8; k++) {
        j = w.next(j);
        if (j >= w.n) return false;
        const ggml_tensor * op = w.nodes[j];
        if (op->op == GGML_OP_MUL_MAT_ID) {
            const ggml_tensor * b = op->src[1];
            return !mmid_uses_tiles(op) && b->data == data && b->ne[0] == K && b->ne[1] * b->ne[2] == rows && K % 32 == 0;
        }
        if (op->op != GGML_OP_SOFT_MAX && op->op != GGML_OP_ARGSORT && op->op != GGML_OP_GET_ROWS && op->op != GGML_OP_SUM_ROWS && op->op != GGML_OP_DIV)
            return false;
    }
    return false;
}

// Do the bytes of two tensors intersect?  A pattern that runs a node ahead of its place in the graph must check this: the
// graph allocator reuses the memory of a tensor once its last reader, in graph order, has run, so a node that comes later may
// write where an earlier, not yet executed node still has to read.
// (This is also why the prefill sequence ROPE(q), MUL_MAT(k), ROPE(k), MUL_MAT(v), CPY(k), CPY(v) stays four glue launches: the
// allocator gives the v product the k product's memory and the k product the unrotated q's, so the products cannot move ahead of
// the rotations, and a single launch would need k and v at once.)
bool bytes_overlap(const ggml_tensor * a, const ggml_tensor * b) {
    const char * a0 = (const char *) a->data, * b0 = (const char *) b->data;
    return a0 < b0 + ggml_nbytes(b) && b0 < a0 + ggml_nbytes(a);
}

// Up to three projections of one activation with their ROPE and f16 cache-store nodes, to be served by ONE launch (decode,
// batch <= 4):  MUL_MAT -> [RESHAPE] -> ROPE [-> CPY to an f16 view]   and   MUL_MAT -> CPY to an f16 view.
// llm_build_kv lists them as  Q, rope(Q), K, rope(K), V, cpy(K), cpy(V): the window takes nodes from `first` on while every
// one of them belongs to such a chain, so nothing outside the window is reordered.
struct qkv_window {
    int n_ch = 0;
    int last = -1;                  // last node the window consumed
    mi355_gemv_rope_mat mats[3];
    mi355_rope_desc rd;
    int n_store = 0;                // cache stores among the epilogues
    bool redirect = false;          // every cache store starts at cell kv_head: address the cache through ctx->cells
    bool ok = false;                // at least one epilogue, whole heads
};

qkv_window match_qkv_window(backend_ctx * ctx, const graph_walk & w, int first, const void * b_data, int64_t K, int64_t B) {
    qkv_window win;
    struct chain {
        const ggml_tensor * mm;     // the product
        const ggml_tensor * out;    // the tensor that currently holds the chain's value (product or its ROPE)
        int out_index;
        mi355_gemv_rope_mat m;
        void * cache_base;          // cache stores that start at cell kv_head: the cache tensor's first byte
        int64_t first_block0;       // ... of a quantized cache: the block index of its cell 0 within the tensor that owns the memory
    } ch[3];
    int n_ch = 0, last = first - 1;
    mi355_rope_desc rd;
    memset(&rd, 0, sizeof(rd));
    bool have_rope = false;
    auto node_index_sole = [&](const ggml_tensor * t, int from, int to) {   // t is a node in [from, to) with one reader
        for (int k = from; k < to; k++)
            if (w.nodes[k] == t) return w.sole_use(k);
        return false;
    };
    for (int k = first; k < w.n && k < first + 24; k++) {
        const ggml_tensor * t = w.nodes[k];
        if (is_noop(t)) continue;
        if (t->op == GGML_OP_MUL_MAT) {
            if (n_ch == 3 || !is_quant_gemv_candidate(t) || t->src[1]->data != b_data || t->src[1]->ne[0] != K || t->src[1]->ne[1] != B ||
                !w.sole_use(k) || t->ne[0] % 2 != 0 || !ggml_is_contiguous(t))
                break;
            chain & c = ch[n_ch++];
            c.mm = t; c.out = t; c.out_index = k;
            c.cache_base = nullptr;
            c.first_block0 = 0;
            c.m.type = to_mi355_type(t->src[0]->type);
            c.m.W = t->src[0]->data;
            c.m.N = t->ne[0];
            c.m.epilogue = MI355_EPI_STORE;
            c.m.dst = t->data;
            c.m.dst_stride = t->ne[0];
            c.m.nb1 = c.m.nb2 = 0;
            last = k;
            continue;
        }
        if (t->op == GGML_OP_ROPE) {
            const ggml_tensor * src = t->src[0];
            chain * c = nullptr;
            for (int q = 0; q < n_ch; q++) {
                if (ch[q].m.epilogue != MI355_EPI_STORE) continue;
                if (src == ch[q].mm) c = &ch[q];
                else if (src->op == GGML_OP_RESHAPE && src->src[0] == ch[q].mm && ggml_is_contiguous(src) && node_index_sole(src, ch[q].out_index + 1, k)) c = &ch[q];
            }
            const int32_t * p = (const int32_t *) t->op_params;
            const int64_t N = c ? c->m.N : 0;
            if (!c || t->src[1]->type != GGML_TYPE_I32 || !ggml_is_contiguous(t) || t->type != GGML_TYPE_F32 || t->ne[0] * t->ne[1] != N || t->ne[2] != B ||
                t->ne[3] != 1 || (t->src[2] && t->src[2]->type != GGML_TYPE_F32) || p[2] != 0 || p[1] % 2 != 0 || p[1] <= 0 || p[1] > t->ne[0] ||
                t->ne[0] % 2 != 0)
                break;
            mi355_rope_desc r;
            memset(&r, 0, sizeof(r));
            r.pos = (const int32_t *) t->src[1]->data;
            r.cells = ctx->iota;
            r.freq_factors = t->src[2] ? (const float *) t->src[2]->data : nullptr;
            r.head_dim = t->ne[0];
            r.n_dims = p[1];
            r.mode = 0;
            r.n_ctx_orig = p[4];
            memcpy(&r.freq_base, p + 5, sizeof(float));
            memcpy(&r.freq_scale, p + 6, sizeof(float));
            memcpy(&r.ext_factor, p + 7, sizeof(float));
            memcpy(&r.attn_factor, p + 8, sizeof(float));
            memcpy(&r.beta_fast, p + 9, sizeof(float));
            memcpy(&r.beta_slow, p + 10, sizeof(float));
            if (have_rope && memcmp(&r, &rd, sizeof(rd)) != 0) break;   // one set of rope parameters per launch
            rd = r;
            have_rope = true;
            c->m.epilogue = MI355_EPI_ROPE;
            c->m.dst = t->data;
            c->m.dst_stride = N;
            c->out = t;
            c->out_index = k;
            last = k;
            continue;
        }
        if (t->op == GGML_OP_CPY) {
            chain * c = nullptr;
            for (int q = 0; q < n_ch; q++)
                if (t->src[0] == ch[q].out && (ch[q].m.epilogue == MI355_EPI_STORE || ch[q].m.epilogue == MI355_EPI_ROPE)) c = &ch[q];
            const ggml_tensor * d = t->src[1];
            const bool quant = d->type == GGML_TYPE_Q8_0 || d->type == GGML_TYPE_Q4_0;
            if (!c || !w.sole_use(c->out_index) || (d->type != GGML_TYPE_F16 && !quant) || !ggml_is_contiguous(d) || ggml_nelements(d) != c->m.N * B ||
                ((uintptr_t) d->data & 1) != 0)
                break;
            if (quant) {   // Q8_0 / Q4_0 cache: the launch quantizes the row's blocks where the CPY node would
                const kv_operand o = kv_operand_of(d);
                if (!o.ok || c->m.N % 32 != 0 || ((uintptr_t) o.base & 1) != 0) break;
                const ptrdiff_t bb = (ptrdiff_t) ggml_type_size(d->type);
                c->m.epilogue = c->m.epilogue == MI355_EPI_ROPE ? MI355_EPI_ROPE_QCACHE : MI355_EPI_QCACHE;
                c->m.dst = (void *) o.base;
                c->m.dst_stride = to_mi355_type(d->type);
                c->m.nb1 = (int64_t) (((const char *) o.p - (const char *) o.base) / bb);   // with rd.cells = iota: row b goes b * N / 32 blocks further
                c->m.nb2 = o.row_blocks;
                c->out = nullptr;
                if (ctx->kv_head >= 0 && d->view_src && d->view_src->data &&
                    (const char *) d->data - (const char *) d->view_src->data == (ptrdiff_t) (ctx->kv_head * (c->m.N / 32) * bb)) {
                    c->cache_base = d->view_src->data;
                    c->first_block0 = (int64_t) (((const char *) d->view_src->data - (const char *) o.base) / bb);
                }
                last = k;
                continue;
            }
            c->m.epilogue = c->m.epilogue == MI355_EPI_ROPE ? MI355_EPI_ROPE_CACHE : MI355_EPI_CACHE;
            c->m.dst = d->data;
            c->m.dst_stride = 0;
            c->m.nb1 = c->m.N * 2;
            c->out = nullptr;
            if (ctx->kv_head >= 0 && d->view_src && d->view_src->data &&
                (const char *) d->data - (const char *) d->view_src->data == (ptrdiff_t) (ctx->kv_head * c->m.N * 2))
                c->cache_base = d->view_src->data;
            last = k;
            continue;
        }
        break;
    }
    bool any_epilogue = false;
    for (int q = 0; q < n_ch; q++) any_epilogue = any_epilogue || ch[q].m.epilogue != MI355_EPI_STORE;
    if (!any_epilogue) return win;
    if (!have_rope) {   // cache stores only: rows are one "head"; any even divisor of every N serves
        rd.cells = ctx->iota;
        rd.head_dim = 2; rd.n_dims = 2; rd.n_ctx_orig = 1; rd.freq_base = 10000.0f; rd.freq_scale = 1.0f; rd.attn_factor = 1.0f; rd.beta_fast = 32.0f; rd.beta_slow = 1.0f;
    }
    bool heads_ok = true;
    int n_base = 0;
    auto quant_store = [](const mi355_gemv_rope_mat & m) { return m.epilogue == MI355_EPI_ROPE_QCACHE || m.epilogue == MI355_EPI_QCACHE; };
    for (int q = 0; q < n_ch; q++) {
        win.mats[q] = ch[q].m;
        if (win.mats[q].epilogue != MI355_EPI_STORE) heads_ok = heads_ok && win.mats[q].N % rd.head_dim == 0;
        if (win.mats[q].epilogue == MI355_EPI_ROPE_CACHE || win.mats[q].epilogue == MI355_EPI_CACHE) win.mats[q].nb2 = rd.head_dim * 2;
        if (win.mats[q].epilogue >= MI355_EPI_ROPE_CACHE) {
            win.n_store++;
            if (ch[q].cache_base) n_base++;
        }
    }
    if (!heads_ok) return win;
    // Cache stores that all start at cell kv_head address the cache tensor through the device-side cell list instead
    // of through the view's own address, so the launch's arguments do not change from token to token.
    if (win.n_store > 0 && n_base == win.n_store) {
        for (int q = 0; q < n_ch; q++) {
            if (!ch[q].cache_base) continue;
            if (quant_store(win.mats[q])) win.mats[q].nb1 = ch[q].first_block0;
            else win.mats[q].dst = ch[q].cache_base;
        }
        rd.cells = ctx->cells;
        win.redirect = true;
    }
    win.n_ch = n_ch;
    win.last = last;
    win.rd = rd;
    win.ok = true;
    return win;
}

void note_window_writes(backend_ctx * ctx, const qkv_window & win, int64_t B) {
    if (win.redirect) ctx->kv_redirected += win.n_store;
    for (int q = 0; q < win.n_ch; q++) {
        if (win.mats[q].epilogue >= MI355_EPI_ROPE_QCACHE) continue;   // a quantized cache is never the source of a cached activation
        const bool f32_out = win.mats[q].epilogue == MI355_EPI_STORE || win.mats[q].epilogue == MI355_EPI_ROPE;
        ctx->note_write(win.mats[q].dst, (size_t) win.mats[q].N * (size_t) B * (f32_out ? sizeof(float) : 2));
    }
}

// Prefill (more than 4 rows): build_llama lists  MUL_MAT(q), ROPE(q), MUL_MAT(k), ROPE(k), MUL_MAT(v), CPY(k -> cache),
// CPY(v -> cache).  The window runs the three products and then ONE launch that rotates q in place, rotates k and stores k and v
// to the f16 cache.  The graph allocator hands the memory of the unrotated q to the k product and that of the unrotated k to
// the v product, so the rotations cannot simply wait for the products: instead the q and k products write straight into the
// memory of their ROPE nodes' results, which nothing else can occupy before those results are read (q by attention, k by its
// cache store), and are rotated there.
// Several K-quant products on one activation at a large batch: those that have tile images go out as one launch of the wide-tile
// GEMM, whatever their K-quant types, so that their tiles fill the compute units together (mi355_mul_mat_q8k_tiled_mixed).  idx: graph
// positions of the products, all reading the same src1.  Returns the mask of the products done (0 or at least two bits).
unsigned tiled_multi(backend_ctx * ctx, hipStream_t s, const graph_walk & w, const int * idx, int n) {
    const ggml_tensor * b = w.nodes[idx[0]]->src[1];
    const int64_t K = b->ne[0], B = b->ne[1];
    // 33 to 128 rows: the Q4_K ones among them as one launch of the weight-streaming kernel on packed rows (mi355_mul_mat_mid_multi)
    {
        mi355_gemv_mat mm_mid[3];
        int64_t Ns[3];
        unsigned mask = 0;
        int m = 0;
        for (int k = 0; k < n && k < 3; k++) {
            const ggml_tensor * mm = w.nodes[idx[k]];
            if (!is_q8k_tile_candidate(mm) || mm->src[1]->data != b->data || mm->src[1]->ne[0] != K || mm->src[1]->ne[1] != B || mm->src[1]->nb[1] != b->nb[1] ||
                mm->type != GGML_TYPE_F32 || mm->nb[0] != sizeof(float) || mm->nb[1] % sizeof(float) != 0 || !takes_mid_kernel(mm))
                continue;
            mm_mid[m].type = MI355_Q4_K;
            mm_mid[m].W = mm->src[0]->data;
            mm_mid[m].N = mm->src[0]->ne[1];
            mm_mid[m].dst = (float *) ctx->out_ptr(mm);
            mm_mid[m].dst_stride = (int64_t) (mm->nb[1] / sizeof(float));
            mm_mid[m].residual = nullptr;
            Ns[m] = mm_mid[m].N;
            m++;
            mask |= 1u << k;
        }
        if (m >= 2) {
            if (!ctx->cached(b->data, K, B, ACT_Q8KT)) {
                void * fresh = ctx->act_slot(mi355_act_q8k_tiled_bytes(K, B));
                MI355_K_OK(mi355_quantize_act_q8k_tiled(s, (const float *) b->data, fresh, K, B, (int64_t) (b->nb[1] / sizeof(float))));
                ctx->cache = act_cache{b->data, K, B, ACT_Q8KT, true, fresh};
            }
            const size_t split_bytes = mi355_mul_mat_mid_multi_ws_bytes(m, Ns, K, B);
            void * split_ws = split_bytes ? ctx->workspace(split_bytes) : nullptr;
            MI355_K_OK(mi355_mul_mat_mid_multi(s, MI355_Q4_K, m, mm_mid, ctx->cache.ptr, K, B, split_ws, split_bytes));
            for (int k = 0; k < m; k++) ctx->note_write(mm_mid[k].dst, (size_t) mm_mid[k].N * (size_t) B * sizeof(float));
            return mask;
        }
    }
    const void * tl[3] = {nullptr, nullptr, nullptr};
    int n_with = 0;
    for (int k = 0; k < n && k < 3; k++) {
        const ggml_tensor * mm = w.nodes[idx[k]];
        if (!is_q8k_tile_candidate(mm) || mm->src[1]->data != b->data || mm->src[1]->ne[0] != K || mm->src[1]->ne[1] != B || mm->src[1]->nb[1] != b->nb[1] ||
            mm->type != GGML_TYPE_F32 || mm->nb[0] != sizeof(float) || mm->nb[1] % sizeof(float) != 0 || takes_mid_kernel(mm) || q8k_format_for(s, mm) != ACT_Q8KT)
            continue;
        tl[k] = tiles().get(s, mm->src[0]);
        n_with += tl[k] != nullptr;
    }
    if (n_with < 2) return 0;
    if (!ctx->cached(b->data, K, B, ACT_Q8KT)) {
        void * fresh = ctx->act_slot(mi355_act_q8k_tiled_bytes(K, B));
        MI355_K_OK(mi355_quantize_act_q8k_tiled(s, (const float *) b->data, fresh, K, B, (int64_t) (b->nb[1] / sizeof(float))));
        ctx->cache = act_cache{b->data, K, B, ACT_Q8KT, true, fresh};
    }
    mi355_tiled_mat mats[3];
    int types[3] = {0, 0, 0};
    unsigned mask = 0;
    int m = 0;
    for (int k = 0; k < n && k < 3; k++) {
        const ggml_tensor * mm = w.nodes[idx[k]];
        if (!tl[k]) continue;
        types[m] = to_mi355_type(mm->src[0]->type);
        mats[m].tiles = tl[k];
        mats[m].dst = (float *) ctx->out_ptr(mm);
        mats[m].residual = nullptr;
        mats[m].N = mm->src[0]->ne[1];
        mats[m].dst_stride = (int64_t) (mm->nb[1] / sizeof(float));
        m++;
        mask |= 1u << k;
    }
    MI355_K_OK(mi355_mul_mat_q8k_tiled_mixed(s, m, types, mats, ctx->cache.ptr, K, B));
    for (int k = 0; k < m; k++) ctx->note_write(mats[k].dst, (size_t) mats[k].N * (size_t) B * sizeof(float));
    return mask;
}

struct prefill_qkv {
    bool ok = false;
    int ik = -1, iv = -1, last = -1;
    const ggml_tensor * rq = nullptr, * rk = nullptr, * mk = nullptr, * mv = nullptr, * ck = nullptr, * cv = nullptr;
};

prefill_qkv match_prefill_qkv(const graph_walk & w, int i) {
    prefill_qkv p;
    const ggml_tensor * mq = w.nodes[i];
    const ggml_tensor * b = mq->src[1];
    const int64_t B = b->ne[1];
    auto product_ok = [&](const ggml_tensor * m, int idx) {
        return m->op == GGML_OP_MUL_MAT && is_weight_type(m->src[0]->type) && m->src[0]->ne[2] == 1 && m->src[0]->ne[3] == 1 && m->src[1] == b &&
               b->ne[2] == 1 && b->ne[3] == 1 && ggml_is_contiguous(m) && m->type == GGML_TYPE_F32 && w.sole_use(idx);
    };
    // the ROPE that reads product m, directly or through a RESHAPE nobody else reads
    auto rope_of = [&](const ggml_tensor * r, const ggml_tensor * m, int from, int to) {
        if (r->op != GGML_OP_ROPE || r->type != GGML_TYPE_F32 || !ggml_is_contiguous(r) || r->ne[3] != 1 || r->ne[2] != B) return false;
        const ggml_tensor * src = r->src[0];
        if (src != m) {
            if (src->op != GGML_OP_RESHAPE || src->src[0] != m || !ggml_is_contiguous(src)) return false;
            bool sole = false;
            for (int k = from; k < to; k++)
                if (w.nodes[k] == src) sole = w.sole_use(k);
            if (!sole) return false;
        }
        const int32_t * q = (const int32_t *) r->op_params;
        return r->ne[0] * r->ne[1] == m->ne[0] && r->src[1]->type == GGML_TYPE_I32 && (!r->src[2] || r->src[2]->type == GGML_TYPE_F32) &&
               (q[2] == 0 || q[2] == 2) && q[1] > 0 && q[1] % 2 == 0 && q[1] <= r->ne[0] && r->ne[0] % 2 == 0 && r->ne[0] <= 2048;
    };
    if (B <= 4 || B > IOTA_N || !product_ok(mq, i)) return p;
    const int j1 = w.next(i);
    if (j1 >= w.n || !rope_of(w.nodes[j1], mq, i + 1, j1)) return p;
    const int j2 = w.next(j1);
    if (j2 >= w.n || !product_ok(w.nodes[j2], j2)) return p;
    const int j3 = w.next(j2);
    if (j3 >= w.n || !rope_of(w.nodes[j3], w.nodes[j2], j2 + 1, j3) || !w.sole_use(j3)) return p;
    const int j4 = w.next(j3);
    if (j4 >= w.n || !product_ok(w.nodes[j4], j4)) return p;
    const int j5 = w.next(j4), j6 = j5 < w.n ? w.next(j5) : w.n;
    if (j6 >= w.n) return p;
    const ggml_tensor * rq = w.nodes[j1], * mk = w.nodes[j2], * rk = w.nodes[j3], * mv = w.nodes[j4], * ck = w.nodes[j5], * cv = w.nodes[j6];
    auto store_ok = [&](const ggml_tensor * c, const ggml_tensor * src) {
        const ggml_tensor * d = c->src[1];
        if (c->op != GGML_OP_CPY || c->src[0] != src || !ggml_is_contiguous(d) || ggml_nelements(d) != ggml_nelements(src) || ((uintptr_t) d->data & 1) != 0)
            return false;
        if (d->type == GGML_TYPE_F16) return true;
        // a Q8_0 / Q4_0 cache: whole blocks per head, adjacent-pair rotation (the launch quantizes 16 lanes x 2 elements per block)
        const int32_t * q = (const int32_t *) rq->op_params;
        return (d->type == GGML_TYPE_Q8_0 || d->type == GGML_TYPE_Q4_0) && kv_operand_of(d).ok && rq->ne[0] % 32 == 0 && q[2] == 0;
    };
    if (!store_ok(ck, rk) || !store_ok(cv, mv)) return p;
    // one set of rope parameters, positions and frequency factors; k and v heads of q's size
    if (memcmp(rq->op_params, rk->op_params, 11 * sizeof(int32_t)) != 0 || rq->src[1] != rk->src[1] || rq->src[2] != rk->src[2]) return p;
    if (rq->ne[0] != rk->ne[0] || mv->ne[0] != mk->ne[0]) return p;
    // what the products write early must not be read or written by anything else inside the window
    if (bytes_overlap(rq, rk) || bytes_overlap(rq, mv) || bytes_overlap(rk, mv) || bytes_overlap(rq, b) || bytes_overlap(rk, b)) return p;
    // ... and what the rotations read late must survive the products: in the last layer the allocator gives the memory of the
    // position vector, whose last reader in graph order is ROPE(k), to the v product
    for (const ggml_tensor * in : {rq->src[1], rq->src[2]}) {
        if (in && (bytes_overlap(in, rq) || bytes_overlap(in, rk) || bytes_overlap(in, mv))) return p;
    }
    p.ok = true;
    p.ik = j2; p.iv = j4; p.last = j6;
    p.rq = rq; p.rk = rk; p.mk = mk; p.mv = mv; p.ck = ck; p.cv = cv;
    return p;
}

// SOFT_MAX (no mask, scale 1) at node i followed by ARGSORT(descending) of its result: expert probabilities and their order
struct moe_route_match {
    bool ok = false;
    int j_argsort = -1;
};
moe_route_match match_moe_route(const graph_walk & w, int i) {
    moe_route_match r;
    const ggml_tensor * node = w.nodes[i];
    const int j = w.next(i);
    const ggml_tensor * nxt = j < w.n ? w.nodes[j] : nullptr;
    if (node->op != GGML_OP_SOFT_MAX || node->src[1] || !nxt || nxt->op != GGML_OP_ARGSORT || nxt->src[0] != node) return r;
    float scale, max_bias;
    memcpy(&scale, (const float *) node->op_params + 0, sizeof(float));
    memcpy(&max_bias, (const float *) node->op_params + 1, sizeof(float));
    const ggml_tensor * x = node->src[0];
    r.ok = scale == 1.0f && max_bias == 0.0f && x->ne[0] <= 64 && x->type == GGML_TYPE_F32 && ggml_is_contiguous(x) && ggml_is_contiguous(node) &&
           ggml_is_contiguous(nxt) && nxt->type == GGML_TYPE_I32 && ((const int32_t *) nxt->op_params)[0] == GGML_SORT_ORDER_DESC;
    r.j_argsort = j;
    return r;
}

// GET_ROWS(probabilities of the selected experts) at node i -> SUM_ROWS -> DIV: normalised expert weights
struct moe_weights_match {
    bool ok = false;
    int last = -1;
    const ggml_tensor * probs = nullptr, * ids = nullptr, * raw = nullptr, * sum = nullptr, * div = nullptr;
    int64_t n_expert = 0, n_used = 0, T = 0, ids_stride = 0;
};
moe_weights_match match_moe_weights(const graph_walk & w, int i) {
    moe_weights_match m;
    const ggml_tensor * node = w.nodes[i];
    const int j = w.next(i);
    const ggml_tensor * nxt = j < w.n ? w.nodes[j] : nullptr;
    if (node->op != GGML_OP_GET_ROWS || !nxt || nxt->op != GGML_OP_SUM_ROWS) return m;
    const ggml_tensor * probs = node->src[0];   // [1, n_expert, T]
    const ggml_tensor * ids = node->src[1];     // [n_used, T]
    const int jd = w.next(j);
    const ggml_tensor * div = jd < w.n ? w.nodes[jd] : nullptr;
    const ggml_tensor * w2d = nxt->src[0];       // [n_used, T] reshape of the GET_ROWS result
    const int64_t n_expert = probs->ne[1], T = probs->ne[2], n_used = ids->ne[0];
    m.ok = div && div->op == GGML_OP_DIV && div->src[0] == w2d && div->src[1] == nxt && w2d->op == GGML_OP_RESHAPE && w2d->src[0] == node &&
           probs->type == GGML_TYPE_F32 && probs->ne[0] == 1 && probs->ne[3] == 1 && ggml_is_contiguous(probs) && ids->type == GGML_TYPE_I32 &&
           ids->nb[0] == sizeof(int32_t) && ids->ne[1] == T && ids->ne[2] == 1 && ids->ne[3] == 1 && n_used <= 64 && n_used <= n_expert &&
           ggml_is_contiguous(node) && node->ne[0] == 1 && node->ne[1] == n_used && node->ne[2] == T && ggml_is_contiguous(w2d) &&
           ggml_is_contiguous(nxt) && ggml_is_contiguous(div) && w2d->ne[0] == n_used && w2d->ne[1] == T && ggml_nelements(nxt) == T;
    m.last = jd;
    m.probs = probs; m.ids = ids; m.raw = node; m.sum = nxt; m.div = div;
    m.n_expert = n_expert; m.n_used = n_used; m.T = T;
    m.ids_stride = (int64_t) (ids->nb[1] / sizeof(int32_t));
    return m;
}

// MUL(expert outputs, weights) at node i -> ADD over the expert slots [-> ADD(residual)]: weighted sum of the selected experts
struct moe_combine_match {
    bool ok = false;
    int last = -1;
    const ggml_tensor * ex = nullptr, * wt = nullptr, * out = nullptr;
    const float * residual = nullptr;
    int64_t n_embd = 0, n_used = 0, T = 0;
};
moe_combine_match match_moe_combine(const graph_walk & w, int i) {
    moe_combine_match c;
    const ggml_tensor * node = w.nodes[i];
    const int j = w.next(i);
    const ggml_tensor * nxt = j < w.n ? w.nodes[j] : nullptr;
    if (node->op != GGML_OP_MUL || node->ne[1] < 2 || node->ne[1] > 64 || node->ne[3] != 1 || !nxt || nxt->op != GGML_OP_ADD) return c;
    const ggml_tensor * ex = node->src[0];
    const ggml_tensor * wt = node->src[1];
    const int64_t n_embd = node->ne[0], n_used = node->ne[1], T = node->ne[2];
    auto slot_view = [&](const ggml_tensor * v, int64_t e) {
        return v && v->op == GGML_OP_VIEW && v->view_src == node && v->view_offs == (size_t) e * node->nb[1] && v->ne[0] == n_embd && v->ne[1] == T &&
               v->ne[2] == 1 && v->ne[3] == 1 && v->nb[1] == node->nb[2] && v->nb[0] == sizeof(float);
    };
    bool ok = ex->type == GGML_TYPE_F32 && wt->type == GGML_TYPE_F32 && ggml_are_same_shape(ex, node) && ggml_is_contiguous(ex) && ggml_is_contiguous(node) &&
              ggml_is_contiguous(wt) && wt->ne[0] == 1 && wt->ne[1] == n_used && wt->ne[2] == T && wt->ne[3] == 1 && n_embd % 4 == 0 && T <= 65535 &&
              (((uintptr_t) ex->data | (uintptr_t) node->data) & 15) == 0;
    int k = j;   // the ADD chain: ((slot0 + slot1) + slot2) + ...
    const ggml_tensor * sum = nullptr;
    for (int64_t e = 1; ok && e < n_used; e++) {
        const ggml_tensor * add = k < w.n ? w.nodes[k] : nullptr;
        ok = add && add->op == GGML_OP_ADD && slot_view(add->src[1], e) && (e == 1 ? slot_view(add->src[0], 0) : add->src[0] == sum) &&
             ggml_is_contiguous(add) && add->type == GGML_TYPE_F32 && ((uintptr_t) add->data & 15) == 0;
        if (ok && e + 1 < n_used) ok = w.sole_use(k);   // intermediate sums are not materialised
        if (ok) {
            sum = add;
            if (e + 1 < n_used) k = w.next(k);
        }
    }
    if (!ok) return c;
    c.last = k;
    c.out = sum;
    const int jr = w.next(k);
    const ggml_tensor * radd = jr < w.n ? w.nodes[jr] : nullptr;
    if (radd && radd->op == GGML_OP_ADD && w.sole_use(k) && (radd->src[0] == sum || radd->src[1] == sum)) {
        const ggml_tensor * res = radd->src[0] == sum ? radd->src[1] : radd->src[0];
        if (res->type == GGML_TYPE_F32 && ggml_are_same_shape(res, sum) && ggml_is_contiguous(res) && ggml_is_contiguous(radd) &&
            (((uintptr_t) res->data | (uintptr_t) radd->data) & 15) == 0) {
            c.residual = (const float *) res->data;
            c.out = radd;
            c.last = jr;
        }
    }
    c.ok = true;
    c.ex = ex; c.wt = wt;
    c.n_embd = n_embd; c.n_used = n_used; c.T = T;
    return c;
}

// The norm + router launch writes y, the logits, the probabilities and the order while it reads x, the norm weights and the router:
// the later tensors must not lie on the earlier ones' memory (the soft-max may be in place on the logits, as in separate launches).
bool router_outputs_apart(const ggml_tensor * x, const ggml_tensor * nw, const ggml_tensor * W, const ggml_tensor * y, const ggml_tensor * logits,
                          const ggml_tensor * probs, const ggml_tensor * order) {
    for (const ggml_tensor * in : {x, nw, W})
        for (const ggml_tensor * o : {logits, probs, order})
            if (bytes_overlap(in, o)) return false;
    if (bytes_overlap(y, logits) || bytes_overlap(y, probs) || bytes_overlap(y, order) || bytes_overlap(order, logits) || bytes_overlap(order, probs)) return false;
    return probs->data == logits->data || !bytes_overlap(probs, logits);
}

// The prefill window of match_prefill_qkv as ONE launch of the wide-tile GEMM: Q, K and V products whose epilogue rotates q and k
// and stores k and v into the f16 cache views (mi355_mul_mat_q8k_tiled_qkv_rope).  Needs tile images of all three matrices, f16
// caches and ROPE in its adjacent-pair mode.  The {cos, sin} table of the batch is written by the first layer's call of a graph.
bool tiled_qkv_rope(backend_ctx * ctx, hipStream_t s, const graph_walk & w, int i, const prefill_qkv & p) {
    const ggml_tensor * mm[3] = {w.nodes[i], p.mk, p.mv};
    const ggml_tensor * b = mm[0]->src[1];
    const ggml_tensor * rq = p.rq;
    const int64_t K = b->ne[0], B = b->ne[1], D = rq->ne[0];
    const int32_t * op = (const int32_t *) rq->op_params;
    const ggml_tensor * dk = p.ck->src[1], * dv = p.cv->src[1];
    if (op[2] != 0 || dk->type != GGML_TYPE_F16 || dv->type != GGML_TYPE_F16 || rq->src[1]->ne[0] != B || !ggml_is_contiguous(rq->src[1]) || B > IOTA_N) return false;
    if (rq->src[2] && !ggml_is_contiguous(rq->src[2])) return false;
    const void * tl[3];
    int types[3];
    for (int k = 0; k < 3; k++) {
        const ggml_tensor * m = mm[k];
        if (!is_q8k_tile_candidate(m) || m->src[1]->data != b->data || m->src[1]->nb[1] != b->nb[1] || takes_mid_kernel(m) || q8k_format_for(s, m) != ACT_Q8KT ||
            m->src[0]->ne[1] % D != 0)
            return false;
        tl[k] = tiles().get(s, m->src[0]);
        if (!tl[k]) return false;
        types[k] = to_mi355_type(m->src[0]->type);
    }
    const int64_t HK = p.rk->ne[1];
    if (mm[1]->src[0]->ne[1] != HK * D || mm[2]->src[0]->ne[1] != HK * D || ((uintptr_t) rq->data & 15) != 0) return false;
    // the batch's rotations: once per graph (positions, frequency factors and parameters are the same in every layer)
    const size_t tab_floats = (size_t) B * (size_t) D;
    const bool tab_ok = ctx->rope_tab && ctx->rope_tab_serial == ctx->graph_serial && ctx->rope_tab_pos == rq->src[1]->data &&
                        ctx->rope_tab_ff == (rq->src[2] ? rq->src[2]->data : nullptr) && ctx->rope_tab_D == D && ctx->rope_tab_T == B &&
                        memcmp(ctx->rope_tab_params, op, sizeof(ctx->rope_tab_params)) == 0;
    if (!tab_ok) {
        if (tab_floats > ctx->rope_tab_floats) {
            if (!ctx->may_allocate()) return false;
            if (ctx->rope_tab) {
                MI355_HIP_OK(hipStreamSynchronize(ctx->stream));
                MI355_HIP_OK(hipFree(ctx->rope_tab));
                ctx->rope_tab = nullptr;
            }
            ctx->rope_tab_floats = tab_floats;
            MI355_HIP_OK(hipMalloc((void **) &ctx->rope_tab, tab_floats * sizeof(float)));
        }
        float freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow;
        memcpy(&freq_base, op + 5, sizeof(float));
        memcpy(&freq_scale, op + 6, sizeof(float));
        memcpy(&ext_factor, op + 7, sizeof(float));
        memcpy(&attn_factor, op + 8, sizeof(float));
        memcpy(&beta_fast, op + 9, sizeof(float));
        memcpy(&beta_slow, op + 10, sizeof(float));
        MI355_K_OK(mi355_rope_table(s, (const int32_t *) rq->src[1]->data, rq->src[2] ? (const float *) rq->src[2]->data : nullptr, ctx->rope_tab, B, D, op[1], op[4],
                                    freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow));
        ctx->rope_tab_serial = ctx->graph_serial;
        ctx->rope_tab_pos = rq->src[1]->data;
        ctx->rope_tab_ff = rq->src[2] ? rq->src[2]->data : nullptr;
        ctx->rope_tab_D = D;
        ctx->rope_tab_T = B;
        memcpy(ctx->rope_tab_params, op, sizeof(ctx->rope_tab_params));
    }
    if (!ctx->cached(b->data, K, B, ACT_Q8KT)) {
        void * fresh = ctx->act_slot(mi355_act_q8k_tiled_bytes(K, B));
        MI355_K_OK(mi355_quantize_act_q8k_tiled(s, (const float *) b->data, fresh, K, B, (int64_t) (b->nb[1] / sizeof(float))));
        ctx->cache = act_cache{b->data, K, B, ACT_Q8KT, true, fresh};
    }
    mi355_tiled_mat mats[3];
    void * dst[3] = {rq->data, dk->data, dv->data};
    for (int k = 0; k < 3; k++) {
        mats[k].tiles = tl[k];
        mats[k].dst = (float *) dst[k];
        mats[k].residual = nullptr;
        mats[k].N = mm[k]->src[0]->ne[1];
        mats[k].dst_stride = mats[k].N;
    }
    MI355_K_OK(mi355_mul_mat_q8k_tiled_qkv_rope(s, types, mats, ctx->cache.ptr, K, B, ctx->rope_tab, ctx->iota, D, op[1], (size_t) (HK * D * 2), (size_t) (D * 2),
                                                (size_t) (HK * D * 2), (size_t) (D * 2)));
    ctx->note_write(rq->data, ggml_nbytes(rq));
    ctx->note_write(dk->data, ggml_nbytes(dk));
    ctx->note_write(dv->data, ggml_nbytes(dv));
    return true;
}

// Runs node i and possibly a few of its successors; returns the index of the last node consumed.
int compute_fused(backend_ctx * ctx, const graph_walk & w, int i) {
    hipStream_t s = ctx->stream;
    ggml_tensor * node = (ggml_tensor *) w.nodes[i];
    const int j = w.next(i);
    ggml_tensor * nxt = j < w.n ? (ggml_tensor *) w.nodes[j] : nullptr;

    if (node == ctx->done_ahead) {   // went out with an earlier product's launch
        ctx->done_ahead = nullptr;
        return i;
    }
    // ---- prefill: Q, K and V products, then both rotations and both cache stores in one launch (see match_prefill_qkv)
    if (node->op == GGML_OP_MUL_MAT && ctx->n_redirect == 0 && node->src[1]->ne[1] > 4) {
        const prefill_qkv p = match_prefill_qkv(w, i);
        if (p.ok) {
            if (tiled_qkv_rope(ctx, s, w, i, p)) return p.last;
            ctx->redirect_node[0] = node;  ctx->redirect_to[0] = p.rq->data;
            ctx->redirect_node[1] = p.mk;  ctx->redirect_to[1] = p.rk->data;
            ctx->n_redirect = 2;
            const int at[3] = {i, p.ik, p.iv};
            const unsigned together = tiled_multi(ctx, s, w, at, 3);   // those with tile images in one launch
            for (int k = 0; k < 3; k++) {
                if (together & (1u << k)) continue;
                const int done = compute_fused(ctx, w, at[k]);
                GGML_ASSERT(done == at[k]);   // a product followed by its ROPE (or by a product, or by the stores) takes nothing with it
            }
            ctx->n_redirect = 0;
            const ggml_tensor * rq = p.rq;
            const int32_t * op = (const int32_t *) rq->op_params;
            float freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow;
            memcpy(&freq_base, op + 5, sizeof(float));
            memcpy(&freq_scale, op + 6, sizeof(float));
            memcpy(&ext_factor, op + 7, sizeof(float));
            memcpy(&attn_factor, op + 8, sizeof(float));
            memcpy(&beta_fast, op + 9, sizeof(float));
            memcpy(&beta_slow, op + 10, sizeof(float));
            const int64_t D = rq->ne[0], H = rq->ne[1], HK = p.rk->ne[1], T = rq->ne[2];
            // an f16 cache view: its data and the byte strides of a cell and a head; a quantized one: the owning tensor's data, the
            // view's first block within it and the owner's blocks per row
            struct store_dest { int type; void * base; int64_t a, b; };
            auto dest_of = [&](const ggml_tensor * d) {
                if (d->type == GGML_TYPE_F16) return store_dest{MI355_F16, d->data, HK * D * 2, D * 2};
                const kv_operand o = kv_operand_of(d);
                return store_dest{to_mi355_type(d->type), (void *) o.base,
                                  (int64_t) (((const char *) o.p - (const char *) o.base) / (ptrdiff_t) ggml_type_size(d->type)), o.row_blocks};
            };
            const store_dest dk = dest_of(p.ck->src[1]), dv = dest_of(p.cv->src[1]);
            MI355_K_OK(mi355_rope_kv_store_typed(s, (float *) rq->data, (const float *) p.rk->data, (const float *) p.mv->data, dk.type, dk.base, dk.a, dk.b,
                                                 dv.type, dv.base, dv.a, dv.b, (const int32_t *) rq->src[1]->data, ctx->iota,
                                                 rq->src[2] ? (const float *) rq->src[2]->data : nullptr, T, H, HK, D, op[1], op[2], op[4], freq_base,
                                                 freq_scale, ext_factor, attn_factor, beta_fast, beta_slow));
            ctx->note_write(rq->data, ggml_nbytes(rq));
            ctx->note_write(p.rk->data, ggml_nbytes(p.rk));
            ctx->note_write(p.ck->src[1]->data, ggml_nbytes(p.ck->src[1]));
            ctx->note_write(p.cv->src[1]->data, ggml_nbytes(p.cv->src[1]));
            return p.last;
        }
    }
    // ---- RMS_NORM -> MUL(weight vector)
    if (node->op == GGML_OP_RMS_NORM && nxt && nxt->op == GGML_OP_MUL && nxt->src[0] == node && w.sole_use(i)) {
        const ggml_tensor * x = node->src[0];
        const ggml_tensor * wt = nxt->src[1];
        const int64_t K = x->ne[0], rows = ggml_nrows(x);
        if (ggml_is_contiguous(x) && ggml_is_contiguous(nxt) && wt->type == GGML_TYPE_F32 && ggml_is_contiguous(wt) && ggml_nelements(wt) == K &&
            K % 32 == 0 && K <= 16384 && x->type == GGML_TYPE_F32 && nxt->type == GGML_TYPE_F32 &&
            (((uintptr_t) x->data | (uintptr_t) nxt->data | (uintptr_t) wt->data) & 15) == 0) {
            float eps;
            memcpy(&eps, node->op_params, sizeof(float));
            void * act = nullptr;
            // one decoded token: the norm goes into the Q/K/V launch when that launch's products are the only readers of the
            // normalised row (every group normalises and quantizes the row for itself; the f32 row is not materialised)
            if (rows == 1 && K <= 4096 && K % 1024 == 0 && !(nxt->flags & GGML_TENSOR_FLAG_OUTPUT)) {
                const int jq = w.next(j);
                if (jq < w.n && is_quant_gemv_candidate(w.nodes[jq]) && w.nodes[jq]->src[1]->data == nxt->data) {
                    const qkv_window win = match_qkv_window(ctx, w, jq, nxt->data, K, 1);
                    if (win.ok && win.n_ch == w.uses[j]) {
                        MI355_K_OK(mi355_rms_norm_mul_mat_vec_q_rope(s, (const float *) x->data, (const float *) wt->data, eps, win.n_ch, win.mats, K, &win.rd));
                        note_window_writes(ctx, win, 1);
                        ctx->cache.valid = false;
                        return win.last;
                    }
                }
            }
            if (rows > 8 && feeds_q8k_tiles(w, j, nxt->data, K, rows)) {   // prefill: the per-super-block form for the tile GEMM
                const int fmt = q8k_format_for(s, w.nodes[w.next(j)]);
                act = ctx->act_slot(fmt == ACT_Q8KT ? mi355_act_q8k_tiled_bytes(K, rows) : mi355_act_q8k_bytes(K, rows));
                if (fmt == ACT_Q8KT)
                    MI355_K_OK(mi355_rms_norm_mul_quant_q8k_tiled(s, (const float *) x->data, K, (const float *) wt->data, (float *) nxt->data, K, act, K, rows, eps));
                else
                    MI355_K_OK(mi355_rms_norm_mul_quant_q8k(s, (const float *) x->data, K, (const float *) wt->data, (float *) nxt->data, K, act, K, rows, eps));
                ctx->cache = act_cache{nxt->data, K, rows, fmt, true, act};
                return j;
            }
            if (rows <= 32 && feeds_quant_gemv(w, j, nxt->data, K, rows)) act = ctx->act_slot(mi355_act_bytes(K, rows));
            // a mixture-of-experts layer: the f32 router product comes first, the experts' MUL_MAT_ID then reads the same rows quantized
            else if (rows <= 8 && router_then_quant_mmid(w, j, nxt->data, K, rows)) {
                act = ctx->act_slot(mi355_act_bytes(K, rows));
                // ... and the router product, its soft-max and the order go out with the norm (one group per row has the row in registers)
                const int jr = w.next(j);
                const ggml_tensor * rt = w.nodes[jr];   // the MUL_MAT (router_then_quant_mmid)
                const ggml_tensor * W = rt->src[0];
                const int js = w.next(jr);
                const moe_route_match r = js < w.n ? match_moe_route(w, js) : moe_route_match();
                if (r.ok && w.nodes[js]->src[0] == rt && w.sole_use(jr) && K <= 4096 && W->ne[0] == K && W->ne[1] <= 64 && W->ne[2] == 1 && W->ne[3] == 1 &&
                    W->nb[0] == sizeof(float) && W->nb[1] % 16 == 0 && ((uintptr_t) W->data & 15) == 0 && rt->src[1]->ne[1] == rows && rt->src[1]->ne[2] == 1 &&
                    rt->src[1]->ne[3] == 1 && ggml_is_contiguous(rt) && rt->type == GGML_TYPE_F32 && rt->ne[0] == W->ne[1] && !(nxt->flags & GGML_TENSOR_FLAG_OUTPUT) &&
                    router_outputs_apart(x, wt, W, nxt, rt, w.nodes[js], w.nodes[r.j_argsort])) {
                    const ggml_tensor * sm = w.nodes[js], * as = w.nodes[r.j_argsort];
                    MI355_K_OK(mi355_rms_norm_mul_quant_router(s, (const float *) x->data, K, (const float *) wt->data, (float *) nxt->data, K, act, K, rows, eps,
                                                               (const float *) W->data, (int64_t) (W->nb[1] / sizeof(float)), (float *) rt->data, (float *) sm->data,
                                                               (int32_t *) as->data, W->ne[1]));
                    ctx->cache = act_cache{nxt->data, K, rows, ACT_Q8_1, true, act};
                    return r.j_argsort;
                }
            }
            MI355_K_OK(mi355_rms_norm_mul_quant(s, (const float *) x->data, K, (const float *) wt->data, (float *) nxt->data, K, act, K, rows, eps));
            ctx->cache = act_cache{nxt->data, K, rows, ACT_Q8_1, act != nullptr, act};
            return j;
        }
    }
    // ---- UNARY(SILU) -> MUL, also across the product that supplies the other factor: llm_build_ffn's graph lists
    //      MUL_MAT(gate), SILU, MUL_MAT(up), MUL; the up product does not read SILU's value, so it runs first and SiLU*up
    //      (+ the quantized form ffn_down reads) is one launch after it
    if (node->op == GGML_OP_UNARY && ggml_get_unary_op(node) == GGML_UNARY_OP_SILU && nxt && w.sole_use(i)) {
        int jm = -1;   // index of the MUL
        if (nxt->op == GGML_OP_MUL && (nxt->src[0] == node || nxt->src[1] == node)) {
            jm = j;
        } else if (nxt->op == GGML_OP_MUL_MAT && nxt->src[0] != node && nxt->src[1] != node) {
            const int j2 = w.next(j);
            const ggml_tensor * m = j2 < w.n ? w.nodes[j2] : nullptr;
            // the product runs ahead of SILU: its result must not land on SILU's input
            if (m && m->op == GGML_OP_MUL && ((m->src[0] == node && m->src[1] == nxt) || (m->src[1] == node && m->src[0] == nxt)) &&
                !bytes_overlap(nxt, node->src[0]))
                jm = j2;
        }
        if (jm >= 0) {
            ggml_tensor * mul = (ggml_tensor *) w.nodes[jm];
            const ggml_tensor * gt = node->src[0];
            const ggml_tensor * up = mul->src[0] == node ? mul->src[1] : mul->src[0];
            const int64_t K = gt->ne[0], rows = ggml_nrows(gt);
            if (ggml_is_contiguous(gt) && ggml_is_contiguous(up) && ggml_is_contiguous(mul) && ggml_are_same_shape(gt, up) && up->type == GGML_TYPE_F32 &&
                gt->type == GGML_TYPE_F32 && mul->type == GGML_TYPE_F32 && K % 32 == 0 && rows <= 65535 &&
                (((uintptr_t) gt->data | (uintptr_t) up->data | (uintptr_t) mul->data) & 15) == 0) {
                if (jm != j) {   // the product first (it may use the activation cached for the gate product)
                    const int done = compute_fused(ctx, w, j);
                    GGML_ASSERT(done == j);   // a MUL_MAT followed by MUL takes nothing with it
                }
                void * act = nullptr;
                if (rows > 8 && feeds_q8k_tiles(w, jm, mul->data, K, rows)) {
                    const int fmt = q8k_format_for(s, w.nodes[w.next(jm)]);
                    act = ctx->act_slot(fmt == ACT_Q8KT ? mi355_act_q8k_tiled_bytes(K, rows) : mi355_act_q8k_bytes(K, rows));
                    if (fmt == ACT_Q8KT)
                        MI355_K_OK(mi355_swiglu_quant_q8k_tiled(s, (const float *) gt->data, (const float *) up->data, K, (float *) mul->data, K, act, K, rows));
                    else
                        MI355_K_OK(mi355_swiglu_quant_q8k(s, (const float *) gt->data, (const float *) up->data, K, (float *) mul->data, K, act, K, rows));
                    ctx->cache = act_cache{mul->data, K, rows, fmt, true, act};
                    return jm;
                }
                if ((rows <= 32 && feeds_quant_gemv(w, jm, mul->data, K, rows)) || (rows <= 8 && feeds_quant_mmid(w, jm, mul->data, K, rows)))
                    act = ctx->act_slot(mi355_act_bytes(K, rows));
                MI355_K_OK(mi355_swiglu_quant(s, (const float *) gt->data, (const float *) up->data, K, (float *) mul->data, K, act, K, rows));
                ctx->cache = act_cache{mul->data, K, rows, ACT_Q8_1, act != nullptr, act};
                return jm;
            }
        }
    }
    // ---- MUL_MAT_ID(up) -> MUL_MAT_ID(gate) -> UNARY(SILU) -> MUL -> [MUL_MAT_ID(down) by GEMV] (llm_build_moe_ffn, one to a few tokens):
    //      one launch for both expert products, SiLU * up and the Q8_1 rows the down experts read; the f32 product is not materialised
    if (node->op == GGML_OP_MUL_MAT_ID && nxt && nxt->op == GGML_OP_MUL_MAT_ID && !mmid_uses_tiles(node) && w.sole_use(i) && w.sole_use(j)) {
        const ggml_tensor * up = node, * gate = nxt;
        const int js = w.next(j), jm = js < w.n ? w.next(js) : w.n;
        if (jm < w.n) {
            const ggml_tensor * silu = w.nodes[js], * mul = w.nodes[jm];
            const ggml_tensor * as_up = up->src[0], * as_gate = gate->src[0], * b = up->src[1], * ids = up->src[2];
            const int64_t K = as_up->ne[0], N = as_up->ne[1], n_expert = as_up->ne[2];
            const int64_t nb1 = b->ne[1], T = b->ne[2], n_used = ids->ne[0], slots = n_used * T;
            const bool chain = silu->op == GGML_OP_UNARY && ggml_get_unary_op(silu) == GGML_UNARY_OP_SILU && silu->src[0] == gate && w.sole_use(js) &&
                               mul->op == GGML_OP_MUL && ((mul->src[0] == silu && mul->src[1] == up) || (mul->src[1] == silu && mul->src[0] == up)) &&
                               w.sole_use(jm) && ggml_is_contiguous(mul) && mul->type == GGML_TYPE_F32 && ggml_are_same_shape(mul, up) &&
                               ggml_are_same_shape(gate, up) && ggml_is_contiguous(up) && ggml_is_contiguous(gate) && ggml_is_contiguous(silu);
            if (chain && gate->src[1]->data == b->data && ggml_are_same_shape(gate->src[1], b) && gate->src[2] == ids && as_gate->type == as_up->type &&
                ggml_are_same_shape(as_gate, as_up) && ((uintptr_t) b->data & 15) == 0 && slots <= 8 && nb1 * T <= 8 && b->type == GGML_TYPE_F32 &&
                ggml_is_contiguous(b) && ids->type == GGML_TYPE_I32 && !bytes_overlap(up, gate) && feeds_quant_mmid(w, jm, mul->data, N, slots) &&
                mi355_moe_gate_up_swiglu_supported(to_mi355_type(as_up->type), as_gate->data, as_up->data, N, K)) {
                const int64_t rows = nb1 * T;
                const size_t in_bytes = mi355_act_bytes(K, rows), out_bytes = mi355_act_bytes(N, slots);
                ctx->act_reserve(in_bytes > out_bytes ? in_bytes : out_bytes);
                if (!ctx->cached(b->data, K, rows, ACT_Q8_1)) {
                    void * fresh = ctx->act_slot(in_bytes);
                    MI355_K_OK(mi355_quantize_act(s, (const float *) b->data, fresh, K, rows, K));
                    ctx->cache = act_cache{b->data, K, rows, ACT_Q8_1, true, fresh};
                }
                const void * act_in = ctx->cache.ptr;
                void * act_out = ctx->act_slot(out_bytes, true);
                MI355_K_OK(mi355_moe_gate_up_swiglu(s, to_mi355_type(as_up->type), as_gate->data, as_up->data, act_in, (const int32_t *) ids->data,
                                                    (int64_t) (ids->nb[1] / sizeof(int32_t)), (float *) gate->data, (float *) up->data, act_out, N, K, n_expert,
                                                    n_used, nb1, T));
                ctx->cache = act_cache{mul->data, N, slots, ACT_Q8_1, true, act_out};
                return jm;
            }
        }
    }
    // ---- MUL_MAT_ID: the quantized rows of src1 are shared by consecutive products (up and gate experts read the same rows)
    if (node->op == GGML_OP_MUL_MAT_ID) {
        const ggml_tensor * as = node->src[0];
        const ggml_tensor * b = node->src[1];
        const ggml_tensor * ids = node->src[2];
        const int64_t K = as->ne[0], N = as->ne[1], n_expert = as->ne[2];
        const int64_t nb1 = b->ne[1], T = b->ne[2], n_used = ids->ne[0], rows = nb1 * T;
        const int64_t ids_stride = (int64_t) (ids->nb[1] / sizeof(int32_t));
        if (((uintptr_t) b->data & 15) == 0 && rows <= 65535 && K % 32 == 0) {
            if (mmid_uses_tiles(node)) {
                if (!ctx->cached(b->data, K, rows, ACT_Q8K)) {
                    void * fresh = ctx->act_slot(mi355_act_q8k_bytes(K, rows));
                    MI355_K_OK(mi355_quantize_act_q8k(s, (const float *) b->data, fresh, K, rows, K));
                    ctx->cache = act_cache{b->data, K, rows, ACT_Q8K, true, fresh};
                }
                const size_t route_bytes = mi355_mul_mat_id_q8k_route_bytes(n_expert, n_used, T);
                void * route = ctx->workspace(route_bytes);
                MI355_K_OK(mi355_mul_mat_id_q8k(s, to_mi355_type(as->type), as->data, ctx->cache.ptr, (const int32_t *) ids->data, ids_stride,
                                                (float *) node->data, N, K, n_expert, n_used, nb1, T, route, route_bytes));
            } else {
                if (!ctx->cached(b->data, K, rows, ACT_Q8_1)) {
                    void * fresh = ctx->act_slot(mi355_act_bytes(K, rows));
                    MI355_K_OK(mi355_quantize_act(s, (const float *) b->data, fresh, K, rows, K));
                    ctx->cache = act_cache{b->data, K, rows, ACT_Q8_1, true, fresh};
                }
                // many slots on experts of a per-32-block type: sorted by expert onto the routed form of their tile kernel
                if (n_used * T >= 32 && mi355_mul_mat_id_q_supported(to_mi355_type(as->type), as->data, N, K, n_expert)) {
                    const size_t route_bytes = mi355_mul_mat_id_q8k_route_bytes(n_expert, n_used, T);
                    void * route = ctx->workspace(route_bytes);
                    MI355_K_OK(mi355_mul_mat_id_q(s, to_mi355_type(as->type), as->data, ctx->cache.ptr, (const int32_t *) ids->data, ids_stride,
                                                  (float *) node->data, N, K, n_expert, n_used, nb1, T, route, route_bytes));
                } else {
                    MI355_K_OK(mi355_mul_mat_id_vec(s, to_mi355_type(as->type), as->data, ctx->cache.ptr, (const int32_t *) ids->data, ids_stride,
                                                    (float *) node->data, N, K, n_expert, n_used, nb1, T));
                }
            }
            ctx->note_write(node->data, ggml_nbytes(node));
            return i;
        }
    }
    // ---- SOFT_MAX -> ARGSORT(descending): expert probabilities and their order (llm_build_moe_ffn)
    if (node->op == GGML_OP_SOFT_MAX) {
        const moe_route_match r = match_moe_route(w, i);
        if (r.ok) {
            const ggml_tensor * x = node->src[0];
            ctx->note_write(node->data, ggml_nbytes(node));
            MI355_K_OK(mi355_moe_route(s, (const float *) x->data, (float *) node->data, (int32_t *) w.nodes[r.j_argsort]->data, x->ne[0], ggml_nrows(x)));
            return r.j_argsort;
        }
    }
    // ---- GET_ROWS(probabilities of the selected experts) -> SUM_ROWS -> DIV: normalised expert weights; with the weighted sum of the
    //      experts' outputs right behind them (a few tokens), both in one launch
    if (node->op == GGML_OP_GET_ROWS) {
        const moe_weights_match m = match_moe_weights(w, i);
        if (m.ok) {
            const int jc = w.next(m.last);
            const moe_combine_match c = jc < w.n ? match_moe_combine(w, jc) : moe_combine_match();
            ctx->note_write(m.raw->data, ggml_nbytes(m.raw));
            ctx->note_write(m.div->data, ggml_nbytes(m.div));
            // One launch for both when the weighted sum is the only reader of the weights (GET_ROWS, SUM_ROWS and DIV results are then not
            // materialised: the allocator has often lent their memory to the sum's own operands by now, e.g. SUM_ROWS' result lies on
            // the probabilities, or the sum on SUM_ROWS' result) and the sum's outputs do not lie on the probabilities or the ids, which
            // every group reads.
            bool one_launch = c.ok && c.wt->data == m.div->data && c.n_used == m.n_used && c.T == m.T && m.T <= 8 && w.sole_use(i) && w.sole_use(w.next(i)) &&
                              w.sole_use(m.last);
            if (one_launch) {
                const ggml_tensor * mul = w.nodes[jc];
                for (int k = i + 1; k < jc; k++) {   // the reshapes in between: [n_used, T] read by SUM_ROWS and DIV, [1, n_used, T] read by the MUL
                    const ggml_tensor * t = w.nodes[k];
                    if (!is_noop(t)) continue;
                    if (t == m.sum->src[0]) one_launch = one_launch && w.uses[k] == 2 && !(t->flags & GGML_TENSOR_FLAG_OUTPUT);
                    else if (t == c.wt) one_launch = one_launch && w.sole_use(k);
                }
                for (const ggml_tensor * in : {m.probs, m.ids})
                    for (const ggml_tensor * o : {mul, c.out}) one_launch = one_launch && !bytes_overlap(in, o);
            }
            if (one_launch) {
                const ggml_tensor * mul = w.nodes[jc];
                ctx->note_write(mul->data, ggml_nbytes(mul));
                ctx->note_write(c.out->data, ggml_nbytes(c.out));
                MI355_K_OK(mi355_moe_weights_combine(s, (const float *) m.probs->data, (const int32_t *) m.ids->data, m.ids_stride, nullptr, nullptr, nullptr,
                                                     m.n_expert, (const float *) c.ex->data, (float *) mul->data, c.residual, (float *) c.out->data, c.n_embd, c.n_used,
                                                     c.T));
                return c.last;
            }
            MI355_K_OK(mi355_moe_weights(s, (const float *) m.probs->data, (const int32_t *) m.ids->data, m.ids_stride, (float *) m.raw->data,
                                         (float *) m.sum->data, (float *) m.div->data, m.n_expert, m.n_used, m.T));
            return m.last;
        }
    }
    // ---- MUL(expert outputs, weights) -> ADD over the expert slots [-> ADD(residual)]: weighted sum of the selected experts
    if (node->op == GGML_OP_MUL) {
        const moe_combine_match c = match_moe_combine(w, i);
        if (c.ok) {
            ctx->note_write(node->data, ggml_nbytes(node));
            ctx->note_write(c.out->data, ggml_nbytes(c.out));
            MI355_K_OK(mi355_moe_combine(s, (const float *) c.ex->data, (const float *) c.wt->data, (float *) node->data, c.residual, (float *) c.out->data, c.n_embd,
                                         c.n_used, c.T));
            return c.last;
        }
    }
    // ---- FLASH_ATTN_EXT whose output feeds a quantized product
    if (node->op == GGML_OP_FLASH_ATTN_EXT) {
        const ggml_tensor * q = node->src[0];
        const int64_t D = q->ne[0], Nq = q->ne[1], Hq = q->ne[2];
        auto cache_type = [](ggml_type t) { return t == GGML_TYPE_F16 || t == GGML_TYPE_Q8_0 || t == GGML_TYPE_Q4_0; };
        if (q->ne[3] == 1 && Nq <= 8 && D % 32 == 0 && cache_type(node->src[1]->type) && cache_type(node->src[2]->type) &&
            feeds_quant_gemv(w, i, node->data, Hq * D, Nq)) {
            const ggml_tensor * k = node->src[1];
            const ggml_tensor * v = node->src[2];
            const ggml_tensor * mask = node->src[3];
            float scale, max_bias, softcap;
            memcpy(&scale, (const float *) node->op_params + 0, sizeof(float));
            memcpy(&max_bias, (const float *) node->op_params + 1, sizeof(float));
            memcpy(&softcap, (const float *) node->op_params + 2, sizeof(float));
            const int64_t Nkv = k->ne[1], Hkv = k->ne[2];
            if (k->type != GGML_TYPE_F16 || v->type != GGML_TYPE_F16) {   // quantized cache, read in place (fewer than 16 query rows)
                const kv_operand ko = kv_operand_of(k), vo = kv_operand_of(v);
                GGML_ASSERT(ko.ok && vo.ok);
                const size_t ws_bytes = mi355_flash_attn_kv_ws_bytes(D, Nq, Nkv, Hq, Hkv, to_mi355_type(k->type), to_mi355_type(v->type));
                void * ws = ctx->workspace(ws_bytes);
                void * act = ctx->act_slot(mi355_act_bytes(Hq * D, Nq));
                MI355_K_OK(mi355_flash_attn_ext_kv(s, (const float *) q->data, ko.p, to_mi355_type(k->type), ko.base, ko.row_blocks, vo.p,
                                                   to_mi355_type(v->type), vo.base, vo.row_blocks, mask ? mask->data : nullptr, (float *) node->data, D, Nq,
                                                   Nkv, Hq, Hkv, q->nb[1], q->nb[2], k->nb[1], k->nb[2], v->nb[1], v->nb[2], mask ? mask->nb[1] : 0, scale,
                                                   max_bias, softcap, ws, ws_bytes, act));
                ctx->cache = act_cache{node->data, Hq * D, Nq, ACT_Q8_1, true, act};
                return i;
            }
            const size_t full = mi355_flash_attn_ws_bytes(D, Nq, Nkv, Hq);
            const size_t ws_bytes = full < (size_t(256) << 20) ? full : (size_t(256) << 20);
            void * ws = ctx->workspace(ws_bytes);
            void * act = ctx->act_slot(mi355_act_bytes(Hq * D, Nq));
            MI355_K_OK(mi355_flash_attn_ext_quant(s, (const float *) q->data, k->data, v->data, mask ? mask->data : nullptr, (float *) node->data, D, Nq, Nkv,
                                                  Hq, Hkv, q->nb[1], q->nb[2], k->nb[1], k->nb[2], v->nb[1], v->nb[2], mask ? mask->nb[1] : 0, scale,
                                                  max_bias, softcap, ws, ws_bytes, act));
            ctx->cache = act_cache{node->data, Hq * D, Nq, ACT_Q8_1, true, act};
            return i;
        }
    }
    // ---- MUL_MAT(gate) -> UNARY(SILU) -> MUL_MAT(up) -> MUL -> [quantized MUL_MAT]: one launch that also leaves the Q8_1 form
    //      of silu(gate)*up for ffn_down; the f32 product is not materialised (its only reader takes the quantized form)
    if (is_quant_gemv_candidate(node) && node->src[1]->ne[1] <= 4 && w.sole_use(i) && nxt && nxt->op == GGML_OP_UNARY &&
        ggml_get_unary_op(nxt) == GGML_UNARY_OP_SILU && nxt->src[0] == node && w.sole_use(j)) {
        const int ju = w.next(j);
        const int jm = ju < w.n ? w.next(ju) : w.n;
        if (jm < w.n) {
            const ggml_tensor * up = w.nodes[ju];
            const ggml_tensor * mul = w.nodes[jm];
            const ggml_tensor * b = node->src[1];
            const int64_t K = b->ne[0], B = b->ne[1], N = node->ne[0];
            const bool mul_ok = mul->op == GGML_OP_MUL && ((mul->src[0] == nxt && mul->src[1] == up) || (mul->src[1] == nxt && mul->src[0] == up)) &&
                                ggml_is_contiguous(mul) && mul->type == GGML_TYPE_F32 && ggml_are_same_shape(mul, node);
            if (mul_ok && is_quant_gemv_candidate(up) && up->src[1]->data == b->data && up->src[1]->ne[0] == K && up->src[1]->ne[1] == B &&
                up->ne[0] == N && w.sole_use(ju) && w.sole_use(jm) && N % 32 == 0 && ggml_is_contiguous(node) && ggml_is_contiguous(up) &&
                !bytes_overlap(node, up) &&   // both products are written before SiLU*up reads them
                feeds_quant_gemv(w, jm, mul->data, N, B)) {
                // this launch reads one quantized activation and writes the next: the two slots
                const size_t in_bytes = mi355_act_bytes(K, B), out_bytes = mi355_act_bytes(N, B);
                ctx->act_reserve(in_bytes > out_bytes ? in_bytes : out_bytes);
                if (!ctx->cached(b->data, K, B, ACT_Q8_1)) {
                    void * fresh = ctx->act_slot(in_bytes);
                    MI355_K_OK(mi355_quantize_act(s, (const float *) b->data, fresh, K, B, K));
                    ctx->cache = act_cache{b->data, K, B, ACT_Q8_1, true, fresh};
                }
                const void * act_in = ctx->cache.ptr;
                void * act_out = ctx->act_slot(out_bytes, true);
                // Gate and up of one type: one launch whose groups each own a 32-row block of both matrices and quantize
                // SiLU*up themselves (15.3 us on 2 x 14336 x 4096 against 15.1 + 4.6 us for product and SiLU*up + Q8_1 apart).
                // Two types: the two launches, which are a little quicker than the launch whose last groups do the tail through
                // arrival counters.  Same bits every way.
                const int tg = to_mi355_type(node->src[0]->type), tu = to_mi355_type(up->src[0]->type);
                unsigned * tickets = tg == tu ? ctx->ticket_buffer((size_t) N / 32 + 1) : nullptr;
                if (tickets) {
                    MI355_K_OK(mi355_ffn_gate_up_swiglu(s, tg, node->src[0]->data, tu, up->src[0]->data, act_in, (float *) node->data, (float *) up->data, N,
                                                        act_out, tickets, N, K, B));
                    ctx->cache = act_cache{mul->data, N, B, ACT_Q8_1, true, act_out};
                    return jm;
                }
                mi355_gemv_mat gu[2];
                gu[0] = mi355_gemv_mat{to_mi355_type(node->src[0]->type), node->src[0]->data, N, (float *) node->data, N, nullptr};
                gu[1] = mi355_gemv_mat{to_mi355_type(up->src[0]->type), up->src[0]->data, N, (float *) up->data, N, nullptr};
                MI355_K_OK(mi355_mul_mat_vec_q_multi(s, 2, gu, act_in, K, B));
                MI355_K_OK(mi355_swiglu_quant(s, (const float *) node->data, (const float *) up->data, N, nullptr, 0, act_out, N, B));
                ctx->cache = act_cache{mul->data, N, B, ACT_Q8_1, true, act_out};
                return jm;
            }
        }
    }
    // ---- the Q/K/V window (see match_qkv_window): projections, rotations and cache stores in one launch
    if (is_quant_gemv_candidate(node) && node->src[1]->ne[1] <= 4 && w.sole_use(i) && nxt && node->ne[0] % 2 == 0) {
        const ggml_tensor * b = node->src[1];
        const int64_t K = b->ne[0], B = b->ne[1];
        const qkv_window win = match_qkv_window(ctx, w, i, b->data, K, B);
        if (win.ok) {
            if (!ctx->cached(b->data, K, B, ACT_Q8_1)) {
                void * fresh = ctx->act_slot(mi355_act_bytes(K, B));
                MI355_K_OK(mi355_quantize_act(s, (const float *) b->data, fresh, K, B, K));
                ctx->cache = act_cache{b->data, K, B, ACT_Q8_1, true, fresh};
            }
            MI355_K_OK(mi355_mul_mat_vec_q_rope(s, win.n_ch, win.mats, ctx->cache.ptr, K, B, &win.rd));
            note_window_writes(ctx, win, B);
            return win.last;
        }
    }
    // ---- runs of quantized products on one activation (batch <= 32): one quantization, multi-matrix GEMV (up to 4 rows) or the
    //      weight-streaming kernel, residual epilogue
    if (is_quant_gemv_candidate(node)) {
        const ggml_tensor * b = node->src[1];
        const int64_t K = b->ne[0], B = b->ne[1];
        int run[4], n_run = 0, last = i;
        for (int k = i; k < w.n && n_run < (B <= 4 ? 4 : 1); k = w.next(k)) {
            const ggml_tensor * mm = w.nodes[k];
            if (!is_quant_gemv_candidate(mm) || mm->src[1]->data != b->data || mm->src[1]->ne[0] != K || mm->src[1]->ne[1] != B) break;
            run[n_run++] = k;
            last = k;
        }
        if (!ctx->cached(b->data, K, B, ACT_Q8_1)) {
            void * fresh = ctx->act_slot(mi355_act_bytes(K, B));
            MI355_K_OK(mi355_quantize_act(s, (const float *) b->data, fresh, K, B, K));
            ctx->cache = act_cache{b->data, K, B, ACT_Q8_1, true, fresh};
        }
        const void * act = ctx->cache.ptr;
        mi355_gemv_mat mats[4];
        for (int r = 0; r < n_run; r++) {
            ggml_tensor * mm = (ggml_tensor *) w.nodes[run[r]];
            mats[r].type = to_mi355_type(mm->src[0]->type);
            mats[r].W = mm->src[0]->data;
            mats[r].N = mm->src[0]->ne[1];
            mats[r].dst = (float *) ctx->out_ptr(mm);
            mats[r].dst_stride = (int64_t) (mm->nb[1] / sizeof(float));
            mats[r].residual = nullptr;
        }
        if (n_run == 1) {   // MUL_MAT -> ADD(residual): write the sum straight into the ADD's tensor
            const int ja = w.next(i);
            ggml_tensor * add = ja < w.n ? (ggml_tensor *) w.nodes[ja] : nullptr;
            if (add && add->op == GGML_OP_ADD && w.sole_use(i) && (add->src[0] == node || add->src[1] == node)) {
                const ggml_tensor * res = add->src[0] == node ? add->src[1] : add->src[0];
                if (res->type == GGML_TYPE_F32 && ggml_are_same_shape(res, node) && ggml_is_contiguous(res) && ggml_is_contiguous(add) &&
                    ggml_is_contiguous(node)) {
                    mats[0].dst = (float *) add->data;
                    mats[0].dst_stride = (int64_t) (add->nb[1] / sizeof(float));
                    mats[0].residual = (const float *) res->data;
                    last = ja;
                }
            }
        }
        if (n_run == 1 && B >= 5 && mi355_mul_mat_skinny_supported(mats[0].type, mats[0].W, K, B)) {
            // with room for the slices along K that products with few rows are split into
            const size_t split_bytes = mi355_mul_mat_skinny_ws_bytes(mats[0].N, K, B);
            void * split_ws = split_bytes ? ctx->workspace(split_bytes) : nullptr;
            MI355_K_OK(mi355_mul_mat_skinny(s, mats[0].type, mats[0].W, act, mats[0].dst, mats[0].residual, mats[0].N, K, B, mats[0].dst_stride, split_ws,
                                            split_bytes));
        } else {
            MI355_K_OK(mi355_mul_mat_vec_q_multi(s, n_run, mats, act, K, B));
        }
        for (int r = 0; r < n_run; r++) ctx->note_write(mats[r].dst, (size_t) mats[r].N * (size_t) B * sizeof(float));
        return last;
    }
    // ---- runs of K-quant products on one activation (batch > 8): one per-super-block quantization
    // (a Q5_K or IQ4_XS matrix without tile images - not in a weights buffer, no memory for them, or a batch below the images'
    // threshold - takes the generic path below)
    if (is_q8k_tile_candidate(node) && !(tiles_or_generic(node->src[0]->type) && q8k_format_for(s, node) != ACT_Q8KT)) {
        const ggml_tensor * b = node->src[1];
        const int64_t K = b->ne[0], B = b->ne[1];
        // MUL_MAT(gate) -> UNARY(SILU) -> MUL_MAT(up) -> MUL: the up product goes out with the gate product (it reads the same
        // activation and nothing in between writes); its node is then passed over when the walk gets there
        if (nxt && nxt->op == GGML_OP_UNARY && ggml_get_unary_op(nxt) == GGML_UNARY_OP_SILU && nxt->src[0] == node && w.sole_use(i) && ctx->done_ahead == nullptr &&
            ctx->n_redirect == 0) {
            const int ju = w.next(j);
            const ggml_tensor * up = ju < w.n ? w.nodes[ju] : nullptr;
            if (up && up->op == GGML_OP_MUL_MAT && up->src[1]->data == b->data && !bytes_overlap(up, node) && !bytes_overlap(up, b) && ggml_is_contiguous(up) &&
                ggml_is_contiguous(node)) {
                const int at[2] = {i, ju};
                if (tiled_multi(ctx, s, w, at, 2) == 3u) {
                    ctx->done_ahead = up;
                    return i;
                }
            }
        }
        // large batches: the wide-tile kernel on tile images of the weights (built on first use) and of the activation
        const int fmt = q8k_format_for(s, node);
        const bool mid = takes_mid_kernel(node);
        const void * tl = fmt == ACT_Q8KT && !mid ? tiles().get(s, node->src[0]) : nullptr;
        if (!ctx->cached(b->data, K, B, fmt)) {
            void * fresh = ctx->act_slot(fmt == ACT_Q8KT ? mi355_act_q8k_tiled_bytes(K, B) : mi355_act_q8k_bytes(K, B));
            if (fmt == ACT_Q8KT) MI355_K_OK(mi355_quantize_act_q8k_tiled(s, (const float *) b->data, fresh, K, B, (int64_t) (b->nb[1] / sizeof(float))));
            else MI355_K_OK(mi355_quantize_act_q8k(s, (const float *) b->data, fresh, K, B, (int64_t) (b->nb[1] / sizeof(float))));
            ctx->cache = act_cache{b->data, K, B, fmt, true, fresh};
        }
        const void * pl = tl || mid ? nullptr : planes().get(s, node->src[0]);   // Q6_K weights: the unpacked planes, built on first use
        const int wtype = to_mi355_type(node->src[0]->type);
        const int64_t N = node->src[0]->ne[1];
        // products with few tiles are split along K through the scratch buffer (0 bytes: this shape is not split)
        const size_t split_bytes = mid ? mi355_mul_mat_mid_ws_bytes(N, K, B) : tl ? mi355_mul_mat_q8k_tiled_ws_bytes(N, K, B) : mi355_mul_mat_q8k_ws_bytes(N, K, B);
        void * split_ws = split_bytes ? ctx->workspace(split_bytes) : nullptr;
        auto product = [&](float * out, const float * residual, int64_t out_stride) {
            if (mid) MI355_K_OK(mi355_mul_mat_mid(s, wtype, node->src[0]->data, ctx->cache.ptr, out, residual, N, K, B, out_stride, split_ws, split_bytes));
            else if (tl) MI355_K_OK(mi355_mul_mat_q8k_tiled(s, wtype, tl, ctx->cache.ptr, out, residual, N, K, B, out_stride, split_ws, split_bytes));
            else if (pl) MI355_K_OK(mi355_mul_mat_q8k_planes_ws(s, wtype, pl, ctx->cache.ptr, out, residual, N, K, B, out_stride, split_ws, split_bytes));
            else MI355_K_OK(mi355_mul_mat_q8k_ws(s, wtype, node->src[0]->data, ctx->cache.ptr, out, residual, N, K, B, out_stride, split_ws, split_bytes));
        };
        // MUL_MAT -> ADD(residual): the sum goes straight into the ADD's tensor
        ggml_tensor * add = nxt;
        if (add && add->op == GGML_OP_ADD && w.sole_use(i) && (add->src[0] == node || add->src[1] == node)) {
            const ggml_tensor * res = add->src[0] == node ? add->src[1] : add->src[0];
            if (res->type == GGML_TYPE_F32 && ggml_are_same_shape(res, node) && ggml_is_contiguous(res) && ggml_is_contiguous(add) && ggml_is_contiguous(node)) {
                // ... -> RMS_NORM -> MUL(norm weight) whose readers are tile products again (wo -> the FFN norm, ffn_down -> the next
                // layer's attention norm): a product that is cut along K adds its slices row by row, and the group that has formed a
                // row normalises and quantizes it on the spot (same bits as the norm launch it replaces)
                if ((tl || mid) && split_ws) {
                    const int jn = w.next(j);
                    const int jm = jn < w.n ? w.next(jn) : w.n;
                    const ggml_tensor * nrm = jn < w.n ? w.nodes[jn] : nullptr;
                    const ggml_tensor * mul = jm < w.n ? w.nodes[jm] : nullptr;
                    if (nrm && mul && nrm->op == GGML_OP_RMS_NORM && nrm->src[0] == add && mul->op == GGML_OP_MUL && mul->src[0] == nrm && w.sole_use(jn) &&
                        add->ne[2] == 1 && add->ne[3] == 1 && ggml_is_contiguous(mul) && mul->type == GGML_TYPE_F32 && N % 256 == 0 && N <= 4096) {
                        const ggml_tensor * wt = mul->src[1];
                        if (wt->type == GGML_TYPE_F32 && ggml_is_contiguous(wt) && ggml_nelements(wt) == N &&
                            (((uintptr_t) add->data | (uintptr_t) mul->data | (uintptr_t) wt->data | (uintptr_t) res->data) & 15) == 0 &&
                            feeds_q8k_tiles(w, jm, mul->data, N, B) && q8k_format_for(s, w.nodes[w.next(jm)]) == ACT_Q8KT &&
                            !bytes_overlap(mul, add) && !bytes_overlap(mul, b) &&
                            mi355_act_q8k_tiled_bytes(N, B) <= ctx->act_size) {   // (a larger slot would move the activation the product reads)
                            float eps;
                            memcpy(&eps, nrm->op_params, sizeof(float));
                            void * act_out = ctx->act_slot(mi355_act_q8k_tiled_bytes(N, B), true);   // the product still reads the other slot
                            if (mid)
                                MI355_K_OK(mi355_mul_mat_mid_norm(s, wtype, node->src[0]->data, ctx->cache.ptr, (float *) add->data, (const float *) res->data, N, K, B,
                                                                  (int64_t) (add->nb[1] / sizeof(float)), split_ws, split_bytes, (const float *) wt->data, eps,
                                                                  (float *) mul->data, N, act_out));
                            else
                                MI355_K_OK(mi355_mul_mat_q8k_tiled_norm(s, wtype, tl, ctx->cache.ptr, (float *) add->data, (const float *) res->data, N, K, B,
                                                                        (int64_t) (add->nb[1] / sizeof(float)), split_ws, split_bytes, (const float *) wt->data, eps,
                                                                        (float *) mul->data, N, act_out));
                            ctx->note_write(add->data, ggml_nbytes(add));
                            ctx->note_write(mul->data, ggml_nbytes(mul));
                            ctx->cache = act_cache{mul->data, N, B, ACT_Q8KT, true, act_out};
                            return jm;
                        }
                    }
                }
                product((float *) add->data, (const float *) res->data, (int64_t) (add->nb[1] / sizeof(float)));
                ctx->note_write(add->data, ggml_nbytes(add));
                return j;
            }
        }
        product((float *) ctx->out_ptr(node), nullptr, (int64_t) (node->nb[1] / sizeof(float)));
        ctx->note_write(ctx->out_ptr(node), ggml_nbytes(node));
        return i;
    }
    ctx->note_write(node->op == GGML_OP_CPY ? node->src[1]->data : node->data, ggml_nbytes(node->op == GGML_OP_CPY ? node->src[1] : node));
    compute_node(ctx, node);
    return i;
}

// ---- HIP-graph replay of decode graphs
// llama.cpp rebuilds the same ~1000-node graph for every decoded token.  Issued launch by launch that is ~230 kernel launches
// from the host per token; replayed as one HIP graph it is one.  A graph is replayed when nothing a launch depends on has
// changed since it was recorded: every node's op, type, shape, strides, parameters and data address, and those of its sources
// (the signature below).  The one thing that does change from token to token is where K and V are stored: the CPY destinations
// are views into the cache at the current cell.  Those stores address the cache through a small device array of cell numbers
// (ctx->cells, written by k_fill_cells before the graph starts), so the recorded launches stay valid; the signature covers
// the cache tensor behind such a view instead of the view's address.  A graph runs launch by launch the first time it is seen
// (scratch buffers get their size), is recorded the second time, and replayed from then on.  Batches above 4 rows, graphs
// whose cache stores are not all taken by the fused Q/K/V launch, and MI355_NO_GRAPH=1 stay launch by launch.
__global__ void k_fill_cells(int32_t * cells, int head) { cells[threadIdx.x] = head + (int) threadIdx.x; }

struct graph_signature {
    uint64_t hash = 0;
    bool capturable = false;
    int64_t kv_head = -1;
    int kv_stores = 0;
};

// One multiply per word: the signature is computed for every graph of every token, ahead of the launch.
inline uint64_t sig_mix(uint64_t h, uint64_t v) {
    h = (h ^ v) * 0x9E3779B97F4A7C15ull;
    return h ^ (h >> 29);
}

// two fields per word (the second spread by an odd multiplier, so that swapping them changes the word)
inline uint64_t sig_pair(uint64_t a, uint64_t b) { return a + b * 0xff51afd7ed558ccdull; }

uint64_t sig_tensor(uint64_t h, const ggml_tensor * t, bool through_cache) {
    h = sig_mix(h, ((uint64_t) t->type << 32) | (uint64_t) t->op);
    h = sig_mix(h, sig_pair((uint64_t) t->ne[0], (uint64_t) t->ne[1]));
    h = sig_mix(h, sig_pair((uint64_t) t->ne[2], (uint64_t) t->ne[3]));
    h = sig_mix(h, sig_pair((uint64_t) t->nb[0], (uint64_t) t->nb[1]));
    h = sig_mix(h, sig_pair((uint64_t) t->nb[2], (uint64_t) t->nb[3]));
    return sig_mix(h, (uint64_t) (uintptr_t) (through_cache ? t->view_src->data : t->data));
}

bool is_cache_store(const ggml_tensor * node) {
    if (node->op != GGML_OP_CPY) return false;
    const ggml_tensor * d = node->src[1];
    return d && (d->type == GGML_TYPE_F16 || d->type == GGML_TYPE_Q8_0 || d->type == GGML_TYPE_Q4_0) && d->view_src && d->view_src->data &&
           ggml_is_contiguous(d);
}

graph_signature sign_graph(ggml_cgraph * cgraph, std::vector<uint64_t> * trace = nullptr) {
    graph_signature g;
    const int n = ggml_graph_n_nodes(cgraph);
    // the views that cache stores write through (they are graph nodes themselves, and sources of the CPY nodes): two per layer
    const ggml_tensor * dests[256];
    int n_dests = 0;
    for (int i = 0; i < n; i++) {
        const ggml_tensor * node = ggml_graph_node(cgraph, i);
        if (node->op == GGML_OP_CPY && is_cache_store(node)) {
            if (n_dests == 256) return g;   // not a graph this path knows: launch by launch (capturable stays false, hash 0)
            dests[n_dests++] = node->src[1];
        }
    }
    auto through_cache = [&](const ggml_tensor * t) {
        if (t->op != GGML_OP_VIEW) return false;   // ggml_view_1d of the cache tensor (llm_build_kv_store)
        for (int k = 0; k < n_dests; k++)
            if (dests[k] == t) return true;
        return false;
    };
    uint64_t h = sig_mix(0x6d693335u, (uint64_t) n);
    int64_t batch = 0;
    bool heads_agree = true;
    for (int i = 0; i < n; i++) {
        const ggml_tensor * node = ggml_graph_node(cgraph, i);
        const bool store = node->op == GGML_OP_CPY && is_cache_store(node);
        const bool via_cache = through_cache(node);
        h = sig_tensor(h, node, via_cache || (store && node->view_src != nullptr && node->data == node->src[1]->data));
        h = sig_mix(h, (uint64_t) node->flags);
        if (!via_cache) {   // a view's parameters hold its offset
            for (size_t k = 0; k < GGML_MAX_OP_PARAMS / sizeof(int32_t); k += 2) {
                const uint64_t pw = ((uint64_t) (uint32_t) node->op_params[k] << 32) | (uint32_t) node->op_params[k + 1];
                if (pw) h = sig_mix(h, pw + k);   // most nodes have no parameters at all
            }
        }
        if (trace) trace->push_back(h);
        for (int k = 0; k < GGML_MAX_SRC; k++) {
            const ggml_tensor * src = node->src[k];
            if (!src) continue;
            // A store destination read by anything but its CPY keeps its own address in the signature.  Sources that are
            // computed (nodes of this graph, signed in full where they are listed) are identified by their address alone.
            if (src->op != GGML_OP_NONE && !(store && k == 1)) h = sig_mix(h, ((uint64_t) (uintptr_t) src->data << 3) | (uint64_t) k);
            else h = sig_tensor(sig_mix(h, (uint64_t) k), src, store && k == 1);
        }
        if (node->op == GGML_OP_MUL_MAT && batch == 0) batch = node->src[1]->ne[1] * node->src[1]->ne[2] * node->src[1]->ne[3];
        if (store) {
            g.kv_stores++;
            const ggml_tensor * d = node->src[1];
            const int64_t off = (const char *) d->data - (const char *) d->view_src->data;
            const int64_t row = batch > 0 ? (int64_t) ggml_nbytes(d) / batch : 0;
            if (row <= 0 || off % row != 0 || (g.kv_head >= 0 && g.kv_head != off / row)) heads_agree = false;
            else g.kv_head = off / row;
        }
    }
    if (!heads_agree) g.kv_head = -1;
    g.hash = h | 1;   // never 0
    g.capturable = batch >= 1 && batch <= 4 && (g.kv_stores == 0 || (g.kv_head >= 0 && g.kv_head + 8 < 0x7fffffff));
    return g;
}

void run_graph_launches(backend_ctx * ctx, ggml_cgraph * cgraph) {
    ctx->cache.valid = false;
    ctx->done_ahead = nullptr;
    ctx->n_redirect = 0;
    const graph_walk w(cgraph);
    static const bool log_graph = getenv("MI355_LOG_GRAPH") != nullptr;   // node list and the nodes each launch sequence consumed
    const uint64_t launches_before = mi355_launch_count(), prep_before = g_prep_launches.load();
    for (int i = 0; i < w.n; i++) {
        if (is_noop(w.nodes[i])) continue;
        const int first = i;
        i = compute_fused(ctx, w, i);
        if (log_graph) {
            for (int k = first; k <= i; k++) {
                const ggml_tensor * t = w.nodes[k];
                fprintf(stderr, "MI355 graph %s%3d %-14s %-24s [%lld %lld %lld %lld] uses %d\n", k == first ? "*" : " ", k, ggml_op_name(t->op), t->name,
                        (long long) t->ne[0], (long long) t->ne[1], (long long) t->ne[2], (long long) t->ne[3], w.uses[k]);
            }
        }
    }
    if (log_graph) {
        int64_t batch = 0, layers = 0;
        for (int i = 0; i < w.n; i++) {
            if (w.nodes[i]->op == GGML_OP_MUL_MAT && batch == 0) batch = w.nodes[i]->src[1]->ne[1];
            if (w.nodes[i]->op == GGML_OP_FLASH_ATTN_EXT) layers++;
        }
        const uint64_t prep = g_prep_launches.load() - prep_before;
        fprintf(stderr, "MI355 graph launches: %d nodes, batch %lld, %lld attention nodes, %llu kernel launches + %llu for one-time weight copies\n", w.n,
                (long long) batch, (long long) layers, (unsigned long long) (mi355_launch_count() - launches_before - prep), (unsigned long long) prep);
    }
    ctx->cache.valid = false;
}

ggml_status backend_graph_compute(ggml_backend_t backend, ggml_cgraph * cgraph) {
    backend_ctx * ctx = (backend_ctx *) backend->context;
    MI355_HIP_OK(hipSetDevice(ctx->device));
    ctx->cache.valid = false;
    ctx->graph_serial++;
    if (!ctx->fuse) {
        const int n = ggml_graph_n_nodes(cgraph);
        for (int i = 0; i < n; i++) {
            ggml_tensor * node = ggml_graph_node(cgraph, i);
            if (!is_noop(node)) compute_node(ctx, node);
        }
        return GGML_STATUS_SUCCESS;
    }
    auto & rp = ctx->replay;
    const int64_t t_start = ggml_time_us();
    graph_signature sig;
    static const bool log_replay = getenv("MI355_GRAPH_STATS") != nullptr && getenv("MI355_GRAPH_STATS")[0] == '2';
    if (rp.enabled && log_replay) {   // also name the first node whose signature differs from the previous graph's
        static std::vector<uint64_t> prev;
        std::vector<uint64_t> cur;
        sig = sign_graph(cgraph, &cur);
        size_t k = 0;
        while (k < cur.size() && k < prev.size() && cur[k] == prev[k]) k++;
        const ggml_tensor * t = k < cur.size() ? ggml_graph_node(cgraph, (int) k) : nullptr;
        fprintf(stderr, "MI355 graph: %d nodes, signature %016llx, %s, %d cache stores at cell %lld; first change at node %zu %s %s\n",
                ggml_graph_n_nodes(cgraph), (unsigned long long) sig.hash, sig.capturable ? "replayable" : "launch by launch", sig.kv_stores,
                (long long) sig.kv_head, k, t ? ggml_op_name(t->op) : "-", t ? t->name : "-");
        prev.swap(cur);
    } else if (rp.enabled) {
        sig = sign_graph(cgraph);
    }
    ctx->kv_head = sig.capturable ? sig.kv_head : -1;
    ctx->kv_redirected = 0;
    if (ctx->kv_head >= 0 && ctx->cells_head != ctx->kv_head) {
        hipLaunchKernelGGL(k_fill_cells, dim3(1), dim3(8), 0, ctx->stream, ctx->cells, (int) ctx->kv_head);
        MI355_HIP_OK(hipGetLastError());
        ctx->cells_head = ctx->kv_head;
    }
    if (sig.capturable && rp.exec && rp.exec_sig == sig.hash && rp.exec_gen == ctx->alloc_gen) {
        MI355_HIP_OK(hipGraphLaunch(rp.exec, ctx->stream));
        rp.replays++;
        rp.host_us += (double) (ggml_time_us() - t_start);
        return GGML_STATUS_SUCCESS;
    }
    const bool record = sig.capturable && sig.hash != rp.bad_sig && rp.seen_sig == sig.hash && rp.seen_gen == ctx->alloc_gen;
    if (record && hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
        (void) hipGetLastError();
        rp.bad_sig = sig.hash;
    } else if (record) {
        ctx->capturing = true;
        ctx->capture_broken = false;
        run_graph_launches(ctx, cgraph);
        ctx->capturing = false;
        hipGraph_t graph = nullptr;
        const hipError_t end = hipStreamEndCapture(ctx->stream, &graph);
        const bool ok = end == hipSuccess && graph != nullptr && !ctx->capture_broken && ctx->kv_redirected == sig.kv_stores;
        if (end != hipSuccess) (void) hipGetLastError();
        hipGraphExec_t exec = nullptr;
        if (ok && hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) == hipSuccess) {
            if (rp.exec) MI355_HIP_OK(hipGraphExecDestroy(rp.exec));
            if (rp.graph) MI355_HIP_OK(hipGraphDestroy(rp.graph));
            rp.exec = exec;
            rp.graph = graph;
            rp.exec_sig = sig.hash;
            rp.exec_gen = ctx->alloc_gen;
            rp.captures++;
            MI355_HIP_OK(hipGraphLaunch(rp.exec, ctx->stream));   // nothing has run yet: recording does not execute
            return GGML_STATUS_SUCCESS;
        }
        (void) hipGetLastError();
        if (graph) (void) hipGraphDestroy(graph);
        rp.bad_sig = sig.hash;   // run it launch by launch, now and from now on
        ctx->kv_redirected = 0;
    }
    run_graph_launches(ctx, cgraph);
    rp.seen_sig = sig.hash;
    rp.seen_gen = ctx->alloc_gen;
    return GGML_STATUS_SUCCESS;   // asynchronous: completion is observed through synchronize()
}

const ggml_backend_i backend_iface = {
    /* .get_name           = */ backend_get_name,
    /* .free               = */ backend_free,
    /* .set_tensor_async   = */ backend_set_tensor_async,
    /* .get_tensor_async   = */ backend_get_tensor_async,
    /* .cpy_tensor_async   = */ backend_cpy_tensor_async,
    /* .synchronize        = */ backend_synchronize,
    /* .graph_plan_create  = */ nullptr,
    /* .graph_plan_free    = */ nullptr,
    /* .graph_plan_update  = */ nullptr,
    /* .graph_plan_compute = */ nullptr,
    /* .graph_compute      = */ backend_graph_compute,
    /* .event_record       = */ backend_event_record,
    /* .event_wait         = */ backend_event_wait,
};

// ------------------------------------------------------------------------------- device
const char * device_get_name(ggml_backend_dev_t dev) { return ((device_ctx *) dev->context)->name.c_str(); }
const char * device_get_description(ggml_backend_dev_t dev) { return ((device_ctx *) dev->context)->description.c_str(); }

void device_get_memory(ggml_backend_dev_t dev, size_t * free, size_t * total) {
    device_ctx * ctx = (device_ctx *) dev->context;
    *free = *total = 0;
    if (hipSetDevice(ctx->device) == hipSuccess) (void) hipMemGetInfo(free, total);
}

enum ggml_backend_dev_type device_get_type(ggml_backend_dev_t) { return GGML_BACKEND_DEVICE_TYPE_GPU; }

void device_get_props(ggml_backend_dev_t dev, ggml_backend_dev_props * props) {
    props->name = device_get_name(dev);
    props->description = device_get_description(dev);
    props->type = GGML_BACKEND_DEVICE_TYPE_GPU;
    device_get_memory(dev, &props->memory_free, &props->memory_total);
    props->caps = { /* async */ true, /* host_buffer */ true, /* buffer_from_host_ptr */ false, /* events */ true };
}

ggml_backend_t device_init_backend(ggml_backend_dev_t dev, const char *) {
    device_ctx * dctx = (device_ctx *) dev->context;
    if (hipSetDevice(dctx->device) != hipSuccess) return nullptr;
    backend_ctx * ctx = new backend_ctx;
    ctx->device = dctx->device;
    ctx->name = dctx->name;
    const char * nf = getenv("MI355_NO_FUSION");
    ctx->fuse = !(nf && nf[0] == '1');
    std::vector<int32_t> iota_host(IOTA_N);
    for (int k = 0; k < IOTA_N; k++) iota_host[k] = k;
    if (hipMalloc((void **) &ctx->iota, IOTA_N * sizeof(int32_t)) != hipSuccess ||
        hipMemcpy(ctx->iota, iota_host.data(), IOTA_N * sizeof(int32_t), hipMemcpyHostToDevice) != hipSuccess) {
        delete ctx;
        return nullptr;
    }
    const char * ng = getenv("MI355_NO_GRAPH");
    ctx->replay.enabled = ctx->fuse && !(ng && ng[0] == '1');
    if (hipMalloc((void **) &ctx->cells, 8 * sizeof(int32_t)) != hipSuccess) {
        (void) hipFree(ctx->iota);
        delete ctx;
        return nullptr;
    }
    if (hipStreamCreate(&ctx->stream) != hipSuccess) {   // default priority, blocking w.r.t. the null stream
        (void) hipFree(ctx->iota);
        (void) hipFree(ctx->cells);
        delete ctx;
        return nullptr;
    }
    return new ggml_backend{ mi355_guid(), backend_iface, dev, ctx };
}

ggml_backend_buffer_type_t device_get_buffer_type(ggml_backend_dev_t dev) { return mi355_buffer_type(((device_ctx *) dev->context)->device); }

ggml_backend_buffer_type_t device_get_host_buffer_type(ggml_backend_dev_t dev) { return mi355_host_buffer_type(dev); }

bool device_supports_buft(ggml_backend_dev_t dev, ggml_backend_buffer_type_t buft) {
    return buft->iface.get_name == buft_get_name && buft->device == dev;
}

ggml_backend_event_t device_event_new(ggml_backend_dev_t dev) {
    device_ctx * ctx = (device_ctx *) dev->context;
    if (hipSetDevice(ctx->device) != hipSuccess) return nullptr;
    hipEvent_t ev = nullptr;
    if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
        (void) hipGetLastError();
        return nullptr;
    }
    return new ggml_backend_event{ /* .device = */ dev, /* .context = */ ev };
}

void device_event_free(ggml_backend_dev_t, ggml_backend_event_t event) {
    (void) hipEventDestroy((hipEvent_t) event->context);
    delete event;
}

void device_event_synchronize(ggml_backend_dev_t, ggml_backend_event_t event) {
    MI355_HIP_OK(hipEventSynchronize((hipEvent_t) event->context));
}

const ggml_backend_device_i device_iface = {
    /* .get_name             = */ device_get_name,
    /* .get_description      = */ device_get_description,
    /* .get_memory           = */ device_get_memory,
    /* .get_type             = */ device_get_type,
    /* .get_props            = */ device_get_props,
    /* .init_backend         = */ device_init_backend,
    /* .get_buffer_type      = */ device_get_buffer_type,
    /* .get_host_buffer_type = */ device_get_host_buffer_type,
    /* .buffer_from_host_ptr = */ nullptr,
    /* .supports_op          = */ device_supports_op,
    /* .supports_buft        = */ device_supports_buft,
    /* .offload_op           = */ nullptr,
    /* .event_new            = */ device_event_new,
    /* .event_free           = */ device_event_free,
    /* .event_synchronize    = */ device_event_synchronize,
};

// ------------------------------------------------------------------------------- reg
struct reg_ctx {
    std::vector<ggml_backend_device *> devices;
    std::vector<ggml_backend_buffer_type *> bufts;
};

const char * reg_get_name(ggml_backend_reg_t) { return "MI355X"; }
size_t reg_get_device_count(ggml_backend_reg_t reg) { return ((reg_ctx *) reg->context)->devices.size(); }
ggml_backend_dev_t reg_get_device(ggml_backend_reg_t reg, size_t index) {
    reg_ctx * ctx = (reg_ctx *) reg->context;
    GGML_ASSERT(index < ctx->devices.size());
    return ctx->devices[index];
}
void * reg_get_proc_address(ggml_backend_reg_t, const char *) { return nullptr; }

const ggml_backend_reg_i reg_iface = {
    /* .get_name         = */ reg_get_name,
    /* .get_device_count = */ reg_get_device_count,
    /* .get_device       = */ reg_get_device,
    /* .get_proc_address = */ reg_get_proc_address,
};

// One GPU only: the first gfx950 device.  Lifetime of these objects is the process (the registry never unloads).
ggml_backend_reg * the_reg() {
    static ggml_backend_reg reg;
    static reg_ctx ctx;
    static std::once_flag once;
    std::call_once(once, [] {
        int count = 0;
        if (hipGetDeviceCount(&count) != hipSuccess) count = 0;
        for (int d = 0; d < count && ctx.devices.empty(); d++) {
            if (mi355_device_supported(d) != 1) continue;
            hipDeviceProp_t prop;
            if (hipGetDeviceProperties(&prop, d) != hipSuccess) continue;
            device_ctx * dctx = new device_ctx;
            dctx->device = d;
            dctx->name = "MI355X" + std::to_string(ctx.devices.size());
            dctx->description = std::string(prop.name) + " (" + prop.gcnArchName + ")";
            ggml_backend_device * dev = new ggml_backend_device{ device_iface, &reg, dctx };
            ctx.devices.push_back(dev);
            ctx.bufts.push_back(new ggml_backend_buffer_type{ buft_iface, dev, nullptr });
        }
        reg.api_version = GGML_BACKEND_API_VERSION;
        reg.iface = reg_iface;
        reg.context = &ctx;
    });
    return &reg;
}

ggml_backend_buffer_type_t mi355_buffer_type(int device) {
    reg_ctx * ctx = (reg_ctx *) the_reg()->context;
    for (size_t i = 0; i < ctx->devices.size(); i++)
        if (((device_ctx *) ctx->devices[i]->context)->device == device) return ctx->bufts[i];
    return nullptr;
}

}  // namespace

// The two symbols the registry looks up (ggml/src/ggml-backend-reg.cpp:229-245); prototypes in include/ggml_mi355.h
extern "C" {

GGML_BACKEND_API ggml_backend_reg_t ggml_backend_init(void) { return the_reg(); }

// 0 = "not supported on this system" (no gfx950 GPU visible); higher scores win among variants
GGML_BACKEND_API int ggml_backend_score(void) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess) return 0;
    for (int d = 0; d < count; d++)
        if (mi355_device_supported(d) == 1) return 100;
    return 0;
}

}

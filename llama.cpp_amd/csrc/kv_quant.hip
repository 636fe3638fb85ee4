// Quantized KV cache: CPY f32 -> Q8_0 / Q4_0 (what llm_build_kv_store does with -ctk / -ctv q8_0, q4_0) and FLASH_ATTN_EXT over
// such a cache.  The copies are quantize_row_q8_0_ref / quantize_row_q4_0_ref (ggml/src/ggml-quants.c:39-72, 194-218) bit for
// bit.  Attention with fewer than 16 query rows (decode) reads the blocks where they lie, every byte of the cache once: one token
// over 1024 or more cells of a cache in the device row layout takes the streaming kernel (fattn_stream.hip: integer block dots
// with q as Q8_0, the reference's own arithmetic; V expanded to f16 inside the wave), everything else the vector kernel, which
// turns the levels into exact f16 values in its registers and applies the block's scale afterwards.  With 16 or more query rows the cells are first expanded into an f16 scratch image ([cell][kv head][D],
// d * level rounded to f16) that the matrix-core kernels then read: the expansion is shared by all rows of the batch.
//
// Where a block lives: a caller with a plain ggml cache passes row_blocks = 0 and blocks sit where ggml puts them (block g of the
// tensor at g * block bytes).  A tensor kept in this library's device row layout (levels of a row first, its scales behind them,
// mi355_weights_scatter) passes the blocks per row of the tensor that owns the memory: block g is then block g % row_blocks of
// row g / row_blocks of that tensor, whatever view of it (1-D for the store, [D, cells, heads] for attention) is being used.
#include "common.hpp"
#include "fattn.hpp"
#include "kv_blocks.hpp"

namespace mi355 {


// A view of a quantized tensor whose rows start on block boundaries: element (i0, i1, i2, i3) of the contiguous f32 side lies in block
// first_block + i0 / 32 + i1 * nbb[0] + i2 * nbb[1] + i3 * nbb[2] of the owner (strides in blocks).  ne0 == 0: consecutive blocks.
struct kv_view {
    int64_t ne0, ne1, ne2;
    int64_t nbb[3];
};
__device__ __forceinline__ int64_t kv_view_block(const kv_view &vw, int64_t e0) {
    if (vw.ne0 == 0) return e0 >> 5;
    const int64_t i0 = e0 % vw.ne0, r = e0 / vw.ne0;
    const int64_t i1 = r % vw.ne1, r2 = r / vw.ne1;
    return (i0 >> 5) + i1 * vw.nbb[0] + (r2 % vw.ne2) * vw.nbb[1] + (r2 / vw.ne2) * vw.nbb[2];
}

// Eight lanes share one 32-element block (4 consecutive elements each); n is a multiple of 32.
__global__ void __launch_bounds__(256) k_cpy_f32_q8_0(const float *__restrict__ x, uint8_t *__restrict__ y, int64_t n, kv_place pl, kv_view vw) {
    const int64_t e0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    const bool live = e0 < n;   // a block is all live or all dead
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (live) v = *(const f32x4 *)(x + e0);
    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
#pragma unroll
    for (int off = 4; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    if (!live) return;
    int64_t lv, sc;
    kv_block_offsets<MI355_Q8_0>(pl, pl.first_block + kv_view_block(vw, e0), lv, sc);
    const int sub = (int)((e0 >> 2) & 7);
    int q[4];
#pragma unroll
    for (int i = 0; i < 4; i++) q[i] = (int)roundf(v[i] * id);
    // plain 34-byte blocks are 2-byte aligned only
    unsigned short *o = (unsigned short *)(y + lv + 4 * sub);
    o[0] = (unsigned short)((q[0] & 0xFF) | ((q[1] & 0xFF) << 8));
    o[1] = (unsigned short)((q[2] & 0xFF) | ((q[3] & 0xFF) << 8));
    if (sub == 0) *(unsigned short *)(y + sc) = float_to_half_bits(d);
}

__global__ void __launch_bounds__(256) k_cpy_f32_q4_0(const float *__restrict__ x, uint8_t *__restrict__ y, int64_t n, kv_place pl, kv_view vw) {
    const int64_t e0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    const bool live = e0 < n;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (live) v = *(const f32x4 *)(x + e0);
    // the value of largest magnitude, the first one among equals (the reference's loop keeps the earlier on a tie)
    const int lane8 = threadIdx.x & 7;
    float amax = 0.0f, vmax = 0.0f;
    int imax = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        if (amax < fabsf(v[i])) {
            amax = fabsf(v[i]);
            vmax = v[i];
            imax = lane8 * 4 + i;
        }
    }
    if (amax == 0.0f) imax = 32;   // "no element yet": loses every tie
#pragma unroll
    for (int off = 4; off > 0; off >>= 1) {
        const float oa = __shfl_xor(amax, off, 64), ov = __shfl_xor(vmax, off, 64);
        const int oi = __shfl_xor(imax, off, 64);
        if (oa > amax || (oa == amax && oi < imax)) {
            amax = oa;
            vmax = ov;
            imax = oi;
        }
    }
    // d = vmax / -8, exact as an eighth with the sign flipped; the stored half takes its sign flip in the half's bits, so that a
    // zero block keeps the reference's -0.0 (a product converted to half may be fused with a +0.0 addend, which loses that sign)
    const float eighth = vmax * 0.125f;
    const float d = -eighth;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    unsigned packed = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int8_t qi = (int8_t)(v[i] * id + 8.5f);
        const unsigned u = (unsigned)(qi < 15 ? qi : 15) & 0xFu;
        packed |= u << (8 * i);
    }
    // byte j of the block pairs element j (low nibble) with element j + 16 (high nibble): lanes 0..3 take lanes 4..7's levels
    const unsigned hi = (unsigned)__shfl_down((int)packed, 4, 8);
    if (!live || lane8 >= 4) return;
    int64_t lv, sc;
    kv_block_offsets<MI355_Q4_0>(pl, pl.first_block + kv_view_block(vw, e0), lv, sc);
    const unsigned bytes = packed | (hi << 4);
    unsigned short *o = (unsigned short *)(y + lv + 4 * lane8);
    o[0] = (unsigned short)(bytes & 0xFFFFu);
    o[1] = (unsigned short)(bytes >> 16);
    if (lane8 == 0) *(unsigned short *)(y + sc) = (unsigned short)(float_to_half_bits(eighth) ^ 0x8000u);
}

// the other direction (ggml_cast of a quantized cache view to f32, the first step of its K-shift): y contiguous f32, four elements
// per lane; dequantize_row_q8_0 / dequantize_row_q4_0 (ggml-quants.c:255-273, 365-380)
template <int TYPE>
__global__ void __launch_bounds__(256) k_cpy_quant_f32(const uint8_t *__restrict__ src, float *__restrict__ y, int64_t n, kv_place pl, kv_view vw) {
    const int64_t e0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (e0 >= n) return;
    const int j = (int)((vw.ne0 == 0 ? e0 : e0 % vw.ne0) & 31);
    int64_t lv, sc;
    kv_block_offsets<TYPE>(pl, pl.first_block + kv_view_block(vw, e0), lv, sc);
    const float d = half_bits_to_float(*(const unsigned short *)(src + sc));
    f32x4 f;
    if constexpr (TYPE == MI355_Q8_0) {
        const unsigned short *p = (const unsigned short *)(src + lv + j);
        const unsigned w = (unsigned)p[0] | ((unsigned)p[1] << 16);
#pragma unroll
        for (int i = 0; i < 4; i++) f[i] = (float)(int8_t)((w >> (8 * i)) & 0xFF) * d;
    } else {
        const unsigned short *p = (const unsigned short *)(src + lv + (j & 15));
        const unsigned w = ((unsigned)p[0] | ((unsigned)p[1] << 16)) >> (j >= 16 ? 4 : 0);
#pragma unroll
        for (int i = 0; i < 4; i++) f[i] = (float)((int)((w >> (8 * i)) & 0xF) - 8) * d;
    }
    *(f32x4 *)(y + e0) = f;
}

// n consecutive blocks (in plain ggml addressing) of one quantized tensor to n consecutive blocks of another of the same type: the
// row copies of a cache defragmentation (build_defrag, src/llama.cpp:1215-1300).  One thread per block; overlapping ranges are the
// caller's business, as with ggml_cpy.
template <int TYPE>
__global__ void __launch_bounds__(256) k_cpy_quant_blocks(const uint8_t *__restrict__ src, kv_place sp, uint8_t *__restrict__ dst, kv_place dp, int64_t n) {
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= n) return;
    constexpr int LB = TYPE == MI355_Q8_0 ? 32 : 16;
    int64_t slv, ssc, dlv, dsc;
    kv_block_offsets<TYPE>(sp, sp.first_block + g, slv, ssc);
    kv_block_offsets<TYPE>(dp, dp.first_block + g, dlv, dsc);
    const unsigned short *a = (const unsigned short *)(src + slv);
    unsigned short *b = (unsigned short *)(dst + dlv);
#pragma unroll
    for (int i = 0; i < LB / 2; i++) b[i] = a[i];
    *(unsigned short *)(dst + dsc) = *(const unsigned short *)(src + ssc);
}

// dst f16 [cell][head][D] = dequantized rows of a typed cache whose (cell, head) row starts at block cell * cb + head * hb (+ the
// view's first block); one lane per 4 elements
struct kv_image {
    const uint8_t *src;
    int64_t cb, hb;
    kv_place pl;
    _Float16 *dst;
};
template <int TYPE>
__device__ __forceinline__ void kv_dequant_quad(const kv_image &im, int D, int HK, int64_t qd) {
    const int per_row = D >> 2;
    const int64_t rowi = qd / per_row;
    const int e0 = (int)(qd % per_row) * 4;
    const int64_t cell = rowi / HK;
    const int head = (int)(rowi % HK);
    const int j = e0 & 31;
    int64_t lv, sc;
    kv_block_offsets<TYPE>(im.pl, im.pl.first_block + cell * im.cb + (int64_t)head * im.hb + (e0 >> 5), lv, sc);
    const float d = half_bits_to_float(*(const unsigned short *)(im.src + sc));
    float f[4];
    if constexpr (TYPE == MI355_Q8_0) {
        const unsigned short *p = (const unsigned short *)(im.src + lv + j);
        const unsigned w = (unsigned)p[0] | ((unsigned)p[1] << 16);
#pragma unroll
        for (int i = 0; i < 4; i++) f[i] = (float)(int8_t)((w >> (8 * i)) & 0xFF) * d;
    } else {
        const unsigned short *p = (const unsigned short *)(im.src + lv + (j & 15));
        const unsigned w = ((unsigned)p[0] | ((unsigned)p[1] << 16)) >> (j >= 16 ? 4 : 0);
#pragma unroll
        for (int i = 0; i < 4; i++) f[i] = (float)((int)((w >> (8 * i)) & 0xF) - 8) * d;
    }
    _Float16 *o = im.dst + rowi * D + e0;
    const f16x2 lo = {(_Float16)f[0], (_Float16)f[1]}, hi = {(_Float16)f[2], (_Float16)f[3]};
    *(f16x2 *)o = lo;
    *(f16x2 *)(o + 2) = hi;
}
// blockIdx.y: 0 = the K image, 1 = the V image (one launch for both; TV < 0: only K)
template <int TK, int TV>
__global__ void __launch_bounds__(256) k_kv_dequant_f16(kv_image k, kv_image v, int D, int HK, int64_t n_quads) {
    const int64_t qd = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (qd >= n_quads) return;
    constexpr int TV2 = TV < 0 ? TK : TV;
    if (TV < 0 || blockIdx.y == 0) kv_dequant_quad<TK>(k, D, HK, qd);
    else kv_dequant_quad<TV2>(v, D, HK, qd);
}

static bool kv_type_ok(int t) { return t == MI355_F16 || t == MI355_Q8_0 || t == MI355_Q4_0; }
static size_t kv_image_bytes(int type, int64_t D, int64_t Nkv, int64_t Hkv) {
    return type == MI355_F16 ? 0 : (((size_t)Nkv * (size_t)Hkv * (size_t)D * 2 + 255) & ~(size_t)255);
}

// From this many query rows on the cache is expanded to f16 once and the matrix-core kernels run on the image (the expansion is
// shared by all rows); below it the vector kernel dequantizes in its registers.
constexpr int64_t KV_IMAGE_MIN_ROWS = 16;

// describes a quantized operand for in-place reads (Nkv cells of Hkv heads of D elements); false when its rows do not start on block
// boundaries or its cells are neither whole rows of the owner apart nor all inside one row of it (then the image path, with its own
// checks, takes it)
static bool kv_in_place(int type, const void *p, const void *base, int64_t row_blocks, size_t nb1, size_t nb2, int64_t D, int64_t Nkv, int64_t Hkv, kv_src &o) {
    const int64_t bb = type == MI355_Q8_0 ? Q8_0_BYTES : Q4_0_BYTES, lb = type == MI355_Q8_0 ? 32 : 16;
    if (base == nullptr) base = p;
    const int64_t off = (const char *)p - (const char *)base;
    if (((uintptr_t)base & 1) != 0 || off < 0 || off % bb != 0 || nb1 % bb != 0 || nb2 % bb != 0 || row_blocks < 0) return false;
    const int64_t cb = (int64_t)(nb1 / bb), hb = (int64_t)(nb2 / bb);
    int64_t first = off / bb;
    // every block of cell 0 lies in one row of the owner (checked below): that row becomes the base, so that the kernels find a block
    // of cell 0 without dividing by the row length
    if (row_blocks > 0) {
        base = (const char *)base + (first / row_blocks) * row_blocks * bb;
        first %= row_blocks;
    }
    o.base = (const uint8_t *)base;
    o.first_block = first;
    o.row_blocks = row_blocks;
    o.head_blocks = hb;
    if (row_blocks == 0 || cb % row_blocks == 0) {
        if (row_blocks > 0 && first % row_blocks + (Hkv - 1) * hb + D / 32 > row_blocks) return false;   // a cell's heads within one row
        o.cell_lv = o.cell_sc = (int64_t)nb1;
        return true;
    }
    // all cells inside one row of the owner: levels and scales advance by their own strides
    if (first % row_blocks + (Nkv - 1) * cb + (Hkv - 1) * hb + D / 32 > row_blocks) return false;
    o.cell_lv = cb * lb;
    o.cell_sc = cb * 2;
    return true;
}

}  // namespace mi355

using namespace mi355;

extern "C" {

int mi355_cpy_f32_quant(void *stream, int type, const float *src, void *dst_base, int64_t dst_first_block, int64_t dst_row_blocks, int64_t n) {
    MI355_REQUIRE(type == MI355_Q8_0 || type == MI355_Q4_0, "cpy_f32_quant: destination type %d is not Q8_0 or Q4_0", type);
    MI355_REQUIRE(n >= 0 && n % 32 == 0 && n / 1024 < 0x7fffffff, "cpy_f32_quant: %lld elements are not whole blocks of 32", (long long)n);
    MI355_REQUIRE(((uintptr_t)src & 15) == 0 && ((uintptr_t)dst_base & 1) == 0 && dst_first_block >= 0 && dst_row_blocks >= 0,
                  "cpy_f32_quant: source must be 16-byte, destination 2-byte aligned");
    if (n == 0) return MI355_OK;
    const kv_place pl = {dst_first_block, dst_row_blocks};
    const kv_view vw = {0, 1, 1, {0, 0, 0}};
    const dim3 grid((unsigned)((n / 4 + 255) / 256));
    if (type == MI355_Q8_0) MI355_LAUNCH(k_cpy_f32_q8_0, grid, dim3(256), 0, (hipStream_t)stream, src, (uint8_t *)dst_base, n, pl, vw);
    else MI355_LAUNCH(k_cpy_f32_q4_0, grid, dim3(256), 0, (hipStream_t)stream, src, (uint8_t *)dst_base, n, pl, vw);
    return launch_status("k_cpy_f32_quant");
}

int mi355_cpy_quant_view(void *stream, int type, int to_f32, float *f32, void *q_base, int64_t q_first_block, int64_t q_row_blocks, const int64_t *ne,
                         const int64_t *stride_blocks) {
    MI355_REQUIRE(type == MI355_Q8_0 || type == MI355_Q4_0, "cpy_quant_view: type %d is not Q8_0 or Q4_0", type);
    MI355_REQUIRE(ne != nullptr && stride_blocks != nullptr && ne[0] > 0 && ne[0] % 32 == 0 && ne[1] > 0 && ne[2] > 0 && ne[3] > 0,
                  "cpy_quant_view: rows must be whole blocks of 32");
    MI355_REQUIRE(stride_blocks[0] >= 0 && stride_blocks[1] >= 0 && stride_blocks[2] >= 0 && q_first_block >= 0 && q_row_blocks >= 0,
                  "cpy_quant_view: negative strides");
    MI355_REQUIRE(((uintptr_t)f32 & 15) == 0 && ((uintptr_t)q_base & 1) == 0, "cpy_quant_view: f32 side must be 16-byte, quantized side 2-byte aligned");
    const int64_t n = ne[0] * ne[1] * ne[2] * ne[3];
    MI355_REQUIRE(n / 1024 < 0x7fffffff, "cpy_quant_view: too many elements for one launch");
    const kv_place pl = {q_first_block, q_row_blocks};
    const kv_view vw = {ne[0], ne[1], ne[2], {stride_blocks[0], stride_blocks[1], stride_blocks[2]}};
    const dim3 grid((unsigned)((n / 4 + 255) / 256));
    hipStream_t s = (hipStream_t)stream;
    if (to_f32) {
        if (type == MI355_Q8_0) MI355_LAUNCH(k_cpy_quant_f32<MI355_Q8_0>, grid, dim3(256), 0, s, (const uint8_t *)q_base, f32, n, pl, vw);
        else MI355_LAUNCH(k_cpy_quant_f32<MI355_Q4_0>, grid, dim3(256), 0, s, (const uint8_t *)q_base, f32, n, pl, vw);
    } else {
        if (type == MI355_Q8_0) MI355_LAUNCH(k_cpy_f32_q8_0, grid, dim3(256), 0, s, (const float *)f32, (uint8_t *)q_base, n, pl, vw);
        else MI355_LAUNCH(k_cpy_f32_q4_0, grid, dim3(256), 0, s, (const float *)f32, (uint8_t *)q_base, n, pl, vw);
    }
    return launch_status("k_cpy_quant_view");
}

int mi355_cpy_quant_blocks(void *stream, int type, const void *src_base, int64_t src_first_block, int64_t src_row_blocks, void *dst_base,
                           int64_t dst_first_block, int64_t dst_row_blocks, int64_t n_blocks) {
    MI355_REQUIRE(type == MI355_Q8_0 || type == MI355_Q4_0, "cpy_quant_blocks: type %d is not Q8_0 or Q4_0", type);
    MI355_REQUIRE(n_blocks >= 0 && n_blocks / 256 < 0x7fffffff && src_first_block >= 0 && dst_first_block >= 0 && src_row_blocks >= 0 && dst_row_blocks >= 0,
                  "cpy_quant_blocks: bad block range");
    MI355_REQUIRE(((uintptr_t)src_base & 1) == 0 && ((uintptr_t)dst_base & 1) == 0, "cpy_quant_blocks: tensors must be 2-byte aligned");
    if (n_blocks == 0) return MI355_OK;
    const kv_place sp = {src_first_block, src_row_blocks}, dp = {dst_first_block, dst_row_blocks};
    const dim3 grid((unsigned)((n_blocks + 255) / 256));
    if (type == MI355_Q8_0) MI355_LAUNCH(k_cpy_quant_blocks<MI355_Q8_0>, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t *)src_base, sp, (uint8_t *)dst_base, dp, n_blocks);
    else MI355_LAUNCH(k_cpy_quant_blocks<MI355_Q4_0>, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t *)src_base, sp, (uint8_t *)dst_base, dp, n_blocks);
    return launch_status("k_cpy_quant_blocks");
}

size_t mi355_flash_attn_kv_ws_bytes(int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, int type_k, int type_v) {
    size_t base = mi355_flash_attn_ws_bytes(D, Nq, Nkv, Hq);
    if (base > ((size_t)256 << 20)) base = (size_t)256 << 20;   // the splits use what they are given
    return ((base + 255) & ~(size_t)255) + kv_image_bytes(type_k, D, Nkv, Hkv) + kv_image_bytes(type_v, D, Nkv, Hkv);
}

// describes one quantized operand for the expansion into its f16 image; `p` points at the first row in plain ggml addressing, `base`
// at the data of the tensor that owns the memory
static int kv_image_of(int type, const void *p, const void *base, int64_t row_blocks, size_t nb1, size_t nb2, void *img, kv_image &o) {
    const int64_t bb = type == MI355_Q8_0 ? Q8_0_BYTES : Q4_0_BYTES;
    if (base == nullptr) base = p;
    const int64_t off = (const char *)p - (const char *)base;
    MI355_REQUIRE(((uintptr_t)base & 1) == 0 && off >= 0 && off % bb == 0 && nb1 % bb == 0 && nb2 % bb == 0 && row_blocks >= 0,
                  "flash_attn_kv: quantized rows must start on block boundaries");
    o.src = (const uint8_t *)base;
    o.cb = (int64_t)nb1 / bb;
    o.hb = (int64_t)nb2 / bb;
    o.pl = kv_place{off / bb, row_blocks};
    o.dst = (_Float16 *)img;
    return MI355_OK;
}

// the f16 images of the quantized operands, K and V in one launch where both are quantized (type F16: nothing to do for that operand)
static int kv_expand(hipStream_t s, int type_k, const kv_image &k, int type_v, const kv_image &v, int64_t D, int64_t Nkv, int64_t Hkv) {
    const int64_t n_quads = Nkv * Hkv * (D / 4);
    MI355_REQUIRE(n_quads / 256 < 0x7fffffff, "flash_attn_kv: cache too large for one launch");
    const unsigned gx = (unsigned)((n_quads + 255) / 256);
    const int Di = (int)D, Hi = (int)Hkv;
    if (type_k != MI355_F16 && type_v != MI355_F16) {
        const dim3 grid(gx, 2);
        if (type_k == MI355_Q8_0 && type_v == MI355_Q8_0) MI355_LAUNCH((k_kv_dequant_f16<MI355_Q8_0, MI355_Q8_0>), grid, dim3(256), 0, s, k, v, Di, Hi, n_quads);
        else if (type_k == MI355_Q8_0) MI355_LAUNCH((k_kv_dequant_f16<MI355_Q8_0, MI355_Q4_0>), grid, dim3(256), 0, s, k, v, Di, Hi, n_quads);
        else if (type_v == MI355_Q8_0) MI355_LAUNCH((k_kv_dequant_f16<MI355_Q4_0, MI355_Q8_0>), grid, dim3(256), 0, s, k, v, Di, Hi, n_quads);
        else MI355_LAUNCH((k_kv_dequant_f16<MI355_Q4_0, MI355_Q4_0>), grid, dim3(256), 0, s, k, v, Di, Hi, n_quads);
    } else {
        const kv_image &one = type_k != MI355_F16 ? k : v;
        const int type = type_k != MI355_F16 ? type_k : type_v;
        if (type == MI355_Q8_0) MI355_LAUNCH((k_kv_dequant_f16<MI355_Q8_0, -1>), dim3(gx), dim3(256), 0, s, one, one, Di, Hi, n_quads);
        else MI355_LAUNCH((k_kv_dequant_f16<MI355_Q4_0, -1>), dim3(gx), dim3(256), 0, s, one, one, Di, Hi, n_quads);
    }
    return launch_status("k_kv_dequant_f16");
}

int mi355_flash_attn_ext_kv(void *stream, const float *q, const void *k, int type_k, const void *k_base, int64_t k_row_blocks, const void *v,
                            int type_v, const void *v_base, int64_t v_row_blocks, const void *mask, float *dst, int64_t D, int64_t Nq, int64_t Nkv,
                            int64_t Hq, int64_t Hkv, size_t q_nb1, size_t q_nb2, size_t k_nb1, size_t k_nb2, size_t v_nb1, size_t v_nb2,
                            size_t mask_nb1, float scale, float max_bias, float logit_softcap, void *ws, size_t ws_bytes, void *act) {
    MI355_REQUIRE(kv_type_ok(type_k) && kv_type_ok(type_v), "flash_attn_kv: cache types %d / %d (f16, Q8_0 and Q4_0 are served)", type_k, type_v);
    if (type_k == MI355_F16 && type_v == MI355_F16)
        return mi355_flash_attn_ext_quant(stream, q, k, v, mask, dst, D, Nq, Nkv, Hq, Hkv, q_nb1, q_nb2, k_nb1, k_nb2, v_nb1, v_nb2, mask_nb1, scale,
                                          max_bias, logit_softcap, ws, ws_bytes, act);
    MI355_REQUIRE(D > 0 && D % 32 == 0 && Nkv > 0 && Hkv > 0, "flash_attn_kv: head size %lld is not a whole number of blocks", (long long)D);
    hipStream_t s = (hipStream_t)stream;
    // A few query rows (decode): the vector kernel reads the blocks where they lie, each byte of the cache once.
    if (Nq < KV_IMAGE_MIN_ROWS) {
        kv_src kq = {nullptr, 0, 0, 0, 0, 0}, vq = {nullptr, 0, 0, 0, 0, 0};
        const bool k_ok = type_k == MI355_F16 || kv_in_place(type_k, k, k_base, k_row_blocks, k_nb1, k_nb2, D, Nkv, Hkv, kq);
        const bool v_ok = type_v == MI355_F16 || kv_in_place(type_v, v, v_base, v_row_blocks, v_nb1, v_nb2, D, Nkv, Hkv, vq);
        if (k_ok && v_ok)
            return fattn_vec_kv(s, q, k, type_k, kq, v, type_v, vq, mask, dst, D, Nq, Nkv, Hq, Hkv, q_nb1, q_nb2, k_nb1, k_nb2, v_nb1, v_nb2, mask_nb1, scale,
                                max_bias, logit_softcap, ws, ws_bytes, act);
    }
    const size_t kb = kv_image_bytes(type_k, D, Nkv, Hkv), vb = kv_image_bytes(type_v, D, Nkv, Hkv);
    MI355_REQUIRE(ws != nullptr && ((uintptr_t)ws & 255) == 0 && ws_bytes >= kb + vb, "flash_attn_kv: the workspace must be 256-byte aligned and hold the f16 images (%zu bytes)", kb + vb);
    // the images sit at the end of the workspace; what is in front of them serves the kv splits as before
    const size_t front = (ws_bytes - kb - vb) & ~(size_t)255;
    uint8_t *kimg = (uint8_t *)ws + front, *vimg = kimg + kb;
    kv_image ki = {nullptr, 0, 0, {0, 0}, nullptr}, vi = ki;
    if (type_k != MI355_F16) {
        int rc = kv_image_of(type_k, k, k_base, k_row_blocks, k_nb1, k_nb2, kimg, ki);
        if (rc != MI355_OK) return rc;
    }
    if (type_v != MI355_F16) {
        int rc = kv_image_of(type_v, v, v_base, v_row_blocks, v_nb1, v_nb2, vimg, vi);
        if (rc != MI355_OK) return rc;
    }
    int rc = kv_expand(s, type_k, ki, type_v, vi, D, Nkv, Hkv);
    if (rc != MI355_OK) return rc;
    if (type_k != MI355_F16) {
        k = kimg;
        k_nb1 = (size_t)Hkv * D * 2;
        k_nb2 = (size_t)D * 2;
    }
    if (type_v != MI355_F16) {
        v = vimg;
        v_nb1 = (size_t)Hkv * D * 2;
        v_nb2 = (size_t)D * 2;
    }
    return mi355_flash_attn_ext_quant(stream, q, k, v, mask, dst, D, Nq, Nkv, Hq, Hkv, q_nb1, q_nb2, k_nb1, k_nb2, v_nb1, v_nb2, mask_nb1, scale,
                                      max_bias, logit_softcap, front ? ws : nullptr, front, act);
}

}  // extern "C"

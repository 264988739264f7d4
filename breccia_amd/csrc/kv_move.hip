// Byte-moving kernels of the paged-KV path for gfx950: K/V append through the block
// table (three row encodings), copy-on-write page copy, page gather/scatter for the
// host swap, a dequantising row gather for parity checks, and small utilities.
// All of it is HBM-bound; the rules that matter are 16-byte accesses, whole-line
// coalescing and several independent loads in flight per lane.
#include <type_traits>

#include "bkv_internal.hpp"
#include "f16_rule.hpp"
#include "quant_encode.hpp"

namespace bkv {

namespace {

constexpr int kBlock = 256;

// 16-byte vector the nontemporal builtins accept.  Streaming copies that will not be re-read
// by this kernel go around the caches' replacement policy (measured on MI355X: 6.2 vs 5.8
// TB/s for a page-granular device copy).
typedef unsigned v4u __attribute__((ext_vector_type(4)));
__device__ __forceinline__ v4u ld_stream(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const v4u*>(p));
}
__device__ __forceinline__ void st_stream(void* p, v4u v) {
    __builtin_nontemporal_store(v, reinterpret_cast<v4u*>(p));
}

__device__ __forceinline__ uint32_t pack2(float lo, float hi) { return f16_store_pair(lo, hi); }

struct MoveGeom {
    int32_t n_kv, hd, page_cells, max_pages_per_seq;
};

// Eight consecutive source values as f32.  Sources are f32 rows, or raw binary16 rows that are
// read under the cache's load rule (so an f16 source appends exactly what the f32 row of its
// widened values would): codes8(const uint16_t*) and load8_unflushed / flush8 below.
__device__ __forceinline__ void load8(const float* p, float (&x)[8]) {
    const v4u a = ld_stream(p), b = ld_stream(p + 4);
    x[0] = __uint_as_float(a.x);
    x[1] = __uint_as_float(a.y);
    x[2] = __uint_as_float(a.z);
    x[3] = __uint_as_float(a.w);
    x[4] = __uint_as_float(b.x);
    x[5] = __uint_as_float(b.y);
    x[6] = __uint_as_float(b.z);
    x[7] = __uint_as_float(b.w);
}
// For the quantising kernels: the values as the hardware converts them (subnormal codes keep
// their value), and the load rule's flush as a separate step.  Where a block's amax is above 2^-6
// the flush changes neither the amax nor a code (|x| < 2^-14 quantises to 0 against a scale above
// 2^-6 / 127 either way), so those kernels only flush when a block is below that.
__device__ __forceinline__ void load8_unflushed(const float* p, float (&x)[8]) { load8(p, x); }
__device__ __forceinline__ void load8_unflushed(const uint16_t* p, float (&x)[8]) {
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    const h8 h = __builtin_bit_cast(h8, ld_stream(p));
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = (float)h[i];
}
template <typename SrcT>
__device__ __forceinline__ void flush8(float (&x)[8]) {
    if (std::is_same<SrcT, uint16_t>::value) {
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = fabsf(x[i]) < 0x1p-14f ? __builtin_copysignf(0.0f, x[i]) : x[i];
    }
}

// Eight consecutive source values as the f16 codes the cache stores for them.
__device__ __forceinline__ v4u codes8(const float* p) {
    float x[8];
    load8(p, x);
    v4u o;
    o.x = pack2(x[0], x[1]);
    o.y = pack2(x[2], x[3]);
    o.z = pack2(x[4], x[5]);
    o.w = pack2(x[6], x[7]);
    return o;
}
// A binary16 source goes through the load rule and then the store rule: a code with exponent field
// 0 becomes a signed zero and a NaN a signed infinity, every other code is stored as it is -- that
// is, codes with exponent field 0 or 31 lose their mantissa bits.  Two codes a word, no conversion:
// e + 0x0400 has none of the bits 0x7800 exactly for those two exponent fields.
// (The packed 16-bit min and multiply are written as instructions: the vector forms crash this
// compiler's instruction selection.)
__device__ __forceinline__ uint32_t f16_rule_pair(uint32_t w) {
    const uint32_t t = ((w & 0x7c007c00u) + 0x04000400u) & 0x78007800u;
    uint32_t ordinary, keep;  // per half: 1 where the mantissa stays, then its mask
    asm("v_pk_min_u16 %0, %1, %2" : "=v"(ordinary) : "v"(t), "v"(0x00010001u));
    asm("v_pk_mul_lo_u16 %0, %1, %2" : "=v"(keep) : "v"(ordinary), "v"(0x03ff03ffu));
    return w & (0xfc00fc00u | keep);
}
__device__ __forceinline__ v4u codes8(const uint16_t* p) {
    v4u a = ld_stream(p);
    a.x = f16_rule_pair(a.x);
    a.y = f16_rule_pair(a.y);
    a.z = f16_rule_pair(a.z);
    a.w = f16_rule_pair(a.w);
    return a;
}

// Pages hold 16 cells (bkv_pool_create accepts nothing else), so cell -> (page, row in page) is a
// shift and a mask; the kernels are compiled for head dim 256 and once more for any other, and the
// usual power-of-two kv head counts divide by a shift: a division by a run-time value is some 25
// instructions (a 64-bit one 100), as much as the rest of an append lane's work.
constexpr unsigned kPageShift = 4, kPageMask = 15;

struct RowOfSeq {
    unsigned t, kvh;  // token within the sequence's rows of this call, kv head
};
__device__ __forceinline__ RowOfSeq split_row(uint64_t r, unsigned n_kv, bool fits32) {
    unsigned t;
    if ((n_kv & (n_kv - 1u)) == 0u)
        t = (unsigned)(r >> (31 - __builtin_clz(n_kv)));
    else
        t = fits32 ? (unsigned)r / n_kv : (unsigned)(r / n_kv);
    return RowOfSeq{t, (unsigned)(r - (uint64_t)t * n_kv)};
}
// the pool row of (sequence s of the call, token t, kv head)
__device__ __forceinline__ size_t pool_row_of(const AppendBatch& b, const MoveGeom& g, const int32_t* tables, int s,
                                              RowOfSeq rs) {
    // cells are below 2^31 (pos0 and the token count are int32 and their sum is checked on the host)
    const unsigned cell = (unsigned)b.pos0[s] + rs.t;
    const int32_t phys = tables[(size_t)b.row[s] * (size_t)g.max_pages_per_seq + (size_t)(cell >> kPageShift)];
    return (((size_t)phys * g.n_kv + rs.kvh) << kPageShift) + (size_t)(cell & kPageMask);
}

// ---- append, f16 rows ---------------------------------------------------------
// One lane converts 8 consecutive elements of one (token, kv head) row of K and of V:
// two 16-byte loads and one 16-byte store per pool.  grid.y = sequence of the call; the rows of a
// sequence are contiguous in the source, so unit u of a sequence is simply its u-th 8-element group.
template <typename SrcT, int HD>
__global__ __launch_bounds__(kBlock) void append_f16_kernel(AppendBatch b, MoveGeom g,
                                                            uint16_t* __restrict__ kpool,
                                                            uint16_t* __restrict__ vpool,
                                                            const int32_t* __restrict__ tables,
                                                            const SrcT* __restrict__ k,
                                                            const SrcT* __restrict__ v) {
    const int s = blockIdx.y;
    const unsigned hd = HD ? HD : g.hd;
    const unsigned lpr = hd / 8;  // lanes of a row
    const int64_t rows_total = (int64_t)b.n_tok[s] * g.n_kv;
    const bool fits32 = rows_total * lpr < (1ll << 32);
    const uint64_t unit = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t r = HD ? unit / lpr : (fits32 ? (uint64_t)((unsigned)unit / lpr) : unit / lpr);
    if ((int64_t)r >= rows_total) return;
    const unsigned li = (unsigned)(unit - r * lpr);
    const size_t row = pool_row_of(b, g, tables, s, split_row(r, (unsigned)g.n_kv, fits32));
    const size_t dst = row * (size_t)hd + (size_t)li * 8;
    const size_t src = (size_t)b.src0[s] * (size_t)(g.n_kv * hd) + (size_t)unit * 8;
    const v4u ko = codes8(k + src), vo = codes8(v + src);
    st_stream(kpool + dst, ko);
    st_stream(vpool + dst, vo);
}

// ---- 8 values at a time: the lane's share of a 32-value block whose other shares the rest of its quad holds --
// Both return the rule's results exactly: codes on a reciprocal with a proof per value, and the rule as
// written for the whole wave when any lane could not prove its codes.
template <typename SrcT>
__device__ __forceinline__ void q8v_quarter(float (&x)[8], float& scale, uint32_t& w0, uint32_t& w1) {
    const float amax = quad_max(amax8(x));
    scale = q8v_scale(amax);
    uint32_t doubt = (std::is_same<SrcT, uint16_t>::value && !(amax > 0x1p-6f)) ? 0x7fc00000u : 0u;
    codes8_on_reciprocal(x, scale, w0, w1, doubt);
    if (__any(codes_in_doubt(doubt))) {
        flush8<SrcT>(x);
        scale = q8v_scale(quad_max(amax8(x)));
        q8_codes8(x, scale, w0, w1);
    }
}
// f32 values only (binary16 rows have a path of their own in append_quant_kernel)
__device__ __forceinline__ void i8h_quarter(const float (&x)[8], uint32_t& scale_bits, uint32_t& w0, uint32_t& w1) {
    scale_bits = i8h_scale_bits(quad_max(amax8(x)));
    uint32_t doubt = 0u;
    codes8_on_reciprocal(x, f16_normal_value(scale_bits), w0, w1, doubt);
    if (__any(codes_in_doubt(doubt))) i8h_codes8(x, f16_load(scale_bits), w0, w1);
}

// Encoded rows put together in LDS leave as whole contiguous rows: piece p of the image goes to the same
// offset of its pool row (16-byte pieces where rows are multiples of 16 bytes, else 4-byte ones).
template <uint32_t PIECE>
__device__ __forceinline__ void image_rows_out(const uint8_t* image, uint8_t* pool, const uint64_t* row_s, int nrows,
                                               uint32_t row_bytes, int tid) {
    const uint32_t ppr = row_bytes / PIECE;  // pieces of a row
    const uint32_t n_pieces = (uint32_t)nrows * ppr;
    for (uint32_t p = (uint32_t)tid; p < n_pieces; p += kBlock) {
        const uint32_t pr = p / ppr, off = (p - pr * ppr) * PIECE;
        uint8_t* dst = pool + (size_t)row_s[pr] * row_bytes + off;
        if (PIECE == 16)
            st_stream(dst, *reinterpret_cast<const v4u*>(image + pr * row_bytes + off));
        else
            *reinterpret_cast<uint32_t*>(dst) = *reinterpret_cast<const uint32_t*>(image + pr * row_bytes + off);
    }
}

// ---- append, quantised rows -----------------------------------------------------------
// Q8V (the reference's BRECCIA_KV_Q8V, shaders/qsa_kv_append.comp:87-133): K f16, V
// [f32 scale][32 x i8] per 32 values.  I8H: K and V rows of [hd x i8][hd/32 x f16 scale].
// A lane takes 8 consecutive elements of one (token, kv head) row of K and of V, like the f16
// kernel (a wave's loads are contiguous 16-byte pieces); the four lanes of a quad share a
// 32-value block and agree its amax by DPP.  The encoded rows are put together in LDS and
// leave as whole contiguous rows, one 16-byte piece a lane (4-byte pieces when the head dim
// makes rows that are not 16-byte multiples).  A work-group owns 256 / (hd / 8) consecutive
// rows of one sequence of the call (grid.y).
template <int LAYOUT, typename SrcT, int HD>
__global__ __launch_bounds__(kBlock) void append_quant_kernel(AppendBatch b, MoveGeom g,
                                                              uint8_t* __restrict__ kpool,
                                                              uint8_t* __restrict__ vpool,
                                                              const int32_t* __restrict__ tables,
                                                              const SrcT* __restrict__ k,
                                                              const SrcT* __restrict__ v) {
    // at most 64 rows (hd 32) of at most 288 bytes (hd 256): rows x row bytes <= 2304 per image
    __shared__ __attribute__((aligned(16))) uint8_t image[2 * 2304];
    __shared__ uint64_t row_s[64];
    const int s = blockIdx.y;
    const int hd = HD ? HD : g.hd;
    const int lpr = hd / 8;           // lanes of a row
    const int rows_wg = kBlock / lpr;
    const int blocks = hd / 32;
    const int64_t rows_total = (int64_t)b.n_tok[s] * g.n_kv;
    const int64_t r0 = (int64_t)blockIdx.x * rows_wg;
    if (r0 >= rows_total) return;
    const int nrows = (int)(rows_total - r0 < rows_wg ? rows_total - r0 : rows_wg);
    const int tid = threadIdx.x;
    const int rl = tid / lpr, li = tid - rl * lpr;
    const bool active = rl < nrows;
    const uint32_t row_bytes = LAYOUT == BKV_LAYOUT_Q8V ? (uint32_t)blocks * 36u : (uint32_t)hd + (uint32_t)blocks * 2u;
    uint8_t* const v_image = image + (LAYOUT == BKV_LAYOUT_I8H ? rows_wg * row_bytes : 0u);

    float kx[8], vx[8];
    v4u ko = v4u{0u, 0u, 0u, 0u};
    size_t row = 0;
    if (active) {
        const uint64_t r = (uint64_t)(r0 + rl);
        row = pool_row_of(b, g, tables, s, split_row(r, (unsigned)g.n_kv, rows_total < (1ll << 32)));
        // the rows of a sequence are contiguous in the source
        const size_t src = ((size_t)b.src0[s] * g.n_kv + (size_t)r) * (size_t)hd + (size_t)li * 8;
        if (LAYOUT == BKV_LAYOUT_Q8V)
            ko = codes8(k + src);
        else
            load8_unflushed(k + src, kx);
        load8_unflushed(v + src, vx);
        if (li == 0) row_s[rl] = (uint64_t)row;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) kx[i] = vx[i] = 0.0f;
    }
    // quads never straddle rows (lanes of a row are a multiple of four), so a quad is active as a whole
    const int blk = li >> 2, quarter = li & 3;
    constexpr bool kSrcF16 = std::is_same<SrcT, uint16_t>::value;
    if (LAYOUT == BKV_LAYOUT_Q8V) {
        if (active) st_stream(reinterpret_cast<uint16_t*>(kpool) + row * (size_t)hd + (size_t)li * 8, ko);
        float scale;
        uint32_t w0, w1;
        q8v_quarter<SrcT>(vx, scale, w0, w1);
        if (active) {
            uint32_t* blk_words = reinterpret_cast<uint32_t*>(v_image + rl * row_bytes + blk * 36);
            if (quarter == 0) blk_words[0] = __float_as_uint(scale);
            blk_words[1 + 2 * quarter] = w0;
            blk_words[2 + 2 * quarter] = w1;
        }
    } else {
        const float ka = quad_max(amax8(kx)), va = quad_max(amax8(vx));
        uint32_t kb = i8h_scale_bits(ka), vb = i8h_scale_bits(va);
        uint32_t k0, k1, v0, v1;
        bool redo;
        if (kSrcF16) {
            // a NaN survives any sum; an infinity shows in the amax
            const float sum = ((kx[0] + kx[1]) + (kx[2] + kx[3])) + ((kx[4] + kx[5]) + (kx[6] + kx[7])) +
                              ((vx[0] + vx[1]) + (vx[2] + vx[3])) + ((vx[4] + vx[5]) + (vx[6] + vx[7]));
            redo = !(ka > 0x1p-6f && va > 0x1p-6f && ka <= 65504.0f && va <= 65504.0f) || sum != sum;
            codes8_f16_on_biased_reciprocal(kx, __builtin_amdgcn_rcpf(f16_normal_value(kb)) * kTieBias, k0, k1);
            codes8_f16_on_biased_reciprocal(vx, __builtin_amdgcn_rcpf(f16_normal_value(vb)) * kTieBias, v0, v1);
        } else {
            uint32_t doubt = 0u;
            codes8_on_reciprocal(kx, f16_normal_value(kb), k0, k1, doubt);
            codes8_on_reciprocal(vx, f16_normal_value(vb), v0, v1, doubt);
            redo = codes_in_doubt(doubt);
        }
        if (__any(redo)) {  // the rule as written, for the whole wave
            flush8<SrcT>(kx);
            flush8<SrcT>(vx);
            kb = i8h_scale_bits(quad_max(amax8(kx)));
            vb = i8h_scale_bits(quad_max(amax8(vx)));
            i8h_codes8(kx, f16_load(kb), k0, k1);
            i8h_codes8(vx, f16_load(vb), v0, v1);
        }
        if (active) {
            uint8_t* kr = image + rl * row_bytes;
            uint8_t* vr = v_image + rl * row_bytes;
            *reinterpret_cast<uint2*>(kr + li * 8) = make_uint2(k0, k1);
            *reinterpret_cast<uint2*>(vr + li * 8) = make_uint2(v0, v1);
            if (quarter == 0) {
                *reinterpret_cast<uint16_t*>(kr + hd + blk * 2) = (uint16_t)kb;
                *reinterpret_cast<uint16_t*>(vr + hd + blk * 2) = (uint16_t)vb;
            }
        }
    }
    __syncthreads();
    constexpr uint32_t kPiece = HD == 256 ? 16u : 4u;
    if (LAYOUT == BKV_LAYOUT_I8H) image_rows_out<kPiece>(image, kpool, row_s, nrows, row_bytes, tid);
    image_rows_out<kPiece>(v_image, vpool, row_s, nrows, row_bytes, tid);
}

// ---- K preparation fused into the append ------------------------------------------
// RMSNorm with gamma per (token, kv head) row, partial NEOX rotary at the token's
// position, then the append; V rows are appended as they are.  Replaces the chain
// Qsa::k_norm -> Qsa::rope_k -> Qsa::kv_append (qsa/mod.rs:1051-1058, :1079-1089,
// :1105-1156; shaders ops_rmsnorm.comp, ops_rope.comp, qsa_kv_append.comp) and its two
// f32 round trips through memory.  The arithmetic is the CPU reference's, operation for
// operation (ops/cpu.rs:52-88, :124-154): f64 sum of squares in element order,
// inv = 1/sqrt(ss/cols + eps), y = (f32)(x * inv * gamma), rotary products and sums in
// f64 without fusing, one f32 rounding per stage -- so the stored codes are bit-identical
// to that path followed by the cache's f16 rule.
struct KPrepParams {
    const float* gamma;        // [hd]
    const float* table;        // [max_pos][n_rot/2] of (cos, sin)
    const int32_t* positions;  // optional: rotary position of cell c; null = c itself
    float eps;
    int32_t n_rot, max_pos;
};

constexpr int kPrepRows = 16;  // (token, kv head) rows per work-group

// The sum stays in element order (the reference's f64 loop, ops/cpu.rs:52-66); the row is read
// 16 bytes at a time and several reads ahead, so that the chain of additions is all a lane waits for.
__device__ __forceinline__ double row_sum_squares(const float* row, int n) {
#pragma clang fp contract(off)
    double ss = 0.0;
#pragma unroll 8
    for (int i = 0; i < n; i += 4) {
        const float4 x = *reinterpret_cast<const float4*>(row + i);
        const double a = (double)x.x, b = (double)x.y, c = (double)x.z, d = (double)x.w;
        ss += a * a;
        ss += b * b;
        ss += c * c;
        ss += d * d;
    }
    return ss;
}

__device__ __forceinline__ void rotate_pair(float& lo, float& hi, float c32, float s32) {
#pragma clang fp contract(off)
    const double a = (double)lo, b = (double)hi, c = (double)c32, sn = (double)s32;
    const double ac = a * c, bs = b * sn, as = a * sn, bc = b * c;
    lo = (float)(ac - bs);
    hi = (float)(as + bc);
}

// HD: the head dim as a compile-time constant (the index arithmetic of every loop divides by it),
// or 0 for the value in the geometry.
template <int LAYOUT, int HD>
__global__ __launch_bounds__(kBlock) void append_kprep_kernel(AppendBatch b, MoveGeom g,
                                                              KPrepParams kp,
                                                              uint8_t* __restrict__ kpool,
                                                              uint8_t* __restrict__ vpool,
                                                              const int32_t* __restrict__ tables,
                                                              const float* __restrict__ k,
                                                              const float* __restrict__ v) {
    // [kPrepRows][hd + 4] floats, then per row: 1/rms, pool row, rotary position
    extern __shared__ __attribute__((aligned(16))) float prep_lds[];
    const int s = blockIdx.y;
    const int hd = HD ? HD : g.hd;
    // rows 16-byte aligned and 4 floats apart in the banks: the 16 lanes that sum a row each read
    // 16 bytes of their own row per step without colliding
    const int stride = hd + 4;
    const int rows_total = b.n_tok[s] * g.n_kv;
    const int r0 = (int)blockIdx.x * kPrepRows;
    if (r0 >= rows_total) return;
    const int nrows = min(kPrepRows, rows_total - r0);
    double* inv_s = reinterpret_cast<double*>(prep_lds + kPrepRows * stride);
    const size_t src_base = ((size_t)b.src0[s] * g.n_kv + (size_t)r0) * (size_t)hd;
    const int tid = threadIdx.x;

    // rows of one sequence are contiguous in the source: one coalesced sweep
    for (int idx = tid; idx < nrows * hd / 4; idx += kBlock) {
        const v4u w = ld_stream(k + src_base + (size_t)idx * 4);
        const int row = (idx * 4) / hd, col = (idx * 4) % hd;
        *reinterpret_cast<v4u*>(prep_lds + row * stride + col) = w;
    }
    __syncthreads();
    // While the first lanes sum their rows, a second wave works out where the rows go: the pool row
    // of (sequence row r) = (token, kv head) and the token's rotary position.
    uint64_t* const row_s = reinterpret_cast<uint64_t*>(inv_s + kPrepRows);
    int32_t* const pos_s = reinterpret_cast<int32_t*>(row_s + kPrepRows);
    if (tid < nrows) {
        const double ss = row_sum_squares(prep_lds + tid * stride, hd);
        inv_s[tid] = 1.0 / sqrt(ss / (double)hd + (double)kp.eps);
    } else if (tid >= 64 && tid - 64 < nrows) {
        const unsigned r = (unsigned)(r0 + tid - 64);
        const unsigned cell = (unsigned)b.pos0[s] + r / (unsigned)g.n_kv;
        const unsigned kvh = r % (unsigned)g.n_kv;
        const int32_t phys = tables[(size_t)b.row[s] * (size_t)g.max_pages_per_seq + (size_t)(cell >> kPageShift)];
        row_s[tid - 64] = (((uint64_t)phys * g.n_kv + kvh) << kPageShift) + (uint64_t)(cell & kPageMask);
        int64_t pos = kp.positions ? (int64_t)kp.positions[cell] : (int64_t)cell;
        pos = pos < 0 ? 0 : (pos > kp.max_pos - 1 ? kp.max_pos - 1 : pos);
        pos_s[tid - 64] = (int32_t)pos;
    }
    __syncthreads();
    for (int idx = tid; idx < nrows * hd; idx += kBlock) {
        const int row = idx / hd, col = idx % hd;
        float* d = prep_lds + row * stride + col;
        *d = (float)((double)*d * inv_s[row] * (double)kp.gamma[col]);
    }
    __syncthreads();
    const int half = kp.n_rot / 2;
    for (int idx = tid; idx < nrows * half; idx += kBlock) {
        const int row = idx / half, j = idx % half;
        const float2 cs = reinterpret_cast<const float2*>(kp.table)[(size_t)pos_s[row] * half + j];
        float* d = prep_lds + row * stride;
        rotate_pair(d[j], d[j + half], cs.x, cs.y);
    }
    __syncthreads();

    const auto pool_row = [&](int row) -> size_t { return (size_t)row_s[row]; };
    const int lpr = hd / 8;  // 8-value groups of a row

    if (LAYOUT == BKV_LAYOUT_F16) {
        // K from LDS, V straight from the source rows
        for (int idx = tid; idx < nrows * lpr; idx += kBlock) {
            const int row = (idx * 8) / hd, col = (idx * 8) % hd;
            const float* x = prep_lds + row * stride + col;
            v4u o;
            o.x = pack2(x[0], x[1]);
            o.y = pack2(x[2], x[3]);
            o.z = pack2(x[4], x[5]);
            o.w = pack2(x[6], x[7]);
            st_stream(reinterpret_cast<uint16_t*>(kpool) + pool_row(row) * (size_t)hd + col, o);
            float y[8];
            load8(v + src_base + (size_t)idx * 8, y);
            o.x = pack2(y[0], y[1]);
            o.y = pack2(y[2], y[3]);
            o.z = pack2(y[4], y[5]);
            o.w = pack2(y[6], y[7]);
            st_stream(reinterpret_cast<uint16_t*>(vpool) + pool_row(row) * (size_t)hd + col, o);
        }
        return;
    }
    // Quantised rows, as in append_quant_kernel: a lane encodes 8 consecutive values (the four lanes of a
    // quad share a 32-value block: 8-value groups of a row are a multiple of four, so a quad is in or
    // out of the loop as a whole), the rows are put together in LDS and leave whole.
    __shared__ __attribute__((aligned(16))) uint8_t image[2 * kPrepRows * 288];
    const int blocks = hd / 32;
    const uint32_t row_bytes = LAYOUT == BKV_LAYOUT_Q8V ? (uint32_t)blocks * 36u : (uint32_t)hd + (uint32_t)blocks * 2u;
    uint8_t* const v_image = image + (LAYOUT == BKV_LAYOUT_I8H ? kPrepRows * row_bytes : 0u);
    for (int idx = tid; idx < nrows * lpr; idx += kBlock) {
        const int row = idx / lpr, li = idx - row * lpr;
        const int blk = li >> 2, quarter = li & 3;
        const float* kxp = prep_lds + row * stride + li * 8;
        const float4 ka = *reinterpret_cast<const float4*>(kxp), kb = *reinterpret_cast<const float4*>(kxp + 4);
        float vx[8];
        load8(v + src_base + (size_t)idx * 8, vx);
        if (LAYOUT == BKV_LAYOUT_Q8V) {
            v4u o;
            o.x = pack2(ka.x, ka.y);
            o.y = pack2(ka.z, ka.w);
            o.z = pack2(kb.x, kb.y);
            o.w = pack2(kb.z, kb.w);
            st_stream(reinterpret_cast<uint16_t*>(kpool) + pool_row(row) * (size_t)hd + (size_t)li * 8, o);
            float scale;
            uint32_t w0, w1;
            q8v_quarter<float>(vx, scale, w0, w1);
            uint32_t* blk_words = reinterpret_cast<uint32_t*>(v_image + row * row_bytes + blk * 36);
            if (quarter == 0) blk_words[0] = __float_as_uint(scale);
            blk_words[1 + 2 * quarter] = w0;
            blk_words[2 + 2 * quarter] = w1;
        } else {
            const float kx[8] = {ka.x, ka.y, ka.z, ka.w, kb.x, kb.y, kb.z, kb.w};
            uint32_t ks, k0, k1, vs, v0, v1;
            i8h_quarter(kx, ks, k0, k1);
            i8h_quarter(vx, vs, v0, v1);
            uint8_t* kr = image + row * row_bytes;
            uint8_t* vr = v_image + row * row_bytes;
            *reinterpret_cast<uint2*>(kr + li * 8) = make_uint2(k0, k1);
            *reinterpret_cast<uint2*>(vr + li * 8) = make_uint2(v0, v1);
            if (quarter == 0) {
                *reinterpret_cast<uint16_t*>(kr + hd + blk * 2) = (uint16_t)ks;
                *reinterpret_cast<uint16_t*>(vr + hd + blk * 2) = (uint16_t)vs;
            }
        }
    }
    __syncthreads();
    constexpr uint32_t kPiece = HD == 256 ? 16u : 4u;
    if (LAYOUT == BKV_LAYOUT_I8H) image_rows_out<kPiece>(image, kpool, row_s, nrows, row_bytes, tid);
    image_rows_out<kPiece>(v_image, vpool, row_s, nrows, row_bytes, tid);
}

// ---- whole-page moves -----------------------------------------------------------
// Four independent 16-byte loads per lane, then four stores: one work-group moves up
// to 16 KiB, which is one f16 K or V page.
__device__ __forceinline__ void move_bytes16(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                             uint32_t n_vec, uint32_t base) {
    v4u r[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t idx = base + (uint32_t)i * kBlock + threadIdx.x;
        if (idx < n_vec) r[i] = ld_stream(src + idx);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t idx = base + (uint32_t)i * kBlock + threadIdx.x;
        if (idx < n_vec) st_stream(dst + idx, r[i]);
    }
}

struct PoolPtrs {
    uint8_t* slab;
    uint64_t layer_stride;  // bytes between consecutive layers
    uint64_t v_offset;      // offset of a layer's V pool behind its K pool
    uint64_t k_page_bytes, v_page_bytes;
    int32_t n_layers;
};

// A unit is one 16 KiB chunk of one (pair, layer, K|V) page image.  A work-group copies
// whole chunks (each wave 4 x 1 KiB contiguous), walking the unit list with a grid stride;
// the (src, dst) pair of the next unit is fetched while the current chunk is in flight.
struct CopyUnit {
    const uint8_t* src;
    uint8_t* dst;
    uint32_t n_vec;  // 16-byte vectors left in the page image from this chunk's start
};

__device__ __forceinline__ CopyUnit copy_unit(const PoolPtrs& pp, const bkv_page_pair pr,
                                              uint32_t pl, uint32_t chunk, uint32_t chunks_k) {
    const uint32_t which = chunk >= chunks_k ? 1u : 0u;
    if (which) chunk -= chunks_k;
    const uint32_t layer = pl % (uint32_t)pp.n_layers;
    const uint64_t pb = which ? pp.v_page_bytes : pp.k_page_bytes;
    uint8_t* pool = pp.slab + (uint64_t)layer * pp.layer_stride + (which ? pp.v_offset : 0);
    const uint64_t off = (uint64_t)chunk * (4u * kBlock * 16u);
    CopyUnit u;
    u.src = pool + (uint64_t)pr.src * pb + off;
    u.dst = pool + (uint64_t)pr.dst * pb + off;
    u.n_vec = (uint32_t)((pb - off) / 16);
    return u;
}

__global__ __launch_bounds__(kBlock) void page_copy_kernel(PoolPtrs pp,
                                                           const bkv_page_pair* __restrict__ pairs,
                                                           uint32_t n_pairs, uint32_t chunks_k,
                                                           uint32_t chunks_v) {
    const uint32_t per_pl = chunks_k + chunks_v;
    const uint32_t total = n_pairs * (uint32_t)pp.n_layers * per_pl;
    uint32_t c = blockIdx.x;
    if (c >= total) return;
    bkv_page_pair pr = pairs[(c / per_pl) / (uint32_t)pp.n_layers];
    while (c < total) {
        const uint32_t pl = c / per_pl;
        const CopyUnit u = copy_unit(pp, pr, pl, c - pl * per_pl, chunks_k);
        const uint32_t c_next = c + gridDim.x;
        if (c_next < total) pr = pairs[(c_next / per_pl) / (uint32_t)pp.n_layers];
        v4u r[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t idx = (uint32_t)i * kBlock + threadIdx.x;
            if (idx < u.n_vec) r[i] = ld_stream(u.src + (size_t)idx * 16);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t idx = (uint32_t)i * kBlock + threadIdx.x;
            if (idx < u.n_vec) st_stream(u.dst + (size_t)idx * 16, r[i]);
        }
        c = c_next;
    }
}

// Staging layout: [page i][layer][K page bytes | V page bytes].
__global__ __launch_bounds__(kBlock) void page_stage_kernel(PoolPtrs pp,
                                                            const int32_t* __restrict__ pages,
                                                            uint8_t* __restrict__ stage,
                                                            int to_stage) {
    const uint32_t u = blockIdx.y;
    const uint32_t which = u & 1u;
    const uint32_t layer = (u >> 1) % (uint32_t)pp.n_layers;
    const uint32_t i = (u >> 1) / (uint32_t)pp.n_layers;
    const uint64_t pb = which ? pp.v_page_bytes : pp.k_page_bytes;
    const uint32_t n_vec = (uint32_t)(pb / 16);
    const uint32_t base = blockIdx.x * (4u * kBlock);
    if (base >= n_vec) return;
    uint8_t* pool = pp.slab + (uint64_t)layer * pp.layer_stride + (which ? pp.v_offset : 0) +
                    (uint64_t)pages[i] * pb;
    const uint64_t slab_bytes = (pp.k_page_bytes + pp.v_page_bytes) * (uint64_t)pp.n_layers;
    uint8_t* st = stage + (uint64_t)i * slab_bytes +
                  (uint64_t)layer * (pp.k_page_bytes + pp.v_page_bytes) +
                  (which ? pp.k_page_bytes : 0);
    if (to_stage)
        move_bytes16(reinterpret_cast<const uint4*>(pool), reinterpret_cast<uint4*>(st), n_vec, base);
    else
        move_bytes16(reinterpret_cast<const uint4*>(st), reinterpret_cast<uint4*>(pool), n_vec, base);
}

// ---- dequantising gather (parity / debugging; one lane per element) ---------------
__global__ __launch_bounds__(kBlock) void gather_kernel(MoveGeom g, int layout,
                                                        const uint8_t* __restrict__ kpool,
                                                        const uint8_t* __restrict__ vpool,
                                                        const int32_t* __restrict__ table_row,
                                                        int64_t cell0, int64_t n,
                                                        float* __restrict__ k_out,
                                                        float* __restrict__ v_out) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t total = n * g.n_kv * g.hd;
    if (idx >= total) return;
    const int d = (int)(idx % g.hd);
    const int kvh = (int)((idx / g.hd) % g.n_kv);
    const int64_t i = idx / ((int64_t)g.hd * g.n_kv);
    const int64_t cell = cell0 + i;
    const int32_t phys = table_row[cell / g.page_cells];
    const size_t row = ((size_t)phys * g.n_kv + kvh) * g.page_cells + (size_t)(cell % g.page_cells);
    float kv, vv;
    if (layout == BKV_LAYOUT_I8H) {
        const size_t rb = (size_t)g.hd + (size_t)(g.hd / 32) * 2;
        const uint8_t* kr = kpool + row * rb;
        const uint8_t* vr = vpool + row * rb;
        const uint32_t ks = *reinterpret_cast<const uint16_t*>(kr + g.hd + (d / 32) * 2);
        const uint32_t vs = *reinterpret_cast<const uint16_t*>(vr + g.hd + (d / 32) * 2);
        kv = (float)(int8_t)kr[d] * f16_load(ks);
        vv = (float)(int8_t)vr[d] * f16_load(vs);
    } else {
        kv = f16_load(reinterpret_cast<const uint16_t*>(kpool)[row * (size_t)g.hd + d]);
        if (layout == BKV_LAYOUT_F16) {
            vv = f16_load(reinterpret_cast<const uint16_t*>(vpool)[row * (size_t)g.hd + d]);
        } else {
            const uint32_t* w =
                reinterpret_cast<const uint32_t*>(vpool) + (row * (size_t)(g.hd / 32) + d / 32) * 9u;
            const int j = d % 32;
            const int8_t q = (int8_t)((w[1 + j / 4] >> (8 * (j % 4))) & 0xffu);
            vv = (float)q * __uint_as_float(w[0]);
        }
    }
    k_out[idx] = kv;
    v_out[idx] = vv;
}

__global__ __launch_bounds__(kBlock) void table_scatter_kernel(int32_t* __restrict__ table,
                                                               const TableUpdate* __restrict__ upd,
                                                               int32_t n) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    // Updates are applied in order of their index only within one launch when offsets
    // are distinct; the host collapses repeated offsets before uploading.
    if (i < n) table[upd[i].offset] = upd[i].value;
}

// A handful of updates travel as kernel arguments: no upload, no ring slot.
struct TableUpdateArgs {
    TableUpdate u[kTableUpdatesInArgs];
};
__global__ __launch_bounds__(64) void table_scatter_args_kernel(int32_t* __restrict__ table, TableUpdateArgs a,
                                                               int32_t n) {
    const int i = threadIdx.x;
    if (i < n) table[a.u[i].offset] = a.u[i].value;
}

__global__ __launch_bounds__(kBlock) void fill_kernel(uint4* __restrict__ dst, uint64_t n_vec,
                                                      uint32_t word) {
    const uint4 w = make_uint4(word, word, word, word);
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n_vec;
         i += (uint64_t)gridDim.x * kBlock)
        dst[i] = w;
}

MoveGeom move_geom(const bkv_pool* p) {
    return MoveGeom{p->g.n_kv, p->g.hd, p->g.page_cells, p->desc.max_pages_per_seq};
}

PoolPtrs pool_ptrs(const bkv_pool* p) {
    PoolPtrs pp;
    pp.slab = p->slab;
    pp.layer_stride = p->g.k_pool_bytes + p->g.v_pool_bytes;
    pp.v_offset = p->g.k_pool_bytes;
    pp.k_page_bytes = p->g.k_page_bytes;
    pp.v_page_bytes = p->g.v_page_bytes;
    pp.n_layers = p->g.n_layers;
    return pp;
}

}  // namespace

template <typename SrcT>
static hipError_t launch_append_from(bkv_pool* p, int32_t layer, const AppendBatch& b,
                                     int32_t max_tok, const SrcT* k, const SrcT* v,
                                     hipStream_t stream) {
    const MoveGeom g = move_geom(p);
    uint8_t* kp = p->k_layer[(size_t)layer];
    uint8_t* vp = p->v_layer[(size_t)layer];
    const int32_t* tables = p->table_dev;
    if (p->g.layout == BKV_LAYOUT_F16) {
        const int64_t lanes = (int64_t)max_tok * (g.n_kv * g.hd / 8);
        dim3 grid((unsigned)((lanes + kBlock - 1) / kBlock), (unsigned)b.n);
        if (g.hd == 256)
            launch_staged(p, BKV_STAGE_APPEND, append_f16_kernel<SrcT, 256>, grid, dim3(kBlock), 0, stream, b, g,
                          (uint16_t*)kp, (uint16_t*)vp, tables, k, v);
        else
            launch_staged(p, BKV_STAGE_APPEND, append_f16_kernel<SrcT, 0>, grid, dim3(kBlock), 0, stream, b, g,
                          (uint16_t*)kp, (uint16_t*)vp, tables, k, v);
        return hipGetLastError();
    }
    const int rows_wg = kBlock / (g.hd / 8);
    const int64_t rows = (int64_t)max_tok * g.n_kv;
    dim3 grid((unsigned)((rows + rows_wg - 1) / rows_wg), (unsigned)b.n);
    if (p->g.layout == BKV_LAYOUT_I8H)  // pools of this layout have head dim 256
        launch_staged(p, BKV_STAGE_APPEND, append_quant_kernel<BKV_LAYOUT_I8H, SrcT, 256>, grid, dim3(kBlock), 0,
                      stream, b, g, kp, vp, tables, k, v);
    else if (g.hd == 256)
        launch_staged(p, BKV_STAGE_APPEND, append_quant_kernel<BKV_LAYOUT_Q8V, SrcT, 256>, grid, dim3(kBlock), 0,
                      stream, b, g, kp, vp, tables, k, v);
    else
        launch_staged(p, BKV_STAGE_APPEND, append_quant_kernel<BKV_LAYOUT_Q8V, SrcT, 0>, grid, dim3(kBlock), 0,
                      stream, b, g, kp, vp, tables, k, v);
    return hipGetLastError();
}

hipError_t launch_append(bkv_pool* p, int32_t layer, const AppendBatch& b, int32_t max_tok,
                         const void* k, const void* v, bool src_is_f16, hipStream_t stream) {
    if (src_is_f16)
        return launch_append_from(p, layer, b, max_tok, (const uint16_t*)k, (const uint16_t*)v, stream);
    return launch_append_from(p, layer, b, max_tok, (const float*)k, (const float*)v, stream);
}

hipError_t launch_append_kprep(bkv_pool* p, int32_t layer, const AppendBatch& b, int32_t max_tok,
                               const float* k, const float* v, const float* gamma, float eps,
                               const float* table, int32_t n_rot, int32_t max_pos,
                               const int32_t* positions, hipStream_t stream) {
    const MoveGeom g = move_geom(p);
    const KPrepParams kp{gamma, table, positions, eps, n_rot, max_pos};
    const int rows = max_tok * g.n_kv;
    dim3 grid((unsigned)((rows + kPrepRows - 1) / kPrepRows), (unsigned)b.n);
    const size_t lds = (size_t)kPrepRows * (g.hd + 4) * sizeof(float) +
                       kPrepRows * (sizeof(double) + sizeof(uint64_t) + sizeof(int32_t));
    uint8_t* kpl = p->k_layer[(size_t)layer];
    uint8_t* vpl = p->v_layer[(size_t)layer];
    const auto launch = [&](auto layout_tag, auto hd_tag) {
        launch_staged(p, BKV_STAGE_APPEND_KPREP, append_kprep_kernel<decltype(layout_tag)::value, decltype(hd_tag)::value>,
                      grid, dim3(kBlock), (uint32_t)lds, stream, b, g, kp, kpl, vpl, (const int32_t*)p->table_dev, k, v);
    };
    const auto by_hd = [&](auto layout_tag) {
        if (g.hd == 256)
            launch(layout_tag, std::integral_constant<int, 256>{});
        else
            launch(layout_tag, std::integral_constant<int, 0>{});
    };
    switch (p->g.layout) {
        case BKV_LAYOUT_F16:
            by_hd(std::integral_constant<int, BKV_LAYOUT_F16>{});
            break;
        case BKV_LAYOUT_Q8V:
            by_hd(std::integral_constant<int, BKV_LAYOUT_Q8V>{});
            break;
        default:
            by_hd(std::integral_constant<int, BKV_LAYOUT_I8H>{});
            break;
    }
    return hipGetLastError();
}

hipError_t launch_page_copy(bkv_pool* p, const bkv_page_pair* pairs_dev, int32_t n_pairs,
                            hipStream_t stream) {
    const PoolPtrs pp = pool_ptrs(p);
    const uint32_t chunks_k = (uint32_t)((pp.k_page_bytes / 16 + 4 * kBlock - 1) / (4 * kBlock));
    const uint32_t chunks_v = (uint32_t)((pp.v_page_bytes / 16 + 4 * kBlock - 1) / (4 * kBlock));
    const uint64_t total = (uint64_t)n_pairs * (uint64_t)pp.n_layers * (chunks_k + chunks_v);
    uint64_t grid = total;
    const uint64_t cap = (uint64_t)(p->n_cu > 0 ? p->n_cu : 256) * 32;
    if (grid > cap) grid = cap;
    launch_staged(p, BKV_STAGE_PAGE_COPY, page_copy_kernel, dim3((unsigned)grid), dim3(kBlock), 0, stream, pp,
                  pairs_dev, (uint32_t)n_pairs, chunks_k, chunks_v);
    return hipGetLastError();
}

hipError_t launch_page_stage(bkv_pool* p, const int32_t* pages_dev, int32_t n_pages,
                             uint8_t* stage, int to_stage, hipStream_t stream) {
    const PoolPtrs pp = pool_ptrs(p);
    const uint64_t pb = pp.k_page_bytes > pp.v_page_bytes ? pp.k_page_bytes : pp.v_page_bytes;
    const unsigned chunks = (unsigned)((pb / 16 + 4 * kBlock - 1) / (4 * kBlock));
    dim3 grid(chunks, (unsigned)n_pages * (unsigned)pp.n_layers * 2u);
    launch_staged(p, BKV_STAGE_PAGE_STAGE, page_stage_kernel, grid, dim3(kBlock), 0, stream, pp, pages_dev, stage, to_stage);
    return hipGetLastError();
}

hipError_t launch_gather(const bkv_pool* p, int32_t layer, int32_t row, int64_t cell0, int64_t n,
                         float* k_out, float* v_out, hipStream_t stream) {
    const MoveGeom g = move_geom(p);
    const int64_t total = n * g.n_kv * g.hd;
    if (total == 0) return hipSuccess;
    const unsigned grid = (unsigned)((total + kBlock - 1) / kBlock);
    gather_kernel<<<grid, kBlock, 0, stream>>>(
        g, p->g.layout, p->k_layer[(size_t)layer], p->v_layer[(size_t)layer],
        p->table_dev + (size_t)row * (size_t)p->desc.max_pages_per_seq, cell0, n, k_out, v_out);
    return hipGetLastError();
}

hipError_t launch_table_scatter(int32_t* table, const TableUpdate* upd_dev, int32_t n,
                                hipStream_t stream) {
    if (n == 0) return hipSuccess;
    table_scatter_kernel<<<(n + kBlock - 1) / kBlock, kBlock, 0, stream>>>(table, upd_dev, n);
    return hipGetLastError();
}

hipError_t launch_table_scatter_args(int32_t* table, const TableUpdate* upd_host, int32_t n, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    if (n > kTableUpdatesInArgs) return hipErrorInvalidValue;
    TableUpdateArgs a{};
    for (int i = 0; i < n; ++i) a.u[i] = upd_host[i];
    table_scatter_args_kernel<<<1, 64, 0, stream>>>(table, a, n);
    return hipGetLastError();
}

hipError_t launch_fill(void* dst, uint64_t bytes, uint32_t word, hipStream_t stream) {
    const uint64_t n_vec = bytes / 16;
    if (n_vec == 0) return hipSuccess;
    uint64_t blocks = (n_vec + kBlock - 1) / kBlock;
    if (blocks > 16384) blocks = 16384;
    fill_kernel<<<(unsigned)blocks, kBlock, 0, stream>>>((uint4*)dst, n_vec, word);
    return hipGetLastError();
}

}  // namespace bkv

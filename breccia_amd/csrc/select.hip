// Block selection for the sparse attention path on gfx950: the indexer score of every
// pooled block against a token's indexer queries, and the top-k over those scores that
// leaves the id list attention consumes.  Replaces the reference's qsa_idx_score.comp and
// its qsa_topk*.comp family (crates/breccia-kernels/src/qsa/mod.rs:1234-1376) and must
// emit exactly the list of the CPU path (qsa/cpu.rs:93-152): descending score, ties to
// the lower block, dead blocks never, the query's own block appended when missed.
//
// The list is only reproducible if the scores are: two blocks whose scores differ in the
// last bits must come out in the CPU's order.  The score kernel therefore computes what
// the CPU computes, operation for operation -- f64 products and sums in index order -- and
// the selection works on those f64 scores.  The work is tiny next to attention (a 32k
// context has 8192 blocks of 128 values).
//
// Top-k = one work-group per list: an 8-bit radix select finds the key of the k-th largest
// score, the survivors (at most k) are compacted in index order, sorted by a bitonic network
// in LDS and written out.  Everything is deterministic: no atomic decides an
// order (the histogram counts are order-independent).
#include <algorithm>

#include "bkv_internal.hpp"

namespace bkv {

namespace {

constexpr int kScoreTile = 64;    // blocks per work-group of the score kernel
constexpr int kScoreThreads = 256;
constexpr int kMaxIdxHead = 8;    // as shaders/qsa_idx_score.comp
constexpr int kMaxIdxDim = 128;

constexpr int kTopkThreads = 1024;
constexpr int kMaxTopk = 2048;    // candidates the sort network holds in LDS
constexpr int kHistCopies = 16;   // copies of the radix histogram (a power of two)
constexpr int kRankKeys = 256;    // keys of a radix bin that are ranked directly instead of split further
constexpr int kBuckets = kTopkThreads;  // buckets the selected keys are ordered through (one per thread)
constexpr int kBucketCap = 64;    // a fuller bucket sends the list to the sorting network instead

struct ScoreParams {
    SelectBatch b;
    const float* q;      // [n][idx_n_head][idx_dim]
    double* scores;      // [n][score_stride]
    int64_t score_stride;
    int32_t idx_n_head, idx_dim, idx_block;
};

// score[b] = (1/sqrt(idx_dim)) * sum_h relu(q_h . pooled_b), -inf for a block that starts
// after the query's position (qsa/cpu.rs:93-123).
// DIM = 128: the indexer's usual width as a compile-time constant, rows moved and read 16 bytes
// at a time (pooled and q must be 16-byte aligned); DIM = 0: any width, element by element (the
// index arithmetic of its loops divides by the run-time width).  The products and the sum keep
// the CPU's order in both.
template <int DIM>
__global__ __launch_bounds__(kScoreThreads) void idx_score_kernel(const ScoreParams P) {
    // rows DIM + 4 (16-byte aligned, 4 banks apart: 16-byte reads of 64 rows do not collide) or
    // D + 1 floats apart (odd: lanes walking one column of 64 rows hit 64 banks)
    __shared__ __attribute__((aligned(16))) float pooled_s[kScoreTile * (kMaxIdxDim + 4)];
    __shared__ __attribute__((aligned(16))) float q_s[kMaxIdxHead * kMaxIdxDim];
    __shared__ double part_s[kMaxIdxHead][kScoreTile];
    const int e = blockIdx.y;
    const int n_blocks = P.b.n_blocks[e];
    const int b0 = (int)blockIdx.x * kScoreTile;
    if (b0 >= n_blocks) return;
    const int nb = min(kScoreTile, n_blocks - b0);
    const int D = DIM ? DIM : P.idx_dim, H = P.idx_n_head;
    const int stride = DIM ? DIM + 4 : D + 1;
    const int tid = threadIdx.x;
    const float* pooled = P.b.pooled[e] + (size_t)b0 * D;
    if constexpr (DIM != 0) {
        constexpr int kRow4 = DIM / 4;
        for (int i = tid; i < nb * kRow4; i += kScoreThreads)
            *reinterpret_cast<float4*>(&pooled_s[(i / kRow4) * stride + (i % kRow4) * 4]) =
                reinterpret_cast<const float4*>(pooled)[i];
        for (int i = tid; i < H * kRow4; i += kScoreThreads)
            reinterpret_cast<float4*>(q_s)[i] = reinterpret_cast<const float4*>(P.q + (size_t)e * H * D)[i];
    } else {
        for (int i = tid; i < nb * D; i += kScoreThreads) pooled_s[(i / D) * stride + i % D] = pooled[i];
        for (int i = tid; i < H * D; i += kScoreThreads) q_s[i] = P.q[(size_t)e * H * D + i];
    }
    __syncthreads();

    const int b = tid % kScoreTile;
    if (b < nb) {
#pragma clang fp contract(off)
        const double scale = 1.0 / sqrt((double)D);
        for (int h = tid / kScoreTile; h < H; h += kScoreThreads / kScoreTile) {
            double dot = 0.0;
            if constexpr (DIM != 0) {
#pragma unroll 8
                for (int d = 0; d < DIM; d += 4) {
                    const float4 qv = *reinterpret_cast<const float4*>(&q_s[h * DIM + d]);
                    const float4 pv = *reinterpret_cast<const float4*>(&pooled_s[b * stride + d]);
                    dot += (double)qv.x * (double)pv.x;
                    dot += (double)qv.y * (double)pv.y;
                    dot += (double)qv.z * (double)pv.z;
                    dot += (double)qv.w * (double)pv.w;
                }
            } else {
                for (int d = 0; d < D; ++d) dot += (double)q_s[h * D + d] * (double)pooled_s[b * stride + d];
            }
            part_s[h][b] = (dot > 0.0 ? dot : 0.0) * scale;
        }
    }
    __syncthreads();
    if (tid < nb) {
#pragma clang fp contract(off)
        double acc = 0.0;
        for (int h = 0; h < H; ++h) acc += part_s[h][tid];
        const int64_t first_cell = (int64_t)(b0 + tid) * P.idx_block;
        P.scores[(size_t)e * P.score_stride + b0 + tid] =
            first_cell > (int64_t)P.b.pos[e] ? -INFINITY : acc;
    }
}

// ---- pooled indexer keys ---------------------------------------------------------------
// pooled[b] = rotary(rmsnorm(mean(raw[4b .. 4b+3])), position 4b) for every block the call
// completes (Qsa::idx_pool, qsa/mod.rs:1167-1207, shaders/qsa_idx_pool.comp; CPU path
// qsa/cpu.rs:154-185): rows of the block come from this call's raw keys or, for cells before
// pos0, from the rolling tail of the previous call.  Arithmetic as on the CPU: the mean adds
// raw/idx_block in f32 in cell order, the norm sums squares in f64 in element order, the
// rotary multiplies and adds in f64 without fusing -- so the pooled rows, and through them
// the selection, are the CPU's bit for bit.
struct PoolKeysParams {
    const float* raw;    // [tokens][idx_dim]
    const float* tail;   // [idx_block - 1][idx_dim]
    const float* gamma;  // [idx_dim]
    const float* table;  // [max_pos][n_rot / 2][2]
    float* pooled;       // [blocks][idx_dim]
    int32_t b0, n_new, pos0, tokens, idx_block, idx_dim, n_rot, max_pos;
    float eps;
};

__global__ __launch_bounds__(kMaxIdxDim) void idx_pool_kernel(const PoolKeysParams P) {
    __shared__ float val[kMaxIdxDim];
    __shared__ double inv_s;
    const int block = P.b0 + (int)blockIdx.x;
    const int d = threadIdx.x;
    if (d < P.idx_dim) {
        float mean = 0.0f;
        for (int k = 0; k < P.idx_block; ++k) {
            const int cell = block * P.idx_block + k;
            const int slot = cell - P.pos0;
            float v = 0.0f;
            if (slot >= 0 && slot < P.tokens)
                v = P.raw[(size_t)slot * P.idx_dim + d];
            else if (cell % P.idx_block + 1 < P.idx_block)
                v = P.tail[(size_t)(cell % P.idx_block) * P.idx_dim + d];
            mean += v / (float)P.idx_block;
        }
        val[d] = mean;
    }
    __syncthreads();
    if (d == 0) {
#pragma clang fp contract(off)
        double ss = 0.0;
        for (int i = 0; i < P.idx_dim; ++i) {
            const double x = (double)val[i];
            ss += x * x;
        }
        inv_s = 1.0 / sqrt(ss / (double)P.idx_dim + (double)P.eps);
    }
    __syncthreads();
    if (d < P.idx_dim) val[d] = (float)((double)val[d] * inv_s * (double)P.gamma[d]);
    __syncthreads();
    const int half = P.n_rot / 2;
    float out = d < P.idx_dim ? val[d] : 0.0f;
    if (d < P.n_rot) {
#pragma clang fp contract(off)
        const int j = d < half ? d : d - half;
        int64_t pos = (int64_t)block * P.idx_block;
        pos = pos > P.max_pos - 1 ? P.max_pos - 1 : pos;
        const double c = (double)P.table[((size_t)pos * half + j) * 2];
        const double sn = (double)P.table[((size_t)pos * half + j) * 2 + 1];
        const double a = (double)val[j], b = (double)val[j + half];
        const double ac = a * c, bs = b * sn, as = a * sn, bc = b * c;
        out = d < half ? (float)(ac - bs) : (float)(as + bc);
    }
    if (d < P.idx_dim) P.pooled[(size_t)block * P.idx_dim + d] = out;
}

// The rows of the last, incomplete block go to the rolling tail (Qsa::idx_tail,
// shaders/qsa_idx_tail.comp): slot = cell % idx_block, the last slot is never needed.
__global__ __launch_bounds__(256) void idx_tail_kernel(const float* __restrict__ raw, float* __restrict__ tail,
                                                       int32_t tokens, int32_t pos0, int32_t idx_dim,
                                                       int32_t idx_block) {
    const int i = (int)blockIdx.x * 256 + (int)threadIdx.x;
    if (i >= tokens * idx_dim) return;
    const int d = i % idx_dim, t = i / idx_dim;
    const int cell = pos0 + t, last_cell = pos0 + tokens - 1;
    const int slot = cell % idx_block;
    if (cell / idx_block == last_cell / idx_block && slot + 1 < idx_block)
        tail[(size_t)slot * idx_dim + d] = raw[i];
}

// ---- top-k ---------------------------------------------------------------------------
// Keys: unsigned integers that order like the scores.  A score is dead (never selected)
// unless it is finite and greater than -1e29: that covers NaN, the infinities (the CPU path
// keeps finite scores only, qsa/cpu.rs:139-143) and the reference shaders' own dead marker -1e30
// (shaders/qsa_topk.comp stops at the first best <= -1e29).  -0 is keyed as +0 so that equal
// scores stay equal.  Live keys are never 0.
__device__ __forceinline__ uint64_t score_key(double s) {
    if (!(s > -1.0e29 && s < INFINITY)) return 0;
    if (s == 0.0) s = 0.0;
    const uint64_t u = (uint64_t)__double_as_longlong(s);
    return (u >> 63) ? ~u : (u | 0x8000000000000000ull);
}
__device__ __forceinline__ uint64_t score_key(float s) {
    if (!(s > -1.0e29f && s < INFINITY)) return 0;
    if (s == 0.0f) s = 0.0f;
    const uint32_t u = __float_as_uint(s);
    const uint32_t k = (u >> 31) ? ~u : (u | 0x80000000u);
    return (uint64_t)k << 32;
}
// the score a live key stands for (-0 comes back as +0)
template <typename T>
__device__ __forceinline__ double key_score(uint64_t k);
template <>
__device__ __forceinline__ double key_score<double>(uint64_t k) {
    const uint64_t u = (k >> 63) ? (k ^ 0x8000000000000000ull) : ~k;
    return __longlong_as_double((long long)u);
}
template <>
__device__ __forceinline__ double key_score<float>(uint64_t k) {
    const uint32_t k32 = (uint32_t)(k >> 32);
    const uint32_t u = (k32 >> 31) ? (k32 ^ 0x80000000u) : ~k32;
    return (double)__uint_as_float(u);
}
template <typename T>
struct KeyBits;
template <>
struct KeyBits<double> {
    static constexpr int kLowShift = 0;
};
template <>
struct KeyBits<float> {
    static constexpr int kLowShift = 32;  // the low half of a float's key is zero
};

// Exclusive prefix sum of one int per thread over the work-group, in thread order.
__device__ __forceinline__ int block_exclusive_scan(int v, int* wave_sums, int* total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int t = __shfl_up(inc, off, 64);
        if (lane >= off) inc += t;
    }
    __syncthreads();  // wave_sums may still be read from the previous scan
    if (lane == 63) wave_sums[wave] = inc;
    __syncthreads();
    int before = 0, all = 0;
    for (int w = 0; w < kTopkThreads / 64; ++w) {
        const int s = wave_sums[w];
        if (w < wave) before += s;
        all += s;
    }
    *total = all;
    return before + inc - v;
}

struct TopkParams {
    SelectBatch b;
    const void* scores;   // [n][score_stride] of T
    int64_t score_stride;
    uint32_t* ids;        // [n][id_stride]
    int64_t id_stride;
    uint32_t* counts;     // [n]
    int32_t topk_blocks, max_ids, idx_block, dense;
};

// kRegKeys = keys a thread keeps in registers: 8 serves lists of up to 8192 blocks (a 32k
// context), 32 up to 32768 (128k); longer lists re-read their scores on every pass.
template <typename T, int kRegKeys>
__global__ __launch_bounds__(kTopkThreads) void topk_blocks_kernel(const TopkParams P) {
    // kHistCopies copies of the 256 bins, a lane adds to copy lane % kHistCopies: scores cluster in a
    // few bins of the first digit (its top bits are exponent bits), and LDS atomics of one wave on
    // one address run one after the other.  257 ints per copy put equal bins of different copies in
    // different banks.
    __shared__ int hist[kHistCopies][257];
    __shared__ int wave_sums[kTopkThreads / 64];
    __shared__ uint64_t cand_key[kMaxTopk + kBucketCap];  // the threshold slice may hold keys that are not kept
    __shared__ uint32_t cand_idx[kMaxTopk + kBucketCap];
    __shared__ uint64_t wave_min[kTopkThreads / 64], wave_max[kTopkThreads / 64];
    __shared__ uint64_t sh_prefix;
    __shared__ int sh_rem, sh_done, sh_cnt;
    __shared__ uint64_t small_key[kRankKeys + 4];
    __shared__ int small_n;
    __shared__ int sh_present, sh_crowded;
    __shared__ int sh_placed;  // keys of the slices at and above the threshold slice
    static_assert(3 * kBuckets <= kHistCopies * 257, "the bucket counters reuse the histogram");

    const int e = blockIdx.x;
    const int tid = threadIdx.x;
    const int N = P.b.n_blocks[e];
    const uint32_t own = (uint32_t)(P.b.pos[e] / P.idx_block);
    uint32_t* ids = P.ids + (size_t)e * P.id_stride;

    if (P.dense) {
        // every visible block in ascending order, unscored (shaders/qsa_topk.comp dense branch,
        // Qsa::topk_dense qsa/mod.rs:1363-1376)
        uint32_t n = min(min((uint32_t)N, own + 1u), (uint32_t)P.max_ids);
        for (uint32_t i = tid; i < n; i += kTopkThreads) ids[i] = i;
        if (tid == 0) {
            if (own >= (uint32_t)N && n < (uint32_t)P.max_ids) ids[n++] = own;
            P.counts[e] = n;
        }
        return;
    }

    const T* sc = reinterpret_cast<const T*>(P.scores) + (size_t)e * P.score_stride;
    if (tid == 0) sh_present = 0;  // read after the barriers of the scans below
    // thread t owns the contiguous index range [lo, hi): compaction keeps index order
    const int per = (N + kTopkThreads - 1) / kTopkThreads;
    const int lo = min(tid * per, N), hi = min(lo + per, N);
    const bool in_regs = per <= kRegKeys;
    uint64_t rk[kRegKeys];
#pragma unroll
    for (int u = 0; u < kRegKeys; ++u) rk[u] = in_regs && lo + u < hi ? score_key(sc[lo + u]) : 0;
    // f(index, key) for every element of this thread, in index order
    const auto for_keys = [&](auto f) {
        if (in_regs) {
#pragma unroll
            for (int u = 0; u < kRegKeys; ++u)
                if (lo + u < hi) f(lo + u, rk[u]);
        } else {
            for (int i = lo; i < hi; ++i) f(i, score_key(sc[i]));
        }
    };

    // live keys, the smallest and the largest of them: one sweep, one wave reduction each, one barrier
    int live = 0;
    uint64_t kmin = ~0ull, kmax = 0;
    for_keys([&](int, uint64_t k) {
        if (k != 0) {
            ++live;
            kmin = min(kmin, k);
            kmax = max(kmax, k);
        }
    });
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        live += __shfl_xor(live, off, 64);
        kmin = min(kmin, (uint64_t)__shfl_xor((unsigned long long)kmin, off, 64));
        kmax = max(kmax, (uint64_t)__shfl_xor((unsigned long long)kmax, off, 64));
    }
    if ((tid & 63) == 0) {
        wave_sums[tid >> 6] = live;
        wave_min[tid >> 6] = kmin;
        wave_max[tid >> 6] = kmax;
    }
    if (tid == 0) sh_done = 0;
    __syncthreads();
    int n_live = 0;
    for (int w = 0; w < kTopkThreads / 64; ++w) {
        n_live += wave_sums[w];
        kmin = min(kmin, wave_min[w]);
        kmax = max(kmax, wave_max[w]);
    }
    const int want = min(min(min(N, P.topk_blocks), n_live), P.max_ids);

    if (want > 0) {
        // ---- radix select: a threshold that exactly `want` live keys pass ------------------
        // All live keys agree on the bits above the highest bit in which the smallest and the
        // largest differ (for scores of similar magnitude that is sign, exponent and more), so
        // the digits start there: the first histogram is already well spread, and the LDS
        // atomics do not pile up on one bin.
        // ---- the usual case: one histogram over equal slices of the score range --------------------
        // Slice = floor((score - least) * kBuckets / (greatest - least)), which never decreases when the
        // score grows (a rounded difference, a rounded product and a truncation are all monotone) and is
        // the same for equal scores.  The counts are summed from the top slice down: the slice in which
        // the sum reaches `want` holds the threshold, every slice above it is selected whole, and a
        // slice's keys own a run of output places.  Every key of those slices is ranked against the
        // others of its slice -- greater keys first, equal keys in index order -- which is the place it
        // is written to; in the threshold slice only ranks below the number still wanted are written.
        // Selection, tie rule and order in one histogram and a handful of barriers.  Scores that crowd a
        // slice (many equal scores, an outlier that stretches the range, a range too narrow or too wide
        // to divide) take the general path below: a radix select on the keys' bits.
        bool done = false;
        {
            int* const bcount = &hist[0][0];
            int* const bfill = bcount + kBuckets;
            int* const bbase = bfill + kBuckets;
            const double least = key_score<T>(kmin);
            const double inv_w = (double)kBuckets / (key_score<T>(kmax) - least);
            if (kmin != kmax && inv_w > 0.0 && inv_w < 1.0e300) {
                const auto slice_of = [&](uint64_t k) {
                    return min(kBuckets - 1, (int)((key_score<T>(k) - least) * inv_w));
                };
                bcount[tid] = 0;
                bfill[tid] = 0;
                if (tid == 0) sh_crowded = 0;
                __syncthreads();
                for_keys([&](int, uint64_t k) {
                    if (k != 0) atomicAdd(&bcount[slice_of(k)], 1);
                });
                __syncthreads();
                const int sl_mine = kBuckets - 1 - tid;  // thread t sums from the top
                const int in_mine = bcount[sl_mine];
                int all;
                const int above = block_exclusive_scan(in_mine, wave_sums, &all);
                bbase[sl_mine] = above;
                if (above < want) {
                    if (in_mine > kBucketCap) sh_crowded = 1;
                    if (above + in_mine >= want) {  // the threshold slice: exactly one thread
                        sh_cnt = sl_mine;
                        sh_placed = above + in_mine;
                    }
                }
                __syncthreads();
                if (!sh_crowded) {
                    const int threshold_slice = sh_cnt;
                    const int placed = sh_placed;
                    for_keys([&](int i, uint64_t k) {
                        if (k != 0) {
                            const int b = slice_of(k);
                            if (b >= threshold_slice) {
                                const int slot = bbase[b] + atomicAdd(&bfill[b], 1);
                                cand_key[slot] = k;
                                cand_idx[slot] = (uint32_t)i;
                            }
                        }
                    });
                    __syncthreads();
                    bool mine = false;
                    for (int sl = tid; sl < placed; sl += kTopkThreads) {
                        const uint64_t k = cand_key[sl];
                        const uint32_t i = cand_idx[sl];
                        const int b = slice_of(k);
                        const int first = bbase[b], n = bcount[b];
                        int rank = first;
                        for (int j = 0; j < n; ++j) {
                            const uint64_t kj = cand_key[first + j];
                            const uint32_t ij = cand_idx[first + j];
                            rank += kj > k || (kj == k && ij < i);
                        }
                        if (rank < want) {
                            ids[rank] = i;
                            mine = mine || i == own;
                        }
                    }
                    if (mine) sh_present = 1;
                    done = true;
                }
            }
        }
        if (!done) {
        uint64_t kth = kmax;    // keys greater than kth are selected ...
        int ties_wanted = want; // ... and the first ties_wanted (by index) of those equal to it
        if (kmin != kmax) {
            int hi_bit = 63 - __builtin_clzll(kmin ^ kmax);
            if (tid == 0) {
                sh_prefix = hi_bit == 63 ? 0 : (kmax >> (hi_bit + 1)) << (hi_bit + 1);
                sh_rem = want;
            }
            bool resolved = false;  // became exact: every bit of the threshold key is known
            while (!resolved) {
                const int width = min(8, hi_bit - KeyBits<T>::kLowShift + 1);
                const int shift = hi_bit - width + 1;
                for (int i = tid; i < kHistCopies * 257; i += kTopkThreads) (&hist[0][0])[i] = 0;
                __syncthreads();
                const uint64_t prefix = sh_prefix;
                const int rem = sh_rem;
                for_keys([&](int, uint64_t k) {
                    const bool match = hi_bit == 63 || ((k ^ prefix) >> (hi_bit + 1)) == 0;
                    if (k != 0 && match)
                        atomicAdd(&hist[tid & (kHistCopies - 1)][(int)((k >> shift) & ((1u << width) - 1u))], 1);
                });
                __syncthreads();
                // The digit of the rem-th largest matching key: wave 0 walks the bins from the top,
                // lane l holding bins 255-4l .. 252-4l; the inclusive running count first reaches
                // rem in exactly one bin.
                if (tid < 64) {
                    int c[4], mine = 0;
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        c[u] = 0;
#pragma unroll
                        for (int cp = 0; cp < kHistCopies; ++cp) c[u] += hist[cp][255 - 4 * tid - u];
                        mine += c[u];
                    }
                    int inc = mine;
#pragma unroll
                    for (int off = 1; off < 64; off <<= 1) {
                        const int t = __shfl_up(inc, off, 64);
                        if (tid >= off) inc += t;
                    }
                    int above = inc - mine;
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if (above < rem && above + c[u] >= rem) {
                            sh_rem = rem - above;
                            sh_prefix = prefix | ((uint64_t)(255 - 4 * tid - u) << shift);
                            sh_done = above + c[u] == rem;  // the whole bin is wanted
                            sh_cnt = c[u];
                        }
                        above += c[u];
                    }
                }
                __syncthreads();
                hi_bit = shift - 1;
                resolved = hi_bit < KeyBits<T>::kLowShift;
                if (sh_done) break;
                if (!resolved && sh_cnt <= kRankKeys) {
                    // Few keys are left in the chosen bin (after one pass over a few thousand spread
                    // scores, a few dozen): they are listed, every thread ranks one of them against
                    // the others, and the one that rem of them reach is the threshold -- instead of
                    // six more passes over the remaining bits.  The list's order is whatever the
                    // atomics made it; the threshold's value does not depend on it.
                    if (tid == 0) small_n = 0;
                    if (tid < kRankKeys + 4) small_key[tid] = 0;
                    __syncthreads();
                    const uint64_t chosen = sh_prefix;
                    const int left = sh_rem;
                    for_keys([&](int, uint64_t k) {
                        if (k != 0 && ((k ^ chosen) >> shift) == 0) small_key[atomicAdd(&small_n, 1)] = k;
                    });
                    __syncthreads();
                    const int c = small_n;
                    if (tid < c) {
                        const uint64_t mine = small_key[tid];
                        int greater = 0, equal = 0;
                        // four independent reads at a time (the list is padded with zeros, which
                        // rank below every live key)
                        for (int i = 0; i < c; i += 4) {
                            const uint64_t o0 = small_key[i], o1 = small_key[i + 1];
                            const uint64_t o2 = small_key[i + 2], o3 = small_key[i + 3];
                            greater += (o0 > mine) + (o1 > mine) + (o2 > mine) + (o3 > mine);
                            equal += (o0 == mine) + (o1 == mine) + (o2 == mine) + (o3 == mine);
                        }
                        // equal keys all write the same pair
                        if (greater < left && left <= greater + equal) {
                            sh_prefix = mine;
                            sh_rem = left - greater;
                        }
                    }
                    __syncthreads();
                    resolved = true;
                    break;
                }
            }
            if (resolved && !sh_done) {
                kth = sh_prefix;
                ties_wanted = sh_rem;
            } else {
                // every key at or above the chosen bin's lowest value is selected
                const uint64_t floor_key = sh_prefix;
                kth = floor_key == 0 ? 0 : floor_key - 1;
                ties_wanted = 0;
            }
        }

        // ---- order: descending key, ascending index among equal keys -------------------------
        int ties = 0, greater = 0;
        for_keys([&](int, uint64_t k) {
            ties += k == kth;
            greater += k > kth;
        });
        int total;
        const int ties_before = block_exclusive_scan(ties, wave_sums, &total);
        // The keys equal to the threshold are the smallest selected ones and go last, in index order:
        // their places follow from the scan above.  The n_g keys above the threshold are ordered through
        // buckets: kBuckets equal slices of the key range (kth, kmax], counted, the counts summed from the
        // top -- a bucket's keys then own a run of output places -- and every key ranked against the few
        // others of its bucket.  A handful of barriers instead of a sorting network's stages.  Key ranges
        // that crowd one bucket (an outlier far above the rest, many equal scores, a selection that spans
        // both signs) go through the network below.
        const int n_g = want - ties_wanted;
        bool ordered = false;
        {
            int* const bcount = &hist[0][0];
            int* const bfill = bcount + kBuckets;
            int* const bbase = bfill + kBuckets;
            int sh = 0;
            if (n_g > 0) {
                const uint64_t span = kmax - kth - 1;  // some key lies above kth, so kmax does
                const int bits = span ? 64 - __builtin_clzll(span) : 0;
                sh = bits > 10 ? bits - 10 : 0;
            }
            const auto bucket_of = [&](uint64_t k) { return (int)((k - kth - 1) >> sh); };
            bcount[tid] = 0;
            bfill[tid] = 0;
            if (tid == 0) sh_crowded = 0;
            __syncthreads();
            for_keys([&](int, uint64_t k) {
                if (k > kth) atomicAdd(&bcount[bucket_of(k)], 1);
            });
            __syncthreads();
            const int in_mine = bcount[kBuckets - 1 - tid];  // thread t sums from the top: bucket kBuckets - 1 - t
            if (in_mine > kBucketCap) sh_crowded = 1;
            int placed;
            bbase[kBuckets - 1 - tid] = block_exclusive_scan(in_mine, wave_sums, &placed);
            __syncthreads();
            if (!sh_crowded) {
                for_keys([&](int i, uint64_t k) {
                    if (k > kth) {
                        const int b = bucket_of(k);
                        const int slot = bbase[b] + atomicAdd(&bfill[b], 1);
                        cand_key[slot] = k;
                        cand_idx[slot] = (uint32_t)i;
                    }
                });
                __syncthreads();
                bool mine = false;
                for (int sl = tid; sl < n_g; sl += kTopkThreads) {
                    const uint64_t k = cand_key[sl];
                    const uint32_t i = cand_idx[sl];
                    const int b = bucket_of(k);
                    const int first = bbase[b], n = bcount[b];
                    int rank = 0;
                    for (int j = 0; j < n; ++j) {
                        const uint64_t kj = cand_key[first + j];
                        const uint32_t ij = cand_idx[first + j];
                        rank += kj > k || (kj == k && ij < i);
                    }
                    ids[first + rank] = i;
                    mine = mine || i == own;
                }
                int tie_rank = ties_before;
                for_keys([&](int i, uint64_t k) {
                    if (k == kth) {
                        if (tie_rank < ties_wanted) {
                            ids[n_g + tie_rank] = (uint32_t)i;
                            mine = mine || (uint32_t)i == own;
                        }
                        ++tie_rank;
                    }
                });
                if (mine) sh_present = 1;
                ordered = true;
            }
        }
        if (!ordered) {
        // ---- compaction in index order, then a sorting network ---------------------------------
        const int take = max(0, min(ties, ties_wanted - ties_before));
        int at = block_exclusive_scan(greater + take, wave_sums, &total);
        int tie_rank = ties_before;
        for_keys([&](int i, uint64_t k) {
            bool keep = k > kth;
            if (k == kth) keep = tie_rank++ < ties_wanted;
            if (keep) {
                cand_key[at] = k;
                cand_idx[at] = (uint32_t)i;
                ++at;
            }
        });
        __syncthreads();

        // ---- order: descending key, ascending index among equal keys -------------------------
        // Bitonic network over the candidates padded to a power of two.  A wave owns a chunk of
        // 128 elements: every stage whose partner distance stays inside a chunk needs no
        // work-group barrier (a wave's LDS operations execute in order), so a 512-entry list
        // costs 3 barriers for its 45 stages.
        int padded = 1;
        while (padded < want) padded <<= 1;
        for (int i = want + tid; i < padded; i += kTopkThreads) {
            cand_key[i] = 0;
            cand_idx[i] = 0xffffffffu;
        }
        __syncthreads();
        if (padded <= kTopkThreads) {
            // One candidate per thread, kept in registers: partners less than a wave apart swap
            // through lane shuffles, the others through LDS.  Same network, same order.
            uint64_t key = tid < padded ? cand_key[tid] : 0;
            uint32_t idx = tid < padded ? cand_idx[tid] : 0xffffffffu;
            for (int k2 = 2; k2 <= padded; k2 <<= 1) {
                for (int j2 = k2 >> 1; j2 > 0; j2 >>= 1) {
                    uint64_t pkey;
                    uint32_t pidx;
                    if (j2 < 64) {
                        pkey = (uint64_t)__shfl_xor((unsigned long long)key, j2, 64);
                        pidx = (uint32_t)__shfl_xor((int)idx, j2, 64);
                    } else {
                        __syncthreads();  // the partners of the previous LDS stage have read
                        if (tid < padded) {
                            cand_key[tid] = key;
                            cand_idx[tid] = idx;
                        }
                        __syncthreads();
                        pkey = tid < padded ? cand_key[tid ^ j2] : 0;
                        pidx = tid < padded ? cand_idx[tid ^ j2] : 0xffffffffu;
                    }
                    // a run is in order (first to last) when its k2 bit is clear, reversed otherwise;
                    // the lower position of a pair keeps the element that comes first in the run's order
                    const bool in_order = (tid & k2) == 0;
                    const bool low = (tid & j2) == 0;
                    const bool mine_first = key > pkey || (key == pkey && idx < pidx);
                    if (mine_first != (low == in_order)) {
                        key = pkey;
                        idx = pidx;
                    }
                }
            }
            __syncthreads();
            if (tid < padded) cand_idx[tid] = idx;
        } else {
        const auto exchange = [&](int a, int b, bool reversed_run) {
            const uint64_t ka = cand_key[a], kb = cand_key[b];
            const uint32_t ia = cand_idx[a], ib = cand_idx[b];
            const bool a_first = ka > kb || (ka == kb && ia < ib);
            if (a_first == reversed_run) {
                cand_key[a] = kb, cand_key[b] = ka;
                cand_idx[a] = ib, cand_idx[b] = ia;
            }
        };
        const int wave = tid >> 6, lane = tid & 63;
        for (int k2 = 2; k2 <= padded; k2 <<= 1) {
            for (int j2 = k2 >> 1; j2 > 0; j2 >>= 1) {
                if (j2 >= 128) {
                    __syncthreads();
                    for (int t = tid; t < padded / 2; t += kTopkThreads) {
                        const int a = (t / j2) * 2 * j2 + t % j2;
                        exchange(a, a + j2, (a & k2) != 0);
                    }
                    __syncthreads();
                } else {
                    const int a = wave * 128 + (lane / j2) * 2 * j2 + lane % j2;
                    if (a + j2 < padded) exchange(a, a + j2, (a & k2) != 0);
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                }
            }
        }
        }
        __syncthreads();
        bool mine = false;
        for (int i = tid; i < want; i += kTopkThreads) {
            const uint32_t id = cand_idx[i];
            ids[i] = id;
            mine = mine || id == own;
        }
        if (mine) sh_present = 1;
        }
        }
    }

    // ---- the query's own block when the selection missed it ------------------------------------
    __syncthreads();
    if (tid == 0) {
        uint32_t count = (uint32_t)want;
        if (!sh_present && count < (uint32_t)P.max_ids) ids[count++] = own;
        P.counts[e] = count;
    }
}

}  // namespace

hipError_t launch_idx_score(bkv_pool* p, const SelectBatch& b, const float* q, int32_t idx_n_head, int32_t idx_dim,
                            int32_t idx_block, double* scores, int64_t score_stride, int32_t max_blocks,
                            hipStream_t stream) {
    ScoreParams sp;
    sp.b = b;
    sp.q = q;
    sp.scores = scores;
    sp.score_stride = score_stride;
    sp.idx_n_head = idx_n_head;
    sp.idx_dim = idx_dim;
    sp.idx_block = idx_block;
    dim3 grid((unsigned)((max_blocks + kScoreTile - 1) / kScoreTile), (unsigned)b.n);
    bool wide = idx_dim == 128 && (reinterpret_cast<uintptr_t>(q) & 15u) == 0;
    for (int i = 0; i < b.n && wide; ++i) wide = (reinterpret_cast<uintptr_t>(b.pooled[i]) & 15u) == 0;
    if (wide)
        launch_staged(p, BKV_STAGE_IDX_SCORE, idx_score_kernel<128>, grid, dim3(kScoreThreads), 0, stream, sp);
    else
        launch_staged(p, BKV_STAGE_IDX_SCORE, idx_score_kernel<0>, grid, dim3(kScoreThreads), 0, stream, sp);
    return hipGetLastError();
}

hipError_t launch_topk_blocks(bkv_pool* p, const SelectBatch& b, const void* scores, bool scores_f64,
                              int64_t score_stride, int32_t topk_blocks, int32_t idx_block, bool dense,
                              uint32_t* ids, int64_t id_stride, uint32_t* counts, int32_t max_ids,
                              hipStream_t stream) {
    TopkParams tp;
    tp.b = b;
    tp.scores = scores;
    tp.score_stride = score_stride;
    tp.ids = ids;
    tp.id_stride = id_stride;
    tp.counts = counts;
    tp.topk_blocks = topk_blocks;
    tp.max_ids = max_ids;
    tp.idx_block = idx_block;
    tp.dense = dense ? 1 : 0;
    int32_t longest = 0;
    for (int i = 0; i < b.n; ++i) longest = std::max(longest, b.n_blocks[i]);
    const bool few = longest <= 8 * kTopkThreads;
    if (scores_f64) {
        if (few)
            launch_staged(p, BKV_STAGE_TOPK, topk_blocks_kernel<double, 8>, dim3((unsigned)b.n), dim3(kTopkThreads), 0, stream, tp);
        else
            launch_staged(p, BKV_STAGE_TOPK, topk_blocks_kernel<double, 32>, dim3((unsigned)b.n), dim3(kTopkThreads), 0, stream, tp);
    } else {
        if (few)
            launch_staged(p, BKV_STAGE_TOPK, topk_blocks_kernel<float, 8>, dim3((unsigned)b.n), dim3(kTopkThreads), 0, stream, tp);
        else
            launch_staged(p, BKV_STAGE_TOPK, topk_blocks_kernel<float, 32>, dim3((unsigned)b.n), dim3(kTopkThreads), 0, stream, tp);
    }
    return hipGetLastError();
}

hipError_t launch_idx_pool(bkv_pool* p, const float* raw, float* tail, const float* gamma, const float* table,
                           float* pooled, int32_t pos0, int32_t tokens, int32_t idx_dim, int32_t idx_block,
                           int32_t n_rot, int32_t max_pos, float eps, hipStream_t stream) {
    PoolKeysParams pp;
    pp.raw = raw;
    pp.tail = tail;
    pp.gamma = gamma;
    pp.table = table;
    pp.pooled = pooled;
    pp.b0 = pos0 / idx_block;
    pp.n_new = (pos0 + tokens) / idx_block - pp.b0;
    pp.pos0 = pos0;
    pp.tokens = tokens;
    pp.idx_block = idx_block;
    pp.idx_dim = idx_dim;
    pp.n_rot = n_rot;
    pp.max_pos = max_pos;
    pp.eps = eps;
    if (pp.n_new > 0) {
        launch_staged(p, BKV_STAGE_IDX_POOL, idx_pool_kernel, dim3((unsigned)pp.n_new), dim3(kMaxIdxDim), 0, stream, pp);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    // the tail is read by the pooling above and rewritten here: stream order keeps them apart
    const int total = tokens * idx_dim;
    launch_staged(p, BKV_STAGE_IDX_POOL, idx_tail_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, raw, tail, tokens, pos0,
                  idx_dim, idx_block);
    return hipGetLastError();
}

int32_t select_max_topk() { return kMaxTopk; }
int32_t select_max_idx_head() { return kMaxIdxHead; }
int32_t select_max_idx_dim() { return kMaxIdxDim; }

}  // namespace bkv

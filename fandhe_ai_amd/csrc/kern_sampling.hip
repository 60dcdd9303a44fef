// Next-token sampling on the device: temperature / top-k softmax weights and one multinomial draw per row,
// with the reference's host arithmetic (crates/autodiff/src/generate/mod.rs:347-369, 432-452;
// crates/tensor-core/src/rng.rs:65-104, 509-539): weights (f32) = f64 exp((logit - max) / t) / f64 sum,
// top-k keeps the k largest by (value descending, index ascending), the draw is the first index whose f64
// cumulative weight exceeds u * total, u the next 53-bit uniform of an xorshift64* generator whose state
// lives on the device; rows draw in row order from the one generator.  Only the order of the f64 sums
// differs from the host loop (a block-wide tree instead of a sequential pass).
// With a policy table every row has a strategy, temperature, k and generator of its own (one request per
// row, each drawing from the generator its own seed started: crates/autodiff/src/generate/scheduler.rs:
// 176-211, 553-562); a greedy row takes the first maximum and draws nothing.
#include "device_utils.hpp"
#include "kernels.hpp"

namespace fa {
namespace k {
using namespace fa::dev;

namespace {

constexpr int kThreads = 1024;

__device__ __forceinline__ uint64_t xorshift64star_next(uint64_t &state) {
    uint64_t x = state;
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    state = x;
    return x * 0x2545F4914F6CDD1Dull;
}

// larger float <-> larger key (finite values)
__device__ __forceinline__ uint32_t order_key(float v) {
    uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// exclusive prefix sums of one value per thread over the block; returns the block total through *total
template <typename T>
__device__ __forceinline__ T block_exclusive_scan(T v, T *buf, T *total) {
    const int t = threadIdx.x;
    buf[t] = v;
    __syncthreads();
    for (int off = 1; off < kThreads; off <<= 1) {
        T add = t >= off ? buf[t - off] : (T)0;
        __syncthreads();
        buf[t] += add;
        __syncthreads();
    }
    T incl = buf[t];
    *total = buf[kThreads - 1];
    __syncthreads();
    return incl - v;
}

// WEIGHTS: the draw is left out and the row's f32 sampling weights are stored instead (one-hot at the first
// maximum for a greedy row; NaN throughout, and status 1, when a logit is not finite).
template <bool WEIGHTS>
__global__ void __launch_bounds__(kThreads)
    sample_rows_kernel(const float *__restrict__ logits, int32_t *__restrict__ tokens, const uint64_t *__restrict__ rng_state,
                       RowPolicy *__restrict__ policy, uint32_t vocab, int top_k_mode, float temperature, uint32_t top_k,
                       float *__restrict__ weights_out, int32_t *__restrict__ status, int greedy_weights) {
    __shared__ double s_d[kThreads];
    __shared__ uint32_t s_u[kThreads];
    __shared__ uint32_t hist[256];
    __shared__ float s_max[kThreads / 64];
    __shared__ uint32_t s_sel[4];            // radix-select state: prefix, remaining; flags
    __shared__ double s_x;
    const uint32_t b = blockIdx.x, t = threadIdx.x;
    const float *row = logits + (uint64_t)b * vocab;
    bool greedy = WEIGHTS && greedy_weights != 0;
    float *wrow = WEIGHTS ? weights_out + (uint64_t)b * vocab : nullptr;
    if (policy) {                                        // uniform over the block
        const RowPolicy pr = policy[b];
        greedy = pr.strategy == 0;
        top_k_mode = pr.strategy == 2;
        temperature = pr.temperature;
        top_k = pr.top_k < vocab ? pr.top_k : vocab;
    }
    const uint32_t seg = (vocab + kThreads - 1) / kThreads;
    const uint32_t lo = t * seg < vocab ? t * seg : vocab, hi = lo + seg < vocab ? lo + seg : vocab;

    // ---- every logit finite (the reference rejects the step otherwise); row maximum
    float mx = -INFINITY;
    bool finite = true;
    for (uint32_t i = lo; i < hi; ++i) {
        float v = row[i];
        finite = finite && (fabsf(v) <= 3.402823466e38f);            // false for NaN and +-inf
        mx = fmaxf(mx, v);
    }
    if (t < 4) s_sel[t] = 0;
    __syncthreads();
    if (!finite) atomicOr(&s_sel[2], 1u);
    mx = wave_max(mx);
    if (t % 64 == 0) s_max[t / 64] = mx;
    __syncthreads();
    if (s_sel[2]) {
        if constexpr (WEIGHTS) {
            for (uint32_t i = lo; i < hi; ++i) wrow[i] = __uint_as_float(0x7fc00000u);
            if (t == 0) status[b] = 1;
        } else {
            if (t == 0) tokens[b] = -1;
        }
        return;
    }
    if (WEIGHTS && t == 0) status[b] = 0;
    mx = s_max[0];
    for (int w = 1; w < kThreads / 64; ++w) mx = fmaxf(mx, s_max[w]);
    if (greedy) {                                        // first index holding the maximum
        if (t == 0) s_sel[0] = 0xffffffffu;
        __syncthreads();
        for (uint32_t i = lo; i < hi; ++i)
            if (row[i] == mx) {
                atomicMin(&s_sel[0], i);
                break;
            }
        __syncthreads();
        if constexpr (WEIGHTS) {
            for (uint32_t i = lo; i < hi; ++i) wrow[i] = i == s_sel[0] ? 1.0f : 0.0f;
        } else {
            if (t == 0) tokens[b] = (int32_t)s_sel[0];
        }
        return;
    }
    const double dmax = (double)mx, dt = (double)temperature;

    // ---- top-k: key of the k-th largest value and how many elements with that key are kept (lowest indices)
    uint32_t thr_key = 0, keep_equal = 0xffffffffu, eq_rank = 0;
    if (top_k_mode) {
        uint32_t prefix = 0, mask = 0, remaining = top_k;
        for (int pass = 0; pass < 4; ++pass) {
            const int shift = 24 - 8 * pass;
            if (t < 256) hist[t] = 0;
            __syncthreads();
            for (uint32_t i = lo; i < hi; ++i) {
                uint32_t key = order_key(row[i]);
                if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
            }
            __syncthreads();
            if (t == 0) {
                uint32_t cum = 0, bin = 255;
                for (;; --bin) {
                    if (cum + hist[bin] >= remaining || bin == 0) break;
                    cum += hist[bin];
                }
                s_sel[0] = prefix | (bin << shift);
                s_sel[1] = remaining - cum;
            }
            __syncthreads();
            prefix = s_sel[0];
            remaining = s_sel[1];
            mask |= 255u << shift;
            __syncthreads();
        }
        thr_key = prefix;
        keep_equal = remaining;
        uint32_t eq = 0;
        for (uint32_t i = lo; i < hi; ++i) eq += order_key(row[i]) == thr_key ? 1u : 0u;
        uint32_t eq_total;
        eq_rank = block_exclusive_scan<uint32_t>(eq, s_u, &eq_total);
    }
    // kept(i): walks the segment in index order with a running rank among the elements equal to the threshold
    auto for_each_kept = [&](auto &&f) {
        uint32_t rank = eq_rank;
        for (uint32_t i = lo; i < hi; ++i) {
            const float v = row[i];
            bool kept = true;
            if (top_k_mode) {
                const uint32_t key = order_key(v);
                if (key == thr_key) {
                    kept = rank < keep_equal;
                    ++rank;
                } else {
                    kept = key > thr_key;
                }
            }
            f(i, v, kept);
        }
    };

    // ---- f64 sum of the exponentials of the kept logits
    double part = 0.0;
    for_each_kept([&](uint32_t, float v, bool kept) {
        if (kept) part += exp(((double)v - dmax) / dt);
    });
    double sum_exp;
    (void)block_exclusive_scan<double>(part, s_d, &sum_exp);

    // ---- f32 weights, their f64 cumulative sums, and the draw
    auto weight = [&](float v, bool kept) -> float { return kept ? (float)(exp(((double)v - dmax) / dt) / sum_exp) : 0.0f; };
    if constexpr (WEIGHTS) {
        for_each_kept([&](uint32_t i, float v, bool kept) { wrow[i] = weight(v, kept); });
        return;
    }
    double wsum = 0.0;
    uint32_t last_pos = 0;
    bool any_pos = false;
    for_each_kept([&](uint32_t i, float v, bool kept) {
        const float w = weight(v, kept);
        wsum += (double)w;
        if (w > 0.0f) {
            last_pos = i;
            any_pos = true;
        }
    });
    double total;
    const double before = block_exclusive_scan<double>(wsum, s_d, &total);
    if (t == 0) {
        uint64_t bits = 0;
        if (policy) {                            // the row's own generator: one draw, state kept for the next step
            uint64_t st = policy[b].rng_state;
            bits = xorshift64star_next(st);
            policy[b].rng_state = st;
        } else {
            uint64_t st = rng_state[0];
            for (uint32_t r = 0; r <= b; ++r) bits = xorshift64star_next(st);     // row b takes the (b + 1)-th draw of the step
        }
        s_x = (double)(bits >> 11) / 9007199254740992.0 * total;
        s_sel[0] = 0xffffffffu;                 // first index whose cumulative weight exceeds x
        s_sel[1] = 0;                           // last index with a positive weight (+ 1)
    }
    __syncthreads();
    const double x = s_x;
    if (any_pos) atomicMax(&s_sel[1], last_pos + 1);
    {
        // Every thread looks for the first positive-weight element of its segment whose cumulative weight
        // exceeds x and the block keeps the smallest such index: in a segment past the crossing that is its
        // first positive element, which loses against the true crossing further left, and the rounding of
        // the scanned offsets against the running sums cannot leave x between two segments unnoticed.
        double acc = before;
        uint32_t found = 0xffffffffu;
        for_each_kept([&](uint32_t i, float v, bool kept) {
            const float w = weight(v, kept);
            acc += (double)w;
            if (found == 0xffffffffu && w > 0.0f && acc > x) found = i;
        });
        if (found != 0xffffffffu) atomicMin(&s_sel[0], found);
    }
    __syncthreads();
    if (t == 0) {
        uint32_t idx = s_sel[0];
        if (idx == 0xffffffffu) idx = s_sel[1] ? s_sel[1] - 1 : vocab - 1;
        tokens[b] = (int32_t)idx;
    }
}

// exclusive prefix sums of one value per thread over the block (wavefront scan, then the wavefront totals
// through LDS); *total receives the block total.  buf: one slot per wavefront.
template <typename T>
__device__ __forceinline__ T block_exclusive_scan_fast(T v, T *buf, T *total) {
    const int lane = threadIdx.x % 64, w = threadIdx.x / 64;
    T sc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const T up = __shfl_up(sc, off);
        if (lane >= off) sc += up;
    }
    __syncthreads();                                      // buf may still be read by an earlier scan
    if (lane == 63) buf[w] = sc;
    __syncthreads();
    T before = (T)0, all = (T)0;
    for (int i = 0; i < kThreads / 64; ++i) {
        if (i == w) before = all;
        all += buf[i];
    }
    *total = all;
    return before + sc - v;
}

// The same sampler for rows of at most 1024 * SEG logits, with the row held in registers: thread t owns the
// SEG consecutive logits from t * SEG on, loads them once (16 bytes at a time where the row's alignment
// allows) and keeps first the logits, then their f64 exponentials, then the f32 weights in registers, so the
// row is read from memory once and every exponential is taken once.  What depends on the index order (which
// of several logits equal to the k-th largest are kept; the cumulative weights of the draw) goes through one
// scan of per-thread totals each.
template <int SEG>
__global__ void __launch_bounds__(kThreads)
    sample_rows_reg_kernel(const float *__restrict__ logits, int32_t *__restrict__ tokens, const uint64_t *__restrict__ rng_state,
                           RowPolicy *__restrict__ policy, uint32_t vocab, int top_k_mode, float temperature, uint32_t top_k) {
    constexpr int kW = kThreads / 64;
    __shared__ double s_d[kW];
    __shared__ uint32_t s_u[kW];
    __shared__ uint32_t hist[256];
    __shared__ float s_max[kW];
    __shared__ uint32_t s_sel[4];
    __shared__ double s_x;
    const uint32_t b = blockIdx.x, t = threadIdx.x, lane = t % 64, w = t / 64;
    const float *row = logits + (uint64_t)b * vocab;
    const uint32_t base = t * SEG;
    bool greedy = false;
    if (policy) {
        const RowPolicy pr = policy[b];
        greedy = pr.strategy == 0;
        top_k_mode = pr.strategy == 2;
        temperature = pr.temperature;
        top_k = pr.top_k < vocab ? pr.top_k : vocab;
    }
    float v[SEG];
    const uint32_t n_own = base >= vocab ? 0u : (vocab - base < (uint32_t)SEG ? vocab - base : (uint32_t)SEG);
    if (vocab % 4 == 0) {                                 // every row starts on a 16-byte boundary, and so does base
#pragma unroll
        for (int q = 0; q < SEG / 4; ++q) {
            float4 x4 = float4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
            if (base + 4 * q < vocab) x4 = *(const float4 *)(row + base + 4 * q);
            v[4 * q] = x4.x;
            v[4 * q + 1] = x4.y;
            v[4 * q + 2] = x4.z;
            v[4 * q + 3] = x4.w;
        }
    } else {
#pragma unroll
        for (int j = 0; j < SEG; ++j) v[j] = (uint32_t)j < n_own ? row[base + j] : -INFINITY;
    }
    float mx = -INFINITY;
    bool finite = true;
#pragma unroll
    for (int j = 0; j < SEG; ++j)
        if ((uint32_t)j < n_own) {
            finite = finite && (fabsf(v[j]) <= 3.402823466e38f);
            mx = fmaxf(mx, v[j]);
        }
    if (t < 4) s_sel[t] = t == 0 ? 0xffffffffu : 0u;      // [0] smallest index found, [1] last positive + 1, [2] not finite
    __syncthreads();
    if (!finite) atomicOr(&s_sel[2], 1u);
    mx = wave_max(mx);
    if (lane == 0) s_max[w] = mx;
    __syncthreads();
    if (s_sel[2]) {
        if (t == 0) tokens[b] = -1;
        return;
    }
    mx = s_max[0];
#pragma unroll
    for (int i = 1; i < kW; ++i) mx = fmaxf(mx, s_max[i]);
    if (greedy) {                                         // first index holding the maximum
        uint32_t first = 0xffffffffu;
#pragma unroll
        for (int j = SEG - 1; j >= 0; --j)
            if ((uint32_t)j < n_own && v[j] == mx) first = base + j;
        if (first != 0xffffffffu) atomicMin(&s_sel[0], first);
        __syncthreads();
        if (t == 0) tokens[b] = (int32_t)s_sel[0];
        return;
    }
    const double dmax = (double)mx, dt = (double)temperature;

    uint32_t kept = n_own >= 32 ? 0xffffffffu : (1u << n_own) - 1u;      // bit j: logit j of this thread takes part
    if (top_k_mode) {
        uint32_t prefix = 0, mask = 0, remaining = top_k;
        for (int pass = 0; pass < 4; ++pass) {
            const int shift = 24 - 8 * pass;
            if (t < 256) hist[t] = 0;
            __syncthreads();
#pragma unroll
            for (int j = 0; j < SEG; ++j) {
                const uint32_t key = order_key(v[j]);
                if ((uint32_t)j < n_own && (key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
            }
            __syncthreads();
            {
                // the highest bin whose count together with all higher bins reaches `remaining`: suffix sums of
                // the 256 bins over four wavefronts (a one-thread walk down the bins costs more than the pass)
                const uint32_t c = t < 256 ? hist[t] : 0u;
                uint32_t sfx = c;
#pragma unroll
                for (int off = 1; off < 64; off <<= 1) {
                    const uint32_t dn = __shfl_down(sfx, off);
                    if ((int)lane + off < 64) sfx += dn;
                }
                if (t < 256 && lane == 0) s_u[w] = sfx;
                __syncthreads();
                if (t < 256) {
                    for (uint32_t i = w + 1; i < 4; ++i) sfx += s_u[i];
                    const uint32_t above = sfx - c;               // count in the bins above this one
                    if ((sfx >= remaining && above < remaining) || (t == 0 && sfx < remaining)) {
                        s_sel[1] = prefix | (t << shift);
                        s_sel[3] = remaining - above;
                    }
                }
            }
            __syncthreads();
            prefix = s_sel[1];
            remaining = s_sel[3];
            mask |= 255u << shift;
            __syncthreads();
        }
        if (t == 0) s_sel[1] = 0;
        const uint32_t thr_key = prefix, keep_equal = remaining;
        uint32_t eq = 0;
#pragma unroll
        for (int j = 0; j < SEG; ++j) eq += ((uint32_t)j < n_own && order_key(v[j]) == thr_key) ? 1u : 0u;
        uint32_t eq_total;
        uint32_t rank = block_exclusive_scan_fast<uint32_t>(eq, s_u, &eq_total);
        uint32_t k2 = 0;
#pragma unroll
        for (int j = 0; j < SEG; ++j) {
            const uint32_t key = order_key(v[j]);
            bool ok = (uint32_t)j < n_own && key > thr_key;
            if ((uint32_t)j < n_own && key == thr_key) {
                ok = rank < keep_equal;
                ++rank;
            }
            k2 |= (ok ? 1u : 0u) << j;
        }
        kept = k2;
    }

    // f64 exponentials of the kept logits and their sum
    double ex[SEG], part = 0.0;
#pragma unroll
    for (int j = 0; j < SEG; ++j) {
        ex[j] = ((kept >> j) & 1u) ? exp(((double)v[j] - dmax) / dt) : 0.0;
        part += ex[j];
        __builtin_amdgcn_sched_barrier(0);                // one exponential at a time: the row fills the registers
    }
    const double sum_exp = block_sum<double, kW>(part, s_d);
    // f32 weights, their f64 sum in index order, the last positive one
    double wsum = 0.0;
    uint32_t last_pos = 0;
#pragma unroll
    for (int j = 0; j < SEG; ++j) {
        const float wt = ((kept >> j) & 1u) ? (float)(ex[j] / sum_exp) : 0.0f;
        v[j] = wt;
        wsum += (double)wt;
        if (wt > 0.0f) last_pos = base + j + 1;
        __builtin_amdgcn_sched_barrier(0);
    }
    if (last_pos) atomicMax(&s_sel[1], last_pos);
    double total;
    const double before = block_exclusive_scan_fast<double>(wsum, s_d, &total);
    if (t == 0) {
        uint64_t bits = 0;
        if (policy) {
            uint64_t st = policy[b].rng_state;
            bits = xorshift64star_next(st);
            policy[b].rng_state = st;
        } else {
            uint64_t st = rng_state[0];
            for (uint32_t r = 0; r <= b; ++r) bits = xorshift64star_next(st);
        }
        s_x = (double)(bits >> 11) / 9007199254740992.0 * total;
    }
    __syncthreads();
    const double x = s_x;
    {
        // as in the kernel above: the smallest first-crossing index over all threads is the crossing
        double acc = before;
        uint32_t found = 0xffffffffu;
#pragma unroll
        for (int j = 0; j < SEG; ++j) {
            acc += (double)v[j];
            if (found == 0xffffffffu && v[j] > 0.0f && acc > x) found = base + j;
        }
        if (found != 0xffffffffu) atomicMin(&s_sel[0], found);
    }
    __syncthreads();
    if (t == 0) {
        uint32_t idx = s_sel[0];
        if (idx == 0xffffffffu) idx = s_sel[1] ? s_sel[1] - 1 : vocab - 1;
        tokens[b] = (int32_t)idx;
    }
}

template <typename... A>
static void launch_sampler(uint32_t rows, uint32_t vocab, hipStream_t s, A... args) {
    if (vocab <= kThreads * 8)
        sample_rows_reg_kernel<8><<<rows, kThreads, 0, s>>>(args...);
    else if (vocab <= kThreads * 16)
        sample_rows_reg_kernel<16><<<rows, kThreads, 0, s>>>(args...);
    else if (vocab <= kThreads * 32)
        sample_rows_reg_kernel<32><<<rows, kThreads, 0, s>>>(args...);
    else
        sample_rows_kernel<false><<<rows, kThreads, 0, s>>>(args..., (float *)nullptr, (int32_t *)nullptr, 0);
}

// Acceptance step of sampled speculative decoding for one sequence (crates/autodiff/src/generate/
// speculative.rs:111-189, 246-279), one block: for draft i, p and q are the f32 weight rows of the target and
// of the draft normalised in f64; the draft is accepted when the next uniform u < (f32)min(1, p[d] / q[d]);
// at the first refusal one token is drawn from max(0, p - q) / sum (cast to f32, drawn like every multinomial
// here) and the kernel stops; if all k drafts are accepted one token is drawn from row k of the target's
// weights.  k = 0 is a plain draw from a weight row.  result: accepted drafts, token, status (0 ok; 2 q(d) not
// positive or a probability not finite; 3 a weight row negative, not finite or summing to zero; 4 the
// residual sums to zero; 5 a draft outside the vocabulary).  The generator state is read once and stored
// back with the draws this call consumed.  The f64 sums are block-wide trees instead of sequential passes.
__global__ void __launch_bounds__(kThreads)
    speculative_accept_kernel(const float *__restrict__ p_w, const float *__restrict__ q_w, DraftTokens drafts, uint32_t k,
                              uint32_t vocab, uint64_t *__restrict__ rng_state, int32_t *__restrict__ result) {
    constexpr int kW = kThreads / 64;
    __shared__ double s_d[kW];
    __shared__ uint32_t s_sel[2];
    __shared__ double s_x;
    __shared__ int s_flag;
    const uint32_t t = threadIdx.x;
    const uint32_t seg = (vocab + kThreads - 1) / kThreads;
    const uint32_t lo = t * seg < vocab ? t * seg : vocab, hi = lo + seg < vocab ? lo + seg : vocab;
    uint64_t st = rng_state[0];                          // only thread 0 advances and stores it
    auto finish = [&](uint32_t n_acc, int32_t token, int32_t status) {
        if (t == 0) {
            result[0] = (int32_t)n_acc;
            result[1] = token;
            result[2] = status;
            rng_state[0] = st;
        }
    };
    // f64 sum of a weight row; ok = every weight finite and not negative
    auto row_sum = [&](const float *w, bool *ok) -> double {
        double part = 0.0;
        int good = 1;
        for (uint32_t i = lo; i < hi; ++i) {
            const float v = w[i];
            good &= (v >= 0.0f && v <= 3.402823466e38f) ? 1 : 0;
            part += (double)v;
        }
        double total;
        (void)block_exclusive_scan_fast<double>(part, s_d, &total);
        *ok = __syncthreads_and(good) != 0;
        return total;
    };
    // one multinomial draw from weights given by index; -1 (and nothing drawn) when they sum to zero
    auto draw = [&](auto &&weight_at) -> int32_t {
        double wsum = 0.0;
        uint32_t last_pos = 0;
        for (uint32_t i = lo; i < hi; ++i) {
            const float w = weight_at(i);
            wsum += (double)w;
            if (w > 0.0f) last_pos = i + 1;
        }
        double total;
        const double before = block_exclusive_scan_fast<double>(wsum, s_d, &total);
        if (!(total > 0.0)) return -1;                   // uniform over the block
        if (t == 0) {
            const uint64_t bits = xorshift64star_next(st);
            s_x = (double)(bits >> 11) / 9007199254740992.0 * total;
            s_sel[0] = 0xffffffffu;
            s_sel[1] = 0;
        }
        __syncthreads();
        const double x = s_x;
        if (last_pos) atomicMax(&s_sel[1], last_pos);
        double acc = before;
        uint32_t found = 0xffffffffu;
        for (uint32_t i = lo; i < hi; ++i) {
            const float w = weight_at(i);
            acc += (double)w;
            if (found == 0xffffffffu && w > 0.0f && acc > x) found = i;
        }
        if (found != 0xffffffffu) atomicMin(&s_sel[0], found);
        __syncthreads();
        uint32_t idx = s_sel[0];
        if (idx == 0xffffffffu) idx = s_sel[1] ? s_sel[1] - 1 : vocab - 1;
        __syncthreads();
        return (int32_t)idx;
    };
    for (uint32_t i = 0; i < k; ++i) {
        const float *pr = p_w + (uint64_t)i * vocab, *qr = q_w + (uint64_t)i * vocab;
        bool okp, okq;
        const double sp = row_sum(pr, &okp);
        const double sq = row_sum(qr, &okq);
        if (!okp || !okq || !(sp > 0.0 && sp <= 1.7976931348623157e308) || !(sq > 0.0 && sq <= 1.7976931348623157e308))
            return finish(i, -1, 3);
        const int32_t d = drafts.d[i];
        if (d < 0 || (uint32_t)d >= vocab) return finish(i, -1, 5);
        const double px = (double)pr[d] / sp, qx = (double)qr[d] / sq;
        if (!(qx > 0.0 && qx <= 1.7976931348623157e308) || !(px >= 0.0 && px <= 1.7976931348623157e308)) return finish(i, -1, 2);
        double ratio = px / qx;
        ratio = ratio > 1.0 ? 1.0 : ratio;
        const float a = (float)ratio;
        if (t == 0) {
            const uint64_t bits = xorshift64star_next(st);
            s_flag = (double)(bits >> 11) / 9007199254740992.0 < (double)a ? 1 : 0;
        }
        __syncthreads();
        const bool accepted = s_flag != 0;
        __syncthreads();
        if (accepted) continue;
        auto residual = [&](uint32_t j) -> double {
            const double r = (double)pr[j] / sp - (double)qr[j] / sq;
            return r > 0.0 ? r : 0.0;
        };
        double part = 0.0;
        for (uint32_t j = lo; j < hi; ++j) part += residual(j);
        double sr;
        (void)block_exclusive_scan_fast<double>(part, s_d, &sr);
        if (!(sr > 0.0 && sr <= 1.7976931348623157e308)) return finish(i, -1, 4);
        const int32_t tok = draw([&](uint32_t j) -> float { return (float)(residual(j) / sr); });
        return finish(i, tok, tok < 0 ? 3 : 0);
    }
    const float *br = p_w + (uint64_t)k * vocab;
    bool ok;
    const double sb = row_sum(br, &ok);
    if (!ok || !(sb > 0.0 && sb <= 1.7976931348623157e308)) return finish(k, -1, 3);
    const int32_t tok = draw([&](uint32_t j) -> float { return br[j]; });
    finish(k, tok, tok < 0 ? 3 : 0);
}

__global__ void advance_rng_kernel(uint64_t *state, uint32_t draws) {
    uint64_t st = state[0];
    for (uint32_t i = 0; i < draws; ++i) (void)xorshift64star_next(st);
    state[0] = st;
}

}  // namespace

void sample_rows(const float *logits, int32_t *tokens, uint64_t *rng_state, uint32_t rows, uint32_t vocab, int top_k_mode,
                 float temperature, uint32_t top_k, hipStream_t s) {
    if (rows == 0 || vocab == 0) return;
    launch_sampler(rows, vocab, s, logits, tokens, (const uint64_t *)rng_state, (RowPolicy *)nullptr, vocab, top_k_mode,
                   temperature, top_k);
    advance_rng_kernel<<<1, 1, 0, s>>>(rng_state, rows);
}

void sampling_weights(const float *logits, float *weights, int32_t *status, uint32_t rows, uint32_t vocab, int mode,
                      float temperature, uint32_t top_k, hipStream_t s) {
    if (rows == 0 || vocab == 0) return;
    sample_rows_kernel<true><<<rows, kThreads, 0, s>>>(logits, (int32_t *)nullptr, (const uint64_t *)nullptr, (RowPolicy *)nullptr,
                                                       vocab, mode == 1, temperature, top_k, weights, status, mode == 2);
}

void speculative_accept(const float *p_weights, const float *q_weights, const DraftTokens &drafts, uint32_t k, uint32_t vocab,
                        uint64_t *rng_state, int32_t *result, hipStream_t s) {
    speculative_accept_kernel<<<1, kThreads, 0, s>>>(p_weights, q_weights, drafts, k, vocab, rng_state, result);
}

void sample_rows_policy(const float *logits, int32_t *tokens, RowPolicy *policy, uint32_t rows, uint32_t vocab, hipStream_t s) {
    if (rows == 0 || vocab == 0) return;
    launch_sampler(rows, vocab, s, logits, tokens, (const uint64_t *)nullptr, policy, vocab, 0, 1.0f, 0u);
}

}  // namespace k
}  // namespace fa

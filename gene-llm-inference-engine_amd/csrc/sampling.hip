// Sampling on the device from rows of 32-bit logits: greedy (arg max, lowest index among equal
// maxima) and temperature sampling by the inverse distribution function with a given uniform
// number per row.  Rules as the reference's host sampler states them
// (src/sampler/sampler.cpp:54-80, 119-128): p_i = exp((l_i - max) / T) in 32-bit, sums in 64-bit,
// tokens walked in index order, the first with r = u * total < cumulative sum wins, the last
// token if rounding lets none win.  (The 64-bit sums are taken in a tree, not one by one: the draw
// can differ from the reference's only where r falls within rounding of a boundary.)
#include "common.h"
#include "geneinfer_no_alloc.h"

#include <mutex>

namespace {

constexpr int NT = 1024;

// Arg max in two stages so that a few rows still fill the chip: stage one takes runs of CHUNK
// logits (one workgroup each), stage two the winners of a row.  Among equal values the lowest index
// wins at every comparison, so the result is the lowest index of the maximum.
constexpr int CHUNK = 4096;

// A thread's values of a run of CHUNK logits (i = begin + thread + 256 u), asked for at once by every thread (an index beyond
// the run is clamped and what it brings not used): a loop that reads and compares one by one is sixteen round trips to memory.
constexpr int PER_THREAD = CHUNK / 256;
__device__ __forceinline__ void load_run(const float* __restrict__ row, int begin, int end, float (&v)[PER_THREAD]) {
#pragma unroll
    for (int u = 0; u < PER_THREAD; ++u) v[u] = row[min(begin + (int)threadIdx.x + 256 * u, end - 1)];
}

__device__ __forceinline__ void better(float& bv, int& bi, float ov, int oi) {
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
}

__global__ __launch_bounds__(256) void argmax_chunks_kernel(const float* __restrict__ logits, float* __restrict__ part_v, int* __restrict__ part_i,
                                                            int vocab, long stride, int n_chunks) {
    __shared__ float sv[4];
    __shared__ int si[4];
    const float* row = logits + (size_t)blockIdx.y * stride;
    const int begin = blockIdx.x * CHUNK, end = min(vocab, begin + CHUNK);
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    float v[PER_THREAD];
    load_run(row, begin, end, v);
#pragma unroll
    for (int u = 0; u < PER_THREAD; ++u) {
        const int i = begin + threadIdx.x + 256 * u;
        if (i < end && (v[u] > bv || bi == 0x7fffffff)) { bv = v[u]; bi = i; }      // ascending i: strict > keeps the lowest index
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) better(bv, bi, __shfl_xor(bv, off, 64), __shfl_xor(bi, off, 64));
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = bv; si[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w) better(bv, bi, sv[w], si[w]);
        part_v[(size_t)blockIdx.y * n_chunks + blockIdx.x] = bv;
        part_i[(size_t)blockIdx.y * n_chunks + blockIdx.x] = bi;
    }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ part_v, const int* __restrict__ part_i, int* __restrict__ out,
                                                          int n_chunks) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int c = threadIdx.x; c < n_chunks; c += 64) better(bv, bi, part_v[(size_t)blockIdx.x * n_chunks + c], part_i[(size_t)blockIdx.x * n_chunks + c]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) better(bv, bi, __shfl_xor(bv, off, 64), __shfl_xor(bi, off, 64));
    if (threadIdx.x == 0) out[blockIdx.x] = bi;
}

// Temperature sampling in three stages, so that a few rows still fill the chip: the maxima of runs of
// CHUNK logits (one workgroup each); with the row's maximum known, the runs' sums of p = exp((l - max) / T)
// in 64-bit; then one workgroup per row finds the run that holds r = u * total (runs in index order),
// gives each of its threads 16 consecutive tokens of that run, finds the thread by a prefix sum, and that
// thread walks its tokens one by one.  Cumulative sums follow index order up to the rounding of 64-bit sums.
// `clear`, if given, is `clear_words` 32-bit words per row that later kernels add to: each workgroup zeroes its share of them.
__global__ __launch_bounds__(256) void chunk_max_kernel(const float* __restrict__ logits, float* __restrict__ part_m, int vocab, long stride,
                                                        int n_chunks, unsigned* __restrict__ clear, int clear_words) {
    __shared__ float red[4];
    if (clear != nullptr) {
        const int share = (clear_words + n_chunks - 1) / n_chunks;
        for (int w = blockIdx.x * share + threadIdx.x; w < min(clear_words, (int)(blockIdx.x + 1) * share); w += 256) clear[(size_t)blockIdx.y * clear_words + w] = 0u;
    }
    const float* row = logits + (size_t)blockIdx.y * stride;
    const int begin = blockIdx.x * CHUNK, end = min(vocab, begin + CHUNK);
    float mx = -INFINITY, v[PER_THREAD];
    load_run(row, begin, end, v);
#pragma unroll
    for (int u = 0; u < PER_THREAD; ++u)
        if (begin + (int)threadIdx.x + 256 * u < end) mx = fmaxf(mx, v[u]);
    mx = wave_max(mx);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
    __syncthreads();
    if (threadIdx.x == 0) part_m[(size_t)blockIdx.y * n_chunks + blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// The row's maximum from its runs' maxima, the same value in every thread of a workgroup of 256: the threads read the runs'
// maxima side by side and meet in LDS (`red`: 4 floats; a barrier inside, so every thread of the workgroup must come here).
__device__ __forceinline__ float row_max(const float* __restrict__ part_m, int n_chunks, float* red) {
    float mx = -INFINITY;
    for (int c = threadIdx.x; c < n_chunks; c += 256) mx = fmaxf(mx, part_m[c]);
    mx = wave_max(mx);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    return mx;
}

// `kept`, if given, receives exp((l - max) / T) of every token ([rows, vocab]) for the kernels that come back to them.
__global__ __launch_bounds__(256) void chunk_sum_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                        const float* __restrict__ part_m, double* __restrict__ part_s, float* __restrict__ kept,
                                                        int vocab, long stride, int n_chunks) {
    __shared__ double red[4];
    __shared__ float red_max[4];
    const float* row = logits + (size_t)blockIdx.y * stride;
    const int begin = blockIdx.x * CHUNK, end = min(vocab, begin + CHUNK);
    float v[PER_THREAD];
    load_run(row, begin, end, v);
    const float temp = temperature[blockIdx.y], mx = row_max(part_m + (size_t)blockIdx.y * n_chunks, n_chunks, red_max);
    double sum = 0.0;
#pragma unroll
    for (int u = 0; u < PER_THREAD; ++u) {
        const int i = begin + threadIdx.x + 256 * u;
        if (i < end) {
            const float e = expf((v[u] - mx) / temp);
            if (kept != nullptr) kept[(size_t)blockIdx.y * vocab + i] = e;
            sum += (double)e;
        }
    }
    sum = wave_sum_f64(sum);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0) part_s[(size_t)blockIdx.y * n_chunks + blockIdx.x] = ((red[0] + red[1]) + red[2]) + red[3];
}

constexpr int RUN = CHUNK / 256;            // tokens a thread of the last stage owns
constexpr int MAX_RUNS = 1024;              // runs of a row that the last stage holds in LDS (a vocabulary of 4 M tokens)

__global__ __launch_bounds__(256) void sample_pick_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                          const float* __restrict__ uniform, const float* __restrict__ part_m,
                                                          const double* __restrict__ part_s, int* __restrict__ out, int vocab, long stride,
                                                          int n_chunks) {
    __shared__ double wave_total[4];
    __shared__ int winner;
    __shared__ float red_max[4];
    __shared__ double run_sums[MAX_RUNS];
    __shared__ double before_run;
    __shared__ int the_run;
    const float* row = logits + (size_t)blockIdx.x * stride;
    const double* sums = part_s + (size_t)blockIdx.x * n_chunks;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int c = tid; c < n_chunks; c += 256) run_sums[c] = sums[c];           // side by side; added up in index order below
    const float temp = temperature[blockIdx.x], mx = row_max(part_m + (size_t)blockIdx.x * n_chunks, n_chunks, red_max);     // (its barriers stand behind the writes above)
    // The reference normalises p by a 32-bit 1/sum before it draws; the draw compares u * sum(p) with
    // cumulative p, which is the same comparison scaled by a constant, so it is made on the
    // unnormalised values here.
    if (tid == 0) {
        double total = 0.0;
        for (int c = 0; c < n_chunks; ++c) total += run_sums[c];
        const double r0 = (double)uniform[blockIdx.x] * total;
        int chunk = n_chunks - 1;            // the run that holds r (the last one if rounding lets none hold it)
        double before = 0.0;
        for (int c = 0; c < n_chunks - 1; ++c) {
            if (r0 < before + run_sums[c]) { chunk = c; break; }
            before += run_sums[c];
        }
        the_run = chunk;
        before_run = before;
        run_sums[0] = r0;                    // (the sums have served)
    }
    __syncthreads();
    const int chunk = the_run;
    double before = before_run;
    const double r = run_sums[0];
    const int begin = chunk * CHUNK, end = min(vocab, begin + CHUNK);
    const int lo = min(end, begin + tid * RUN), hi = min(end, lo + RUN);
    float mine_p[RUN];                       // the thread's tokens' p, asked for at once
#pragma unroll
    for (int u = 0; u < RUN; ++u) mine_p[u] = row[min(lo + u, vocab - 1)];
    double mine = 0.0;
#pragma unroll
    for (int u = 0; u < RUN; ++u) {
        mine_p[u] = expf((mine_p[u] - mx) / temp);
        if (lo + u < hi) mine += (double)mine_p[u];
    }
    double c = mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {                  // inclusive prefix sum over the lanes of a wave
        const double below = __shfl_up(c, off, 64);
        if (lane >= off) c += below;
    }
    if (lane == 63) wave_total[wave] = c;
    const double c_below = __shfl_up(c, 1, 64);
    if (tid == 0) winner = min(end, vocab - 1);              // if rounding leaves r beyond the run: the next token in index order
    __syncthreads();
    for (int w = 0; w < wave; ++w) before += wave_total[w];
    // A thread's tokens start where the thread before it stops, as the same sum: taken as `run_stop - mine` the start would fall
    // back onto an earlier thread's tokens wherever those weigh less than the last bit of this thread's (u = 0 before a heavy token).
    const double run_start = lane ? before + c_below : before, run_stop = before + c;
    if (lo < hi && r >= run_start && r < run_stop) {          // at most one thread
        double walk = run_start;
        int pick = min(hi, vocab - 1);
        bool found = false;
#pragma unroll
        for (int u = 0; u < RUN; ++u) {
            if (!found && lo + u < hi) {
                walk += (double)mine_p[u];
                if (r < walk) { pick = lo + u; found = true; }
            }
        }
        winner = pick;
    }
    __syncthreads();
    if (tid == 0) out[blockIdx.x] = winner;
}


// ------------------------------------------------------------------ top-k and top-p
// The reference sorts a row's tokens by probability descending, index ascending among equal ones, keeps the first k, then the
// shortest prefix whose mass reaches top_p times the kept mass, and walks what is left until the cumulative mass exceeds u times
// its mass (src/sampler/sampler.cpp:84-128).  Nothing is sorted here.  All three are the same question, "where in that order does
// a running count, or a running mass, cross a target", and the order is that of the probabilities' bit patterns (a 32-bit float
// that is not negative grows with its pattern).  One workgroup owns a row and walks the pattern down from its high bits, 11, 11
// and 10 at a time: a histogram in LDS holds count and mass of the tokens under each value of those bits (among the tokens that
// share the bits chosen so far), a prefix sum over it from the highest value down finds the value at which the target is
// crossed, and the next level looks inside that value.  The first level's histogram takes every token, is made once and
// serves all three questions: a filter's result ends inside one of its values and leaves the higher ones whole.  After three levels the probability of the token at the crossing is
// known exactly; the tokens that have it come in index order, and a count over the row finds the one.  Probabilities are
// p = exp((l - max) / T) * (float)(1 / sum) in 32-bit as in the reference (:73-81); masses are summed as integers, in units of
// 2^-60, so that a sum does not depend on the order in which the workgroup's threads add to it.  A sum differs from the
// reference's 64-bit floating one by less than vocab * 2^-60: a result differs only where a target falls that close to a
// boundary.
constexpr int FT = 1024;                    // threads of the workgroup that owns a row
constexpr int FW = FT / 64;
constexpr int DIGITS = 2048;                // values of the bits that one level looks at
typedef unsigned long long u64;

struct OrderPlace {                         // a token's place in the order: its probability's pattern and its index
    unsigned key;
    int idx;
};
struct OrderPrefix {                        // the tokens up to and including `last`: how many, and their mass
    OrderPlace last;
    unsigned count;
    u64 mass;
};
struct Histogram {
    unsigned cnt[DIGITS];
    u64 mass[DIGITS];
};
struct FilterShared {
    Histogram top;                          // every token of the row under the high 11 bits of its probability: made once
    Histogram low;                          // the tokens that share the bits chosen so far, under the next bits,
    int low_idx[DIGITS];                    // and one of the tokens under each value: the token, where a value has one
    unsigned wave_cnt[FW];
    u64 wave_mass[FW];
    unsigned digit, cnt_before, cnt_here;
    u64 mass_before;
    int found, idx;
};

// floor(p * 2^60) of the probability with this pattern (0 <= p <= 1): its 24 leading bits moved to their place.
__device__ __forceinline__ u64 mass_of(unsigned key) {
    const int ex = (int)(key >> 23);
    const u64 lead = (u64)((key & 0x7fffffu) | 0x800000u);              // p = lead * 2^(ex - 150)
    return ex >= 90 ? lead << (ex - 90) : ex > 66 ? lead >> (90 - ex) : 0;
}
__device__ __forceinline__ bool within(unsigned key, int i, OrderPlace last) { return key > last.key || (key == last.key && i <= last.idx); }

// One token per lane (those with `take`) into a histogram; every lane of the wave calls it.  Many tokens of a row share few
// values (all of them one, if the logits are equal), and additions to one address queue up: the lanes that share the first
// taker's value add as one.
__device__ __forceinline__ void add_tokens(Histogram& h, bool take, unsigned digit, u64 q, int lane) {
    const u64 takers = __ballot(take);
    if (takers == 0) return;
    const int head = __ffsll((long long)takers) - 1;
    const unsigned head_digit = __shfl(digit, head, 64);
    const bool same = take && digit == head_digit;
    const u64 group = __ballot(same);
    if (__popcll(group) >= 8) {
        u64 sum = same ? q : 0;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
        if (lane == head) {
            atomicAdd(&h.cnt[head_digit], (unsigned)__popcll(group));
            atomicAdd(&h.mass[head_digit], sum);
        }
        take = take && !same;
    }
    if (take) {
        atomicAdd(&h.cnt[digit], 1u);
        if (q != 0) atomicAdd(&h.mass[digit], q);
    }
}

// Every thread of the workgroup calls `f(i, pattern of p_i, i < vocab)` for its share of a row's tokens (and for a few places
// beyond the row's end, so that whole waves call it; there the pattern is that of a negative number, which no probability
// has), in no particular order.  A pass over a row is a chain of loads from the second-level cache, each waited for: a thread
// has eight loads in flight at a time, of four tokens each where the row allows.
template <typename F>
__device__ __forceinline__ void for_each_token(const float* __restrict__ e, float inv, int vocab, F f) {
    constexpr int AT_ONCE = 8;
    if ((vocab & 3) == 0 && ((size_t)e & 15) == 0) {
        const int fours = vocab >> 2;
        for (int first = 0; first < fours; first += FT * AT_ONCE) {
            float4 v[AT_ONCE];
#pragma unroll
            for (int u = 0; u < AT_ONCE; ++u) {
                const int at = first + u * FT + (int)threadIdx.x;
                v[u] = at < fours ? reinterpret_cast<const float4*>(e)[at] : float4{-1.0f, -1.0f, -1.0f, -1.0f};
            }
#pragma unroll
            for (int u = 0; u < AT_ONCE; ++u) {
                const int at = first + u * FT + (int)threadIdx.x;
                if (first + u * FT >= fours) break;
                f(4 * at, __float_as_uint(v[u].x * inv), at < fours);
                f(4 * at + 1, __float_as_uint(v[u].y * inv), at < fours);
                f(4 * at + 2, __float_as_uint(v[u].z * inv), at < fours);
                f(4 * at + 3, __float_as_uint(v[u].w * inv), at < fours);
            }
        }
        return;
    }
    for (int first = 0; first < vocab; first += FT * AT_ONCE) {
        float v[AT_ONCE];
#pragma unroll
        for (int u = 0; u < AT_ONCE; ++u) {
            const int i = first + u * FT + (int)threadIdx.x;
            v[u] = i < vocab ? e[i] : -1.0f;
        }
#pragma unroll
        for (int u = 0; u < AT_ONCE; ++u) {
            const int i = first + u * FT + (int)threadIdx.x;
            if (first + u * FT < vocab) f(i, __float_as_uint(v[u] * inv), i < vocab);
        }
    }
}

// COUNT: the prefix of `target` tokens.  REACH: the shortest prefix whose mass is >= target.  EXCEED: the shortest whose mass
// is > target.
enum { COUNT = 0, REACH = 1, EXCEED = 2 };

// The value of a level's bits at which the running count or mass, from the highest value down and on top of what lies before
// the level, crosses the target; what lies before that value, and how many tokens have it.  The histogram is complete (a
// barrier lies behind its last addition).  With `cut`, `kept` ends inside the value `cut_digit`: lower values hold nothing, and
// that value holds what is left of `kept`.  False if nothing crosses.
template <int MODE>
__device__ bool choose(const Histogram& h, int values, bool cut, unsigned cut_digit, const OrderPrefix& kept, u64 target, unsigned& digit,
                       unsigned& cnt_before, u64& mass_before, unsigned& cnt_here, FilterShared& sh) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    unsigned c[2];                                          // two values per thread, a prefix sum over the threads
    u64 m[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        const int value = values - 1 - (2 * tid + s);
        const bool holds = value >= 0 && !(cut && (unsigned)value <= cut_digit);
        c[s] = holds ? h.cnt[value] : 0;
        m[s] = holds ? h.mass[value] : 0;
    }
    const unsigned c_mine = c[0] + c[1];
    const u64 m_mine = m[0] + m[1];
    unsigned c_upto = c_mine;
    u64 m_upto = m_mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const unsigned cb = __shfl_up(c_upto, off, 64);
        const u64 mb = __shfl_up(m_upto, off, 64);
        if (lane >= off) {
            c_upto += cb;
            m_upto += mb;
        }
    }
    if (lane == 63) {
        sh.wave_cnt[wave] = c_upto;
        sh.wave_mass[wave] = m_upto;
    }
    if (tid == 0) sh.found = 0;
    __syncthreads();
    unsigned c_run = cnt_before + (c_upto - c_mine);
    u64 m_run = mass_before + (m_upto - m_mine);
    for (int w = 0; w < wave; ++w) {
        c_run += sh.wave_cnt[w];
        m_run += sh.wave_mass[w];
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        const int value = values - 1 - (2 * tid + s);
        if (cut && value == (int)cut_digit) {               // everything above it is whole, so the running sums are right here
            c[s] = kept.count - c_run;
            m[s] = kept.mass - m_run;
        }
        const unsigned c_next = c_run + c[s];
        const u64 m_next = m_run + m[s];
        const bool crossed = MODE == COUNT ? (c_run < target && c_next >= target)
                           : MODE == REACH ? (m_run < target && m_next >= target)
                                           : (m_run <= target && m_next > target);
        if (crossed) {                                       // sums only grow: at most one value of one thread
            sh.found = 1;
            sh.digit = (unsigned)value;
            sh.cnt_before = c_run;
            sh.mass_before = m_run;
            sh.cnt_here = c[s];
        }
        c_run = c_next;
        m_run = m_next;
    }
    __syncthreads();
    const bool found = sh.found != 0;
    digit = sh.digit;
    cnt_before = sh.cnt_before;
    mass_before = sh.mass_before;
    cnt_here = sh.cnt_here;
    __syncthreads();                                         // everyone has read the choice before anything clears it
    return found;
}

// Only tokens within `kept` exist.  If no prefix does it (the caller's targets do not allow that), `kept` itself.
template <int MODE>
__device__ OrderPrefix find_prefix(const float* __restrict__ e, float inv, int vocab, const OrderPrefix& kept, u64 target, FilterShared& sh) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool cut = kept.last.idx < vocab;                  // otherwise every token is within it
    unsigned chosen = 0, digit = 0, cnt_before = 0, cnt_here = 0;
    u64 mass_before = 0;
    if (!choose<MODE>(sh.top, DIGITS, cut, kept.last.key >> 21, kept, target, chosen, cnt_before, mass_before, cnt_here, sh)) return kept;
#pragma unroll
    for (int level = 1; level < 3; ++level) {
        const int shift = level == 1 ? 10 : 0, width = level == 1 ? 11 : 10, values = 1 << width;
        for (int b = tid; b < DIGITS; b += FT) {
            sh.low.cnt[b] = 0;
            sh.low.mass[b] = 0;
        }
        __syncthreads();
        for_each_token(e, inv, vocab, [&](int i, unsigned key, bool) {
            const bool shares = (key >> (shift + width)) == chosen;         // (a place beyond the row's end has a negative number: never)
            if (__ballot(shares) == 0) return;                              // most waves most of the time: a few instructions per token
            const bool take = shares && (!cut || within(key, i, kept.last));
            add_tokens(sh.low, take, (key >> shift) & (values - 1), mass_of(key), lane);
            if (take) sh.low_idx[(key >> shift) & (values - 1)] = i;
        });
        __syncthreads();
        if (!choose<MODE>(sh.low, values, false, 0u, kept, target, digit, cnt_before, mass_before, cnt_here, sh)) return kept;
        chosen = (chosen << width) | digit;
        if (cnt_here == 1) {                                 // the usual end: one token has these bits, the prefix ends with it
            const int idx = sh.low_idx[digit];
            const unsigned key = __float_as_uint(e[idx] * inv);
            return OrderPrefix{OrderPlace{key, idx}, cnt_before + 1, mass_before + mass_of(key)};
        }
    }
    // Every token left has the probability whose pattern is `chosen`; they come in index order.  How many of them the prefix takes:
    const u64 each = mass_of(chosen);
    u64 n_taken = MODE == COUNT ? target - cnt_before : MODE == REACH ? (target - mass_before + each - 1) / each : (target - mass_before) / each + 1;
    if (n_taken > cnt_here) n_taken = cnt_here;
    // Which token is that: each wave counts a run of the row, the wave that holds it counts once more.
    const int per_wave = (((vocab + FW - 1) / FW) + 63) & ~63;
    const int begin = wave * per_wave, end = min(vocab, begin + per_wave);
    const bool any_index = !cut || chosen > kept.last.key;   // else only those up to kept's last are within it
    unsigned mine = 0;
    for (int first = begin; first < end; first += 64 * 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = first + u * 64 + lane < end ? e[first + u * 64 + lane] : -1.0f;       // no probability is negative
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const bool is = __float_as_uint(v[u] * inv) == chosen && (any_index || first + u * 64 + lane <= kept.last.idx);
            mine += (unsigned)__popcll(__ballot(is));
        }
    }
    if (lane == 0) sh.wave_cnt[wave] = mine;
    if (tid == 0) sh.idx = kept.last.idx;
    __syncthreads();
    unsigned before = 0;
    for (int w = 0; w < wave; ++w) before += sh.wave_cnt[w];
    if (before < n_taken && n_taken <= before + mine) {
        bool seen = false;
        for (int first = begin; first < end && !seen; first += 64 * 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = first + u * 64 + lane < end ? e[first + u * 64 + lane] : -1.0f;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int i = first + u * 64 + lane;
                const bool is = __float_as_uint(v[u] * inv) == chosen && (any_index || i <= kept.last.idx);
                const u64 which = __ballot(is);
                const unsigned n = (unsigned)__popcll(which);
                if (!seen && before + n >= n_taken) {
                    if (is && before + (unsigned)__popcll(which & ((1ull << lane) - 1ull)) + 1 == n_taken) sh.idx = i;
                    seen = true;
                }
                before += n;
            }
        }
    }
    __syncthreads();
    const int idx = sh.idx;
    __syncthreads();
    return OrderPrefix{OrderPlace{chosen, idx}, cnt_before + (unsigned)n_taken, mass_before + n_taken * each};
}

// The first level's histogram of every row, TOP_SHARES workgroups a row (it is the one pass that every token adds to, and the
// first that reads the row, from wherever the kernel before left it): each takes a stretch of the row into a histogram in LDS
// and adds what that holds to the row's in memory, which starts at zero.  Sums of integers: the order does not matter.
constexpr int TOP_SHARES = 8;

__global__ __launch_bounds__(FT) void top_histogram_kernel(const float* __restrict__ e_all, const double* __restrict__ part_s, Histogram* __restrict__ tops,
                                                           int vocab, int n_chunks) {
    __shared__ Histogram h;
    const int row = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
    double total = 0.0;
    for (int c = 0; c < n_chunks; ++c) total += part_s[(size_t)row * n_chunks + c];
    const float inv = (float)(1.0 / total);                  // sampler.cpp:80
    const int share = (((vocab + TOP_SHARES - 1) / TOP_SHARES) + FT - 1) / FT * FT;
    const int begin = min(vocab, (int)blockIdx.x * share), n = min(vocab, begin + share) - begin;
    if (n <= 0) return;
    for (int b = tid; b < DIGITS; b += FT) {
        h.cnt[b] = 0;
        h.mass[b] = 0;
    }
    __syncthreads();
    for_each_token(e_all + (size_t)row * vocab + begin, inv, n, [&](int, unsigned key, bool there) { add_tokens(h, there, key >> 21, mass_of(key), lane); });
    __syncthreads();
    for (int b = tid; b < DIGITS; b += FT)
        if (h.cnt[b] != 0) {
            atomicAdd(&tops[row].cnt[b], h.cnt[b]);
            if (h.mass[b] != 0) atomicAdd(&tops[row].mass[b], h.mass[b]);
        }
}

// One workgroup per row: exp((l - max) / T) of its tokens, the runs' sums and the first level's histogram are there.
__global__ __launch_bounds__(FT) void sample_filtered_kernel(const float* __restrict__ e_all, const double* __restrict__ part_s,
                                                             const Histogram* __restrict__ tops, const int* __restrict__ top_k,
                                                             const float* __restrict__ top_p, const float* __restrict__ uniform,
                                                             int* __restrict__ out, int vocab, int n_chunks) {
    __shared__ FilterShared sh;
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float* e = e_all + (size_t)row * vocab;
    double total = 0.0;
    for (int c = 0; c < n_chunks; ++c) total += part_s[(size_t)row * n_chunks + c];
    const float inv = (float)(1.0 / total);                  // sampler.cpp:80
    for (int b = tid; b < DIGITS; b += FT) {
        sh.top.cnt[b] = tops[row].cnt[b];
        sh.top.mass[b] = tops[row].mass[b];
    }
    __syncthreads();
    u64 all = sh.top.mass[2 * tid] + sh.top.mass[2 * tid + 1];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) all += __shfl_xor(all, off, 64);
    if (lane == 0) sh.wave_mass[wave] = all;
    __syncthreads();
    OrderPrefix kept{OrderPlace{0u, vocab}, (unsigned)vocab, 0};       // every token
    for (int w = 0; w < FW; ++w) kept.mass += sh.wave_mass[w];
    __syncthreads();
    const int k = top_k[row];
    if (k > 0 && k < vocab) kept = find_prefix<COUNT>(e, inv, vocab, kept, (u64)k, sh);
    const float p_keep = top_p[row];
    if (p_keep < 1.0f) {                                      // cum >= top_p * total (:104-111), in units of 2^-60
        u64 target = (u64)ceil((double)p_keep * (double)kept.mass);
        target = target < 1 ? 1 : target > kept.mass ? kept.mass : target;
        kept = find_prefix<REACH>(e, inv, vocab, kept, target, sh);
    }
    u64 r = (u64)((double)uniform[row] * (double)kept.mass);  // r < cum (:121-126); the last kept token if rounding lets none win
    if (kept.mass > 0 && r >= kept.mass) r = kept.mass - 1;
    const OrderPrefix drawn = find_prefix<EXCEED>(e, inv, vocab, kept, r, sh);
    if (tid == 0) out[row] = min(drawn.last.idx, vocab - 1);
}

}  // namespace

// Chunks per row, so that the caller can size the scratch: n_rows * chunks floats and as many ints.
GI_API int gi_argmax_chunks(int vocab) { return (vocab + CHUNK - 1) / CHUNK; }

GI_API int gi_argmax(const float* logits, int* out, float* part_v, int* part_i, int n_rows, int vocab, long stride, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_rows <= 65535 && vocab > 0 && stride >= vocab, "argmax: bad sizes (rows %d, vocab %d, stride %ld)", n_rows, vocab, stride);
    GI_REQUIRE(part_v != nullptr && part_i != nullptr, "argmax: scratch is missing");
    const int n_chunks = gi_argmax_chunks(vocab);
    argmax_chunks_kernel<<<dim3(n_chunks, n_rows), 256, 0, stream>>>(logits, part_v, part_i, vocab, stride, n_chunks);
    GI_CHECK_LAUNCH("argmax (chunks)");
    argmax_final_kernel<<<n_rows, 64, 0, stream>>>(part_v, part_i, out, n_chunks);
    GI_CHECK_LAUNCH("argmax (final)");
    return 0;
}

// part_m: n_rows * gi_argmax_chunks(vocab) floats, part_s: as many doubles.
GI_API int gi_sample_temperature(const float* logits, const float* temperature, const float* uniform, int* out, float* part_m, double* part_s,
                                 int n_rows, int vocab, long stride, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_rows <= 65535 && vocab > 0 && stride >= vocab, "sample_temperature: bad sizes (rows %d, vocab %d, stride %ld)", n_rows, vocab, stride);
    GI_REQUIRE(part_m != nullptr && part_s != nullptr, "sample_temperature: scratch is missing");
    const int n_chunks = gi_argmax_chunks(vocab);
    GI_REQUIRE(n_chunks <= MAX_RUNS, "sample_temperature: a vocabulary of %d tokens is more than %d runs of %d", vocab, MAX_RUNS, CHUNK);
    chunk_max_kernel<<<dim3(n_chunks, n_rows), 256, 0, stream>>>(logits, part_m, vocab, stride, n_chunks, nullptr, 0);
    GI_CHECK_LAUNCH("sample_temperature (maxima)");
    chunk_sum_kernel<<<dim3(n_chunks, n_rows), 256, 0, stream>>>(logits, temperature, part_m, part_s, nullptr, vocab, stride, n_chunks);
    GI_CHECK_LAUNCH("sample_temperature (sums)");
    sample_pick_kernel<<<n_rows, 256, 0, stream>>>(logits, temperature, uniform, part_m, part_s, out, vocab, stride, n_chunks);
    GI_CHECK_LAUNCH("sample_temperature (pick)");
    return 0;
}

// Top-k, then top-p, then the draw, of rows of which every one has a filter (top_k in 1..vocab-1, or top_p < 1; a top_k of 0
// or of vocab and more, or a top_p of 1, leaves that filter out).  part_m, part_s as for gi_sample_temperature; kept: n_rows * vocab floats;
// tops: n_rows * gi_sample_filtered_histogram_bytes() bytes, 8-byte aligned.
GI_API int gi_sample_filtered(const float* logits, const float* temperature, const int* top_k, const float* top_p, const float* uniform, int* out,
                              float* part_m, double* part_s, float* kept, void* tops, int n_rows, int vocab, long stride, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_rows <= 65535 && vocab > 0 && stride >= vocab, "sample_filtered: bad sizes (rows %d, vocab %d, stride %ld)", n_rows, vocab, stride);
    GI_REQUIRE(part_m != nullptr && part_s != nullptr && kept != nullptr && tops != nullptr && (size_t)tops % 8 == 0, "sample_filtered: scratch is missing");
    const int n_chunks = gi_argmax_chunks(vocab);
    chunk_max_kernel<<<dim3(n_chunks, n_rows), 256, 0, stream>>>(logits, part_m, vocab, stride, n_chunks, (unsigned*)tops, (int)(sizeof(Histogram) / 4));
    GI_CHECK_LAUNCH("sample_filtered (maxima)");
    chunk_sum_kernel<<<dim3(n_chunks, n_rows), 256, 0, stream>>>(logits, temperature, part_m, part_s, kept, vocab, stride, n_chunks);
    GI_CHECK_LAUNCH("sample_filtered (sums)");
    top_histogram_kernel<<<dim3(TOP_SHARES, n_rows), FT, 0, stream>>>(kept, part_s, (Histogram*)tops, vocab, n_chunks);
    GI_CHECK_LAUNCH("sample_filtered (first histogram)");
    sample_filtered_kernel<<<n_rows, FT, 0, stream>>>(kept, part_s, (const Histogram*)tops, top_k, top_p, uniform, out, vocab, n_chunks);
    GI_CHECK_LAUNCH("sample_filtered (draw)");
    return 0;
}

// Bytes of `tops` per row.
GI_API int gi_sample_filtered_histogram_bytes(void) { return (int)sizeof(Histogram); }

// ------------------------------------------------------------------ arg max without a scratch argument
// The partial results of gi_argmax's first stage live in a static array in device memory instead of memory the caller
// brings.  In host code the array's name is only a handle for hipGetSymbolAddress: every GPU holds its own copy at its
// own address, which is asked for once per device and kept; kernels, and anything else on the host that needs the
// memory, get that address.
static __device__ __align__(256) unsigned char scratch[GI_NO_ALLOC_ARGMAX_MAX_PARTS * (sizeof(float) + sizeof(int))];

namespace {
constexpr int MAX_DEVICES = 64;
void* g_scratch_of_device[MAX_DEVICES] = {};
std::mutex g_scratch_mutex;

// This GPU's copy of `scratch` (the current device's), or nullptr with the error recorded.
void* scratch_of_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        gi_fail("no_alloc: no current HIP device (or more than %d devices)", MAX_DEVICES);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_of_device[dev] == nullptr) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            gi_fail("no_alloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_of_device[dev] = ptr;
    }
    return g_scratch_of_device[dev];
}
}  // namespace

GI_API int gi_no_alloc_prepare(void) { return scratch_of_current_device() != nullptr ? 0 : -1; }

GI_API int gi_argmax_no_alloc(const float* logits, int* out, int n_rows, int vocab, long stride, hipStream_t stream) {
    GI_REQUIRE(logits != nullptr && out != nullptr, "argmax_no_alloc: logits and out must be given");
    GI_REQUIRE(n_rows > 0 && n_rows <= 65535 && vocab > 0 && stride >= vocab, "argmax_no_alloc: bad sizes (rows %d, vocab %d, stride %ld)", n_rows, vocab, stride);
    const int n_chunks = gi_argmax_chunks(vocab);
    GI_REQUIRE((long)n_rows * n_chunks <= GI_NO_ALLOC_ARGMAX_MAX_PARTS,
               "argmax_no_alloc: %d rows x %d runs of %d logits need %ld partial results, the static scratch holds %d; use gi_argmax with scratch of your own",
               n_rows, n_chunks, CHUNK, (long)n_rows * n_chunks, GI_NO_ALLOC_ARGMAX_MAX_PARTS);
    unsigned char* ptr = (unsigned char*)scratch_of_current_device();
    if (ptr == nullptr) return -1;
    float* part_v = (float*)ptr;
    int* part_i = (int*)(ptr + (size_t)GI_NO_ALLOC_ARGMAX_MAX_PARTS * sizeof(float));
    argmax_chunks_kernel<<<dim3(n_chunks, n_rows), 256, 0, stream>>>(logits, part_v, part_i, vocab, stride, n_chunks);
    GI_CHECK_LAUNCH("argmax_no_alloc (chunks)");
    argmax_final_kernel<<<n_rows, 64, 0, stream>>>(part_v, part_i, out, n_chunks);
    GI_CHECK_LAUNCH("argmax_no_alloc (final)");
    return 0;
}

// Sampling over rows of float logits [B, V]: argmax, and the reference's sampler
// (crates/braidinfer-runtime/src/sampling.rs:49-171) in its order: logit bias,
// repetition penalty, temperature, top-k, min-p, top-p, softmax, inverse CDF with a
// uniform number the host supplies.  One block per row; every reduction and scan has a
// fixed order, so a row samples the same token alone or inside any batch.
#include "common.h"

#define SBLOCK 256

// order-preserving map float -> uint32 (larger float = larger key).  -0 takes the key of +0: the
// two are equal in the reference's order (a sort by value, the lower index first among equals),
// so which of a row's zeros a cut keeps is decided by their indices alone.
__device__ __forceinline__ uint32_t f2key(float f) {
    uint32_t u = __float_as_uint(f);
    if (u == 0x80000000u) u = 0u;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key2f(uint32_t k) {
    uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __uint_as_float(u);
}

// ---------------------------------------------------------------------- argmax -----
// out[b] = index of the largest logit of row b; the lowest index wins ties (the
// reference's GPU kernel keeps the first maximum within a thread's stripe,
// kernels/argmax.hip:21-27; its host argmax keeps the last, generate.rs:493-500; one
// rule is fixed here).  NaN never wins.
__device__ __forceinline__ void argmax_combine(float& v, int& i, float ov, int oi) {
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

#define ABLOCK 1024
// ADVANCE: the row's token also becomes the next single-token step's input, on the device:
// for a live row (slot >= 0) tokens[b] = the token, and the row's position and length grow
// by one, so the same recorded step can be replayed without the host writing its arrays.
template <bool ADVANCE>
__global__ __launch_bounds__(ABLOCK) void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int V,
                                                        int* __restrict__ tokens, int* __restrict__ positions,
                                                        const int* __restrict__ slots, int* __restrict__ ctx) {
    __shared__ float sv[ABLOCK / 64];
    __shared__ int si[ABLOCK / 64];
    const float* r = logits + (size_t)blockIdx.x * V;
    float bv = -INFINITY; int bi = 0x7fffffff;
    // eight loads in flight per thread: one load per trip would wait a memory latency each time
    for (int i0 = threadIdx.x; i0 < V; i0 += 8 * ABLOCK) {
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = i0 + k * ABLOCK < V ? r[i0 + k * ABLOCK] : -INFINITY;
#pragma unroll
        for (int k = 0; k < 8; ++k)
            if (i0 + k * ABLOCK < V) argmax_combine(bv, bi, v[k], i0 + k * ABLOCK);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        float ov = __shfl_xor(bv, o, 64); int oi = __shfl_xor(bi, o, 64);
        argmax_combine(bv, bi, ov, oi);
    }
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = bv; si[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < ABLOCK / 64; ++w) argmax_combine(bv, bi, sv[w], si[w]);
        const int tok = (bi == 0x7fffffff) ? 0 : bi;
        out[blockIdx.x] = tok;
        if (ADVANCE && slots[blockIdx.x] >= 0) {
            tokens[blockIdx.x] = tok;
            positions[blockIdx.x] += 1;
            ctx[blockIdx.x] += 1;
        }
    }
}

extern "C" int br_argmax(const float* logits, int* out, int B, int V, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (V <= 0) return BR_BAD_ARG;
    argmax_kernel<false><<<B, ABLOCK, 0, s>>>(logits, out, V, nullptr, nullptr, nullptr, nullptr);
    return br_check_launch();
}

// argmax of every row, and the rows' step arrays moved on by one token (see ADVANCE)
extern "C" int br_argmax_advance(const float* logits, int* out, int B, int V, int* tokens, int* positions,
                                 const int* slots, int* ctx, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (V <= 0 || !tokens || !positions || !slots || !ctx) return BR_BAD_ARG;
    argmax_kernel<true><<<B, ABLOCK, 0, s>>>(logits, out, V, tokens, positions, slots, ctx);
    return br_check_launch();
}

// The step arrays of n live rows moved on by the tokens a sampler drew for them: tokens[i] =
// drawn[i], the row's position and length one more (what ADVANCE does for the argmax).
__global__ void step_advance_kernel(const int* __restrict__ drawn, int* __restrict__ tokens, int* __restrict__ positions,
                                    const int* __restrict__ slots, int* __restrict__ ctx, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && slots[i] >= 0) {
        tokens[i] = drawn[i];
        positions[i] += 1;
        ctx[i] += 1;
    }
}

extern "C" int br_step_advance(const int* drawn, int* tokens, int* positions, const int* slots, int* ctx, int n,
                               hipStream_t s) {
    if (n <= 0) return BR_OK;
    if (!drawn || !tokens || !positions || !slots || !ctx) return BR_BAD_ARG;
    step_advance_kernel<<<(n + 255) / 256, 256, 0, s>>>(drawn, tokens, positions, slots, ctx, n);
    return br_check_launch();
}

// --------------------------------------------------- bias, penalty, temperature ----
// work[b, :] = logits[b, :]; then per row, in the reference's order (sampling.rs:57-87):
// bias entries (token, delta) are added; every history token's logit is divided by the
// penalty when positive, multiplied otherwise, once per occurrence; everything is divided by
// the temperature when it is not 0.  The bias lists are ragged: entries of row b are
// [off[b], off[b+1]).  The history is a table counts[B, V] of occurrences per token (null: none),
// which br_sample_draw_count keeps up to date on the device.
#define PSEG 2048      // entries of a row that one workgroup prepares
__global__ __launch_bounds__(SBLOCK) void sample_prepare_kernel(
    const float* __restrict__ logits, float* __restrict__ work, int V,
    const int* __restrict__ bias_off, const int* __restrict__ bias_tok, const float* __restrict__ bias_val,
    const float* __restrict__ penalty, const float* __restrict__ temperature, const int* __restrict__ counts) {
    __shared__ float seg[PSEG];
    const int b = blockIdx.y, lo = blockIdx.x * PSEG;
    const int n = V - lo < PSEG ? V - lo : PSEG;
    const float* r = logits + (size_t)b * V + lo;
    float* w = work + (size_t)b * V + lo;
    for (int i = threadIdx.x; i < n; i += SBLOCK) seg[i] = r[i];
    if (bias_off) {
        __syncthreads();
        // entries of one row may repeat a token: one thread applies those of this segment in order
        if (threadIdx.x == 0)
            for (int e = bias_off[b]; e < bias_off[b + 1]; ++e) {
                const int tk = bias_tok[e] - lo;
                if (tk >= 0 && tk < n) seg[tk] += bias_val[e];
            }
        __syncthreads();
    }
    const float pen = penalty ? penalty[b] : 1.f;
    const bool penalised = counts && pen != 1.f;
    const int* cn = penalised ? counts + (size_t)b * V + lo : nullptr;
    const float temp = temperature[b];
    for (int i = threadIdx.x; i < n; i += SBLOCK) {
        float v = seg[i];
        if (penalised) {
            const int c_ = cn[i];
            for (int c = 0; c < c_; ++c) v = (v > 0.f) ? v / pen : v * pen;
        }
        if (temp != 0.f) v = v / temp;
        w[i] = v;
    }
}

extern "C" int br_sample_prepare(const float* logits, float* work, int B, int V, const int* bias_off,
                                 const int* bias_tok, const float* bias_val, const int* counts,
                                 const float* penalty, const float* temperature, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (V <= 0 || B > 65535) return BR_BAD_ARG;
    sample_prepare_kernel<<<dim3((V + PSEG - 1) / PSEG, B), SBLOCK, 0, s>>>(logits, work, V, bias_off, bias_tok, bias_val,
                                                                          penalty, temperature, counts);
    return br_check_launch();
}

// counts[row[e], tok[e]] += cnt[e] for n entries (a history put into the table)
__global__ void sample_count_add_kernel(int* __restrict__ counts, int V, const int* __restrict__ row,
                                        const int* __restrict__ tok, const int* __restrict__ cnt, int n) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n && tok[e] >= 0 && tok[e] < V) atomicAdd(counts + (size_t)row[e] * V + tok[e], cnt[e]);
}

extern "C" int br_sample_count_add(int* counts, int B, int V, const int* row, const int* tok, const int* cnt, int n,
                                   hipStream_t s) {
    if (n <= 0) return BR_OK;
    if (!counts || B <= 0 || V <= 0) return BR_BAD_ARG;
    sample_count_add_kernel<<<(n + 255) / 256, 256, 0, s>>>(counts, V, row, tok, cnt, n);
    return br_check_launch();
}

// The first index i in [0, n) at which the running sum of f(0..i) reaches `target` (as
// `target <= sum`), or n.  The sums run in index order: every wave takes a run of consecutive
// indices, 64 at a time with a scan inside the wave and the run's sum carried on; the runs'
// totals, added in wave order, give each run its start.  Two passes over the run (its total,
// then the search) with one barrier between them: no barrier per 64 indices, which is what a
// row of a whole vocabulary would cost otherwise.  Every thread of the block calls it; `wsum`
// holds one float per wave, `found` one int.
template <typename F>
__device__ __forceinline__ int block_first_reach(int n, float target, F f, float* wsum, int* found) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int nblk = (n + 63) >> 6, bpw = (nblk + nw - 1) / nw;
    const int lo = wv * bpw * 64;
    int hi = lo + bpw * 64;
    if (hi > n) hi = n;
    __syncthreads();                  // the caller may still be reading what `wsum` or `found` held
    if (threadIdx.x == 0) *found = 0x7fffffff;
    float run = 0.f;
    for (int i0 = lo; i0 < hi; i0 += 64) {
        const int i = i0 + lane;
        float sc = i < n ? f(i) : 0.f;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) { float t = __shfl_up(sc, o, 64); if (lane >= o) sc += t; }
        run += __shfl(sc, 63, 64);
    }
    if (lane == 0) wsum[wv] = run;
    __syncthreads();
    float acc = 0.f;
    for (int x = 0; x < wv; ++x) acc += wsum[x];
    int first = 0x7fffffff;
    for (int i0 = lo; i0 < hi; i0 += 64) {
        const int i = i0 + lane;
        float sc = i < n ? f(i) : 0.f;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) { float t = __shfl_up(sc, o, 64); if (lane >= o) sc += t; }
        if (i < n && first == 0x7fffffff && target <= acc + sc) first = i;
        acc += __shfl(sc, 63, 64);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { const int t = __shfl_xor(first, o, 64); first = t < first ? t : first; }
    if (lane == 0 && first != 0x7fffffff) atomicMin(found, first);
    __syncthreads();
    const int r = *found;
    __syncthreads();
    return r == 0x7fffffff ? n : r;
}

// ------------------------------------------------- top-k / min-p / top-p filter ----
// Masks entries of work[b, :] to -inf as sampling.rs:89-151 does: top-k keeps the k
// largest; min-p keeps values with exp(v - max) >= min_p; top-p keeps the shortest prefix,
// in descending order, of the survivors whose probabilities (softmax over the survivors)
// sum to >= top_p.  Order is by value, the lower index first among equals.
//
// Nothing is sorted.  Both cuts are "the largest value T such that the entries from T upwards
// weigh at least so much": for top-k an entry weighs 1 and so much is k; for top-p a survivor
// weighs exp(v - max) as a whole number of 2^-40ths and so much is top_p times the survivors'
// total (whole numbers: the sums are exact, whatever the order the atomics add them in).  T
// comes from a radix descent over the value keys, 8 bits a pass, each pass a 256-bin table of
// weights in LDS whose bins four waves scan from the top.  Of the entries equal to T the
// lowest indices are kept, as many as are still needed: found by one count in index order,
// and only when not all of them are.
#define FBLOCK 1024
#define FIL_RESIDENT 32768      // a row of up to so many entries is read once and its value keys kept in LDS

__device__ __forceinline__ unsigned long long comp_key(float v, int i) {
    return ((unsigned long long)f2key(v) << 32) | (uint32_t)(~(uint32_t)i);
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[w] = v;
    __syncthreads();
    float t = -INFINITY;
    for (int i = 0; i < nw; ++i) t = fmaxf(t, scratch[i]);
    return t;
}

__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// weight of a survivor of value v in the top-p cut: exp(v - vmax) in 2^-40ths, at most 2^40
__device__ __forceinline__ unsigned long long mass_of(float v, float vmax) {
    return __float2ull_rn(expf(v - vmax) * 1099511627776.f);
}

template <bool RES>
__global__ __launch_bounds__(FBLOCK) void sample_filter_kernel(
    float* __restrict__ work, int V, const int* __restrict__ top_k, const float* __restrict__ min_p,
    const float* __restrict__ top_p, const float* __restrict__ temperature) {
    __shared__ unsigned long long hist[3 * 256];
    __shared__ unsigned long long wtot[FBLOCK / 64];
    __shared__ float red[16];
    __shared__ int wcnt[FBLOCK / 64];
    __shared__ int sh_idx;
    const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int k = top_k[b];
    const float mp = min_p[b], tp = top_p[b];
    const bool use_k = k > 0 && k < V, use_mp = mp > 0.f, use_tp = tp < 1.f;
    if (temperature[b] == 0.f || !(use_k || use_mp || use_tp)) return;
    float* w = work + (size_t)b * V;
    // wave wv takes the run of bpw * 64 consecutive entries from lo on, 64 at a time: entry j of a lane is
    // i = lo + 64 j + lane; its value key stands in sk[i] (RES) or is made from the row again
    extern __shared__ uint32_t sk[];
    const int nblk = (V + 63) >> 6, bpw = (nblk + FBLOCK / 64 - 1) / (FBLOCK / 64);
    const int lo = wv * bpw * 64;
    if (RES)
        for (int j = 0; j < bpw; ++j) {
            const int i = lo + 64 * j + lane;
            if (i < V) sk[i] = f2key(w[i]);          // read back by the same lane only
        }
#define FIL_ROW(j, i) _Pragma("unroll 4") for (int j = 0; j < bpw; ++j) if (const int i = lo + 64 * j + lane; i < V)
#define FIL_KEY(j, i) (RES ? sk[i] : f2key(w[i]))
    for (int t = tid; t < 3 * 256; t += FBLOCK) hist[t] = 0ull;
    uint32_t kmax = 0;
    FIL_ROW(j, i) { const uint32_t key = FIL_KEY(j, i); kmax = key > kmax ? key : kmax; }
    const float vmax = block_max(key2f(kmax), red);          // its barriers also stand behind the clearing

    // The largest key T such that the entries with pred and a key >= T weigh at least `need` (need >= 1, and
    // all of them together do): T in `pick_T`, what the entries equal to T still have to bring in `pick_rest`
    // (>= 1) and what they weigh together in `pick_at`.  A pass: every thread adds its entries' weights into
    // the pass's table, one barrier, then every wave reads the table for itself (four bins a lane, from the
    // top) and finds the bin.  Three tables in turn, each cleared two passes before it is used, so that the
    // barrier of the pass between stands between the clearing and both its neighbours.
    uint32_t pick_T;
    unsigned long long pick_rest, pick_at;
    int table = 0;                    // the table of the next pass; tables table + 1 and + 2 (mod 3) are clear
#define FIL_PICK(TYPE, PRED, MASS, NEED)                                                                      \
    do {                                                                                                      \
        uint32_t prefix_ = 0, bits_ = 0;                                                                      \
        TYPE need_ = (TYPE)(NEED), at_ = 0;                                                                   \
        for (int shift_ = 24; shift_ >= 0; shift_ -= 8) {                                                     \
            TYPE* h_ = (TYPE*)(hist + 256 * table);                                                           \
            FIL_ROW(j, i) {                                                                                   \
                const uint32_t key = FIL_KEY(j, i);                                                           \
                if ((key & bits_) == prefix_ && (PRED)) atomicAdd(&h_[(key >> shift_) & 255], (TYPE)(MASS));  \
            }                                                                                                 \
            __syncthreads();                                                                                  \
            if (tid < 256) hist[256 * ((table + 2) % 3) + tid] = 0ull;      /* for the pass after the next */ \
            /* lane l reads bins 255 - 4 l down to 252 - 4 l */                                               \
            TYPE b_[4], run_ = 0;                                                                             \
            _Pragma("unroll") for (int q = 0; q < 4; ++q) { b_[q] = h_[255 - 4 * lane - q]; run_ += b_[q]; } \
            TYPE sc_ = run_;                                                                                  \
            _Pragma("unroll") for (int o = 1; o < 64; o <<= 1) {                                              \
                const TYPE t_ = __shfl_up(sc_, o, 64);                                                        \
                if (lane >= o) sc_ += t_;                                                                     \
            }                                                                                                 \
            const unsigned long long m_ = __ballot(sc_ >= need_);                                             \
            const int first_ = m_ ? __ffsll((long long)m_) - 1 : 63;      /* none: the lowest bin */          \
            TYPE above_ = sc_ - run_;                                       /* weight of the bins above this lane's */ \
            int bin_ = 252 - 4 * lane;                                                                        \
            TYPE here_ = b_[3];                                                                               \
            {                                                                                                 \
                TYPE c_ = above_;                                                                             \
                bool done_ = false;                                                                           \
                _Pragma("unroll") for (int q = 0; q < 4; ++q)                                                 \
                    if (!done_ && (c_ + b_[q] >= need_ || q == 3)) {                                          \
                        bin_ = 255 - 4 * lane - q; here_ = b_[q]; above_ = c_; done_ = true;                  \
                    } else if (!done_) c_ += b_[q];                                                           \
            }                                                                                                 \
            bin_ = __shfl(bin_, first_, 64);                                                                  \
            above_ = __shfl(above_, first_, 64);                                                              \
            here_ = __shfl(here_, first_, 64);                                                                \
            prefix_ |= (uint32_t)bin_ << shift_;                                                              \
            bits_ |= 255u << shift_;                                                                          \
            need_ -= above_;                                                                                  \
            at_ = here_;                                                                                      \
            table = (table + 1) % 3;                                                                          \
        }                                                                                                     \
        pick_T = prefix_; pick_rest = need_; pick_at = at_;                                                   \
    } while (0)

    // The index of the n-th entry (n >= 1), in index order, with key T and pred; V if there are fewer.
    int nth_idx;
#define FIL_NTH(PRED, T_, N_)                                                                                 \
    do {                                                                                                      \
        int cnt_ = 0;                                                                                         \
        FIL_ROW(j, i) { const uint32_t key = FIL_KEY(j, i); if (key == (T_) && (PRED)) ++cnt_; }              \
        _Pragma("unroll") for (int o = 32; o > 0; o >>= 1) cnt_ += __shfl_xor(cnt_, o, 64);                   \
        if (lane == 0) wcnt[wv] = cnt_;                                                                       \
        if (tid == 0) sh_idx = V;                                                                             \
        __syncthreads();                                                                                      \
        int before_ = 0;                                                                                      \
        for (int x = 0; x < wv; ++x) before_ += wcnt[x];                                                      \
        if (before_ < (N_) && before_ + cnt_ >= (N_)) {          /* the wave whose run holds it */            \
            for (int j = 0; j < bpw; ++j) {                                                                   \
                {                                                                                             \
                    const int i = lo + 64 * j + lane;                                                         \
                    const uint32_t key = i < V ? FIL_KEY(j, i) : 0u;                                          \
                    const bool f_ = i < V && key == (T_) && (PRED);                                           \
                    const unsigned long long m_ = __ballot(f_);                                               \
                    const int rank_ = before_ + __popcll(m_ & ((1ull << lane) - 1ull));                       \
                    if (f_ && rank_ == (N_) - 1) sh_idx = i;                                                  \
                    before_ += __popcll(m_);                                                                  \
                }                                                                                             \
            }                                                                                                 \
        }                                                                                                     \
        __syncthreads();                                                                                      \
        nth_idx = sh_idx;                                                                                     \
        __syncthreads();                                                                                      \
    } while (0)

    // top-k: the entries above Tk and, of those equal to it, the ones up to index idx_k
    uint32_t Tk = 0;
    int idx_k = V;
    if (use_k) {
        FIL_PICK(unsigned int, true, 1u, k);
        Tk = pick_T;
        if (pick_rest < pick_at) { FIL_NTH(true, Tk, (int)pick_rest); idx_k = nth_idx; }
    }
#define FIL_SURVIVES(key, i)                                                                                 \
    ((!use_k || (key) > Tk || ((key) == Tk && (i) <= idx_k)) && key2f(key) > -INFINITY &&                   \
     !(use_mp && expf(key2f(key) - vmax) < mp))
    if (!use_tp) {
        FIL_ROW(j, i) { const uint32_t key = FIL_KEY(j, i); if (!FIL_SURVIVES(key, i)) w[i] = -INFINITY; }
        return;
    }
    // top-p over the survivors
    unsigned long long part = 0;
    FIL_ROW(j, i) { const uint32_t key = FIL_KEY(j, i); if (FIL_SURVIVES(key, i)) part += mass_of(key2f(key), vmax); }
    part = wave_sum_u64(part);
    __syncthreads();
    if (lane == 0) wtot[wv] = part;
    __syncthreads();
    unsigned long long total = 0;
    for (int x = 0; x < FBLOCK / 64; ++x) total += wtot[x];
    __syncthreads();
    if (total == 0) {                 // nothing survives with any weight (every entry was -inf): mask all
        FIL_ROW(j, i) w[i] = -INFINITY;
        return;
    }
    unsigned long long target = (unsigned long long)ceil((double)tp * (double)total);
    target = target < 1 ? 1 : (target > total ? total : target);
    FIL_PICK(unsigned long long, FIL_SURVIVES(key, i), mass_of(key2f(key), vmax), target);
    const uint32_t Tp = pick_T;
    int idx_p = V;
    {
        const unsigned long long each = mass_of(key2f(Tp), vmax);
        const unsigned long long n = each ? (pick_rest + each - 1) / each : 1ull;
        if (each == 0 || n * each < pick_at) { FIL_NTH(FIL_SURVIVES(key, i), Tp, (int)n); idx_p = nth_idx; }
    }
    FIL_ROW(j, i) {
        const uint32_t key = FIL_KEY(j, i);
        if (!(FIL_SURVIVES(key, i) && (key > Tp || (key == Tp && i <= idx_p)))) w[i] = -INFINITY;
    }
#undef FIL_ROW
#undef FIL_KEY
#undef FIL_PICK
#undef FIL_NTH
#undef FIL_SURVIVES
}

extern "C" int br_sample_filter(float* work, int B, int V, const int* top_k, const float* min_p, const float* top_p,
                                const float* temperature, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (V <= 0) return BR_BAD_ARG;
    if (V <= FIL_RESIDENT) {
        static bool set = false;
        if (!set) {
            if (hipFuncSetAttribute((const void*)sample_filter_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    FIL_RESIDENT * (int)sizeof(uint32_t)) != hipSuccess)
                return BR_LAUNCH_FAILED;
            set = true;
        }
        sample_filter_kernel<true><<<B, FBLOCK, (size_t)V * sizeof(uint32_t), s>>>(work, V, top_k, min_p, top_p, temperature);
    } else {
        sample_filter_kernel<false><<<B, FBLOCK, 0, s>>>(work, V, top_k, min_p, top_p, temperature);
    }
    return br_check_launch();
}

// The same masks the plain way, for tests to hold against the kernel above: the whole row is
// sorted once as 64-bit keys (value key << 32 | ~index) by a bitonic network in `keys`
// ([B, n2], n2 = V rounded up to a power of two), and the probabilities are added in that
// order in float.  With `slow` given, only the rows it flags are treated.
__global__ __launch_bounds__(FBLOCK) void sample_filter_sort_kernel(
    float* __restrict__ work, unsigned long long* __restrict__ keys, int V, int n2,
    const int* __restrict__ top_k, const float* __restrict__ min_p, const float* __restrict__ top_p,
    const float* __restrict__ temperature, const int* __restrict__ slow) {
    __shared__ float red[16];
    __shared__ float wsum[FBLOCK / 64];
    __shared__ int keep_s;
    const int b = blockIdx.x;
    if (slow && !slow[b]) return;
    const int k = top_k[b]; const float mp = min_p[b], tp = top_p[b];
    const bool use_k = k > 0 && k < V, use_mp = mp > 0.f, use_tp = tp < 1.f;
    if (temperature[b] == 0.f || !(use_k || use_mp || use_tp)) return;
    float* w = work + (size_t)b * V;
    unsigned long long* ks = keys + (size_t)b * n2;
    for (int i = threadIdx.x; i < n2; i += FBLOCK) ks[i] = i < V ? comp_key(w[i], i) : 0ull;
    __syncthreads();
    for (int size = 2; size <= n2; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int i = threadIdx.x; i < n2 / 2; i += FBLOCK) {
                const int lo = 2 * i - (i & (stride - 1)), hi = lo + stride;
                const bool desc = (lo & size) == 0;
                unsigned long long a = ks[lo], c = ks[hi];
                if ((a < c) == desc) { ks[lo] = c; ks[hi] = a; }
            }
            __syncthreads();
        }
    }
    int keep = use_k ? k : V;         // survivors are a prefix [0, keep) of the sorted order
    const float vmax = key2f((uint32_t)(ks[0] >> 32));
    float cnt = 0.f, part = 0.f;
    for (int i = threadIdx.x; i < keep; i += FBLOCK) {
        const float v = key2f((uint32_t)(ks[i] >> 32));
        if (v > -INFINITY && !(use_mp && expf(v - vmax) < mp)) { cnt += 1.f; part += expf(v - vmax); }
    }
    keep = (int)(block_sum(cnt, red) + 0.5f);
    const float sum = block_sum(part, red);
    if (use_tp) {
        const int hit = block_first_reach(keep, tp, [&](int i) {
            return expf(key2f((uint32_t)(ks[i] >> 32)) - vmax) / sum; }, wsum, &keep_s);
        if (hit < keep) keep = hit + 1;
    }
    for (int i = keep + threadIdx.x; i < V; i += FBLOCK) w[~(uint32_t)(ks[i] & 0xffffffffu)] = -INFINITY;
}

// every row through the sort (tests)
extern "C" int br_sample_filter_sort(float* work, unsigned long long* keys, int B, int V, int n2, const int* top_k,
                                     const float* min_p, const float* top_p, const float* temperature,
                                     hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (V <= 0 || !keys || n2 < V || (n2 & (n2 - 1))) return BR_BAD_ARG;
    sample_filter_sort_kernel<<<B, FBLOCK, 0, s>>>(work, keys, V, n2, top_k, min_p, top_p, temperature, nullptr);
    return br_check_launch();
}

// ----------------------------------------------------------- softmax + draw --------
// out[b] = first index i with u <= sum_{j<=i} softmax(work[b])_j  (sampling.rs:153-170);
// argmax of the row when temperature is 0 (:81-84) or when rounding leaves u above the
// last partial sum (:170).  Sums run over indices in ascending order (see block_first_reach).
#define DBLOCK 1024
//
// The row's uniform number comes from u[b], or, with `rng_key`, is made here: 24 bits of
// splitmix64(rng_key[b] ^ draw * 0xCA5A826395121157), draw = rng_draw[b], which then goes up by
// one (every call, whatever the temperature): the numbers of sampling/params.py::uniform for
// draws 0, 1, 2, ... of a request, without a copy from the host per step.
__device__ __forceinline__ unsigned long long splitmix64(unsigned long long x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

#define DRAW_K 32      // a row of up to DRAW_K * DBLOCK entries is read once and kept in registers
template <bool REG>
__global__ __launch_bounds__(DBLOCK) void sample_draw_kernel(const float* __restrict__ work, int* __restrict__ out,
                                                             int V, const float* __restrict__ temperature,
                                                             const float* __restrict__ u, int* __restrict__ counts,
                                                             const unsigned long long* __restrict__ rng_key,
                                                             int* __restrict__ rng_draw) {
    __shared__ float red[16];
    __shared__ float wsum[DBLOCK / 64];
    __shared__ int found;
    __shared__ float sv[DBLOCK / 64];
    __shared__ int si[DBLOCK / 64];
    const int b = blockIdx.x;
    const float* w = work + (size_t)b * V;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    // read before the first barrier; thread 0 moves the count on behind it
    const int draw = rng_key ? rng_draw[b] : 0;
    const float ub = rng_key ? (float)(splitmix64(rng_key[b] ^ ((unsigned long long)draw * 0xCA5A826395121157ull)) >> 40) *
                                   (1.f / 16777216.f)
                             : u[b];
    // REG: wave wv holds the run of bpw * 64 consecutive entries from lo on, 64 at a time (the runs of block_first_reach)
    const int nblk = (V + 63) >> 6, bpw = (nblk + DBLOCK / 64 - 1) / (DBLOCK / 64);
    const int lo = wv * bpw * 64;
    float x[DRAW_K];
    // argmax (lowest index wins)
    float bv = -INFINITY; int bi = 0x7fffffff;
    if (REG) {
#pragma unroll
        for (int k = 0; k < DRAW_K; ++k) {
            const int i = lo + k * 64 + lane;
            const bool in = k < bpw && i < V;
            x[k] = in ? w[i] : -INFINITY;
            if (in) argmax_combine(bv, bi, x[k], i);
        }
    } else {
        for (int i = threadIdx.x; i < V; i += DBLOCK) argmax_combine(bv, bi, w[i], i);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        float ov = __shfl_xor(bv, o, 64); int oi = __shfl_xor(bi, o, 64);
        argmax_combine(bv, bi, ov, oi);
    }
    if (lane == 0) { sv[wv] = bv; si[wv] = bi; }
    __syncthreads();
    for (int ww = 0; ww < DBLOCK / 64; ++ww) argmax_combine(bv, bi, sv[ww], si[ww]);
    if (bi == 0x7fffffff) bi = 0;
    if (temperature[b] == 0.f) {
        if (threadIdx.x == 0) {
            out[b] = bi;
            if (counts) counts[(size_t)b * V + bi] += 1;
            if (rng_key) rng_draw[b] = draw + 1;
        }
        return;
    }
    const float vmax = bv;
    float part = 0.f;
    int hit;
    if (REG) {
#pragma unroll
        for (int k = 0; k < DRAW_K; ++k) {
            const bool in = k < bpw && lo + k * 64 + lane < V;
            x[k] = in ? expf(x[k] - vmax) : 0.f;
            part += x[k];
        }
        const float sum = block_sum(part, red);
        // the running sums as in block_first_reach, from the registers
        if (threadIdx.x == 0) found = 0x7fffffff;
        float run = 0.f;
#pragma unroll
        for (int k = 0; k < DRAW_K; ++k)
            if (k < bpw) {
                x[k] = x[k] / sum;
                float sc = x[k];
#pragma unroll
                for (int o = 1; o < 64; o <<= 1) { float t = __shfl_up(sc, o, 64); if (lane >= o) sc += t; }
                run += __shfl(sc, 63, 64);
            }
        if (lane == 0) wsum[wv] = run;
        __syncthreads();
        float acc = 0.f;
        for (int ww = 0; ww < wv; ++ww) acc += wsum[ww];
        int first = 0x7fffffff;
#pragma unroll
        for (int k = 0; k < DRAW_K; ++k)
            if (k < bpw) {
                float sc = x[k];
#pragma unroll
                for (int o = 1; o < 64; o <<= 1) { float t = __shfl_up(sc, o, 64); if (lane >= o) sc += t; }
                const int i = lo + k * 64 + lane;
                if (i < V && first == 0x7fffffff && ub <= acc + sc) first = i;
                acc += __shfl(sc, 63, 64);
            }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) { const int t = __shfl_xor(first, o, 64); first = t < first ? t : first; }
        if (lane == 0 && first != 0x7fffffff) atomicMin(&found, first);
        __syncthreads();
        hit = found == 0x7fffffff ? V : found;
    } else {
        for (int i = threadIdx.x; i < V; i += DBLOCK) part += expf(w[i] - vmax);
        const float sum = block_sum(part, red);
        hit = block_first_reach(V, ub, [&](int i) { return expf(w[i] - vmax) / sum; }, wsum, &found);
    }
    if (threadIdx.x == 0) {
        const int tok = hit < V ? hit : bi;
        out[b] = tok;
        if (counts) counts[(size_t)b * V + tok] += 1;       // the row's history grows by its new token
        if (rng_key) rng_draw[b] = draw + 1;
    }
}

static int launch_draw(const float* work, int* out, int B, int V, const float* temperature, const float* u, int* counts,
                       const unsigned long long* rng_key, int* rng_draw, hipStream_t s) {
    if (V <= DRAW_K * DBLOCK)
        sample_draw_kernel<true><<<B, DBLOCK, 0, s>>>(work, out, V, temperature, u, counts, rng_key, rng_draw);
    else
        sample_draw_kernel<false><<<B, DBLOCK, 0, s>>>(work, out, V, temperature, u, counts, rng_key, rng_draw);
    return br_check_launch();
}

extern "C" int br_sample_draw(const float* work, int* out, int B, int V, const float* temperature,
                              const float* u, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (V <= 0) return BR_BAD_ARG;
    if (!u) return BR_BAD_ARG;
    return launch_draw(work, out, B, V, temperature, u, nullptr, nullptr, nullptr, s);
}

// The same, and counts[b, token drawn] += 1 (the dense history of br_sample_prepare_dense; null: none).
extern "C" int br_sample_draw_count(const float* work, int* out, int B, int V, const float* temperature,
                                    const float* u, int* counts, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (V <= 0) return BR_BAD_ARG;
    if (!u) return BR_BAD_ARG;
    return launch_draw(work, out, B, V, temperature, u, counts, nullptr, nullptr, s);
}

// The same with the uniform numbers made on the device: rng_key[b] (the request's key, see the
// kernel) and rng_draw[b] (its next draw, moved on by the call); counts may be null.
extern "C" int br_sample_draw_random(const float* work, int* out, int B, int V, const float* temperature,
                                     const unsigned long long* rng_key, int* rng_draw, int* counts, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (V <= 0 || !rng_key || !rng_draw) return BR_BAD_ARG;
    return launch_draw(work, out, B, V, temperature, nullptr, counts, rng_key, rng_draw, s);
}

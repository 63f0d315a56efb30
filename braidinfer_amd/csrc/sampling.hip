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
// sum to >= top_p.  Order is by value, the lower index first among equals: every entry
// has a 64-bit key (value key << 32 | ~index), all distinct, and "kept" is "key >= some
// key", so the mask is one pass once that key is known.
//
// sample_filter_select_kernel finds it without sorting the row: a radix select over the
// value keys picks the (at most 1024) largest entries, which are sorted in LDS; top-k,
// min-p and top-p are then decided on that short list.  A row it cannot decide there
// (top_k above 1024, or no top-k and a top-p that the 1024 largest do not reach) is
// flagged in `slow` and left untouched for sample_filter_sort_kernel, which sorts the
// whole row in global memory.
#define FBLOCK 1024
#define CAND 1024

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

#define SEL_K 32       // a row of up to SEL_K * FBLOCK entries is read once and its keys kept in registers
template <bool REG>
__global__ __launch_bounds__(FBLOCK) void sample_filter_select_kernel(
    float* __restrict__ work, int V, const int* __restrict__ top_k, const float* __restrict__ min_p,
    const float* __restrict__ top_p, const float* __restrict__ temperature, int* __restrict__ slow) {
    __shared__ unsigned long long ck[CAND];
    __shared__ int hist[256];
    __shared__ float red[16];
    __shared__ float wsum[FBLOCK / 64];
    __shared__ int sh_bin, sh_need, sh_ties, sh_cnt, keep_s;
    __shared__ int wtot[4];
    const int b = blockIdx.x, tid = threadIdx.x;
    const int k = top_k[b];
    const float mp = min_p[b], tp = top_p[b];
    const bool use_k = k > 0 && k < V, use_mp = mp > 0.f, use_tp = tp < 1.f;
    if (tid == 0) slow[b] = 0;
    if (temperature[b] == 0.f || !(use_k || use_mp || use_tp)) return;
    if (use_k && k > CAND) { if (tid == 0) slow[b] = 1; return; }
    float* w = work + (size_t)b * V;
    // entry j of this thread is i = j * FBLOCK + tid; its value key stands in kx[j] (REG) or is read again
    const int per = (V + FBLOCK - 1) / FBLOCK;
    uint32_t kx[SEL_K];
    if (REG) {
#pragma unroll
        for (int j = 0; j < SEL_K; ++j) {
            const int i = j * FBLOCK + tid;
            kx[j] = i < V ? f2key(w[i]) : 0u;
        }
    }
#define SEL_ROW(j, i) _Pragma("unroll") for (int j = 0; j < (REG ? SEL_K : per); ++j) if (const int i = j * FBLOCK + tid; i < V)
#define SEL_KEY(j, i) (REG ? kx[j] : f2key(w[i]))
    uint32_t kmax = 0;
    SEL_ROW(j, i) { const uint32_t key = SEL_KEY(j, i); kmax = key > kmax ? key : kmax; }
    const float vmax = block_max(key2f(kmax), red);
    if (!use_k && !use_tp) {          // min-p alone is a threshold on the value
        SEL_ROW(j, i) {
            const float v = key2f(SEL_KEY(j, i));
            if (v > -INFINITY && expf(v - vmax) < mp) w[i] = -INFINITY;
        }
        return;
    }
    const int cand = use_k ? k : (V < CAND ? V : CAND);
    // radix select: the value key T of the cand-th largest entry, 8 bits a pass
    uint32_t prefix = 0, bits = 0;
    int need = cand, ties = 0;
    for (int shift = 24; shift >= 0; shift -= 8) {
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        SEL_ROW(j, i) {
            const uint32_t key = SEL_KEY(j, i);
            if ((key & bits) == prefix) atomicAdd(&hist[(key >> shift) & 255], 1);
        }
        __syncthreads();
        // the highest bin at which the count from the top reaches `need` (bin 0 if none does): thread t
        // of the first four waves stands for bin 255 - t and scans the counts from the top
        const int lane = tid & 63, wv = tid >> 6;
        int h = 0, sc = 0;
        if (tid < 256) {
            h = hist[255 - tid];
            sc = h;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) { int t = __shfl_up(sc, o, 64); if (lane >= o) sc += t; }
            if (lane == 63) wtot[wv] = sc;
        }
        if (tid == 0) sh_bin = 255;
        __syncthreads();
        if (tid < 256) {
            for (int x = 0; x < wv; ++x) sc += wtot[x];
            const unsigned long long m = __ballot(sc >= need);
            if (m && lane == __ffsll((long long)m) - 1) atomicMin(&sh_bin, tid);
        }
        __syncthreads();
        if (tid == sh_bin) { sh_need = need - (sc - h); sh_ties = h; }
        __syncthreads();
        const int bin = 255 - sh_bin;
        prefix |= (uint32_t)bin << shift;
        bits |= 255u << shift;
        need = sh_need;
        ties = sh_ties;
        __syncthreads();
    }
    const uint32_t T = prefix;        // take every key above T and `need` of the `ties` keys equal to it
    if (tid == 0) sh_cnt = 0;
    __syncthreads();
    SEL_ROW(j, i) {
        const uint32_t key = SEL_KEY(j, i);
        if (key > T) ck[atomicAdd(&sh_cnt, 1)] = ((unsigned long long)key << 32) | (uint32_t)(~(uint32_t)i);
    }
    __syncthreads();
    const int ngt = sh_cnt;
    if (ties == need) {
        SEL_ROW(j, i) {
            const uint32_t key = SEL_KEY(j, i);
            if (key == T) ck[atomicAdd(&sh_cnt, 1)] = ((unsigned long long)key << 32) | (uint32_t)(~(uint32_t)i);
        }
    } else {
        // more equal values than places: the lowest indices win, found by an ordered scan
        const int lane = tid & 63, wv = tid >> 6;
        int base = 0;
        for (int j = 0; j < per && base < need; ++j) {
            const int i = j * FBLOCK + tid;
            const int flag = (i < V && f2key(w[i]) == T) ? 1 : 0;
            int sc = flag;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) { int t = __shfl_up(sc, o, 64); if (lane >= o) sc += t; }
            __syncthreads();
            if (lane == 63) hist[wv] = sc;
            __syncthreads();
            int before = base, tot = base;
            for (int x = 0; x < FBLOCK / 64; ++x) { if (x < wv) before += hist[x]; tot += hist[x]; }
            const int rank = before + sc - flag;
            if (flag && rank < need) ck[ngt + rank] = ((unsigned long long)T << 32) | (uint32_t)(~(uint32_t)i);
            base = tot;
            __syncthreads();
        }
    }
    // bitonic sort of the candidates in LDS, descending, over the least power of two that holds them
    int sortn = 64;
    while (sortn < cand) sortn <<= 1;
    for (int t = cand + tid; t < sortn; t += FBLOCK) ck[t] = 0ull;
    __syncthreads();
    for (int size = 2; size <= sortn; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            if (tid < sortn / 2) {
                const int lo = 2 * tid - (tid & (stride - 1)), hi = lo + stride;
                const bool desc = (lo & size) == 0;
                const unsigned long long a = ck[lo], c = ck[hi];
                if ((a < c) == desc) { ck[lo] = c; ck[hi] = a; }
            }
            __syncthreads();
        }
    }
    // survivors are a prefix [0, keep) of the candidates
    int keep = cand;
    float cnt = 0.f, part = 0.f;
    for (int i = tid; i < cand; i += FBLOCK) {
        const float v = key2f((uint32_t)(ck[i] >> 32));
        if (v > -INFINITY && !(use_mp && expf(v - vmax) < mp)) { cnt += 1.f; part += expf(v - vmax); }
    }
    keep = (int)(block_sum(cnt, red) + 0.5f);
    float sum = block_sum(part, red);
    bool covered = true;              // do the candidates hold every survivor?
    if (!use_k) {
        // without top-k the survivors are all entries that pass min-p: count and add them all
        float call = 0.f, pall = 0.f;
        SEL_ROW(j, i) {
            const float v = key2f(SEL_KEY(j, i));
            if (v > -INFINITY && !(use_mp && expf(v - vmax) < mp)) { call += 1.f; pall += expf(v - vmax); }
        }
        covered = (int)(block_sum(call, red) + 0.5f) <= keep;
        sum = block_sum(pall, red);
    }
    if (use_tp) {
        const int hit = block_first_reach(keep, tp, [&](int i) {
            return expf(key2f((uint32_t)(ck[i] >> 32)) - vmax) / sum; }, wsum, &keep_s);
        if (hit < keep) keep = hit + 1;
        else if (!covered) { if (tid == 0) slow[b] = 1; return; }
    }
    const unsigned long long last = ck[keep - 1];
    SEL_ROW(j, i) {
        if ((((unsigned long long)SEL_KEY(j, i) << 32) | (uint32_t)(~(uint32_t)i)) < last) w[i] = -INFINITY;
    }
#undef SEL_ROW
#undef SEL_KEY
}

static int launch_filter_select(float* work, int B, int V, const int* top_k, const float* min_p, const float* top_p,
                                const float* temperature, int* slow, hipStream_t s) {
    if (V <= SEL_K * FBLOCK)
        sample_filter_select_kernel<true><<<B, FBLOCK, 0, s>>>(work, V, top_k, min_p, top_p, temperature, slow);
    else
        sample_filter_select_kernel<false><<<B, FBLOCK, 0, s>>>(work, V, top_k, min_p, top_p, temperature, slow);
    return br_check_launch();
}

// The general form: the whole row is sorted once as 64-bit keys by a bitonic network in
// `keys` ([B, n2], n2 = V rounded up to a power of two).  With `slow` given, only the rows
// it flags are treated.
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

// The general form for rows of up to LDS_SORT_MAX entries (padded to a power of two): only the
// 32-bit value keys are sorted, in LDS.  The values in descending order are what the running
// sum needs; which entries are kept follows from the last kept value T and from how many
// entries equal to T are among the kept: those with the lowest indices, found by one scan in
// index order.  The same masks as the sort of 64-bit keys in global memory, about twenty
// times sooner at 32,768 entries.
#define LDS_SORT_MAX 32768
__global__ __launch_bounds__(FBLOCK) void sample_filter_sort_lds_kernel(
    float* __restrict__ work, int V, int n2, const int* __restrict__ top_k, const float* __restrict__ min_p,
    const float* __restrict__ top_p, const float* __restrict__ temperature, const int* __restrict__ slow) {
    extern __shared__ uint32_t sk[];
    __shared__ float red[16];
    __shared__ float wsum[FBLOCK / 64];
    __shared__ int wcnt[FBLOCK / 64];
    __shared__ int keep_s, last_s;
    const int b = blockIdx.x, tid = threadIdx.x;
    if (slow && !slow[b]) return;
    const int k = top_k[b]; const float mp = min_p[b], tp = top_p[b];
    const bool use_k = k > 0 && k < V, use_mp = mp > 0.f, use_tp = tp < 1.f;
    if (temperature[b] == 0.f || !(use_k || use_mp || use_tp)) return;
    float* w = work + (size_t)b * V;
    for (int i = tid; i < n2; i += FBLOCK) sk[i] = i < V ? f2key(w[i]) : 0u;
    __syncthreads();
    for (int size = 2; size <= n2; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int i = tid; i < n2 / 2; i += FBLOCK) {
                const int lo = 2 * i - (i & (stride - 1)), hi = lo + stride;
                const bool desc = (lo & size) == 0;
                const uint32_t a = sk[lo], c = sk[hi];
                if ((a < c) == desc) { sk[lo] = c; sk[hi] = a; }
            }
            __syncthreads();
        }
    }
    int keep = use_k ? k : V;         // survivors are a prefix [0, keep) of the sorted order
    const float vmax = key2f(sk[0]);
    float cnt = 0.f, part = 0.f;
    for (int i = tid; i < keep; i += FBLOCK) {
        const float v = key2f(sk[i]);
        if (v > -INFINITY && !(use_mp && expf(v - vmax) < mp)) { cnt += 1.f; part += expf(v - vmax); }
    }
    keep = (int)(block_sum(cnt, red) + 0.5f);
    const float sum = block_sum(part, red);
    if (use_tp) {
        const int hit = block_first_reach(keep, tp, [&](int i) { return expf(key2f(sk[i]) - vmax) / sum; }, wsum, &keep_s);
        if (hit < keep) keep = hit + 1;
    }
    if (keep <= 0) {                  // nothing survives (every entry was -inf): mask all, as the sort of whole keys does
        for (int i = tid; i < V; i += FBLOCK) w[i] = -INFINITY;
        return;
    }
    const uint32_t T = sk[keep - 1];
    // entries above T come first in the order: their number by bisection, the same in every thread
    int lo = 0, hi = keep - 1;        // sk[hi] == T; find the first index with sk[i] == T
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (sk[mid] > T) lo = mid + 1; else hi = mid;
    }
    const int need = keep - lo;       // kept entries equal to T: the `need` lowest indices among the equals
    if (tid == 0) last_s = V;
    __syncthreads();
    const int lane = tid & 63, wv = tid >> 6;
    int base = 0;
    for (int i0 = 0; i0 < V && base < need; i0 += FBLOCK) {
        const int i = i0 + tid;
        const int flag = (i < V && f2key(w[i]) == T) ? 1 : 0;
        int sc = flag;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) { int t = __shfl_up(sc, o, 64); if (lane >= o) sc += t; }
        __syncthreads();
        if (lane == 63) wcnt[wv] = sc;
        __syncthreads();
        int before = base, tot = base;
        for (int x = 0; x < FBLOCK / 64; ++x) { if (x < wv) before += wcnt[x]; tot += wcnt[x]; }
        if (flag && before + sc == need) last_s = i;         // the last kept one among the equals
        base = tot;
        __syncthreads();
    }
    __syncthreads();
    const int last = last_s;
    for (int i = tid; i < V; i += FBLOCK) {
        const uint32_t key = f2key(w[i]);
        if (key < T || (key == T && i > last)) w[i] = -INFINITY;
    }
}

static int launch_filter_sort(float* work, unsigned long long* keys, int B, int V, int n2, const int* top_k,
                              const float* min_p, const float* top_p, const float* temperature, const int* slow,
                              int in_lds, hipStream_t s) {
    if (in_lds) {
        const size_t lds = (size_t)n2 * sizeof(uint32_t);
        static bool set = false;
        if (!set) {
            if (hipFuncSetAttribute((const void*)sample_filter_sort_lds_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    LDS_SORT_MAX * (int)sizeof(uint32_t)) != hipSuccess)
                return BR_LAUNCH_FAILED;
            set = true;
        }
        sample_filter_sort_lds_kernel<<<B, FBLOCK, lds, s>>>(work, V, n2, top_k, min_p, top_p, temperature, slow);
    } else {
        sample_filter_sort_kernel<<<B, FBLOCK, 0, s>>>(work, keys, V, n2, top_k, min_p, top_p, temperature, slow);
    }
    return br_check_launch();
}

// slow: int [B] scratch.  keys: [B, n2] scratch, needed only when `with_sort` (some row may
// take the general form: top_k above 1024, or top-p without top-k) and n2 is beyond
// LDS_SORT_MAX (shorter rows are sorted in LDS).
extern "C" int br_sample_filter(float* work, unsigned long long* keys, int B, int V, int n2, const int* top_k,
                                const float* min_p, const float* top_p, const float* temperature, int* slow,
                                int with_sort, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (V <= 0 || !slow || (with_sort && (n2 < V || (n2 & (n2 - 1)) || (n2 > LDS_SORT_MAX && !keys)))) return BR_BAD_ARG;
    int rc = launch_filter_select(work, B, V, top_k, min_p, top_p, temperature, slow, s);
    if (rc != BR_OK || !with_sort) return rc;
    return launch_filter_sort(work, keys, B, V, n2, top_k, min_p, top_p, temperature, slow, n2 <= LDS_SORT_MAX, s);
}

// the general form alone, for every row (tests compare the forms): in_lds 0 sorts whole keys in
// `keys`, 1 the value keys in LDS (n2 up to LDS_SORT_MAX; `keys` is not used)
extern "C" int br_sample_filter_sort(float* work, unsigned long long* keys, int B, int V, int n2, const int* top_k,
                                     const float* min_p, const float* top_p, const float* temperature, int in_lds,
                                     hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (V <= 0 || n2 < V || (n2 & (n2 - 1)) || (in_lds ? n2 > LDS_SORT_MAX : !keys)) return BR_BAD_ARG;
    return launch_filter_sort(work, keys, B, V, n2, top_k, min_p, top_p, temperature, nullptr, in_lds, s);
}

extern "C" int br_sample_lds_sort_max() { return LDS_SORT_MAX; }

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

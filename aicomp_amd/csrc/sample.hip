// Token sampling: temperature -> top-k -> top-p (nucleus) -> multinomial, one launch.
//
// Replaces the step after the attention path,
//   opt_prime/opt_prime/inference.py:786-843 (_sample_token):
//     logits / temperature; remove logits < k-th largest; sort descending, cumulative
//     softmax, remove entries whose preceding cumulative mass exceeds top_p (the first
//     entry always stays); softmax of what is left; torch.multinomial
// which in PyTorch is a full-vocabulary sort plus about ten elementwise / scan launches
// per token.  Greedy decoding (do_sample == False, :806-808) is the argmax.
//
// One workgroup of 1024 lanes per row; nothing is sorted.
//   1  row maximum and argmax on the raw logits (a positive temperature keeps the order)
//   2  top-k (k <= 1024, the usual case): the k-th largest of the 1024 per-lane maxima bounds the
//      row's k-th largest value from below, so a second pass over the row collects the
//      candidates (about k) into LDS; selection of the k-th value, the nucleus threshold and the
//      draw then run on that list.  Two passes over the row in total, neither dividing nor
//      exponentiating more than the candidates.
//   2' without top-k, or when the candidates do not fit (masses of equal logits): radix select
//      over the whole row on order-preserving integer keys (digits of 11, 11 and 10 bits, count
//      histograms in LDS), nucleus threshold by the same walk over MASS histograms, and a draw
//      located by wave segment, lane chunk and element.
// Probability mass is carried as 2^-40 fixed point in 64-bit integers, so every sum is
// exact, order independent and reproducible; ties at the nucleus threshold are kept in
// index order (what a stable descending sort would do).
//
// Not HBM-bound: a row (128 K logits = 512 KB in fp32) belongs to one CU, whose instruction
// rate bounds a pass; the full-row histogram passes are LDS-atomic bound when many logits
// share the leading key bits.
#include "common.h"

#include <type_traits>

namespace aicomp {

namespace {

constexpr int NT = 1024;                 // lanes per workgroup
constexpr int NW = NT / 64;              // waves
constexpr int BINS = 2048;
constexpr int LIST_CAP = 4096;          // candidate list of the top-k fast path (64 KB of LDS with weights)
constexpr uint32_t LIST_SLACK = 64;      // raw values below the bound that may still tie with it after the division
constexpr float LIST_MAX_TEMPERATURE = 32.f;   // at most ~T+1 raw values share a quotient: 64 covers this
constexpr float W_ONE = 1099511627776.f; // 2^40: weight of the row maximum

struct SampleParams {
    int64_t* out;                        // [B] token ids
    const void* logits;                  // [B, V]
    int64_t row_stride;                  // elements
    float* probs_out;                    // optional [B, V]: the distribution drawn from
    const float* uniforms;               // [B] in [0, 1)
    int vocab;
    float temperature;
    int top_k;                           // <= 0 or >= V: off
    float top_p;                         // >= 1: off
    int greedy;
};

// float -> key with the same order (larger float, larger key).  -0.0 gets the key of +0.0: the
// reference compares floats (`logits < kth`), for which the two zeros are one value.
__device__ __forceinline__ uint32_t order_key(float x) {
    uint32_t b = __float_as_uint(x);
    if (b == 0x80000000u) b = 0u;
    return b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
    const uint32_t b = (k & 0x80000000u) ? (k ^ 0x80000000u) : ~k;
    return __uint_as_float(b);
}

template <typename T>
__device__ __forceinline__ float scaled_logit(const T* row, int i, float temperature);
template <>
__device__ __forceinline__ float scaled_logit<float>(const float* row, int i, float temperature) {
    return temperature == 1.f ? row[i] : row[i] / temperature;
}
template <>
__device__ __forceinline__ float scaled_logit<bf16_t>(const bf16_t* row, int i, float temperature) {
    const float x = bf16_to_f32(row[i].bits);
    // the division of a bf16 tensor is rounded back to bf16, as the eager division is
    return temperature == 1.f ? x : (float)(__bf16)(x / temperature);
}

template <>
__device__ __forceinline__ float scaled_logit<f16_t>(const f16_t* row, int i, float temperature) {
    const float x = f16_to_f32(row[i].bits);
    return temperature == 1.f ? x : (float)(_Float16)(x / temperature);
}

// four consecutive logits in one load (16 bytes of fp32, 8 bytes of bf16 / fp16)
template <typename T> struct Load4;
template <> struct Load4<float> {
    __device__ __forceinline__ static void get(const float* p, float* x) {
        const float4 v = *(const float4*)p;
        x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    }
};
template <> struct Load4<bf16_t> {
    __device__ __forceinline__ static void get(const bf16_t* p, float* x) {
        const uint2 v = *(const uint2*)p;
        x[0] = __uint_as_float(v.x << 16); x[1] = __uint_as_float(v.x & 0xffff0000u);
        x[2] = __uint_as_float(v.y << 16); x[3] = __uint_as_float(v.y & 0xffff0000u);
    }
};
template <> struct Load4<f16_t> {
    __device__ __forceinline__ static void get(const f16_t* p, float* x) {
        const uint2 v = *(const uint2*)p;
        x[0] = f16_to_f32((uint16_t)(v.x & 0xffffu)); x[1] = f16_to_f32((uint16_t)(v.x >> 16));
        x[2] = f16_to_f32((uint16_t)(v.y & 0xffffu)); x[3] = f16_to_f32((uint16_t)(v.y >> 16));
    }
};
// For fp16 rows: a raw value below which the scaled, rounded logit is certainly below `q_scaled`.
// A quotient rounds up by at most half a unit in the last place of the result, 2^-25 in fp16's
// subnormal range, so everything from q - max(2^-24, |q| 2^-10) up may still reach q; the
// float division adds a relative 2^-24.  Other types: +inf (no extra lowering).
template <typename T> __device__ __forceinline__ float f16_raw_bound(float q_scaled, float temperature) {
    if constexpr (std::is_same<T, f16_t>::value) {
        const float y = (q_scaled - fmaxf(5.9604645e-8f, fabsf(q_scaled) * 9.765625e-4f)) * temperature;
        return y - fabsf(y) * 9.5367431640625e-7f;
    } else {
        (void)q_scaled; (void)temperature;
        return 0.f;                                    // not used for the other types
    }
}
template <typename T> __device__ __forceinline__ float apply_temperature(float x, float temperature);
template <> __device__ __forceinline__ float apply_temperature<float>(float x, float temperature) {
    return temperature == 1.f ? x : x / temperature;
}
template <> __device__ __forceinline__ float apply_temperature<bf16_t>(float x, float temperature) {
    return temperature == 1.f ? x : (float)(__bf16)(x / temperature);
}
template <> __device__ __forceinline__ float apply_temperature<f16_t>(float x, float temperature) {
    return temperature == 1.f ? x : (float)(_Float16)(x / temperature);
}

// f(index, scaled logit) over the elements [begin, end) owned by `rank` of `nranks` lanes.
// With 16-byte aligned rows a lane takes four consecutive elements per load and keeps eight
// loads in flight; each lane visits its elements in ascending index order.
template <typename T, typename F>
__device__ __forceinline__ void for_each_logit(const T* row, int begin, int end, float temperature,
                                               int rank, int nranks, bool vec_ok, F f) {
    int tail = begin;
    if (vec_ok) {
        const int n4 = (end - begin) / 4;              // begin is a multiple of 4 for every caller
        constexpr int U = 16;                          // loads in flight per lane: the passes are latency bound
        for (int j0 = rank; j0 < n4; j0 += U * nranks) {
            float a[U][4];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = j0 + u * nranks;
                Load4<T>::get(row + begin + 4 * (j < n4 ? j : j0), a[u]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = j0 + u * nranks;
                if (j < n4) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) f(begin + 4 * j + e, apply_temperature<T>(a[u][e], temperature));
                }
            }
        }
        tail = begin + 4 * n4;
    }
    for (int i = tail + rank; i < end; i += nranks) f(i, scaled_logit<T>(row, i, temperature));
}

// 2^-40 fixed-point weight exp(x - m) of a logit (x <= m, so the weight is in [0, 1]): the hardware
// exponential, then the two 32-bit halves of w * 2^40 from two float -> uint32 conversions (a
// float -> uint64 conversion is a long instruction sequence, and this runs once per logit in the
// full-row passes).  A NaN logit gets weight 0.
__device__ __forceinline__ uint64_t weight_of(float x, float m) {
    const float w = __builtin_amdgcn_exp2f((x - m) * LOG2E);
    const float s8 = w * 256.f;                                  // exact scaling, [0, 256]
    const float hi_f = floorf(s8);
    const uint32_t hi = (uint32_t)hi_f;                          // w * 2^8, integer part
    const uint32_t lo = (uint32_t)((s8 - hi_f) * 4294967296.f);  // fraction * 2^32 (the difference is exact)
    return ((uint64_t)hi << 32) | lo;
}

__device__ __forceinline__ uint64_t shfl64(uint64_t v, int src) {
    const uint32_t lo = __shfl((uint32_t)v, src), hi = __shfl((uint32_t)(v >> 32), src);
    return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ uint64_t shfl_up64(uint64_t v, int d) {
    const uint32_t lo = __shfl_up((uint32_t)v, d), hi = __shfl_up((uint32_t)(v >> 32), d);
    return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ uint64_t wave_sum64(uint64_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const uint32_t lo = __shfl_xor((uint32_t)v, o), hi = __shfl_xor((uint32_t)(v >> 32), o);
        v += ((uint64_t)hi << 32) | lo;
    }
    return v;
}
__device__ __forceinline__ uint64_t wave_incl_scan64(uint64_t v, int lane) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint64_t o = shfl_up64(v, d);
        if (lane >= d) v += o;
    }
    return v;
}

// Shared state of the radix walks (one row)
struct Shared {
    alignas(16) unsigned long long mass[BINS];
    alignas(16) unsigned int cnt[BINS];
    unsigned long long seg_mass[NW];
    unsigned int seg_tied[NW];
    float red_f[NW];
    int red_i[NW];
    // results broadcast by wave 0
    unsigned int sel_digit;
    unsigned long long sel_above_mass;
    unsigned int sel_above_cnt;
    // candidates of the top-k fast path
    unsigned int n_list;
    alignas(16) unsigned int list_key[LIST_CAP];
    alignas(16) unsigned int list_idx[LIST_CAP];
    alignas(16) unsigned long long list_w[LIST_CAP];
};

// Wave 0: walking the bins from the top, find the bin that holds the k-th element
// (by count).  Returns digit and the count strictly above it.
__device__ void pick_by_count(Shared& s, int nbins, unsigned int k, int lane) {
    // lane owns bins [hi - 32*lane - 31, hi - 32*lane], i.e. lane 0 the top 32 bins: read as eight
    // 16-byte vectors (independent loads; a dependent chain of 32 LDS reads costs microseconds)
    constexpr int per = BINS / 64;
    const int top = nbins - 1 - lane * per;            // highest bin of this lane; nbins is a multiple of per
    unsigned int c[per];                               // c[j] = count of bin top - j
    if (top >= per - 1) {
        const uint4* v = (const uint4*)&s.cnt[top - (per - 1)];
#pragma unroll
        for (int q = 0; q < per / 4; ++q) {
            const uint4 x = v[q];
            c[per - 1 - 4 * q] = x.x; c[per - 2 - 4 * q] = x.y; c[per - 3 - 4 * q] = x.z; c[per - 4 - 4 * q] = x.w;
        }
    } else {
#pragma unroll
        for (int j = 0; j < per; ++j) c[j] = 0;
    }
    unsigned int local = 0;
#pragma unroll
    for (int j = 0; j < per; ++j) local += c[j];
    unsigned int incl = local;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const unsigned int o = __shfl_up(incl, d);
        if (lane >= d) incl += o;
    }
    const unsigned int excl = incl - local;
    // first lane (from the top) whose inclusive count reaches k
    const unsigned long long hit = __ballot(incl >= k);
    const int owner = hit ? __ffsll((long long)hit) - 1 : 63;
    if (lane == owner) {
        unsigned int run = excl;
        int chosen = 0;
        unsigned int above = excl;
        bool done = false;
#pragma unroll
        for (int j = 0; j < per; ++j) {
            if (!done && top - j >= 0) {
                chosen = top - j;
                above = run;
                run += c[j];
                done = run >= k;
            }
        }
        s.sel_digit = (unsigned int)chosen;
        s.sel_above_cnt = above;
    }
}

// Wave 0: lowest bin d with mass(bins > d) <= limit.  Returns digit and that mass.
__device__ void pick_by_mass(Shared& s, int nbins, unsigned long long limit, int lane) {
    const int per = BINS / 64;
    unsigned long long local = 0;
    for (int j = 0; j < per; ++j) {
        const int b = nbins - 1 - (lane * per + j);
        if (b >= 0) local += s.mass[b];
    }
    const unsigned long long incl = wave_incl_scan64(local, lane);
    const unsigned long long excl = incl - local;
    // mass above the LAST bin of a lane's range is incl - mass[last]; the walk continues past a
    // lane while even the mass above the first bin of the next lane (= incl) is <= limit
    const unsigned long long cont = __ballot(incl <= limit);
    // owner: first lane from the top for which incl > limit (the walk stops inside it); if none, the last lane
    const unsigned long long stop = ~cont;
    const int last_lane = nbins / per - 1;        // lanes beyond it own no bins
    int owner = stop ? __ffsll((long long)stop) - 1 : 63;
    if (owner > last_lane) owner = last_lane;
    if (lane == owner) {
        unsigned long long above = excl;          // mass above the current bin
        int chosen = nbins - 1 - lane * per;
        for (int j = 0; j < per; ++j) {
            const int b = nbins - 1 - (lane * per + j);
            if (b < 0) break;
            if (above > limit) break;             // cannot happen at j == 0 (excl <= limit for the owner)
            chosen = b;
            s.sel_above_mass = above;
            above += s.mass[b];
        }
        s.sel_digit = (unsigned int)chosen;
    }
}

constexpr int SHIFTS[3] = {21, 10, 0};
constexpr int WIDTHS[3] = {11, 11, 10};

// Key of the k-th largest element of a source (all lanes call; `src(f)` runs f(index, value) over
// the lane's share of the elements).  Three histogram rounds over digits of 11, 11 and 10 bits.
// With fewer than three levels the result is the lower edge of the bin that holds the k-th largest
// element at that resolution: a lower bound of its key.
template <typename Src>
__device__ __forceinline__ uint32_t select_kth(Shared& s, Src src, unsigned int k, int tid, int lane, int wave,
                                               int levels = 3) {
    uint32_t prefix = 0, pmask = 0;
    for (int lvl = 0; lvl < levels; ++lvl) {
        const int nb = 1 << WIDTHS[lvl];
        const int sh = SHIFTS[lvl];
        __syncthreads();
        for (int b = tid; b < BINS; b += NT) s.cnt[b] = 0;
        __syncthreads();
        src([&](int, float x) {
            const uint32_t key = order_key(x);
            if ((key & pmask) == prefix) atomicAdd(&s.cnt[(key >> sh) & (nb - 1)], 1u);
        });
        __syncthreads();
        if (wave == 0) pick_by_count(s, nb, k, lane);
        __syncthreads();
        k -= s.sel_above_cnt;
        prefix |= s.sel_digit << sh;
        pmask |= (uint32_t)(nb - 1) << sh;
    }
    return prefix;
}

struct Nucleus {
    uint32_t key_t;              // keep key > key_t ...
    unsigned int tie_keep;       // ... plus the first tie_keep elements (index order) with key == key_t
    bool tie_rule;               // false: keep every key >= key_t
};

// Nucleus threshold over the elements with key >= key_k: the same radix walk on mass histograms.
template <typename Src>
__device__ __forceinline__ Nucleus nucleus_threshold(Shared& s, Src src, uint32_t key_k, float m, float top_p,
                                                     int tid, int lane, int wave, int first_level = 0,
                                                     uint32_t prefix0 = 0, uint32_t pmask0 = 0,
                                                     unsigned long long limit0 = 0) {
    // first_level > 0: the caller has already walked the upper digit levels (prefix, mask and what is
    // left of the mass limit below the bins above the chosen one)
    uint32_t prefix = prefix0, pmask = pmask0;
    unsigned long long limit = limit0;
    for (int lvl = first_level; lvl < 3; ++lvl) {
        const int nb = 1 << WIDTHS[lvl];
        const int sh = SHIFTS[lvl];
        __syncthreads();
        for (int b = tid; b < BINS; b += NT) { s.mass[b] = 0; s.cnt[b] = 0; }
        __syncthreads();
        src([&](int, float x) {
            const uint32_t key = order_key(x);
            if (key >= key_k && (key & pmask) == prefix) {
                const int b = (key >> sh) & (nb - 1);
                atomicAdd(&s.mass[b], (unsigned long long)weight_of(x, m));
                atomicAdd(&s.cnt[b], 1u);
            }
        });
        __syncthreads();
        if (lvl == 0) {
            // total mass after top-k: sum of the first-level bins (every kept element is in one)
            unsigned long long z = 0;
            for (int b = tid; b < BINS; b += NT) z += s.mass[b];
            z = wave_sum64(z);
            if (lane == 0) s.seg_mass[wave] = z;
            __syncthreads();
            z = 0;
            for (int w = 0; w < NW; ++w) z += s.seg_mass[w];
            limit = (unsigned long long)((double)fmaxf(top_p, 0.f) * (double)z);
            __syncthreads();
        }
        if (wave == 0) pick_by_mass(s, nb, limit, lane);
        __syncthreads();
        limit -= s.sel_above_mass;
        prefix |= s.sel_digit << sh;
        pmask |= (uint32_t)(nb - 1) << sh;
    }
    // the last chosen bin holds exactly the elements with key == prefix
    const unsigned int n_t = s.cnt[s.sel_digit];
    const unsigned long long m_t = s.mass[s.sel_digit];
    Nucleus r;
    r.key_t = prefix;
    r.tie_rule = true;
    if (n_t == 0) r.tie_keep = 0;
    else {
        const unsigned long long w_t = m_t / n_t;              // identical keys, identical weights
        const unsigned long long c = w_t ? limit / w_t + 1 : (unsigned long long)n_t;
        r.tie_keep = (unsigned int)(c < n_t ? c : n_t);
    }
    if (r.key_t < key_k) { r.key_t = key_k; r.tie_rule = false; r.tie_keep = 0xffffffffu; }   // nucleus wider than top-k
    __syncthreads();
    return r;
}

template <typename T>
__global__ void __launch_bounds__(NT)
sample_kernel(SampleParams p) {
    __shared__ Shared s;
    const int row_idx = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const T* row = (const T*)p.logits + (int64_t)row_idx * p.row_stride;
    const int V = p.vocab;
    const float temp = p.greedy ? 1.f : p.temperature;

    // ---------------------------------------------------------------- 1. maximum (greedy: argmax)
    // On the raw logits: dividing by a positive temperature keeps the order, so the maximum of
    // the scaled row is the scaled maximum and no division is needed in this pass.  Sampling only
    // needs the value (one v_max per element); the index is found by a second pass in the rare
    // case that asks for it (greedy decoding, or a row without any finite mass).
    const bool vec_ok = ((uintptr_t)row % 16) == 0;
    auto block_argmax = [&]() -> int {
        float best = -INFINITY;
        int best_i = 0x7fffffff;
        for_each_logit<T>(row, 0, V, 1.f, tid, NT, vec_ok, [&](int i, float x) {
            if (x > best) { best = x; best_i = i; }       // lowest index wins ties within a lane (ascending i)
        });
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o);
            const int oi = __shfl_xor(best_i, o);
            if (ob > best || (ob == best && oi < best_i)) { best = ob; best_i = oi; }
        }
        __syncthreads();
        if (lane == 0) { s.red_f[wave] = best; s.red_i[wave] = best_i; }
        __syncthreads();
        best = s.red_f[0]; best_i = s.red_i[0];
        for (int w = 1; w < NW; ++w) {
            const float ob = s.red_f[w];
            const int oi = s.red_i[w];
            if (ob > best || (ob == best && oi < best_i)) { best = ob; best_i = oi; }
        }
        return best_i == 0x7fffffff ? 0 : best_i;
    };
    if (p.greedy) {
        const int best_i = block_argmax();
        if (tid == 0) p.out[row_idx] = best_i;
        if (p.probs_out)
            for (int i = tid; i < V; i += NT) p.probs_out[(int64_t)row_idx * V + i] = i == best_i ? 1.f : 0.f;
        return;
    }
    // a row without finite mass (all -inf, NaN): the argmax, and an all-zero distribution
    auto no_mass = [&]() {
        const int best_i = block_argmax();
        if (tid == 0) p.out[row_idx] = best_i;
        if (p.probs_out)
            for (int i = tid; i < V; i += NT) p.probs_out[(int64_t)row_idx * V + i] = 0.f;
    };
    float lane_best = -INFINITY;                      // raw maximum of this lane's share of the row
    for_each_logit<T>(row, 0, V, 1.f, tid, NT, vec_ok, [&](int, float x) { lane_best = fmaxf(lane_best, x); });
    float best = lane_best;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) best = fmaxf(best, __shfl_xor(best, o));
    if (lane == 0) s.red_f[wave] = best;
    __syncthreads();
    best = s.red_f[0];
    for (int w = 1; w < NW; ++w) best = fmaxf(best, s.red_f[w]);
    const float m = apply_temperature<T>(best, temp);

    auto over_row = [&](auto f) { for_each_logit<T>(row, 0, V, temp, tid, NT, vec_ok, f); };
    auto over_list = [&](auto f) {
        const int n = (int)s.n_list;
        for (int j = tid; j < n; j += NT) f((int)s.list_idx[j], key_value(s.list_key[j]));
    };

    // ---------------------------------------------------------------- 2. top-k: key of the k-th largest
    // With k <= 1024 the k-th largest of the 1024 per-lane maxima is a lower bound of the row's k-th
    // largest value (the maxima are elements of the row), so one more pass collects every
    // candidate (about k of them) into LDS, and selection, nucleus walk and draw run on that
    // list.  The pass compares raw keys against the bound lowered by LIST_SLACK representable
    // values (several raw values can divide to the same scaled value, and ties at the k-th
    // scaled value all stay) and divides only what passes.  A row whose candidates do not fit
    // (masses of equal values) takes the full-row walk.
    uint32_t key_k = 0;                          // keep keys >= key_k
    bool use_list = false;
    int nuc_first = 0;                           // nucleus walk already done down to this digit level (no top-k) ...
    uint32_t nuc_prefix = 0, nuc_pmask = 0;      // ... with this key prefix ...
    unsigned long long nuc_limit = 0;            // ... and this much of the mass limit left
    const bool topk_on = p.top_k > 0 && p.top_k < V;
    if (topk_on && p.top_k <= NT && temp <= LIST_MAX_TEMPERATURE) {
        auto over_lane_max = [&](auto f) { f(tid, lane_best); };
        // two digit levels (22 of 32 key bits): a bound 2^-13 relative below the k-th largest maximum
        // lets in a few more candidates and saves a histogram round
        const uint32_t key_l = select_kth(s, over_lane_max, (unsigned int)p.top_k, tid, lane, wave, 2);
        const uint32_t key_ls = order_key(apply_temperature<T>(key_value(key_l), temp));
        const uint32_t slack = LIST_SLACK * (sizeof(T) == 2 ? 0x10000u : 1u);     // bf16 values are 2^16 keys apart
        const uint32_t key_lo = key_l > slack ? key_l - slack : 0u;
        if (tid == 0) s.n_list = 0;
        __syncthreads();
        // prefilter on the raw float, one compare per element.  It lets through whatever the key
        // order would (plus -0.0 next to +0.0, and everything when the bound is below -inf, whose
        // key decodes to a NaN); the exact test on the scaled key follows.
        float raw_lo = key_value(key_lo);              // may be a NaN (a bound below -inf): lets everything through
        if constexpr (std::is_same<T, f16_t>::value) {
            const float b = f16_raw_bound<T>(key_value(key_ls), temp);
            if (b < raw_lo) raw_lo = b;
        }
        for_each_logit<T>(row, 0, V, 1.f, tid, NT, vec_ok, [&](int i, float x) {
            if (!(x < raw_lo)) {
                const uint32_t key = order_key(apply_temperature<T>(x, temp));
                if (key >= key_ls) {
                    const unsigned int j = atomicAdd(&s.n_list, 1u);
                    if (j < LIST_CAP) { s.list_key[j] = key; s.list_idx[j] = (unsigned int)i; }
                }
            }
        });
        __syncthreads();
        use_list = s.n_list <= LIST_CAP;
    }
    // ---------------------------------------------------------------- at most one candidate per lane
    // No histograms: every lane ranks its candidate in the descending order a stable sort would give
    // (key, then index); with top-k the lane of rank k-1 holds the k-th largest key; the mass that
    // precedes a candidate in that order decides the nucleus; the draw walks the kept candidates in
    // index order.  Plain loops over the list in LDS, exact 64-bit sums.  Without top-k the list is
    // everything above a cut of the whole row and z_row the mass of the whole row.
    auto draw_from_small_list = [&](bool has_topk, unsigned long long z_row) {
        const int n = (int)s.n_list;
        const bool mine = tid < n;
        const uint32_t key = mine ? s.list_key[tid] : 0u;
        const unsigned int idx = mine ? s.list_idx[tid] : 0xffffffffu;
        // the loops below read the list eight entries at a time (independent LDS reads; entries past
        // n are inside the arrays and masked out)
        unsigned int rank = 0;
        if (mine)
            for (int i0 = 0; i0 < n; i0 += 8) {
                uint32_t kk[8], ii[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) { kk[u] = s.list_key[i0 + u]; ii[u] = s.list_idx[i0 + u]; }
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    rank += (i0 + u < n) && ((kk[u] > key) || (kk[u] == key && ii[u] < idx));
            }
        if (has_topk && mine && rank == (unsigned int)p.top_k - 1u) s.sel_digit = key;   // ranks are a permutation: one writer
        __syncthreads();
        const uint32_t kth = has_topk ? s.sel_digit : 0u;
        uint64_t w = (mine && key >= kth) ? weight_of(key_value(key), m) : 0;   // ties at the k-th value all stay
        if (mine) { s.cnt[tid] = rank; s.list_w[tid] = w; }
        unsigned long long z = wave_sum64(w);
        if (lane == 0) s.seg_mass[wave] = z;
        __syncthreads();
        z = 0;
        for (int wv = 0; wv < NW; ++wv) z += s.seg_mass[wv];
        if (p.top_p < 1.f) {
            // an entry stays while the mass before it (in sorted order) is at most top_p of the total
            // (of the row's total when the list is a cut of the whole row rather than its top k)
            const unsigned long long limit = (unsigned long long)((double)fmaxf(p.top_p, 0.f) * (double)(has_topk ? z : z_row));
            unsigned long long before = 0;
            if (w)
                for (int i0 = 0; i0 < n; i0 += 8) {
                    uint32_t rr[8];
                    unsigned long long ww[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) { rr[u] = s.cnt[i0 + u]; ww[u] = s.list_w[i0 + u]; }
#pragma unroll
                    for (int u = 0; u < 8; ++u) before += (i0 + u < n && rr[u] < rank) ? ww[u] : 0ull;
                }
            if (before > limit) w = 0;
            __syncthreads();                       // every lane has read the unfiltered weights
            if (mine) s.list_w[tid] = w;
            z = wave_sum64(w);
            if (lane == 0) s.seg_mass[wave] = z;
            __syncthreads();
            z = 0;
            for (int wv = 0; wv < NW; ++wv) z += s.seg_mass[wv];
        }
        if (z == 0) {                                  // non-finite logits: fall back to the argmax
            no_mass();
            return;
        }
        unsigned long long target = (unsigned long long)((double)p.uniforms[row_idx] * (double)z);
        if (target >= z) target = z - 1;
        if (p.probs_out) {
            for (int i = tid; i < V; i += NT) p.probs_out[(int64_t)row_idx * V + i] = 0.f;
            __syncthreads();
        }
        if (w) {
            unsigned long long before = 0;             // kept mass at lower indices
            for (int i0 = 0; i0 < n; i0 += 8) {
                uint32_t ii[8];
                unsigned long long ww[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) { ii[u] = s.list_idx[i0 + u]; ww[u] = s.list_w[i0 + u]; }
#pragma unroll
                for (int u = 0; u < 8; ++u) before += (i0 + u < n && ii[u] < idx) ? ww[u] : 0ull;
            }
            if (before <= target && target < before + w) p.out[row_idx] = idx;
            const double inv_z = 1.0 / (double)z;
            if (p.probs_out) p.probs_out[(int64_t)row_idx * V + idx] = (float)((double)w * inv_z);
        }
    };
    if (use_list && s.n_list <= NT && s.n_list >= (unsigned int)p.top_k) {
        draw_from_small_list(true, 0ull);
        return;
    }

    // ---------------------------------------------------------------- 2b. nucleus without top-k
    // One pass gives the exact mass of the row and, for the logits within NUCLEUS_SPAN of the
    // maximum only (the rest cannot hold the threshold unless the row is very flat, and would cost
    // an LDS atomic each), a first-level mass histogram.  If the walk finds the threshold bin inside
    // that region, everything from that bin up is collected and, when it fits one candidate per
    // lane, handled like a top-k list.  Otherwise the full-row walk below runs.
    if (!topk_on && p.top_p < 1.f) {
        constexpr float NUCLEUS_SPAN = 12.f;
        const float cut_f = m - NUCLEUS_SPAN;
        const int nb0 = 1 << WIDTHS[0];
        for (int b2 = tid; b2 < BINS; b2 += NT) { s.mass[b2] = 0; s.cnt[b2] = 0; }
        if (tid == 0) s.n_list = 0;
        __syncthreads();
        unsigned long long zacc = 0;
        over_row([&](int, float x) {
            const uint64_t w = weight_of(x, m);
            zacc += w;
            if (x >= cut_f) {
                const int b2 = (int)(order_key(x) >> SHIFTS[0]) & (nb0 - 1);
                atomicAdd(&s.mass[b2], (unsigned long long)w);
                atomicAdd(&s.cnt[b2], 1u);
            }
        });
        zacc = wave_sum64(zacc);
        if (lane == 0) s.seg_mass[wave] = zacc;
        __syncthreads();
        unsigned long long z_row = 0;
        for (int wv = 0; wv < NW; ++wv) z_row += s.seg_mass[wv];
        if (z_row == 0) {
            no_mass();
            return;
        }
        const unsigned long long limit = (unsigned long long)((double)fmaxf(p.top_p, 0.f) * (double)z_row);
        if (wave == 0) pick_by_mass(s, nb0, limit, lane);
        __syncthreads();
        const uint32_t d0 = s.sel_digit;
        if (d0 > (order_key(cut_f) >> SHIFTS[0])) {               // the whole bin lies inside the histogrammed region
            // candidates from that bin up
            unsigned int c = (tid >= (int)d0 ? s.cnt[tid] : 0u) + (tid + NT >= (int)d0 ? s.cnt[tid + NT] : 0u);
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o);
            if (lane == 0) s.seg_tied[wave] = c;
            __syncthreads();
            unsigned int n_est = 0;
            for (int wv = 0; wv < NW; ++wv) n_est += s.seg_tied[wv];
            const uint32_t key_lo_s = d0 << SHIFTS[0];
            if (n_est <= (unsigned int)NT) {
                // raw prefilter: the scaled bound times the temperature, lowered by more than the division
                // (and, for bf16 rows, the rounding of the quotient) can move a value
                const float t_raw = key_value(key_lo_s) * temp;
                float raw_lo = temp == 1.f ? key_value(key_lo_s)
                                           : t_raw - fabsf(t_raw) * (sizeof(T) == 2 ? 0.0078125f : 9.5367431640625e-7f);
                if constexpr (std::is_same<T, f16_t>::value) {
                    const float b = f16_raw_bound<T>(key_value(key_lo_s), temp);
                    if (b < raw_lo) raw_lo = b;
                }
                for_each_logit<T>(row, 0, V, 1.f, tid, NT, vec_ok, [&](int i, float x) {
                    if (!(x < raw_lo)) {
                        const uint32_t key = order_key(apply_temperature<T>(x, temp));
                        if (key >= key_lo_s) {
                            const unsigned int j = atomicAdd(&s.n_list, 1u);
                            if (j < LIST_CAP) { s.list_key[j] = key; s.list_idx[j] = (unsigned int)i; }
                        }
                    }
                });
                __syncthreads();
                if (s.n_list <= NT) {
                    draw_from_small_list(false, z_row);
                    return;
                }
            }
            // too many for a list: the full-row walk continues below from the second digit level
            nuc_first = 1;
            nuc_prefix = key_lo_s;
            nuc_pmask = (uint32_t)(nb0 - 1) << SHIFTS[0];
            nuc_limit = limit - s.sel_above_mass;
        }
        __syncthreads();
    }
    if (topk_on)
        key_k = use_list ? select_kth(s, over_list, (unsigned int)p.top_k, tid, lane, wave)
                         : select_kth(s, over_row, (unsigned int)p.top_k, tid, lane, wave);

    // ---------------------------------------------------------------- 3. nucleus threshold
    Nucleus nu;
    nu.key_t = key_k; nu.tie_keep = 0xffffffffu; nu.tie_rule = false;
    if (p.top_p < 1.f)
        nu = use_list ? nucleus_threshold(s, over_list, key_k, m, p.top_p, tid, lane, wave)
                      : nucleus_threshold(s, over_row, key_k, m, p.top_p, tid, lane, wave, nuc_first, nuc_prefix,
                                          nuc_pmask, nuc_limit);
    const uint32_t key_t = nu.key_t;
    const unsigned int tie_keep = nu.tie_keep;
    const bool tie_rule = nu.tie_rule;
    __syncthreads();

    if (use_list) {
        // ------------------------------------------------------------ 4a. draw from the candidate list
        // Every kept element is on the list.  Weights first (a tied element needs its rank among
        // the tied ones in index order), then each entry's mass-before in index order; both by
        // plain loops over the list, which holds about k entries.
        const int n = (int)s.n_list;
        const uint64_t w_tie = tie_rule ? weight_of(key_value(key_t), m) : 0;
        for (int j = tid; j < n; j += NT) {
            const uint32_t key = s.list_key[j];
            const unsigned int idx = s.list_idx[j];
            uint64_t w = 0;
            if (tie_rule ? key > key_t : key >= key_t) w = weight_of(key_value(key), m);
            else if (tie_rule && key == key_t) {
                unsigned int rank = 0;
                for (int i0 = 0; i0 < n; i0 += 8) {
                    uint32_t kk[8], ii[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) { kk[u] = s.list_key[min(i0 + u, n - 1)]; ii[u] = s.list_idx[min(i0 + u, n - 1)]; }
#pragma unroll
                    for (int u = 0; u < 8; ++u) rank += i0 + u < n && kk[u] == key_t && ii[u] < idx;
                }
                if (rank < tie_keep) w = w_tie;
            }
            s.list_w[j] = w;
        }
        __syncthreads();
        unsigned long long part = 0;
        for (int j = tid; j < n; j += NT) part += s.list_w[j];
        part = wave_sum64(part);
        if (lane == 0) s.seg_mass[wave] = part;
        __syncthreads();
        unsigned long long z2 = 0;
        for (int w = 0; w < NW; ++w) z2 += s.seg_mass[w];
        if (z2 == 0) {                                 // non-finite logits: fall back to the argmax
            no_mass();
            return;
        }
        unsigned long long target = (unsigned long long)((double)p.uniforms[row_idx] * (double)z2);
        if (target >= z2) target = z2 - 1;
        if (p.probs_out) {
            for (int i = tid; i < V; i += NT) p.probs_out[(int64_t)row_idx * V + i] = 0.f;
            __syncthreads();
        }
        const double inv_z = 1.0 / (double)z2;
        if (p.probs_out)
            for (int j = tid; j < n; j += NT) {
                const uint64_t w = s.list_w[j];
                if (w) p.probs_out[(int64_t)row_idx * V + s.list_idx[j]] = (float)((double)w * inv_z);
            }
        // The draw in index order without comparing every pair of entries: kept mass per bucket of
        // consecutive indices (one bucket per lane), a scan over the buckets to find the one that
        // holds the target, then the few entries of that bucket among themselves.
        int sh = 0;
        while (((V - 1) >> sh) >= NT) ++sh;
        __syncthreads();
        s.mass[tid] = 0;                               // NT <= BINS buckets
        if (tid == 0) s.sel_above_cnt = 0;
        __syncthreads();
        for (int j = tid; j < n; j += NT) {
            const uint64_t w = s.list_w[j];
            if (w) atomicAdd(&s.mass[s.list_idx[j] >> sh], (unsigned long long)w);
        }
        __syncthreads();
        const unsigned long long mine_b = s.mass[tid];
        unsigned long long incl = wave_incl_scan64(mine_b, lane);
        if (lane == 63) s.seg_mass[wave] = incl;
        __syncthreads();
        unsigned long long base = 0;
        for (int w = 0; w < wave; ++w) base += s.seg_mass[w];
        incl += base;
        if (mine_b && incl - mine_b <= target && target < incl) {      // exactly one bucket
            s.sel_digit = (unsigned int)tid;
            s.sel_above_mass = incl - mine_b;
        }
        __syncthreads();
        const unsigned int bucket = s.sel_digit;
        const unsigned long long bucket_base = s.sel_above_mass;
        // the list positions of that bucket's entries go to the key array (the keys are no longer needed)
        for (int j = tid; j < n; j += NT)
            if (s.list_w[j] && (s.list_idx[j] >> sh) == bucket) s.list_key[atomicAdd(&s.sel_above_cnt, 1u)] = (unsigned int)j;
        __syncthreads();
        const int nb = (int)s.sel_above_cnt;           // at most n
        for (int a = tid; a < nb; a += NT) {
            const int j = (int)s.list_key[a];
            const unsigned int idx = s.list_idx[j];
            const unsigned long long w = s.list_w[j];
            unsigned long long before = bucket_base;
            for (int b = 0; b < nb; ++b) {
                const int i = (int)s.list_key[b];
                before += s.list_idx[i] < idx ? s.list_w[i] : 0ull;
            }
            if (before <= target && target < before + w) p.out[row_idx] = idx;
        }
        return;
    }

    // ---------------------------------------------------------------- 4. draw in index order
    // wave w owns the contiguous segment [w*seg, (w+1)*seg)
    const int seg = ((V + NW - 1) / NW + 63) / 64 * 64;
    const int s0 = wave * seg, s1 = min(V, s0 + seg);
    unsigned long long mass_gt = 0;
    unsigned int n_tied = 0;
    uint64_t w_t_val = 0;
    for_each_logit<T>(row, s0, max(s0, s1), temp, lane, 64, vec_ok, [&](int, float x) {
        const uint32_t key = order_key(x);
        if (tie_rule ? key > key_t : key >= key_t) mass_gt += weight_of(x, m);
        else if (tie_rule && key == key_t) ++n_tied;
    });
    if (tie_rule) w_t_val = weight_of(key_value(key_t), m);
    mass_gt = wave_sum64(mass_gt);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) n_tied += __shfl_xor(n_tied, o);
    if (lane == 0) { s.seg_mass[wave] = mass_gt; s.seg_tied[wave] = n_tied; }
    __syncthreads();
    unsigned long long z2 = 0, my_base = 0, my_total = 0;
    unsigned int tied_base = 0, my_tied_base = 0;
    for (int w = 0; w < NW; ++w) {
        const unsigned int nt = s.seg_tied[w];
        const unsigned int kept = tie_rule ? (tied_base >= tie_keep ? 0u : min(nt, tie_keep - tied_base)) : 0u;
        const unsigned long long tot = s.seg_mass[w] + (unsigned long long)kept * w_t_val;
        if (w == wave) { my_base = z2; my_tied_base = tied_base; my_total = tot; }
        z2 += tot;
        tied_base += nt;
    }
    if (z2 == 0) {                                 // no mass at all (non-finite logits): fall back to the argmax
        no_mass();
        return;
    }
    unsigned long long target = (unsigned long long)((double)p.uniforms[row_idx] * (double)z2);
    if (target >= z2) target = z2 - 1;
    const float inv_z = (float)(1.0 / (double)z2);
    auto weight_or_tie = [&](float x, bool& tied) -> uint64_t {
        const uint32_t key = order_key(x);
        tied = false;
        if (tie_rule ? key > key_t : key >= key_t) return weight_of(x, m);
        tied = tie_rule && key == key_t;
        return 0;
    };

    if (p.probs_out) {
        // the distribution itself, on request: every wave walks its segment in steps of 64 with a
        // running count of the tied elements seen so far
        unsigned int tied_seen = my_tied_base;
        for (int i0 = s0; i0 < s1; i0 += 64) {
            const int i = i0 + lane;
            uint64_t w = 0;
            bool tied = false;
            if (i < s1) w = weight_or_tie(scaled_logit<T>(row, i, temp), tied);
            const unsigned long long tb = __ballot(tied);
            if (tied && tied_seen + __popcll(tb & ((1ull << lane) - 1ull)) < tie_keep) w = w_t_val;
            tied_seen += __popcll(tb);
            if (i < s1) p.probs_out[(int64_t)row_idx * V + i] = (float)((double)w * (double)inv_z);
        }
    }

    // only the wave whose segment holds the target goes on
    if (!(my_base <= target && target < my_base + my_total)) return;

    // lane chunks of the segment: totals per lane, scans over the wave, then the owning lane's chunk
    // is walked by the whole wave
    const int chunk = ((s1 - s0 + 63) / 64 + 3) / 4 * 4;
    const int c0 = min(s1, s0 + lane * chunk), c1 = min(s1, c0 + chunk);
    unsigned long long lane_mass = 0;
    unsigned int lane_tied = 0;
    for_each_logit<T>(row, c0, c1, temp, 0, 1, vec_ok, [&](int, float x) {
        bool tied;
        lane_mass += weight_or_tie(x, tied);
        lane_tied += tied;
    });
    unsigned int tied_incl = lane_tied;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const unsigned int o = __shfl_up(tied_incl, d);
        if (lane >= d) tied_incl += o;
    }
    const unsigned int lane_tied_base = my_tied_base + tied_incl - lane_tied;
    if (tie_rule && lane_tied_base < tie_keep)
        lane_mass += (unsigned long long)min(lane_tied, tie_keep - lane_tied_base) * w_t_val;
    const unsigned long long incl = my_base + wave_incl_scan64(lane_mass, lane);
    const unsigned long long hit = __ballot(lane_mass != 0 && incl > target);
    if (!hit) return;                                          // cannot happen: the segment holds the target
    const int owner = __ffsll((long long)hit) - 1;
    unsigned long long running = shfl64(incl, owner) - shfl64(lane_mass, owner);
    unsigned int tied_seen = __shfl(lane_tied_base, owner);
    const int w0 = __shfl(c0, owner), w1 = __shfl(c1, owner);
    for (int i0 = w0; i0 < w1; i0 += 64) {
        const int i = i0 + lane;
        uint64_t w = 0;
        bool tied = false;
        if (i < w1) w = weight_or_tie(scaled_logit<T>(row, i, temp), tied);
        const unsigned long long tb = __ballot(tied);
        if (tied && tied_seen + __popcll(tb & ((1ull << lane) - 1ull)) < tie_keep) w = w_t_val;
        tied_seen += __popcll(tb);
        const unsigned long long sc = wave_incl_scan64(w, lane);
        const unsigned long long h2 = __ballot(w != 0 && running + sc > target);
        if (h2) {
            if (lane == __ffsll((long long)h2) - 1) p.out[row_idx] = i;
            return;
        }
        running += shfl64(sc, 63);
    }
}

}  // namespace

int launch_sample(int64_t* out, const void* logits, int64_t row_stride, float* probs_out,
                  const float* uniforms, int batch, int vocab, float temperature, int top_k, float top_p,
                  int greedy, int dtype, hipStream_t stream) {
    SampleParams p;
    p.out = out; p.logits = logits; p.row_stride = row_stride; p.probs_out = probs_out;
    p.uniforms = uniforms; p.vocab = vocab; p.temperature = temperature; p.top_k = top_k;
    p.top_p = top_p; p.greedy = greedy;
    if (dtype == AICOMP_KV_F32) hipLaunchKernelGGL((sample_kernel<float>), dim3(batch), dim3(NT), 0, stream, p);
    else if (dtype == AICOMP_KV_F16) hipLaunchKernelGGL((sample_kernel<f16_t>), dim3(batch), dim3(NT), 0, stream, p);
    else hipLaunchKernelGGL((sample_kernel<bf16_t>), dim3(batch), dim3(NT), 0, stream, p);
    AICOMP_HIP_LAUNCH_CHECK();
    return AICOMP_KV_OK;
}

}  // namespace aicomp

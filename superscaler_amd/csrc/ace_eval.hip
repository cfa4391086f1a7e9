// MI355X (gfx950) batched plan evaluator: kernels and C ABI (see include/ace_eval.h).
//
// Scoring kernel: one plan per lane.  All lanes of a workgroup walk the op sequence in
// lockstep, so the op type at each step is wave-uniform: the row of profiled values for
// that type sits in LDS at a scalar base address and each lane only adds its own
// (micro-batch, tp, algo) offset -- at most n_tp*n_algo distinct, consecutive entries per
// sub-table, i.e. LDS reads without bank conflicts.  Plan bytes are stored plan-minor
// ([16-op group][plan][16 bytes]) so a wavefront's load covers 1 KiB of consecutive HBM.
// Every plan's sums run sequentially in op order in fp64, which reproduces the reference's
// Python floats bit for bit.  When the rows of all op types do not fit in LDS the op
// sequence is cut into windows and the workgroup restages the rows at each window boundary.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <algorithm>
#include <mutex>
#include <new>
#include <vector>

#include "ace_edit_kernels.h"
#include "ace_score_loop.h"

// Scratch of ace_score_batch_static: the deferred-stage-tail records of up to ACE_STATIC_MAX_PLANS plans (the
// layout ace_score_body's DEFER variant uses: [workgroup][stage][lane][ACE_WS_REC]).  Every GPU the library runs on holds
// its own copy of this array until the process ends.  In host code the array's name is only a stand-in for
// hipGetSymbolAddress(): kernels get the per-device pointer that call returned (static_scratch_ptr), never the name.
static __device__ __align__(256) double scratch[(size_t)ACE_STATIC_MAX_PLANS * ACE_MAX_STAGES * ACE_WS_REC];

namespace {

#ifndef ACE_BLOCK
#define ACE_BLOCK 1024
#endif
constexpr int kBlock = ACE_BLOCK;        // lanes (= plans) per workgroup: 16 wavefronts, 4 per SIMD
constexpr int kSmallBlock = 256;         // ... for small batches: 4 wavefronts, 1 per SIMD
#ifndef ACE_SMALL_BATCH_BLOCKS
#define ACE_SMALL_BATCH_BLOCKS 128
#endif
constexpr int kSmallBatchBlocks = ACE_SMALL_BATCH_BLOCKS;   // batches of fewer than this many kBlock workgroups use kSmallBlock
constexpr uint32_t kMaxLds = 160 * 1024;  // CDNA4 LDS per workgroup
static_assert(ACE_STATIC_MAX_PLANS % ACE_BLOCK == 0, "the static scratch holds whole workgroups");

thread_local char g_hip_err[256] = "";

constexpr int kMaxDevices = 64;
double *g_static_ptr[kMaxDevices];     // device address of `scratch` by device ordinal; filled once per device
std::mutex g_static_mutex;

#define ACE_HIP(call)                                                                          \
    do {                                                                                       \
        hipError_t e_ = (call);                                                                \
        if (e_ != hipSuccess) {                                                                \
            snprintf(g_hip_err, sizeof(g_hip_err), "%s failed: %s", #call, hipGetErrorString(e_)); \
            return ACE_EHIP;                                                                   \
        }                                                                                      \
    } while (0)

// BD / RANGED / WIN / DEFER: see ace_score_body (ace_score_loop.h), which holds the whole kernel.
// BLOCK: kBlock lanes for large batches; kSmallBlock for batches that would otherwise occupy only a
// few CUs (a workgroup keeps a CU to itself either way: the tables fill its LDS): the walk over the
// op sequence is sequential per wavefront, so a small batch finishes soonest with one wavefront per
// SIMD on as many CUs as it can reach.
// COLL: tables compiled with consider_collective_memory (large workgroups only: a switch few callers set).
template <bool BD, bool RANGED, bool WIN, bool DEFER, int BLOCK, bool COLL = false>
__global__ __launch_bounds__(BLOCK) void ace_score_kernel(const AceKernelArgs a) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    ace_score_body<BD, RANGED, WIN, DEFER, BLOCK, COLL>(a, lds_raw, 0u, (int)threadIdx.x, (long long)blockIdx.x, gridDim.x);
}

// ------------------------------------------------------------------------------------------
// top-k: radix select on the order-preserving 64-bit image of the iteration time, then a
// gather of everything below the k-th key plus the lowest-indexed ties, then a small sort.
// ------------------------------------------------------------------------------------------
constexpr int kTopBlock = 256;
constexpr int kRadixBits = 11;
constexpr int kRadix = 1 << kRadixBits;
constexpr int kPasses = 6;               // 6 * 11 = 66 >= 64 key bits
constexpr unsigned long long kInfKey = 0xffffffffffffffffull;

struct TopkState {                     // lives in the caller's workspace
    unsigned long long prefix;         // key bits fixed so far (from the top)
    unsigned long long thr;            // final k-th smallest key
    unsigned int k_rem;                // how many still to pick inside the current bucket
    unsigned int n_feasible;
    unsigned int n_less;               // entries with key < thr
    unsigned int n_out_less;           // atomic cursor for the gather of "< thr"
    unsigned int n_ties;               // atomic cursor for tie candidates
    unsigned int pad;
};

__device__ __forceinline__ unsigned long long time_key(double t, uint8_t feasible) {
    // positive doubles order like their bit patterns; infeasible or NaN plans sort last
    if (!feasible || !(t == t)) return kInfKey;
    if (t == 0.0) t = 0.0;          // (-0.0 compares equal to 0.0 in the reference's float order: one key for both)
    unsigned long long b = (unsigned long long)__double_as_longlong(t);
    return (b >> 63) ? ~b : (b | 0x8000000000000000ull);
}

__device__ __forceinline__ int pass_shift(int pass) {
    int s = 64 - kRadixBits * (pass + 1);
    return s < 0 ? 0 : s;
}
__device__ __forceinline__ int pass_bits(int pass) {
    int hi = 64 - kRadixBits * pass;
    int lo = pass_shift(pass);
    return hi - lo;
}

__global__ void topk_init(TopkState *st, unsigned int *hist, int k) {
    for (int j = threadIdx.x; j < kRadix; j += blockDim.x) hist[j] = 0;
    if (threadIdx.x == 0) {
        st->prefix = 0; st->thr = 0; st->k_rem = (unsigned)k; st->n_feasible = 0;
        st->n_less = 0; st->n_out_less = 0; st->n_ties = 0; st->pad = 0;
    }
}

__global__ __launch_bounds__(kTopBlock) void topk_hist(const double *t, const uint8_t *f, size_t n, int pass,
                                                       const TopkState *st, unsigned int *hist) {
    __shared__ unsigned int lh[kRadix];
    for (int j = threadIdx.x; j < kRadix; j += kTopBlock) lh[j] = 0;
    __syncthreads();
    const int shift = pass_shift(pass);
    const int bits = pass_bits(pass);
    const unsigned long long prefix = st->prefix;
    const int hi_shift = shift + bits;   // bits above this are already fixed
    for (size_t i = (size_t)blockIdx.x * kTopBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kTopBlock) {
        unsigned long long key = time_key(t[i], f[i]);
        bool match = hi_shift >= 64 ? true : ((key >> hi_shift) == (prefix >> hi_shift));
        if (match) atomicAdd(&lh[(unsigned)((key >> shift) & ((1ull << bits) - 1))], 1u);
    }
    __syncthreads();
    for (int j = threadIdx.x; j < kRadix; j += kTopBlock)
        if (lh[j]) atomicAdd(&hist[j], lh[j]);
}

__global__ __launch_bounds__(kTopBlock) void topk_pick(TopkState *st, unsigned int *hist, int pass) {
    // single workgroup: find the bucket holding the k_rem-th entry of the current prefix, descend into it
    constexpr int kPer = kRadix / kTopBlock;          // buckets per lane
    __shared__ unsigned int part[kTopBlock];
    const int tid = threadIdx.x;
    unsigned int loc[kPer];
    unsigned int sum = 0;
#pragma unroll
    for (int j = 0; j < kPer; ++j) { loc[j] = hist[tid * kPer + j]; sum += loc[j]; }
    part[tid] = sum;
    __syncthreads();
    for (int off = 1; off < kTopBlock; off <<= 1) {   // inclusive scan of the per-lane sums
        unsigned int v = tid >= off ? part[tid - off] : 0u;
        __syncthreads();
        part[tid] += v;
        __syncthreads();
    }
    const unsigned int rem = st->k_rem;
    const unsigned int incl = part[tid], excl = incl - sum;
    const unsigned int total = part[kTopBlock - 1];
    const int shift = pass_shift(pass);
    __syncthreads();
    bool mine = excl < rem && rem <= incl;            // exactly one lane when total >= rem
    if (total < rem) mine = (tid == kTopBlock - 1);   // fewer entries than asked for: take the last bucket
    if (mine) {
        unsigned int acc = excl;
        int b = tid * kPer;
        if (total >= rem) {
            for (int j = 0; j < kPer; ++j) {
                if (acc + loc[j] >= rem) { b = tid * kPer + j; break; }
                acc += loc[j];
            }
        } else {
            const int nb = 1 << pass_bits(pass);
            b = nb - 1;
            acc = total - hist[b];
        }
        st->prefix |= ((unsigned long long)b) << shift;
        st->k_rem = rem - acc;
        st->n_less += acc;
        if (pass == kPasses - 1) st->thr = st->prefix;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kPer; ++j) hist[tid * kPer + j] = 0;
}

struct Cand { unsigned long long key; long long idx; };

__global__ __launch_bounds__(kTopBlock) void topk_gather(const double *t, const uint8_t *f, size_t n, TopkState *st,
                                                         Cand *less, Cand *ties, unsigned int cap_less, unsigned int cap_ties) {
    const unsigned long long thr = st->thr;
    for (size_t i = (size_t)blockIdx.x * kTopBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kTopBlock) {
        unsigned long long key = time_key(t[i], f[i]);
        if (key == kInfKey) continue;
        if (key < thr) {
            unsigned int p = atomicAdd(&st->n_out_less, 1u);
            if (p < cap_less) less[p] = Cand{key, (long long)i};
        } else if (key == thr) {
            unsigned int p = atomicAdd(&st->n_ties, 1u);
            if (p < cap_ties) ties[p] = Cand{key, (long long)i};
        }
    }
}

// When more ties than fit were seen, pick the lowest-indexed ones: one workgroup reads the input in index order, 8,192
// entries per step (512 consecutive ones per wavefront, the loads of the next step in flight), ranks the entries equal to
// the k-th key by wavefront ballots and one exchange of the wavefronts' counts through LDS, and stops as soon as it has
// enough.  Exact whatever the number of ties.
constexpr int kTieBlock = 1024;
__global__ __launch_bounds__(kTieBlock) void topk_ties_exact(const double *t, const uint8_t *f, size_t n, TopkState *st,
                                                             Cand *ties, unsigned int want) {
    constexpr int kCh = 8;                                      // a wavefront's share of a step: kCh * 64 consecutive entries
    constexpr size_t kStep = (size_t)kCh * kTieBlock;
    __shared__ unsigned int s_cnt[16];
    const unsigned long long thr = st->thr;
    // nothing to redo unless the gather overflowed its tie buffer (every lane reads the same value;
    // it is only rewritten after the last barrier below)
    if (st->n_ties <= want || thr == kInfKey) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t mine = (size_t)wave * (kCh * 64) + (size_t)lane;   // entry c of this lane in a step: start + mine + c * 64
    unsigned int found = 0;
    // (the entries of the step after the current one are asked for before the current one is ranked)
    double nt[kCh];
    uint8_t nf[kCh];
#pragma unroll
    for (int c = 0; c < kCh; ++c) {
        const size_t i = mine + (size_t)c * 64;
        nt[c] = 0.0; nf[c] = 0;
        if (i < n) { nt[c] = t[i]; nf[c] = f[i]; }
    }
    for (size_t start = 0; start < n && found < want; start += kStep) {
        unsigned long long mask[kCh];
        unsigned int wave_total = 0;
#pragma unroll
        for (int c = 0; c < kCh; ++c) {
            const size_t i = start + mine + (size_t)c * 64;
            mask[c] = __ballot(i < n && time_key(nt[c], nf[c]) == thr);
            wave_total += (unsigned int)__popcll(mask[c]);
        }
#pragma unroll
        for (int c = 0; c < kCh; ++c) {
            const size_t i = start + kStep + mine + (size_t)c * 64;
            if (i < n) { nt[c] = t[i]; nf[c] = f[i]; }
        }
        if (lane == 0) s_cnt[wave] = wave_total;
        __syncthreads();
        unsigned int before = found, total = 0;
        for (int w = 0; w < 16; ++w) { const unsigned int v = s_cnt[w]; before += w < wave ? v : 0u; total += v; }
#pragma unroll
        for (int c = 0; c < kCh; ++c) {
            const unsigned int rank = before + (unsigned int)__popcll(mask[c] & ((1ull << lane) - 1ull));
            if (((mask[c] >> lane) & 1ull) && rank < want) ties[rank] = Cand{thr, (long long)(start + mine + (size_t)c * 64)};
            before += (unsigned int)__popcll(mask[c]);
        }
        found += total;                                        // (the same for every lane)
        __syncthreads();
    }
    if (tid == 0) st->n_ties = found < want ? found : want;
}

// Sort the candidates (key asc, index asc) in one workgroup (bitonic, in global memory for
// sizes beyond LDS) and write the first k.
__global__ __launch_bounds__(1024) void topk_finish(TopkState *st, Cand *less, Cand *ties, unsigned int cap_ties, int k,
                                                    Cand *buf, unsigned int buf_pow2, long long *out_idx, double *out_val,
                                                    int *out_count) {
    const unsigned int n_less = st->n_less;
    unsigned int n_ties = st->n_ties < cap_ties ? st->n_ties : cap_ties;
    const unsigned int total = n_less + n_ties;
    for (unsigned int j = threadIdx.x; j < buf_pow2; j += blockDim.x) {
        Cand c{kInfKey, 0x7fffffffffffffffll};
        if (j < n_less) c = less[j];
        else if (j < total) c = ties[j - n_less];
        buf[j] = c;
    }
    __syncthreads();
    for (unsigned int size = 2; size <= buf_pow2; size <<= 1) {
        for (unsigned int stride = size >> 1; stride > 0; stride >>= 1) {
            for (unsigned int j = threadIdx.x; j < buf_pow2; j += blockDim.x) {
                unsigned int partner = j ^ stride;
                if (partner > j) {
                    Cand x = buf[j], y = buf[partner];
                    bool up = (j & size) == 0;
                    bool gt = x.key > y.key || (x.key == y.key && x.idx > y.idx);
                    if (gt == up) { buf[j] = y; buf[partner] = x; }
                }
            }
            __syncthreads();
        }
    }
    unsigned int cnt = total < (unsigned)k ? total : (unsigned)k;
    for (unsigned int j = threadIdx.x; j < (unsigned)k; j += blockDim.x) {
        if (j < cnt) {
            Cand c = buf[j];
            unsigned long long b = c.key;
            b = (b >> 63) ? (b & 0x7fffffffffffffffull) : ~b;
            out_idx[j] = c.idx;
            out_val[j] = __longlong_as_double((long long)b);
        } else {
            out_idx[j] = -1;
            out_val[j] = __longlong_as_double(0x7ff0000000000000ll);
        }
    }
    if (threadIdx.x == 0 && out_count) *out_count = (int)cnt;
}

// ------------------------------------------------------------------------------------------
// top-k, short form (small k): three launches instead of seventeen.  The k-th smallest key of an evenly spaced SAMPLE
// bounds the k-th smallest key of the whole input from above, so one pass keeps everything at or below it (about
// n * k / kSample entries), and one workgroup then selects among those (held in registers, or in LDS): radix select on the 96-bit order
// (key, index), which makes ties fall to the lower index, a gather of the k winners and a small sort.
// ------------------------------------------------------------------------------------------
constexpr int kSample = 8192;            // sampled keys, selected from by one workgroup (eight per lane)
static_assert(kSample == 1 << 13, "topk_sample's index arithmetic");
constexpr unsigned kCandCap = 12000;     // candidates the last kernel can hold in LDS (12 bytes each)
constexpr int kShortMaxK = 256;
constexpr size_t kShortMaxNK = 1ull << 26;   // n * k up to this: about kSample candidates expected, kCandCap is 4 sigma above
// Equal keys: the threshold is the sample's exact k-th key; entries below it and entries equal to it are kept apart,
// and of the equal ones only the lowest indices are ever needed (k minus the number of entries below).  Few of them go
// into a list of their own; masses of them (a search neighbourhood whose plans share the bottleneck stage all have the
// same time) are only COUNTED per filter workgroup, and the last kernel reads the first few of them from the input in
// index order.  Cost: 0.03-0.05 ms at n = 2^20, k = 64 whatever the keys; only when more than kCandCap entries lie
// strictly below the sample's k-th key (feasible plans crowded between the sampled positions) does the last kernel
// select from the whole input in global memory instead (ShortSource below): one workgroup, about nine passes over
// n entries, 3.8 ms at n = 2^20.
constexpr unsigned kTieCap = 2048;       // equal-to-threshold entries listed one by one; beyond that: per-workgroup counts
constexpr unsigned kMaxFilterGroups = 8192;   // n <= kShortMaxNK entries in workgroups of 8,192
static_assert(kShortMaxNK / (1024 * 8) <= kMaxFilterGroups, "one count per filter workgroup");

struct ShortTopk { unsigned long long thr; unsigned int count; unsigned int count_eq; };

// Which of the kRadix buckets of `hist` (LDS) holds the rem-th entry (1-based), counting buckets in order: returns the
// bucket, the entries before it in `before` and the total in `total` to every lane of the 1024-lane workgroup (no bucket:
// total < rem, and the return value is meaningless).  Two buckets per lane, wavefront scans, one exchange through LDS.
__device__ __forceinline__ unsigned int short_pick(const unsigned int *hist, unsigned int rem, unsigned int *wsum /* [16 + 3] */,
                                                   unsigned int &before, unsigned int &total) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const unsigned int h0 = hist[2 * tid], h1 = hist[2 * tid + 1];
    unsigned int incl = h0 + h1;
    for (int off = 1; off < 64; off <<= 1) {
        const unsigned int v = __shfl_up(incl, off, 64);
        if (lane >= off) incl += v;
    }
    if (lane == 63) wsum[wave] = incl;
    __syncthreads();
    unsigned int base = 0, all = 0;
    for (int w2 = 0; w2 < 16; ++w2) {
        const unsigned int v = wsum[w2];
        if (w2 < wave) base += v;
        all += v;
    }
    incl += base;
    const unsigned int excl = incl - (h0 + h1);
    if (all >= rem && excl < rem && rem <= incl) {       // exactly one lane
        const bool second = excl + h0 < rem;
        wsum[16] = 2 * tid + (second ? 1 : 0);
        wsum[17] = excl + (second ? h0 : 0u);
    }
    __syncthreads();
    const unsigned int bucket = wsum[16];
    before = wsum[17];
    total = all;
    __syncthreads();                                       // (wsum is reused by the next call)
    return bucket;
}

// Smallest and largest finite key of a strided view of the lanes' own keys (kmin = kInfKey: none), to every lane.  The bits
// above the highest bit in which the two differ are common to all keys: the radix passes start below them, where the
// histogram spreads (a pass over common bits would send every LDS atomic to one bucket, one after the other).
// `cnt`: the lane's number of finite keys; `total` their number in all.
__device__ __forceinline__ void short_minmax(unsigned long long mn, unsigned long long mx, unsigned long long cnt,
                                             unsigned long long *wmm /* [48] */, unsigned long long &kmin, unsigned long long &kmax,
                                             unsigned long long &total) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int off = 32; off > 0; off >>= 1) {
        const unsigned long long a = __shfl_xor(mn, off, 64), b = __shfl_xor(mx, off, 64);
        cnt += __shfl_xor(cnt, off, 64);
        mn = a < mn ? a : mn;
        mx = b > mx ? b : mx;
    }
    if (lane == 0) { wmm[3 * wave] = mn; wmm[3 * wave + 1] = mx; wmm[3 * wave + 2] = cnt; }
    __syncthreads();
    kmin = kInfKey; kmax = 0; total = 0;
    for (int w2 = 0; w2 < 16; ++w2) {
        const unsigned long long a = wmm[3 * w2], b = wmm[3 * w2 + 1];
        kmin = a < kmin ? a : kmin;
        kmax = b > kmax ? b : kmax;
        total += wmm[3 * w2 + 2];
    }
    __syncthreads();
}

// The sample's k-th smallest key: an upper bound of the input's k-th smallest key (with fewer than k feasible entries in
// the sample: the largest finite key, so that every feasible entry is kept).
__global__ __launch_bounds__(1024) void topk_sample(const double *t, const uint8_t *f, size_t n, int k, ShortTopk *st) {
    constexpr int kPer = kSample / 1024;
    __shared__ unsigned int hist[kRadix];
    __shared__ unsigned int wsum[20];
    __shared__ unsigned long long s_wref[16];
    __shared__ unsigned long long small_keys[64];
    __shared__ unsigned long long s_kth;
    __shared__ unsigned int s_nsmall, s_nfin, s_cur;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) { s_nfin = 0; s_cur = 0; }
    // the sample: evenly spaced runs of consecutive entries (consecutive entries share cache lines); all of a short input.
    // 64 runs of 128 entries up to 2^18 entries, then more and shorter runs, so that the stretch between two runs stays at
    // about 4,096 entries (8,192 single entries from 2^25 on): an input in which the best entries are neighbours -- times
    // that fall or rise along the batch -- then leaves fewer of them between two runs than the last kernel can hold.
    // The keys stay in registers, eight per lane: no pass of the selection reads anything.
    const size_t m = n < (size_t)kSample ? n : (size_t)kSample;
    int run_shift = 7;                                          // log2(entries per run)
    while (run_shift > 0 && (n >> (13 - run_shift)) > 4096) --run_shift;
    const size_t run_step = n >> (13 - run_shift);              // (kSample = 2^13 entries in 2^(13 - run_shift) runs)
    unsigned long long rk[kPer];
#pragma unroll
    for (int q = 0; q < kPer; ++q) {
        const int j = tid + q * 1024;
        const size_t i = n <= (size_t)kSample ? (size_t)j : (size_t)(j >> run_shift) * run_step + (size_t)(j & ((1 << run_shift) - 1));
        rk[q] = (size_t)j < m ? time_key(t[i], f[i]) : kInfKey;
    }
    // how many keys are finite, and which bits vary among them: the highest bit in which any key differs from one of
    // them (the first finite key in lane order), one 32-bit maximum over the workgroup
    unsigned long long mine = kInfKey;
    unsigned int wave_cnt = 0;
#pragma unroll
    for (int q = kPer - 1; q >= 0; --q) {
        const bool fin = rk[q] != kInfKey;
        if (fin) mine = rk[q];
        wave_cnt += (unsigned int)__popcll(__ballot(fin));
    }
    const unsigned long long has = __ballot(mine != kInfKey);
    const unsigned long long wave_ref = __shfl(mine, has ? __ffsll((long long)has) - 1 : 0, 64);
    __syncthreads();                                           // (the counters are zero)
    if (lane == 0) {
        s_wref[wave] = wave_ref;
        if (wave_cnt) atomicAdd(&s_nfin, wave_cnt);
    }
    __syncthreads();
    unsigned long long ref = kInfKey;
    for (int w2 = 15; w2 >= 0; --w2) {
        const unsigned long long v = s_wref[w2];
        if (v != kInfKey) ref = v;
    }
    const unsigned long long nfin = s_nfin;
    int hb = 0;
#pragma unroll
    for (int q = 0; q < kPer; ++q) {
        if (rk[q] != kInfKey) {
            const unsigned long long x = rk[q] ^ ref;
            const int b = x ? 64 - __clzll((long long)x) : 0;
            hb = b > hb ? b : hb;
        }
    }
    for (int off = 32; off > 0; off >>= 1) {
        const int o = __shfl_xor(hb, off, 64);
        hb = o > hb ? o : hb;
    }
    if (lane == 0 && hb) atomicMax(&s_cur, (unsigned int)hb);
    __syncthreads();
    int cur = nfin == 0 ? 0 : (int)s_cur;                      // the low `cur` bits vary
    unsigned long long prefix = cur >= 64 ? 0ull : (ref >> cur) << cur;
    unsigned int rem = (unsigned)k;
    bool enough = nfin >= (unsigned long long)k;           // fewer than k feasible entries in the sample: keep every feasible entry
    for (int pass = 0; pass < 8 && enough && cur > 0; ++pass) {
        for (int j = tid; j < kRadix; j += 1024) hist[j] = 0;
        __syncthreads();
        const int bits = cur < kRadixBits ? cur : kRadixBits, shift = cur - bits;
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
            const unsigned long long x = rk[q];
            if (x != kInfKey && (cur >= 64 || (x >> cur) == (prefix >> cur)))
                atomicAdd(&hist[(unsigned)((x >> shift) & ((1ull << bits) - 1ull))], 1u);
        }
        __syncthreads();
        unsigned int before, total;
        const unsigned int b = short_pick(hist, rem, wsum, before, total);
        (void)total;
        prefix |= (unsigned long long)b << shift;
        rem -= before;
        cur = shift;
        const unsigned int in_bucket = hist[b];
        __syncthreads();                                       // (hist[b] read by all before anything clears it)
        if (cur > 0 && in_bucket <= 64u) {
            // a handful of keys left in the bucket (distinct keys: after two passes): the rem-th smallest of them directly,
            // each wavefront ranking some of them by ballot
            if (tid == 0) s_nsmall = 0;
            __syncthreads();
#pragma unroll
            for (int q = 0; q < kPer; ++q) {
                const unsigned long long x = rk[q];
                if (x != kInfKey && (x >> cur) == (prefix >> cur)) small_keys[atomicAdd(&s_nsmall, 1u) & 63u] = x;
            }
            __syncthreads();
            for (unsigned int i = (unsigned int)wave; i < in_bucket; i += 16) {
                const unsigned long long me = small_keys[i];
                bool less = false;
                if ((unsigned int)lane < in_bucket) {
                    const unsigned long long o = small_keys[lane];
                    less = o < me || (o == me && (unsigned int)lane < i);
                }
                const unsigned int rank = (unsigned int)__popcll(__ballot(less));
                if (lane == 0 && rank + 1u == rem) s_kth = me;
            }
            __syncthreads();
            prefix = s_kth;
            cur = 0;
        }
    }
    if (tid == 0) {
        // the sample's k-th smallest key itself (all digits found; all sampled keys equal: that key)
        unsigned long long thr = enough ? prefix : kInfKey;
        if (thr == kInfKey) thr = kInfKey - 1;
        st->thr = thr; st->count = 0; st->count_eq = 0;
    }
}

constexpr int kFilterPer = 8;             // entries per lane of topk_filter
__global__ __launch_bounds__(1024) void topk_filter(const double *t, const uint8_t *f, size_t n, ShortTopk *st, Cand *cand,
                                                    Cand *tiecand, unsigned int *group_ties) {
    // One atomic on each shared counter per WORKGROUP (atomics on one address are served one after the other, about ten
    // nanoseconds each): the lanes count their hits in LDS first.  Below the threshold: a candidate.  Equal to it: counted
    // for this workgroup's stretch of the input (group_ties), and listed while the list has room.
    __shared__ unsigned int s_hits, s_base, s_ties, s_tbase;
    const unsigned long long thr = st->thr;
    const size_t i0 = (size_t)blockIdx.x * 1024 * kFilterPer + threadIdx.x;
    unsigned long long key[kFilterPer];
    if (threadIdx.x == 0) { s_hits = 0; s_ties = 0; }
#pragma unroll
    for (int q = 0; q < kFilterPer; ++q) {
        const size_t i = i0 + (size_t)q * 1024;
        key[q] = i < n ? time_key(t[i], f[i]) : kInfKey;
    }
    __syncthreads();
    unsigned int mine = 0, mine_eq = 0;
#pragma unroll
    for (int q = 0; q < kFilterPer; ++q) { mine += key[q] < thr ? 1u : 0u; mine_eq += key[q] == thr ? 1u : 0u; }
    unsigned int first = 0, first_eq = 0;
    if (mine) first = atomicAdd(&s_hits, mine);
    if (mine_eq) first_eq = atomicAdd(&s_ties, mine_eq);
    __syncthreads();
    if (threadIdx.x == 0) {
        if (s_hits) s_base = atomicAdd(&st->count, s_hits);
        if (s_ties) s_tbase = atomicAdd(&st->count_eq, s_ties);
        group_ties[blockIdx.x] = s_ties;
    }
    __syncthreads();
    if (mine) {
        unsigned int p = s_base + first;
#pragma unroll
        for (int q = 0; q < kFilterPer; ++q) {
            if (key[q] < thr) {
                if (p < kCandCap) cand[p] = Cand{key[q], (long long)(i0 + (size_t)q * 1024)};
                ++p;
            }
        }
    }
    if (mine_eq) {
        unsigned int p = s_tbase + first_eq;
#pragma unroll
        for (int q = 0; q < kFilterPer; ++q) {
            if (key[q] == thr) {
                if (p < kTieCap) tiecand[p] = Cand{key[q], (long long)(i0 + (size_t)q * 1024)};
                ++p;
            }
        }
    }
}

// Entry j of the selection's input: the candidates in LDS, or -- when more entries passed the filter than LDS holds --
// the whole input again, read from global memory (slow, exact, and rare: see kShortMaxNK).
struct ShortSource {
    const unsigned long long *lkey; const unsigned int *lidx;     // LDS
    const double *t; const uint8_t *f;                             // global
    bool global;
    __device__ __forceinline__ void get(size_t j, unsigned long long &key, unsigned int &idx) const {
        if (global) { key = time_key(t[j], f[j]); idx = (unsigned int)j; }
        else { key = lkey[j]; idx = lidx[j]; }
    }
};

// Rank of `me` among the first `cnt` entries of `list` (LDS) in (key, index) order, for a whole wavefront at once: every
// lane compares one entry, the ballots are counted (a lane that walks the list alone waits for one LDS read per entry).
__device__ __forceinline__ unsigned int short_rank(const Cand *list, unsigned int cnt, const Cand me) {
    const unsigned int lane = threadIdx.x & 63u;
    unsigned int rank = 0;
    for (unsigned int c = 0; c < cnt; c += 64) {
        const unsigned int j = c + lane;
        bool less = false;
        if (j < cnt) {
            const Cand o = list[j];
            less = o.key < me.key || (o.key == me.key && o.idx < me.idx);
        }
        rank += (unsigned int)__popcll(__ballot(less));
    }
    return rank;
}

// (the selection in general: candidates in LDS or the whole input in global memory, equal keys at the threshold)
__device__ __forceinline__ void short_final_any(unsigned char *smem, const double *t, const uint8_t *f, size_t n, ShortTopk *st,
                                                const Cand *cand, const Cand *tiecand, const unsigned int *group_ties, int k,
                                                long long *out_idx, double *out_val, int *out_count) {
    unsigned long long *lkey = reinterpret_cast<unsigned long long *>(smem);                       // [kCandCap]
    unsigned int *lidx = reinterpret_cast<unsigned int *>(smem + (size_t)kCandCap * 8);            // [kCandCap]
    unsigned int *hist = lidx + kCandCap;                                                          // [kRadix]
    Cand *win = reinterpret_cast<Cand *>(hist + kRadix);                                           // [kShortMaxK]
    __shared__ unsigned int wsum[20];
    __shared__ unsigned int s_nwin;
    const int tid = threadIdx.x;
    const unsigned int count_lt = st->count, count_eq = st->count_eq;
    ShortSource src{lkey, lidx, t, f, count_lt > kCandCap};
    // Entries equal to the threshold matter only if fewer than k lie below it.  Then: all of them join the candidates if
    // they were listed one by one and fit; otherwise every entry below wins, and the lowest-indexed equal ones are read
    // from the input (tie_scan, after the selection).
    const bool want_ties = !src.global && count_lt < (unsigned)k && count_eq > 0;
    const bool ties_listed = want_ties && count_eq <= kTieCap && count_lt + count_eq <= kCandCap;
    const bool tie_scan = want_ties && !ties_listed;
    const unsigned int count = count_lt + (ties_listed ? count_eq : 0u);
    const size_t m = src.global ? n : (size_t)count;
    if (!src.global) {
        for (unsigned j = tid; j < count_lt; j += 1024) { const Cand c = cand[j]; lkey[j] = c.key; lidx[j] = (unsigned int)c.idx; }
        if (ties_listed)
            for (unsigned j = tid; j < count_eq; j += 1024) { const Cand c = tiecand[j]; lkey[count_lt + j] = c.key; lidx[count_lt + j] = (unsigned int)c.idx; }
    }
    if (tid == 0) s_nwin = 0;
    // radix select on the 96-bit order (key, index): 6 passes over the key bits, then 3 over the index bits of the entries
    // whose key is the selected one -- cut short as soon as the bucket that holds the k-th entry is small enough to be sorted
    // as it is (usually after two passes).  State is kept by every lane alike (short_pick returns the same values to all).
    constexpr unsigned kSmall = 512;                           // bucket entries that fit the histogram's LDS as (key, index) pairs
    Cand *bucket = reinterpret_cast<Cand *>(hist);
    __shared__ unsigned int s_nbucket;
    __shared__ unsigned long long wmm[48];
    unsigned long long mn = kInfKey, mx = 0, nf = 0;
    __syncthreads();
    for (size_t j = tid; j < m; j += 1024) {
        unsigned long long key; unsigned int idx;
        src.get(j, key, idx);
        if (key != kInfKey) { mn = key < mn ? key : mn; mx = key > mx ? key : mx; ++nf; }
    }
    unsigned long long kmin, kmax, nfin;
    short_minmax(mn, mx, nf, wmm, kmin, kmax, nfin);
    const bool all = nfin < (unsigned long long)k;             // fewer (feasible) candidates than asked for: all of them win
    int cur = (nfin == 0 || kmin == kmax) ? 0 : 64 - __clzll((long long)(kmin ^ kmax));      // the low `cur` key bits vary
    unsigned long long prefix = cur >= 64 ? 0ull : (kmin >> cur) << cur;
    unsigned int iprefix = 0, rem = (unsigned)k;
    bool small = false;
    int small_shift = 0, icur = 32;
    if (tid == 0) s_nbucket = 0;
    // key digits from the highest varying bit down, then index digits among the entries with the selected key
    while (!all && !small && (cur > 0 || icur > 0)) {
        for (int j = tid; j < kRadix; j += 1024) hist[j] = 0;
        __syncthreads();
        const bool on_key = cur > 0;
        const int top = on_key ? cur : icur;
        const int bits = top < kRadixBits ? top : kRadixBits, shift = top - bits;
        for (size_t j = tid; j < m; j += 1024) {
            unsigned long long key; unsigned int idx;
            src.get(j, key, idx);
            if (key == kInfKey) continue;
            if (on_key) {
                if (cur >= 64 || (key >> cur) == (prefix >> cur))
                    atomicAdd(&hist[(unsigned)((key >> shift) & ((1ull << bits) - 1ull))], 1u);
            } else if (key == prefix) {
                if (icur >= 32 || (idx >> icur) == (iprefix >> icur)) atomicAdd(&hist[(idx >> shift) & ((1u << bits) - 1u)], 1u);
            }
        }
        __syncthreads();
        unsigned int before, total;
        const unsigned int b = short_pick(hist, rem, wsum, before, total);
        (void)total;
        rem -= before;
        if (on_key) {
            prefix |= (unsigned long long)b << shift;
            cur = shift;
            if (hist[b] <= kSmall) { small = true; small_shift = shift; }
        } else {
            iprefix |= b << shift;
            icur = shift;
        }
        __syncthreads();                                       // (hist[b] read by all before the next pass clears it)
    }
    // gather the winners
    for (size_t j = tid; j < m; j += 1024) {
        unsigned long long key; unsigned int idx;
        src.get(j, key, idx);
        if (key == kInfKey) continue;
        bool wins;
        if (all) wins = true;
        else if (small) {
            // the key bits from small_shift up are fixed: below the bucket -> a winner; in it -> sorted below
            const unsigned long long hk = key >> small_shift, hp = prefix >> small_shift;
            wins = hk < hp;
            if (hk == hp) {
                const unsigned int p = atomicAdd(&s_nbucket, 1u);
                if (p < kSmall) bucket[p] = Cand{key, (long long)idx};
            }
        } else wins = key < prefix || (key == prefix && idx <= iprefix);
        if (wins) {
            const unsigned int p = atomicAdd(&s_nwin, 1u);
            if (p < (unsigned)kShortMaxK) win[p] = Cand{key, (long long)idx};
        }
    }
    __syncthreads();
    if (small) {
        // the `rem` smallest (key, index) of the bucket join the winners: an entry's rank is the number of entries before
        // it in that order (the pairs are distinct); a wavefront ranks one entry at a time by ballot
        const unsigned int nb = s_nbucket < kSmall ? s_nbucket : kSmall;
        const unsigned int base = s_nwin;
        for (unsigned int i = (unsigned int)tid >> 6; i < nb; i += 16) {
            const Cand me = bucket[i];
            const unsigned int rank = short_rank(bucket, nb, me);
            if ((tid & 63) == 0 && rank < rem && base + rank < (unsigned)kShortMaxK) win[base + rank] = me;
        }
        __syncthreads();
        if (tid == 0) s_nwin = base + rem;
    }
    __syncthreads();
    if (tie_scan) {
        // every candidate below the threshold has won (there are fewer than k: `all`); the rest of the k are the entries
        // EQUAL to the threshold with the lowest indices.  group_ties[g] says how many of them stretch g of the input
        // (8,192 consecutive entries) holds: stretches without any are skipped, the others read 1,024 entries at a time
        // in index order, each lane ranking its entry among the equal ones of the step (wavefront ballots, one
        // exchange through LDS), until enough are found.
        const unsigned long long thr = st->thr;
        const unsigned int need = (unsigned)k - s_nwin, base = s_nwin;
        const unsigned int n_groups = (unsigned int)((n + 1024 * (size_t)kFilterPer - 1) / (1024 * (size_t)kFilterPer));
        __shared__ unsigned int s_wave_ties[16];
        unsigned int found = 0;
        for (unsigned int g = 0; g < n_groups && found < need; ++g) {
            if (group_ties[g] == 0) continue;                  // (the same for every lane)
            for (int c = 0; c < kFilterPer && found < need; ++c) {
                const size_t i = (size_t)g * 1024 * kFilterPer + (size_t)c * 1024 + (size_t)tid;
                const bool eq = i < n && time_key(t[i], f[i]) == thr;
                const unsigned long long mask = __ballot(eq);
                const int lane = tid & 63, wave = tid >> 6;
                if (lane == 0) s_wave_ties[wave] = (unsigned int)__popcll(mask);
                __syncthreads();
                unsigned int before = 0, total = 0;
                for (int w = 0; w < 16; ++w) { const unsigned int v = s_wave_ties[w]; before += w < wave ? v : 0u; total += v; }
                const unsigned int rank = found + before + (unsigned int)__popcll(mask & ((1ull << lane) - 1ull));
                if (eq && rank < need && base + rank < (unsigned)kShortMaxK) win[base + rank] = Cand{thr, (long long)i};
                found += total;
                __syncthreads();
            }
        }
        if (tid == 0) s_nwin = base + (found < need ? found : need);
        __syncthreads();
    }
    const unsigned int nwin = s_nwin < (unsigned)k ? s_nwin : (unsigned)k;
    // the winners in ascending (key, index) order, by rank as above
    for (unsigned j = tid; j < (unsigned)k; j += 1024) {
        if (j >= nwin) {
            out_idx[j] = -1;
            out_val[j] = __longlong_as_double(0x7ff0000000000000ll);
        }
    }
    for (unsigned int i = (unsigned int)tid >> 6; i < nwin; i += 16) {
        const Cand me = win[i];
        const unsigned int rank = short_rank(win, nwin, me);
        if ((tid & 63) == 0) {
            unsigned long long b = me.key;
            b = (b >> 63) ? (b & 0x7fffffffffffffffull) : ~b;
            out_idx[rank] = me.idx;
            out_val[rank] = __longlong_as_double((long long)b);
        }
    }
    if (tid == 0 && out_count) *out_count = (int)nwin;
}

// The selection's common case -- at least k candidates below the threshold and no more than LDS-sized lists were made
// for -- with the candidates in REGISTERS (twelve per lane, read once from global memory): the same radix select on
// (key, index), but no pass reads anything, the bits that vary are found from key XOR threshold (every candidate lies
// below the threshold, so the bits above the highest differing one are the threshold's: one 32-bit maximum over the
// workgroup instead of a 64-bit minimum and maximum), and the two small sorts rank by ballot.
__device__ __forceinline__ void short_final_fast(unsigned char *smem, const ShortTopk *st, const Cand *cand, unsigned int m, int k,
                                                 long long *out_idx, double *out_val, int *out_count) {
    constexpr int kPer = (int)((kCandCap + 1023u) / 1024u);
    constexpr unsigned kSmall = 512;                           // bucket entries that fit the histogram's LDS as (key, index) pairs
    unsigned int *hist = reinterpret_cast<unsigned int *>(smem);                                   // [kRadix]
    Cand *bucket = reinterpret_cast<Cand *>(hist);                                                 // [kSmall], after the passes
    Cand *win = reinterpret_cast<Cand *>(hist + kRadix);                                           // [kShortMaxK]
    __shared__ unsigned int wsum[20];
    __shared__ unsigned int s_nwin, s_nbucket, s_cur;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    unsigned long long rk[kPer];
    unsigned int ri[kPer];
#pragma unroll
    for (int q = 0; q < kPer; ++q) {
        const unsigned int j = (unsigned int)tid + (unsigned int)q * 1024u;
        rk[q] = kInfKey;
        ri[q] = 0;
        if (j < m) { const Cand c = cand[j]; rk[q] = c.key; ri[q] = (unsigned int)c.idx; }
    }
    if (tid == 0) { s_nwin = 0; s_nbucket = 0; s_cur = 0; }
    const unsigned long long thr = st->thr;
    int hb = 0;
#pragma unroll
    for (int q = 0; q < kPer; ++q) {
        if (rk[q] != kInfKey) {
            const int b = 64 - __clzll((long long)(rk[q] ^ thr));
            hb = b > hb ? b : hb;
        }
    }
    for (int off = 32; off > 0; off >>= 1) {
        const int o = __shfl_xor(hb, off, 64);
        hb = o > hb ? o : hb;
    }
    __syncthreads();
    if (lane == 0) atomicMax(&s_cur, (unsigned int)hb);
    __syncthreads();
    int cur = (int)s_cur;                                      // the low `cur` key bits vary (>= 1: every key differs from thr)
    unsigned long long prefix = cur >= 64 ? 0ull : (thr >> cur) << cur;
    unsigned int iprefix = 0, rem = (unsigned)k;
    bool small = false;
    int small_shift = 0, icur = 32;
    // key digits from the highest varying bit down, then index digits among the entries with the selected key
    while (!small && (cur > 0 || icur > 0)) {
        for (int j = tid; j < kRadix; j += 1024) hist[j] = 0;
        __syncthreads();
        const bool on_key = cur > 0;
        const int top = on_key ? cur : icur;
        const int bits = top < kRadixBits ? top : kRadixBits, shift = top - bits;
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
            const unsigned long long key = rk[q];
            if (key == kInfKey) continue;
            if (on_key) {
                if (cur >= 64 || (key >> cur) == (prefix >> cur))
                    atomicAdd(&hist[(unsigned)((key >> shift) & ((1ull << bits) - 1ull))], 1u);
            } else if (key == prefix) {
                if (icur >= 32 || (ri[q] >> icur) == (iprefix >> icur)) atomicAdd(&hist[(ri[q] >> shift) & ((1u << bits) - 1u)], 1u);
            }
        }
        __syncthreads();
        unsigned int before, total;
        const unsigned int b = short_pick(hist, rem, wsum, before, total);
        (void)total;
        rem -= before;
        if (on_key) {
            prefix |= (unsigned long long)b << shift;
            cur = shift;
            if (hist[b] <= kSmall) { small = true; small_shift = shift; }
        } else {
            iprefix |= b << shift;
            icur = shift;
        }
        __syncthreads();                                       // (hist[b] read by all before the next pass clears it)
    }
    // gather the winners (the bucket's entries go where the histogram was)
#pragma unroll
    for (int q = 0; q < kPer; ++q) {
        const unsigned long long key = rk[q];
        if (key == kInfKey) continue;
        bool wins;
        if (small) {
            const unsigned long long hk = key >> small_shift, hp = prefix >> small_shift;
            wins = hk < hp;
            if (hk == hp) {
                const unsigned int p = atomicAdd(&s_nbucket, 1u);
                if (p < kSmall) bucket[p] = Cand{key, (long long)ri[q]};
            }
        } else wins = key < prefix || (key == prefix && ri[q] <= iprefix);
        if (wins) {
            const unsigned int p = atomicAdd(&s_nwin, 1u);
            if (p < (unsigned)kShortMaxK) win[p] = Cand{key, (long long)ri[q]};
        }
    }
    __syncthreads();
    if (small) {
        // the `rem` smallest (key, index) of the bucket join the winners, each at its rank
        const unsigned int nb = s_nbucket < kSmall ? s_nbucket : kSmall;
        const unsigned int base = s_nwin;
        for (unsigned int i = (unsigned int)wave; i < nb; i += 16) {
            const Cand me = bucket[i];
            const unsigned int rank = short_rank(bucket, nb, me);
            if (lane == 0 && rank < rem && base + rank < (unsigned)kShortMaxK) win[base + rank] = me;
        }
        __syncthreads();
        if (tid == 0) s_nwin = base + rem;
    }
    __syncthreads();
    const unsigned int nwin = s_nwin < (unsigned)k ? s_nwin : (unsigned)k;
    for (unsigned j = tid; j < (unsigned)k; j += 1024) {
        if (j >= nwin) {
            out_idx[j] = -1;
            out_val[j] = __longlong_as_double(0x7ff0000000000000ll);
        }
    }
    // the winners in ascending (key, index) order
    for (unsigned int i = (unsigned int)wave; i < nwin; i += 16) {
        const Cand me = win[i];
        const unsigned int rank = short_rank(win, nwin, me);
        if (lane == 0) {
            unsigned long long b = me.key;
            b = (b >> 63) ? (b & 0x7fffffffffffffffull) : ~b;
            out_idx[rank] = me.idx;
            out_val[rank] = __longlong_as_double((long long)b);
        }
    }
    if (tid == 0 && out_count) *out_count = (int)nwin;
}

__global__ __launch_bounds__(1024) void topk_short_final(const double *t, const uint8_t *f, size_t n, ShortTopk *st, const Cand *cand,
                                                         const Cand *tiecand, const unsigned int *group_ties, int k,
                                                         long long *out_idx, double *out_val, int *out_count) {
    extern __shared__ __align__(16) unsigned char smem[];
    const unsigned int count_lt = st->count;
    if (count_lt >= (unsigned)k && count_lt <= kCandCap) short_final_fast(smem, st, cand, count_lt, k, out_idx, out_val, out_count);
    else short_final_any(smem, t, f, n, st, cand, tiecand, group_ties, k, out_idx, out_val, out_count);
}
constexpr size_t kShortLds = (size_t)kCandCap * 12 + (size_t)kRadix * 4 + (size_t)kShortMaxK * sizeof(Cand);

unsigned int next_pow2(unsigned int v) {
    unsigned int p = 1;
    while (p < v) p <<= 1;
    return p;
}

}  // namespace

struct ace_handle {
    int device;
    AceGeom geom;
    int32_t n_windows, row_doubles, rk_bytes, stg_words, num_types;
    uint32_t lds_bytes;
    // device copies
    double *d_rows;
    uint32_t *d_pos_info;
    uint32_t *d_pos_types;     // d_pos_info with row indices in place of LDS slots (windowed rows, at most 256 of them; else null)
    ace_u4 *d_pos4;            // per position, for the assembly op loop (null when its pair-kind table has no room in LDS)
    ace_u4 *d_win_dma;         // windowed rows: what the assembly op loop fetches its windows by (setup_windowed_asm), or null
    AceGeom geom_wa;           // ... and the LDS layout of the kernel that runs it
    uint32_t lds_bytes_wa;
    uint8_t *d_pair_kinds;
    uint32_t *d_stage_lut;
    double *d_nbm1;
    int32_t *d_win_pos, *d_win_row_begin;
    uint32_t *d_win_rows;
    int32_t flat_rows16;       // see AceKernelArgs
    double *d_stage_ws;        // grow-only workspace for deferred stage tails
    size_t stage_ws_plans;     // capacity in plans
    int stage_ws_fixed;        // ace_reserve(..., fixed): a larger batch is an error instead of a reallocation
};

// The bodies of these kernels live in ace_edit_kernels.h (shared with the host build of the tests).
__global__ __launch_bounds__(256) void apply_moves_kernel(const ace_u4 *tmpl_codes, const ace_u4 *tmpl_hdr, int n_templates,
                                                          const ace_u4 *moves, unsigned long long n, int G, int a_shift,
                                                          ace_u4 *codes_out, ace_u4 *hdr_out, unsigned long long *key_out) {
    apply_moves_body((unsigned long long)blockIdx.x * 256 + threadIdx.x, tmpl_codes, tmpl_hdr, n_templates, moves, n, G, a_shift,
                     codes_out, hdr_out, key_out);
}

__global__ __launch_bounds__(256) void group_keys_kernel(const ace_u4 *codes, const ace_u4 *hdr, unsigned long long n, int G, int N,
                                                         unsigned long long *keys) {
    group_keys_body((unsigned long long)blockIdx.x * 256 + threadIdx.x, codes, hdr, n, G, N, keys);
}

__global__ __launch_bounds__(256) void gather_plans_kernel(const ace_u4 *codes_in, const ace_u4 *hdr_in, const uint32_t *perm,
                                                           unsigned long long n, int G, ace_u4 *codes_out, ace_u4 *hdr_out) {
    gather_plans_body((unsigned long long)blockIdx.x * 256 + threadIdx.x, codes_in, hdr_in, perm, n, G, codes_out, hdr_out);
}

__global__ void rc_groups_kernel(RcTables t, int n, const int32_t *q_plan, const int32_t *q_lo, const int32_t *q_hi,
                                 const int32_t *q_nsb, const uint32_t *q_mrow, double *sum_size, int32_t *first_pos,
                                 int32_t *bad) {
    rc_groups_body((int)(blockIdx.x * blockDim.x + threadIdx.x), t, n, q_plan, q_lo, q_hi, q_nsb, q_mrow, sum_size, first_pos, bad);
}

__global__ void rc_select_kernel(RcTables t, uint8_t *codes_rw, int n, const int32_t *q_plan, const int32_t *q_lo,
                                 const int32_t *q_hi, const int32_t *q_nsb, const uint32_t *q_mrow, const double *sum_size,
                                 const int32_t *first_pos, uint8_t *recomputed, const double *mem, double memory_limit,
                                 uint8_t *alive) {
    rc_select_body((int)(blockIdx.x * blockDim.x + threadIdx.x), t, codes_rw, n, q_plan, q_lo, q_hi, q_nsb, q_mrow, sum_size,
                   first_pos, recomputed, mem, memory_limit, alive);
}

extern "C" {

int ace_abi_version(void) { return ACE_ABI_VERSION; }

const char *ace_strerror(int code) {
    switch (code) {
        case ACE_OK: return "ok";
        case ACE_EINVAL: return "invalid argument";
        case ACE_ETOOBIG: return "table row larger than LDS";
        case ACE_EHIP: return "HIP runtime error";
        case ACE_ENOMEM: return "out of memory";
        case ACE_EVERSION: return "ABI version mismatch";
        case ACE_EFIXED: return "the batch needs a larger workspace than the one fixed with ace_reserve";
        default: return "unknown error";
    }
}

const char *ace_last_hip_error(void) { return g_hip_err; }

static int upload(void **dst, const void *src, size_t bytes, size_t alloc_bytes = 0) {
    *dst = nullptr;
    if (alloc_bytes < bytes) alloc_bytes = bytes;
    if (alloc_bytes == 0) alloc_bytes = 16;
    ACE_HIP(hipMalloc(dst, alloc_bytes));
    if (alloc_bytes > bytes) ACE_HIP(hipMemset(*dst, 0, alloc_bytes));
    if (src && bytes) ACE_HIP(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
    return ACE_OK;
}

}  // extern "C"

template <bool BD, bool RANGED, bool WIN, bool DEFER> static int allow_big_lds() {
    ACE_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&ace_score_kernel<BD, RANGED, WIN, DEFER, kBlock>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    ACE_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&ace_score_kernel<BD, RANGED, WIN, DEFER, kSmallBlock>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    if (!DEFER)
        ACE_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&ace_score_kernel<BD, RANGED, WIN, false, kBlock, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    return ACE_OK;
}

// Per op position, what the assembly form of the op loop (ace_score_loop_asm.inc) reads with scalar loads: the LDS
// address of the position's row at its hot sub-table and at its collective-cost tables, the LDS address of the
// 32-bit pair-kind block of the (this op, next op) pair, and two flags (bit 0: the rule "ordinary op followed by a layer
// start" does NOT apply here, bit 1: ordinary op).  Positions past the last op point at row 0 and pair kind 0.
static int upload_pos4(ace_handle *h, const ace_tables_t *t, size_t pos_entries, uint32_t pk32_off) {
    h->d_pos4 = nullptr;
    if (!pk32_off || t->n_windows != 1) return ACE_OK;       // (windowed rows: setup_windowed_asm)
    ace_u4 *p4 = new (std::nothrow) ace_u4[pos_entries];
    if (!p4) return ACE_ENOMEM;
    const uint32_t row_bytes = (uint32_t)t->row_doubles * 8u, kind_stride = (uint32_t)t->n_glog * ACE_PK32_BLOCK;   // (words of the 32-bit table per pair kind)
    for (size_t i = 0; i < pos_entries; ++i) {
        const uint32_t info = i < (size_t)t->num_ops ? t->pos_info[i] : 0u;
        const uint32_t row = (info & 0xffu) * row_bytes;
        p4[i].x = row + (uint32_t)t->hot_off * 8u;
        p4[i].y = row + (uint32_t)t->z_off * 8u;
        p4[i].z = pk32_off + ((info >> 16) & 0xffu) * kind_stride * 4u;
        // (rows as the evaluation of the stage tails indexes them: LDS slots)
        const uint32_t ids = info & 0xffffu;
        p4[i].w = (((info >> 24) & 1u) ^ 1u) | (((info >> 25) & 1u) << 1) | (ids << 8);
    }
    const int rc = upload((void **)&h->d_pos4, p4, pos_entries * sizeof(ace_u4));
    delete[] p4;
    return rc;
}

// Windowed rows: the position descriptors with each row's index in `rows` where its LDS slot is.
static int upload_pos_types(ace_handle *h, const ace_tables_t *t, size_t pos_entries) {
    h->d_pos_types = nullptr;
    if (t->n_windows <= 1 || t->num_types > 256) return ACE_OK;
    uint32_t *pt = new (std::nothrow) uint32_t[pos_entries];
    if (!pt) return ACE_ENOMEM;
    ace_pos_types(t, pt, pos_entries);
    const int rc = upload((void **)&h->d_pos_types, pt, pos_entries * 4);
    delete[] pt;
    return rc;
}

// Windowed rows, for the assembly op loop.  That loop reads only the hot sub-table and the collective-cost tables of a
// row (the boundary sub-tables are read from global memory when the stage tails are evaluated), so it keeps its own,
// denser windows: per row those two parts back to back, consecutive windows in alternate halves of the region in front of
// the small tables, so that a window is fetched while the one before it is walked.  Built here: the LDS layout
// (h->geom_wa), the per-position table (h->d_pos4) and the fetch records (h->d_win_dma): per fetch event and wavefront
// (sixteen) 80 bytes = {first position of the window after the one being entered, bit 0: wait for the fetch (else it
// completes before the next event) | number of loads << 8, address of the rows} and eight LDS-direct loads {byte offset
// in the rows, LDS address} of 1 KB each.  Events: 0 fetches window 0 and waits, 1 fetches window 1, and entering window
// w >= 1 fetches window w + 1 (the last one fetches window w - 1 again, into the half nobody reads).
// Leaves the handle without them (plain scoring then takes the C++ loop) where the layout does not work out.
static int setup_windowed_asm(ace_handle *h, const ace_tables_t *t, size_t pos_entries, int32_t rk_bytes, int32_t stg_words) {
    h->d_win_dma = nullptr;
    if (t->n_windows <= 1 || !h->d_pos_types || (t->flags & ACE_F_COLLECTIVE_MEM) || t->num_ops >= 32768) return ACE_OK;
    if ((int64_t)(t->n_z > 0 ? t->n_z : 1) * t->z_table_doubles * 8 > 65536) return ACE_OK;
    const uint64_t row_bytes = (uint64_t)t->row_doubles * 8u;
    if ((uint64_t)t->num_types * row_bytes > 0xffffffffull) return ACE_OK;
    if (!(t->hot_off < t->start_off && t->start_off <= t->z_off && t->z_off <= t->row_doubles)) return ACE_OK;
    const uint32_t hot_len = (uint32_t)(t->start_off - t->hot_off) * 8u, z_len = (uint32_t)(t->row_doubles - t->z_off) * 8u;
    if (hot_len < 1024u || (z_len != 0u && z_len < 1024u) || (hot_len & 15u) || (z_len & 15u)) return ACE_OK;
    const uint32_t crow = hot_len + z_len;
    // the most rows per half that leave room for the small tables
    uint32_t slots = 127, stg_off = 0, lut2_off = 0, pk32_off = 0, lut2a_off = 0, lds_end = 0;
    for (; slots >= 5u; --slots) {
        lut2a_off = (ace_lds_pk32(ace_lds_layout(2u * slots * crow, (uint32_t)rk_bytes, (uint32_t)stg_words, &stg_off, &lut2_off),
                                  (uint32_t)rk_bytes, &pk32_off) + 15u) & ~15u;
        lds_end = lut2a_off + (uint32_t)stg_words * 8u;
        if (lds_end <= kMaxLds) break;
    }
    if (slots < 5u) return ACE_OK;
    const int N = t->num_ops;
    std::vector<uint32_t> types(pos_entries);
    ace_pos_types(t, types.data(), pos_entries);
    // windows end at multiples of 4 ops (or at the last op) and hold at most `slots` different rows
    std::vector<int> win_start;
    std::vector<std::vector<uint32_t>> win_types;
    for (int i = 0; i < N;) {
        std::vector<uint32_t> seen;
        int good = -1;
        size_t good_n = 0;
        for (int j = i; j < N;) {
            const uint32_t ty = types[j] & 0xffu;
            if (std::find(seen.begin(), seen.end(), ty) == seen.end()) {
                if (seen.size() >= slots) break;
                seen.push_back(ty);
            }
            ++j;
            if (j == N || (j & 3) == 0) { good = j; good_n = seen.size(); }
        }
        if (good < 0) return ACE_OK;
        seen.resize(good_n);
        win_start.push_back(i);
        win_types.push_back(seen);
        i = good;
    }
    const int n_w = (int)win_start.size();
    if (n_w < 2) return ACE_OK;
    auto row_addr = [&](int w, uint32_t ty) {
        const std::vector<uint32_t> &v = win_types[w];
        return (uint32_t)((w & 1) * slots + (uint32_t)(std::find(v.begin(), v.end(), ty) - v.begin())) * crow;
    };
    // the per-position table
    std::vector<ace_u4> p4(pos_entries);
    const uint32_t kind_stride = (uint32_t)t->n_glog * ACE_PK32_BLOCK;
    for (size_t i = 0, w = 0; i < pos_entries; ++i) {
        if (i >= (size_t)N) { p4[i] = ace_u4{0u, hot_len, pk32_off, 0u}; continue; }
        while ((int)w + 1 < n_w && (size_t)win_start[w + 1] <= i) ++w;
        const uint32_t info = t->pos_info[i], at = row_addr((int)w, types[i] & 0xffu);
        p4[i] = ace_u4{at, at + hot_len, pk32_off + ((info >> 16) & 0xffu) * kind_stride * 4u,
                       (((info >> 24) & 1u) ^ 1u) | (((info >> 25) & 1u) << 1) | ((types[i] & 0xffffu) << 8)};
    }
    // the loads of each window, dealt to the wavefronts in turn (the last load of a part ends with the part: it may
    // overlap the one before it)
    std::vector<std::vector<ace_u2>> loads(n_w);
    for (int w = 0; w < n_w; ++w)
        for (uint32_t ty : win_types[w]) {
            const uint32_t at = row_addr(w, ty), src = (uint32_t)(ty * row_bytes);
            for (int part = 0; part < 2; ++part) {
                const uint32_t len = part ? z_len : hot_len, from = src + (uint32_t)(part ? t->z_off : t->hot_off) * 8u;
                for (uint32_t off = 0; off < len; off += 1024u) {
                    const uint32_t o = off + 1024u <= len ? off : len - 1024u;
                    loads[w].push_back(ace_u2{from + o, at + (part ? hot_len : 0u) + o});
                }
            }
        }
    for (int w = 0; w < n_w; ++w)
        if (loads[w].size() > 16u * 8u) return ACE_OK;
    const int n_ev = n_w + 1;
    std::vector<ace_u4> blob((size_t)n_ev * 16u * 5u, ace_u4{0u, 0u, 0u, 0u});
    const uint64_t rows_at = (uint64_t)(uintptr_t)h->d_rows;
    for (int e = 0; e < n_ev; ++e) {
        const int entering = e < 2 ? 0 : e - 1;                        // the window walked after this event
        int fetch = e == 0 ? 0 : entering + 1;
        if (fetch >= n_w) fetch = entering - 1;
        const uint32_t nextwin = entering + 1 < n_w ? (uint32_t)win_start[entering + 1] : 0x7fffffffu;
        for (uint32_t v = 0; v < 16u; ++v) {
            ace_u4 *rec = &blob[((size_t)e * 16u + v) * 5u];
            uint32_t d[16] = {0};
            uint32_t n = 0;
            for (size_t c = v; c < loads[fetch].size(); c += 16u, ++n) { d[2 * n] = loads[fetch][c].x; d[2 * n + 1] = loads[fetch][c].y; }
            rec[0] = ace_u4{nextwin, (e == 0 ? 1u : 0u) | (n << 8), (uint32_t)rows_at, (uint32_t)(rows_at >> 32)};
            for (int q = 0; q < 4; ++q) rec[1 + q] = ace_u4{d[4 * q], d[4 * q + 1], d[4 * q + 2], d[4 * q + 3]};
        }
    }
    int rc = upload((void **)&h->d_win_dma, blob.data(), blob.size() * sizeof(ace_u4));
    if (rc == ACE_OK) rc = upload((void **)&h->d_pos4, p4.data(), p4.size() * sizeof(ace_u4));
    if (rc != ACE_OK) return rc;
    h->geom_wa = h->geom;
    h->geom_wa.rk_lds_off = 2u * slots * crow;
    h->geom_wa.stg_lds_off = stg_off; h->geom_wa.lut2_lds_off = lut2_off; h->geom_wa.pk32_lds_off = pk32_off; h->geom_wa.pace_lds_off = 0; h->geom_wa.lut2a_lds_off = lut2a_off;
    h->lds_bytes_wa = lds_end;
    return ACE_OK;
}

// The device address of `scratch` on the current device (looked up once per device).
static int static_scratch_ptr(double **out) {
    int dev = -1;
    ACE_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return ACE_EINVAL;
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_ptr[dev]) {
        void *p = nullptr;
        ACE_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return ACE_EHIP;
        g_static_ptr[dev] = static_cast<double *>(p);
    }
    *out = g_static_ptr[dev];
    return ACE_OK;
}

extern "C" {

int ace_create(const ace_tables_t *t, ace_handle_t **out) {
    if (!t || !out) return ACE_EINVAL;
    *out = nullptr;
    if (t->abi_version != ACE_ABI_VERSION) return ACE_EVERSION;
    if (t->num_ops <= 0 || t->num_types <= 0 || t->n_mbs <= 0 || t->n_mbs > 15 || t->n_tp <= 0 || t->n_tp > 4 ||
        (t->n_algo != 1 && t->n_algo != 2) || t->n_diag <= 0 || t->n_diag > 14 || t->n_glog <= 0 || t->n_glog > 16 ||
        t->n_z < 0 || t->n_z == 1 || t->n_z > 15 || ((t->flags & ACE_F_RESHARDING) && t->n_z < 2) || t->z_table_doubles <= 0 || (t->z_table_doubles & (t->z_table_doubles - 1)) || t->n_pair_kinds <= 0 || t->n_pair_kinds > 255 || t->row_doubles <= 0 ||
        (t->row_doubles & 1) || t->n_windows <= 0 || t->lds_row_bytes <= 0 || (t->lds_row_bytes & 15) ||
        !t->rows || !t->pos_info || !t->pair_kinds || !t->stage_lut || !t->nb_minus_1 || !t->win_pos ||
        !t->win_row_begin || !t->win_rows)
        return ACE_EINVAL;
    const int C = t->n_tp * t->n_algo;
    // sub-tables must lie inside a row and be 16-byte aligned
    const int64_t hot_end = (int64_t)t->hot_off + (int64_t)(t->n_diag + 1) * C * 6;
    const int64_t start_end = (int64_t)t->start_off + (int64_t)t->n_diag * C * 3;
    const int64_t out_end = (int64_t)t->out_off + (int64_t)t->n_mbs * t->n_tp * t->n_algo * 2;
    if ((t->flags & ACE_F_COLLECTIVE_MEM) && !(t->flags & ACE_F_RESHARDING)) return ACE_EINVAL;
    const int64_t z_end = (int64_t)t->z_off + (int64_t)t->n_z * t->z_table_doubles * ((t->flags & ACE_F_COLLECTIVE_MEM) ? 2 : 1);
    if (t->z_table_doubles < t->n_diag * C) return ACE_EINVAL;
    if ((t->hot_off & 1) || (t->start_off & 1) || (t->out_off & 1) || (t->z_off & 1) || t->hot_off < 0 ||
        t->start_off < 0 || t->out_off < 0 || t->z_off < 0 ||
        hot_end > t->row_doubles || start_end > t->row_doubles || out_end > t->row_doubles || z_end > t->row_doubles)
        return ACE_EINVAL;
    const int64_t row_bytes = (int64_t)t->row_doubles * 8;
    if (row_bytes > t->lds_row_bytes || t->lds_row_bytes > (int32_t)kMaxLds) return ACE_ETOOBIG;
    const int32_t rk_bytes = t->n_pair_kinds * t->n_glog * 64;
    const int32_t stg_words = t->n_mbs * 16;
    const uint32_t rk_off = (uint32_t)t->lds_row_bytes;
    uint32_t stg_off, lut2_off;
    uint32_t lds_bytes = ace_lds_layout(rk_off, (uint32_t)rk_bytes, (uint32_t)stg_words, &stg_off, &lut2_off);
    if (lds_bytes > kMaxLds) return ACE_ETOOBIG;
    // the assembly loop's pair-kind table, where the table has room and its entries can hold the offsets (otherwise plain
    // scoring takes the C++ form of the loop)
    uint32_t pk32_off = 0, pace_off = 0, lut2a_off = 0;
    if (t->n_windows == 1) {                               // (windowed rows: setup_windowed_asm lays LDS out anew)
        uint32_t off;
        const uint32_t end = ace_lds_pk32(lds_bytes, (uint32_t)rk_bytes, &off);
        // (behind it: the loop's arrival counters and its own per-(micro-batch, stage size) offset pairs)
        if (end + 128u + (uint32_t)stg_words * 8u + 16u <= kMaxLds && ((int64_t)(t->n_z > 0 ? t->n_z : 1) * t->z_table_doubles * 8) <= 65536) {
            pk32_off = off;
            pace_off = (end + 15u) & ~15u;
            lut2a_off = pace_off + 128u;
            lds_bytes = lut2a_off + (uint32_t)stg_words * 8u;
        }
    }
    // (the in-kernel sort keeps its bins and its permutation in the first 128 + 2 * kBlock bytes of LDS before the
    // tables are staged there: tiny tables still get that much)
    const uint32_t lds_floor = 128u + 2u * (uint32_t)kBlock;
    const uint32_t lds_alloc = lds_bytes < lds_floor ? lds_floor : lds_bytes;
    // window tables: window starts are multiples of 4 ops; every referenced row must fit the
    // resident region; every position's row offsets must point at a row start inside it
    const int32_t n_win_rows = t->win_row_begin[t->n_windows];
    if (t->win_pos[0] != 0 || t->win_row_begin[0] != 0 || n_win_rows <= 0) return ACE_EINVAL;
    for (int w = 0; w < t->n_windows; ++w) {
        if (t->win_pos[w + 1] <= t->win_pos[w] || t->win_row_begin[w + 1] < t->win_row_begin[w] || (t->win_pos[w] & 3))
            return ACE_EINVAL;
    }
    if (t->win_pos[t->n_windows] < t->num_ops) return ACE_EINVAL;
    for (int r = 0; r < n_win_rows; ++r) {
        if (t->win_rows[2 * r] >= (uint32_t)t->num_types) return ACE_EINVAL;
        if ((int64_t)t->win_rows[2 * r + 1] + row_bytes > t->lds_row_bytes || (t->win_rows[2 * r + 1] & 15u)) return ACE_EINVAL;
    }
    for (int i = 0; i <= t->num_ops; ++i) {
        const uint32_t pi = t->pos_info[i];
        if ((int64_t)((pi & 0xffu) + 1) * row_bytes > t->lds_row_bytes || (int64_t)(((pi >> 8) & 0xffu) + 1) * row_bytes > t->lds_row_bytes ||
            ((pi >> 16) & 0xffu) >= (uint32_t)t->n_pair_kinds)
            return ACE_EINVAL;
    }
    for (int j = 0; j < stg_words; ++j) {
        // the diag of every (micro-batch, stage size) pair must exist (n_diag = the all-NaN one)
        if ((t->stage_lut[j] & 0xffffu) > (uint32_t)t->n_diag) return ACE_EINVAL;
    }
    for (int j = 0; j < rk_bytes; ++j) {
        const uint32_t lim = t->n_z ? (uint32_t)t->n_z : 1u;
        if ((t->pair_kinds[j] & 15u) >= lim || (uint32_t)(t->pair_kinds[j] >> 4) >= lim) return ACE_EINVAL;
    }

    ace_handle *h = new (std::nothrow) ace_handle();
    if (!h) return ACE_ENOMEM;
    memset(h, 0, sizeof(*h));
    AceGeom &g = h->geom;
    g.N = t->num_ops; g.P = 0; g.G = (t->num_ops + 15) / 16;
    g.C = C; g.A_shift = t->n_algo == 2 ? 1 : 0;
    g.n_mbs = t->n_mbs; g.n_tp = t->n_tp; g.n_algo = t->n_algo; g.n_glog = t->n_glog; g.n_pair_kinds = t->n_pair_kinds;
    g.hot_off = (uint32_t)t->hot_off * 8u; g.start_off = (uint32_t)t->start_off * 8u;
    g.out_off = (uint32_t)t->out_off * 8u; g.z_off = (uint32_t)t->z_off * 8u;
    g.z_shift = 3;
    while ((1 << (g.z_shift - 3)) < t->z_table_doubles) ++g.z_shift;
    g.zm_delta = (uint32_t)t->n_z << g.z_shift;
    g.rk_lds_off = rk_off; g.stg_lds_off = stg_off; g.lut2_lds_off = lut2_off; g.pk32_lds_off = pk32_off; g.pace_lds_off = pace_off; g.lut2a_lds_off = lut2a_off;
    g.rk_kind_stride = (uint32_t)(t->n_glog * 64);
    g.row_bytes = (uint32_t)row_bytes;
    g.flags = t->flags; g.main_params = t->main_params; g.optimizer = t->optimizer;
    g.mem_limit = 0.0; g.strict = 0;
    h->n_windows = t->n_windows; h->row_doubles = t->row_doubles; h->rk_bytes = rk_bytes; h->stg_words = stg_words;
    // rows resident, slot r of LDS holding row r: the kernels stage them as one block
    h->flat_rows16 = 0;
    if (t->n_windows == 1 && (row_bytes & 15) == 0) {
        bool flat = true;
        for (int r = 0; r < n_win_rows; ++r)
            flat = flat && t->win_rows[2 * r] == (uint32_t)r && t->win_rows[2 * r + 1] == (uint32_t)(r * row_bytes);
        if (flat) h->flat_rows16 = (int32_t)(n_win_rows * row_bytes / 16);
    }
    h->num_types = t->num_types; h->lds_bytes = lds_alloc;
    const size_t pos_entries = (size_t)((t->num_ops + 15) / 16) * 16 + 16;
    int rc;
    double *scratch_here = nullptr;
    if ((rc = hipGetDevice(&h->device) == hipSuccess ? ACE_OK : ACE_EHIP) ||
        (rc = static_scratch_ptr(&scratch_here)) ||
        (rc = upload((void **)&h->d_rows, t->rows, (size_t)t->num_types * row_bytes)) ||
        (rc = upload((void **)&h->d_pos_info, t->pos_info, (size_t)(t->num_ops + 1) * 4, pos_entries * 4)) ||
        (rc = upload_pos4(h, t, pos_entries, pk32_off)) ||
        (rc = upload_pos_types(h, t, pos_entries)) ||
        (rc = upload((void **)&h->d_pair_kinds, t->pair_kinds, (size_t)rk_bytes)) ||
        (rc = upload((void **)&h->d_stage_lut, t->stage_lut, (size_t)stg_words * 4)) ||
        (rc = upload((void **)&h->d_nbm1, t->nb_minus_1, (size_t)t->n_mbs * 8)) ||
        (rc = upload((void **)&h->d_win_pos, t->win_pos, (size_t)(t->n_windows + 1) * 4)) ||
        (rc = upload((void **)&h->d_win_row_begin, t->win_row_begin, (size_t)(t->n_windows + 1) * 4)) ||
        (rc = upload((void **)&h->d_win_rows, t->win_rows, (size_t)n_win_rows * 8)) ||
        (rc = setup_windowed_asm(h, t, pos_entries, rk_bytes, stg_words)) ||
        (rc = hipFuncSetAttribute(reinterpret_cast<const void *>(&topk_short_final), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)kShortLds) == hipSuccess ? ACE_OK : ACE_EHIP) ||
        (rc = allow_big_lds<false, false, false, false>()) || (rc = allow_big_lds<false, false, true, false>()) ||
        (rc = allow_big_lds<false, false, false, true>()) || (rc = allow_big_lds<false, false, true, true>()) ||
        (rc = allow_big_lds<true, false, false, false>()) || (rc = allow_big_lds<true, false, true, false>()) ||
        (rc = allow_big_lds<true, true, false, false>()) || (rc = allow_big_lds<true, true, true, false>())) {
        ace_destroy(h);
        return rc;
    }
    *out = h;
    return ACE_OK;
}

void ace_destroy(ace_handle_t *h) {
    if (!h) return;
    (void)hipFree(h->d_rows); (void)hipFree(h->d_pos_info); (void)hipFree(h->d_pos_types); (void)hipFree(h->d_pair_kinds);
    if (h->d_pos4) (void)hipFree(h->d_pos4);
    if (h->d_win_dma) (void)hipFree(h->d_win_dma);
    (void)hipFree(h->d_stage_lut); (void)hipFree(h->d_nbm1); (void)hipFree(h->d_win_pos);
    (void)hipFree(h->d_win_row_begin); (void)hipFree(h->d_win_rows);
    if (h->d_stage_ws) (void)hipFree(h->d_stage_ws);
    delete h;
}

static int fill_args(ace_handle_t *h, const ace_batch_t *b, double memory_limit, int strict, double *d_iter_ms,
                     double *d_peak_mb, uint8_t *d_feasible, uint8_t *d_status, double *d_stage_out, AceKernelArgs *a) {
    if (!h || !b || !b->d_codes || !b->d_hdr || !d_iter_ms || !d_peak_mb || !d_feasible) return ACE_EINVAL;
    if (b->n_plans == 0 || b->n_plans > 0x7fffffffull) return ACE_EINVAL;
    if (((uintptr_t)b->d_codes & 15u) || ((uintptr_t)b->d_hdr & 15u) || ((uintptr_t)b->d_range & 7u) || ((uintptr_t)b->d_order & 3u))
        return ACE_EINVAL;
    if (b->d_range && !d_stage_out) return ACE_EINVAL;   // single-stage queries are read from their stage record
    a->g = h->geom;
    a->g.P = (int32_t)b->n_plans;
    a->g.mem_limit = memory_limit;
    a->g.strict = strict ? 1 : 0;
    a->codes = reinterpret_cast<const ace_u4 *>(b->d_codes);
    a->hdr = reinterpret_cast<const ace_u4 *>(b->d_hdr);
    a->range = reinterpret_cast<const ace_u2 *>(b->d_range);
    a->order = b->d_order;
    a->rows = h->d_rows; a->pos_info = h->d_pos_info; a->pos_types = h->d_pos_types; a->pos4 = h->d_pos4; a->win_dma = h->d_win_dma; a->pair_kinds = h->d_pair_kinds; a->stage_lut = h->d_stage_lut;
    a->nbm1 = h->d_nbm1; a->win_pos = h->d_win_pos; a->win_row_begin = h->d_win_row_begin; a->win_rows = h->d_win_rows;
    a->n_windows = h->n_windows; a->row_doubles = h->row_doubles; a->rk_bytes = h->rk_bytes; a->stg_words = h->stg_words;
    a->flat_rows16 = h->flat_rows16;
    a->iter_ms = d_iter_ms; a->peak_mb = d_peak_mb; a->feasible = d_feasible; a->status = d_status; a->stage_out = d_stage_out;
    a->stage_ws = nullptr;
    return ACE_OK;
}

}  // extern "C"

template <bool BD, bool RANGED, bool WIN, bool DEFER>
static void launch_score_b(const ace_handle_t *h, const AceKernelArgs &a, hipStream_t s) {
    const size_t P = (size_t)a.g.P;
    if (a.g.flags & ACE_F_COLLECTIVE_MEM) {
        if (!DEFER)         // (ensure_stage_ws never hands such tables to the deferred kernel)
            hipLaunchKernelGGL((ace_score_kernel<BD, RANGED, WIN, false, kBlock, true>), dim3((unsigned)((P + kBlock - 1) / kBlock)),
                               dim3(kBlock), h->lds_bytes, s, a);
    } else if (WIN && DEFER && h->d_win_dma) {
        // the assembly op loop over windowed rows lays LDS out its own way (batches of any size: with the next window
        // arriving while a window is walked, the large workgroup is the faster one from a single plan on)
        AceKernelArgs b = a;
        b.g = h->geom_wa;
        b.g.P = a.g.P; b.g.mem_limit = a.g.mem_limit; b.g.strict = a.g.strict;
        hipLaunchKernelGGL((ace_score_kernel<BD, RANGED, WIN, DEFER, kBlock>), dim3((unsigned)((P + kBlock - 1) / kBlock)),
                           dim3(kBlock), h->lds_bytes_wa, s, b);
    } else if ((P + kBlock - 1) / kBlock < (size_t)kSmallBatchBlocks)
        hipLaunchKernelGGL((ace_score_kernel<BD, RANGED, WIN, DEFER, kSmallBlock>), dim3((unsigned)((P + kSmallBlock - 1) / kSmallBlock)),
                           dim3(kSmallBlock), h->lds_bytes, s, a);
    else
        hipLaunchKernelGGL((ace_score_kernel<BD, RANGED, WIN, DEFER, kBlock>), dim3((unsigned)((P + kBlock - 1) / kBlock)),
                           dim3(kBlock), h->lds_bytes, s, a);
}

template <bool BD, bool RANGED>
static void launch_score_w(const ace_handle_t *h, const AceKernelArgs &a, hipStream_t s) {
    if (h->n_windows > 1) launch_score_b<BD, RANGED, true, false>(h, a, s);
    else launch_score_b<BD, RANGED, false, false>(h, a, s);
}

static void launch_score(const ace_handle_t *h, const AceKernelArgs &a, hipStream_t s) {
    if (a.range) launch_score_w<true, true>(h, a, s);
    else if (a.stage_out) launch_score_w<true, false>(h, a, s);
    else if (a.stage_ws && h->n_windows > 1) launch_score_b<false, false, true, true>(h, a, s);
    else if (a.stage_ws) launch_score_b<false, false, false, true>(h, a, s);
    else launch_score_w<false, false>(h, a, s);
}

// Plain scoring with every row resident uses the deferred-stage-tail kernel, which needs a
// per-plan workspace; the handle keeps one and grows it on demand.
static int ensure_stage_ws(ace_handle_t *h, AceKernelArgs *a) {
    a->stage_ws = nullptr;
    if (a->range || a->stage_out || (h->n_windows > 1 && !h->d_pos_types) || h->geom.N >= 32768 || (h->geom.flags & ACE_F_COLLECTIVE_MEM)) return ACE_OK;
    const size_t need = (((size_t)a->g.P + kBlock - 1) / kBlock) * kBlock;
    if (need * ACE_MAX_STAGES * (ACE_WS_REC / 2) > 0xffffffffull) return ACE_OK;   // (a workspace of 64 GiB and more: such batches take the plain kernel)
    if (need > h->stage_ws_plans) {
        if (h->stage_ws_fixed) return ACE_EFIXED;
        if (h->d_stage_ws) ACE_HIP(hipFree(h->d_stage_ws));
        h->d_stage_ws = nullptr;
        h->stage_ws_plans = 0;
        ACE_HIP(hipMalloc((void **)&h->d_stage_ws, need * ACE_MAX_STAGES * ACE_WS_REC * sizeof(double)));
        h->stage_ws_plans = need;
    }
    a->stage_ws = h->d_stage_ws;
    return ACE_OK;
}

extern "C" {

int ace_reserve(ace_handle_t *h, size_t max_plans, int fixed) {
    if (!h || max_plans > 0x7fffffffull) return ACE_EINVAL;
    if (max_plans) {
        AceKernelArgs a;
        memset(&a, 0, sizeof(a));
        a.g.P = (int32_t)max_plans;
        const int was_fixed = h->stage_ws_fixed;
        h->stage_ws_fixed = 0;
        const int rc = ensure_stage_ws(h, &a);
        h->stage_ws_fixed = was_fixed;
        if (rc) return rc;
    }
    h->stage_ws_fixed = fixed ? 1 : 0;
    return ACE_OK;
}

int ace_score_batch(ace_handle_t *h, const ace_batch_t *batch, double memory_limit, int strict, double *d_iter_ms,
                    double *d_peak_mb, uint8_t *d_feasible, uint8_t *d_status, double *d_stage_out, void *stream) {
    AceKernelArgs a;
    int rc = fill_args(h, batch, memory_limit, strict, d_iter_ms, d_peak_mb, d_feasible, d_status, d_stage_out, &a);
    if (rc) return rc;
    if ((rc = ensure_stage_ws(h, &a))) return rc;
    launch_score(h, a, (hipStream_t)stream);
    ACE_HIP(hipGetLastError());
    return ACE_OK;
}

int ace_score_batch_static(ace_handle_t *h, const ace_batch_t *batch, double memory_limit, int strict, double *d_iter_ms,
                           double *d_peak_mb, uint8_t *d_feasible, uint8_t *d_status, void *stream) {
    if (batch && (batch->d_range || batch->n_plans > (size_t)ACE_STATIC_MAX_PLANS)) return batch->d_range ? ACE_EINVAL : ACE_ETOOBIG;
    AceKernelArgs a;
    int rc = fill_args(h, batch, memory_limit, strict, d_iter_ms, d_peak_mb, d_feasible, d_status, nullptr, &a);
    if (rc) return rc;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev != h->device || dev < 0 || dev >= kMaxDevices) return ACE_EINVAL;
    // (the same test as ensure_stage_ws: tables that take the kernels without deferred stage tails need no scratch)
    const bool deferred = !((h->n_windows > 1 && !h->d_pos_types) || h->geom.N >= 32768 || (h->geom.flags & ACE_F_COLLECTIVE_MEM));
    // looked up by ace_create on this device; the padded plan count of either workgroup size fits: ACE_STATIC_MAX_PLANS is a multiple of kBlock
    a.stage_ws = deferred ? g_static_ptr[dev] : nullptr;
    if (deferred && !a.stage_ws) return ACE_EINVAL;
    launch_score(h, a, (hipStream_t)stream);
    ACE_HIP(hipGetLastError());
    return ACE_OK;
}

int ace_time_score_kernel(ace_handle_t *h, const ace_batch_t *batch, double memory_limit, int strict, double *d_iter_ms,
                          double *d_peak_mb, uint8_t *d_feasible, int reps, void *stream, double *avg_ms) {
    if (reps <= 0 || !avg_ms) return ACE_EINVAL;
    AceKernelArgs a;
    int rc = fill_args(h, batch, memory_limit, strict, d_iter_ms, d_peak_mb, d_feasible, nullptr, nullptr, &a);
    if (rc) return rc;
    if ((rc = ensure_stage_ws(h, &a))) return rc;
    hipStream_t s = (hipStream_t)stream;
    hipEvent_t e0, e1;
    ACE_HIP(hipEventCreate(&e0));
    ACE_HIP(hipEventCreate(&e1));
    ACE_HIP(hipEventRecord(e0, s));
    for (int r = 0; r < reps; ++r) launch_score(h, a, s);
    ACE_HIP(hipEventRecord(e1, s));
    ACE_HIP(hipEventSynchronize(e1));
    float ms = 0.f;
    ACE_HIP(hipEventElapsedTime(&ms, e0, e1));
    ACE_HIP(hipEventDestroy(e0));
    ACE_HIP(hipEventDestroy(e1));
    ACE_HIP(hipGetLastError());
    *avg_ms = (double)ms / reps;
    return ACE_OK;
}

// workspace layout: TopkState | hist[kRadix] | less[cap] | ties[cap] | buf[pow2(2*cap)]
static unsigned int topk_cap(int k) { return (unsigned)k; }

size_t ace_topk_workspace_bytes(size_t n, int k) {
    (void)n;
    if (k <= 0) return 0;
    const unsigned cap = topk_cap(k);
    const unsigned p2 = next_pow2(2 * cap);
    // (the last part: state and candidates of the short form)
    return 256 + sizeof(unsigned int) * kRadix + sizeof(Cand) * ((size_t)cap * 2 + p2) + 256 + sizeof(Cand) * (kCandCap + kTieCap) +
           sizeof(unsigned int) * kMaxFilterGroups;
}

int ace_topk(ace_handle_t *h, const double *d_iter_ms, const uint8_t *d_feasible, size_t n, int k, int64_t *d_idx,
             double *d_val, int32_t *d_count, void *d_workspace, size_t workspace_bytes, void *stream) {
    if (!h || !d_iter_ms || !d_feasible || !d_idx || !d_val || !d_workspace || n == 0 || k <= 0 || k > (1 << 20)) return ACE_EINVAL;
    if (workspace_bytes < ace_topk_workspace_bytes(n, k) || ((uintptr_t)d_workspace & 15u)) return ACE_EINVAL;
    hipStream_t s = (hipStream_t)stream;
    unsigned char *ws = (unsigned char *)d_workspace;
    TopkState *st = (TopkState *)ws;
    unsigned int *hist = (unsigned int *)(ws + 256);
    const unsigned cap = topk_cap(k);
    const unsigned p2 = next_pow2(2 * cap);
    Cand *less = (Cand *)(ws + 256 + sizeof(unsigned int) * kRadix);
    Cand *ties = less + cap;
    Cand *buf = ties + cap;
    unsigned blocks = (unsigned)((n + kTopBlock * 8 - 1) / (kTopBlock * 8));
    if (blocks < 1) blocks = 1;
    if (blocks > 2048) blocks = 2048;
    if (k <= kShortMaxK && n * (size_t)k <= kShortMaxNK && n <= 0xffffffffull) {
        ShortTopk *sst = (ShortTopk *)(buf + p2);
        Cand *cand = (Cand *)((unsigned char *)sst + 256);
        Cand *tiecand = cand + kCandCap;
        unsigned int *group_ties = (unsigned int *)(tiecand + kTieCap);      // (at most kMaxFilterGroups filter workgroups: n <= kShortMaxNK)
        hipLaunchKernelGGL(topk_sample, dim3(1), dim3(1024), 0, s, d_iter_ms, d_feasible, n, k, sst);
        hipLaunchKernelGGL(topk_filter, dim3((unsigned)((n + 1024 * kFilterPer - 1) / (1024 * kFilterPer))), dim3(1024), 0, s, d_iter_ms,
                           d_feasible, n, sst, cand, tiecand, group_ties);
        hipLaunchKernelGGL(topk_short_final, dim3(1), dim3(1024), kShortLds, s, d_iter_ms, d_feasible, n, sst, cand, tiecand, group_ties, k,
                           (long long *)d_idx, d_val, d_count);
        ACE_HIP(hipGetLastError());
        return ACE_OK;
    }
    hipLaunchKernelGGL(topk_init, dim3(1), dim3(256), 0, s, st, hist, k);
    for (int pass = 0; pass < kPasses; ++pass) {
        hipLaunchKernelGGL(topk_hist, dim3(blocks), dim3(kTopBlock), 0, s, d_iter_ms, d_feasible, n, pass, st, hist);
        hipLaunchKernelGGL(topk_pick, dim3(1), dim3(kTopBlock), 0, s, st, hist, pass);
    }
    hipLaunchKernelGGL(topk_gather, dim3(blocks), dim3(kTopBlock), 0, s, d_iter_ms, d_feasible, n, st, less, ties, cap, cap);
    // ties: the gather keeps an arbitrary subset when more than `cap` plans share the k-th time;
    // redo them exactly (lowest indices first): a single-workgroup scan that stops early.
    hipLaunchKernelGGL(topk_ties_exact, dim3(1), dim3(kTieBlock), 0, s, d_iter_ms, d_feasible, n, st, ties, cap);
    hipLaunchKernelGGL(topk_finish, dim3(1), dim3(1024), 0, s, st, less, ties, cap, k, buf, p2, (long long *)d_idx, d_val, d_count);
    ACE_HIP(hipGetLastError());
    return ACE_OK;
}

int ace_apply_moves(const uint8_t *d_template_codes, const uint32_t *d_template_hdr, int n_templates,
                    const uint32_t *d_moves, size_t n_moves, int num_ops, int n_algo, uint8_t *d_codes_out,
                    uint32_t *d_hdr_out, uint64_t *d_keys_out, void *stream) {
    if (!d_template_codes || !d_template_hdr || !d_moves || !d_codes_out || !d_hdr_out || n_templates <= 0 ||
        n_templates > 65536 || n_moves == 0 || n_moves > 0x7fffffffull || num_ops <= 0 || num_ops >= 65536 ||
        (n_algo != 1 && n_algo != 2))
        return ACE_EINVAL;
    if (((uintptr_t)d_template_codes & 15u) || ((uintptr_t)d_template_hdr & 15u) || ((uintptr_t)d_moves & 15u) ||
        ((uintptr_t)d_codes_out & 15u) || ((uintptr_t)d_hdr_out & 15u) || ((uintptr_t)d_keys_out & 7u))
        return ACE_EINVAL;
    const int G = (num_ops + 15) / 16;
    const unsigned long long total = (unsigned long long)n_moves * (unsigned long long)G;
    const unsigned long long blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffull) return ACE_ETOOBIG;
    hipLaunchKernelGGL(apply_moves_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<const ace_u4 *>(d_template_codes), reinterpret_cast<const ace_u4 *>(d_template_hdr),
                       n_templates, reinterpret_cast<const ace_u4 *>(d_moves), (unsigned long long)n_moves, G,
                       n_algo == 2 ? 1 : 0, reinterpret_cast<ace_u4 *>(d_codes_out), reinterpret_cast<ace_u4 *>(d_hdr_out),
                       reinterpret_cast<unsigned long long *>(d_keys_out));
    ACE_HIP(hipGetLastError());
    return ACE_OK;
}

int ace_group_keys(const uint8_t *d_codes, const uint32_t *d_hdr, size_t n_plans, int num_ops, uint64_t *d_keys, void *stream) {
    if (!d_codes || !d_hdr || !d_keys || n_plans == 0 || n_plans > 0x7fffffffull || num_ops <= 0 || num_ops >= (1 << 20)) return ACE_EINVAL;
    if (((uintptr_t)d_codes & 15u) || ((uintptr_t)d_hdr & 15u) || ((uintptr_t)d_keys & 7u)) return ACE_EINVAL;
    const int G = (num_ops + 15) / 16;
    hipLaunchKernelGGL(group_keys_kernel, dim3((unsigned)((n_plans + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<const ace_u4 *>(d_codes), reinterpret_cast<const ace_u4 *>(d_hdr),
                       (unsigned long long)n_plans, G, num_ops, reinterpret_cast<unsigned long long *>(d_keys));
    ACE_HIP(hipGetLastError());
    return ACE_OK;
}

int ace_gather_plans(const uint8_t *d_codes_in, const uint32_t *d_hdr_in, const uint32_t *d_perm, size_t n_plans, int num_ops,
                     uint8_t *d_codes_out, uint32_t *d_hdr_out, void *stream) {
    if (!d_codes_in || !d_hdr_in || !d_perm || !d_codes_out || !d_hdr_out || n_plans == 0 || n_plans > 0x7fffffffull ||
        num_ops <= 0 || num_ops >= (1 << 20) || d_codes_in == d_codes_out || d_hdr_in == d_hdr_out)
        return ACE_EINVAL;
    if (((uintptr_t)d_codes_in & 15u) || ((uintptr_t)d_hdr_in & 15u) || ((uintptr_t)d_codes_out & 15u) ||
        ((uintptr_t)d_hdr_out & 15u) || ((uintptr_t)d_perm & 3u))
        return ACE_EINVAL;
    const int G = (num_ops + 15) / 16;
    const unsigned long long blocks = ((unsigned long long)n_plans * G + 255) / 256;
    if (blocks > 0x7fffffffull) return ACE_ETOOBIG;
    hipLaunchKernelGGL(gather_plans_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<const ace_u4 *>(d_codes_in), reinterpret_cast<const ace_u4 *>(d_hdr_in), d_perm,
                       (unsigned long long)n_plans, G, reinterpret_cast<ace_u4 *>(d_codes_out), reinterpret_cast<ace_u4 *>(d_hdr_out));
    ACE_HIP(hipGetLastError());
    return ACE_OK;
}

int ace_recompute_groups(const ace_rc_tables_t *t, int n_stages, const int32_t *d_plan, const int32_t *d_lo,
                         const int32_t *d_hi, const int32_t *d_nsb, const uint32_t *d_mrow, double *d_sum_size,
                         int32_t *d_first_pos, int32_t *d_bad, void *stream) {
    if (!t || n_stages <= 0 || !d_plan || !d_lo || !d_hi || !d_nsb || !d_mrow || !d_sum_size || !d_first_pos || !d_bad ||
        !t->d_codes || !t->d_type_of_pos || !t->d_activations || !t->d_no_recompute || t->num_ops <= 0 || t->num_types <= 0 ||
        t->n_tp <= 0 || t->n_tp > 4 || (t->n_algo != 1 && t->n_algo != 2) || t->n_mbs <= 0 || t->n_mbs > 15 || t->n_plans == 0)
        return ACE_EINVAL;
    RcTables k{t->d_codes, (unsigned long long)t->n_plans, t->d_type_of_pos, t->d_activations, t->d_no_recompute,
               t->num_ops, t->num_types, t->n_mbs, t->n_tp, t->n_algo, t->n_algo == 2 ? 1 : 0};
    hipLaunchKernelGGL(rc_groups_kernel, dim3((n_stages + 127) / 128), dim3(128), 0, (hipStream_t)stream, k, n_stages,
                       d_plan, d_lo, d_hi, d_nsb, d_mrow, d_sum_size, d_first_pos, d_bad);
    ACE_HIP(hipGetLastError());
    return ACE_OK;
}

int ace_recompute_select(const ace_rc_tables_t *t, uint8_t *d_codes_rw, int n_stages, const int32_t *d_plan,
                         const int32_t *d_lo, const int32_t *d_hi, const int32_t *d_nsb, const uint32_t *d_mrow,
                         const double *d_sum_size, const int32_t *d_first_pos, uint8_t *d_recomputed, const double *d_mem,
                         double memory_limit, uint8_t *d_alive, void *stream) {
    if (!t || !d_codes_rw || n_stages <= 0 || !d_plan || !d_lo || !d_hi || !d_nsb || !d_mrow || !d_sum_size ||
        !d_first_pos || !d_recomputed || !d_mem || !d_alive || !t->d_codes || !t->d_type_of_pos || !t->d_activations ||
        !t->d_no_recompute || t->num_ops <= 0 || t->num_types <= 0 || t->n_tp <= 0 || t->n_tp > 4 ||
        (t->n_algo != 1 && t->n_algo != 2) || t->n_mbs <= 0 || t->n_mbs > 15 || t->n_plans == 0)
        return ACE_EINVAL;
    RcTables k{t->d_codes, (unsigned long long)t->n_plans, t->d_type_of_pos, t->d_activations, t->d_no_recompute,
               t->num_ops, t->num_types, t->n_mbs, t->n_tp, t->n_algo, t->n_algo == 2 ? 1 : 0};
    hipLaunchKernelGGL(rc_select_kernel, dim3((n_stages + 127) / 128), dim3(128), 0, (hipStream_t)stream, k, d_codes_rw,
                       n_stages, d_plan, d_lo, d_hi, d_nsb, d_mrow, d_sum_size, d_first_pos, d_recomputed, d_mem,
                       memory_limit, d_alive);
    ACE_HIP(hipGetLastError());
    return ACE_OK;
}

}  // extern "C"

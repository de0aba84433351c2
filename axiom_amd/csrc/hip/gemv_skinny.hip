// Skinny-M (1 <= M <= 16) fp32 route: C[M,N] = act(A[M,K] * B[K,N] + bias[n]).
//
// The work is one pass over B (K*N*4 bytes): HBM-bound.  A workgroup of 256 threads owns 64
// columns (16 lanes x float4 = 256 contiguous bytes per B row) and a K range; its 16 lane
// groups share the rows of that range.  The M activations of a k row are wave-uniform only per
// lane group, so they come from LDS (staged once per workgroup); the first batch of weight
// loads is issued before that staging so HBM latency overlaps it.  Up to M = 8 the products run
// on the vector ALU out of a ring of U weight registers per lane that is refilled slot by slot
// (k_skinny_stream); from M = 9 on they run on the matrix cores (v_mfma_f32_16x16x4_f32, which
// sums a wave's four k rows itself; k_skinny_mfma); rows off the 16-byte grid take k_skinny_any.
// The 16 lane groups' sums are joined through LDS in a fixed order.
//
// When K is split over several workgroups the splits of a strip are joined in a fixed binary
// tree (leaf = split, a node = left + right, an odd node out passes up unchanged), inside the
// launch, in one of two ways.  Exchange tree: every output element is joined on its own; a
// thread exchanges its sum into the node's slot (one device-scope atomic exchange); whoever
// finds the slot empty is done, whoever finds the sibling's sum adds it, empties the slot and
// carries the node's sum one level up.  fp32 addition is commutative, so the result does not
// depend on who arrives first; the value travels inside the atomic, so nothing has to be
// ordered around it, and the last arriver pays one trip to memory per tree level — but a
// device-scope exchange per element and level: good for few rows and few levels.  Tile join:
// every split stores its partial tile, arrives on a per-strip counter, and the last one loads
// the tiles and adds them in the same tree order — three trips whatever the tree's depth, and
// plain loads and stores: used for M >= 5 with more than four splits, and always with a head
// (below), where one workgroup must end up with the whole finished strip.  Both give the same
// bits.  The sum order is fixed, results are bit-identical run to run, and there is no second
// launch.  (Measured on 4096 x 4096 with 8 splits, over the time with the join switched off:
// exchange tree +1.3 us at M = 1, +3.9 at M = 8; tile join +2.0 ... +2.4.)
#include "common.h"

namespace {
using namespace axhip;

// A weight vector.  Every byte of the weights is read once per launch; with STREAM the loads are marked non-temporal,
// which lets large weights that come from HBM arrive 3-6 % faster and costs weights small enough to be met again in
// the caches as much (4096 x 784: 7.0 -> 7.5 us), so the launcher sets it from 32 MiB of weights on.
typedef const __attribute__((address_space(1))) v4f *global_v4f_ptr;
template <bool STREAM>
__device__ __forceinline__ v4f ldw(const float *p) {
    const global_v4f_ptr g = (global_v4f_ptr)p;           // weights are in global memory: never a flat load
    if (STREAM) return __builtin_nontemporal_load(g);
    return *g;
}

// A byte offset every lane of the wave holds the same value of, pinned to scalar registers: a load from
// base + that offset + a 32-bit lane offset then takes the scalar-base addressing form, with no vector
// arithmetic per load.
__device__ __forceinline__ int64_t wave_uniform(int64_t v) {
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)(uint64_t)v), hi = __builtin_amdgcn_readfirstlane((unsigned)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

constexpr int COLS = 64;        // columns per workgroup (k_skinny_mfma, k_skinny_any and the classic stream form)
constexpr int KGROUPS = 16;     // lane groups per workgroup of 256 threads, each 16 lanes x float4
constexpr int UNROLL = 8;       // weight loads in flight per lane (k_skinny_mfma, k_skinny_any)
constexpr int kJoinChunk = 16;              // splits whose partials the finishing workgroup of a head launch requests at once
constexpr int kMfmaFromM = 9;              // from this M on the products run on the matrix cores (16-byte aligned rows); below, the vector ALU form measured faster (M = 8, 4096 x 32000: 107 us against 117)
constexpr unsigned kEmptySlot = 0xFFFFFFFFu;    // a join slot nobody has written (a NaN pattern no sum is allowed to take)
constexpr unsigned kOtherNan = 0x7FC00000u;     // what a sum with exactly that pattern is exchanged as

// A narrow layer riding on this one: out2[m, j] = act2(sum_n C[m, n] * W[n, j] + bias2[j]), j < nh <= 16
// (a hidden layer followed by a classifier head).  The workgroup that finishes a strip has that strip's 64
// finished outputs per row in hand and multiplies them by the head's 64 x nh block of weights at once;
// the strips' contributions are joined like the splits of a strip: partial vectors out, an arrival counter,
// the last strip adds them in strip order.  That is one more join at the end of this launch instead of a
// launch of its own, whose time would be almost all fixed cost.
struct SkinnyHead {
    const float *W;        // [N, nh] dense; null: no head
    const float *bias;     // [nh] or null
    float *out;            // [MR, nh] dense
    float *part;           // [strips][MR][nh] partial vectors
    int *counter;          // one arrival counter, zero between launches
    int nh, act, strips;
    int keep;              // also write this layer's own output C
};

struct SkinnyArgs {
    const float *A;
    int64_t lda;
    const float *B;
    int64_t ldb;
    float *join;               // splits > 1: join slots [node][MR][N] (exchange tree) or partial tiles [split][MR][N] (tile join)
    int64_t N, K, k_per_split;
    int xp;                    // floats per activation row in LDS
    const float *bias;
    int act, splits;
    float *C;
    int64_t ldc;
    int *counters;             // per-strip arrival counters (tile join)
    int tile_join;             // splits > 1: 0 = element-wise exchange tree, 1 = partial tiles and an arrival counter
};

// Adds n <= 16 values in the join tree's order: v[i] = v[2i] + v[2i+1], an odd one out passes up.
__device__ __forceinline__ float tree16(float (&v)[kJoinChunk], int n) {
#pragma unroll
    for (int width = kJoinChunk / 2; width >= 1; width >>= 1) {
#pragma unroll
        for (int i = 0; i < width; i++) v[i] = (2 * i + 1 < n) ? v[2 * i] + v[2 * i + 1] : v[2 * i];
        n = (n + 1) >> 1;
    }
    return v[0];
}

// The end of every skinny kernel.  `red` holds NPART partial tiles [part][MR][COLS] of this workgroup
// (visible to all threads); behind them LDS has room for the head's [MR][COLS] finished outputs and its
// [COLS][nh] block of weights.  Sums the partial tiles in part order, joins the splits of the strip,
// applies bias and activation, writes C and runs the head.
template <int MR, int NPART, int COLS = 64, int THREADS = 256>
__device__ __forceinline__ void strip_finish(const SkinnyArgs &p, const SkinnyHead &head, float *red,
                                             const float (&hw)[(COLS * 16 + THREADS - 1) / THREADS], int tid, int64_t n0) {
    __shared__ int head_last, last_flag;
    constexpr int OUTS = (MR * COLS + THREADS - 1) / THREADS;
    constexpr int HWN = (COLS * 16 + THREADS - 1) / THREADS;
    float *hs = red + NPART * MR * COLS;                          // the strip's finished outputs, for the head
    float *hws = hs + MR * COLS;                                  // the head's [64][nh] block of weights
    const int64_t N = p.N;

    // The head's share of a finished strip (every thread of the finishing workgroup calls this).
    auto head_tail = [&]() {
        const int nh = head.nh, hm = tid / nh, hj = tid - hm * nh;
#pragma unroll
        for (int q = 0; q < HWN; q++)
            if (tid + q * THREADS < COLS * nh) hws[tid + q * THREADS] = hw[q];
        __syncthreads();                                          // hs and hws are complete
        const bool mine = tid < MR * nh;
        if (mine) {
            float sum = 0.0f;
            const int cols = N - n0 < COLS ? (int)(N - n0) : COLS;
#pragma unroll 16
            for (int c = 0; c < cols; c++) sum = __builtin_fmaf(hs[hm * COLS + c], hws[c * nh + hj], sum);
            __hip_atomic_store(reinterpret_cast<int *>(head.part + ((int64_t)blockIdx.x * MR + hm) * nh + hj), __float_as_int(sum),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // The partial vector is written with device-scope stores; the wait makes this thread's stores
        // complete before the barrier and the barrier orders them before thread 0's increment.  This
        // relies on the target writing device-scope atomic stores through to the level all XCDs share
        // before they count as complete (gfx942 / gfx950), which a formal release would not add to.
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (tid == 0) {
            const int arrived = __hip_atomic_fetch_add(head.counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            head_last = (arrived == head.strips - 1);
        }
        __syncthreads();
        if (!head_last) return;
        // The last strip adds the strips' partial vectors.  T = 2^t threads share an output (as many as the workgroup
        // allows, at most 16): thread q of them adds strips q*L .. q*L + L - 1 in order, all of its requests in
        // flight at once when L <= 16, and the T sums are added across lanes in a butterfly, which every lane
        // evaluates with the same pairs, so the order is fixed.
        const int outs = MR * nh;
        int T = 16;
        while (T > 1 && outs * T > THREADS) T >>= 1;
        const int oi = tid / T, q = tid - oi * T;                 // output, share
        const bool live = oi < outs;
        const int L = (head.strips + T - 1) / T;
        float sum = 0.0f;
        if (live) {
            const float *pp = head.part + oi;                     // oi = hm * nh + hj
            const int64_t step = (int64_t)MR * nh;
            const int s_begin = q * L, s_end = s_begin + L < head.strips ? s_begin + L : head.strips;
            for (int s0 = s_begin; s0 < s_end; s0 += 16) {
                float v[16];
#pragma unroll
                for (int u = 0; u < 16; u++)
                    v[u] = s0 + u < s_end
                               ? __int_as_float(__hip_atomic_load(reinterpret_cast<const int *>(pp + (s0 + u) * step),
                                                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
                               : 0.0f;
#pragma unroll
                for (int u = 0; u < 16; u++)
                    if (s0 + u < s_end) sum += v[u];
            }
        }
        for (int off = 1; off < T; off <<= 1) sum += __shfl_xor(sum, off, 64);
        if (live && q == 0) {
            const int hj2 = oi % nh;
            if (head.bias) sum += head.bias[hj2];
            head.out[oi] = apply_act(sum, head.act);
        }
        if (tid == 0) __hip_atomic_store(head.counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };

    // this workgroup's own sums, in part order
    float s[OUTS];
    bool ok[OUTS];
    int om[OUTS];
    int64_t on[OUTS];
#pragma unroll
    for (int o = 0; o < OUTS; o++) {
        const int i = tid + o * THREADS, m = i / COLS, c = i % COLS;
        om[o] = m;
        on[o] = n0 + c;
        ok[o] = i < MR * COLS && n0 + c < N;
        float t = 0.0f;
        if (i < MR * COLS)
#pragma unroll
            for (int w = 0; w < NPART; w++) t += red[(w * MR + m) * COLS + c];
        s[o] = t;
    }
    auto write_out = [&](int o, float r) {
        if (p.bias) r += p.bias[on[o]];
        r = apply_act(r, p.act);
        if (!head.W || head.keep) p.C[om[o] * p.ldc + on[o]] = r;
        if (head.W) hs[tid + o * THREADS] = r;
    };

    if (p.splits == 1) {
#pragma unroll
        for (int o = 0; o < OUTS; o++)
            if (ok[o]) write_out(o, s[o]);
        if (head.W) head_tail();
        return;
    }

    const int64_t tile = (int64_t)MR * N;          // floats per join slot / partial tile
    if (!p.tile_join) {
        // element-wise join up the tree: one exchange per level this split is paired on
        bool alive[OUTS];
#pragma unroll
        for (int o = 0; o < OUTS; o++) alive[o] = ok[o];
        int idx = blockIdx.y, n = p.splits;
        int64_t node_base = 0;
        while (n > 1) {
            if ((idx ^ 1) < n) {
                unsigned *slot[OUTS], old[OUTS];
#pragma unroll
                for (int o = 0; o < OUTS; o++) {
                    slot[o] = reinterpret_cast<unsigned *>(p.join + (node_base + (idx >> 1)) * tile + om[o] * N + on[o]);
                    if (alive[o]) {
                        unsigned mine = __float_as_uint(s[o]);
                        if (mine == kEmptySlot) mine = kOtherNan;
                        old[o] = __hip_atomic_exchange(slot[o], mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
#pragma unroll
                for (int o = 0; o < OUTS; o++)
                    if (alive[o]) {
                        if (old[o] == kEmptySlot) {
                            alive[o] = false;                     // first at this node: the sibling carries on
                        } else {
                            s[o] += __uint_as_float(old[o]);
                            __hip_atomic_store(slot[o], kEmptySlot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
                        }
                    }
            }
            node_base += n >> 1;
            n = (n + 1) >> 1;
            idx >>= 1;
        }
#pragma unroll
        for (int o = 0; o < OUTS; o++)
            if (alive[o]) write_out(o, s[o]);
        return;
    }

    // Tile join: publish this split's partial tile, then find out whether every split of the strip is in.
    // Partials, counter and the reads below are all device-scope accesses, so no cache-wide write-back or
    // invalidate is needed (a __threadfence here costs ~150 us per launch: it flushes the XCD's whole L2);
    // the wait makes this thread's stores complete before the barrier, the barrier orders them before
    // thread 0's increment (see head_tail for what that relies on).
#pragma unroll
    for (int o = 0; o < OUTS; o++)
        if (ok[o])
            __hip_atomic_store(reinterpret_cast<int *>(p.join + blockIdx.y * tile + om[o] * N + on[o]), __float_as_int(s[o]),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0) {
        const int arrived = __hip_atomic_fetch_add(p.counters + blockIdx.x, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_flag = (arrived == p.splits - 1);
    }
    __syncthreads();
    if (!last_flag) return;
    // All partials of a chunk of 16 splits are requested before the first is used (one trip to memory per
    // chunk); a chunk is a whole subtree, and the chunks' sums are joined like a binary counter, which is
    // the same tree again.
    float pend[OUTS][12];
    unsigned pending = 0;                          // bit l: pend[.][l] holds a node 4 + l levels up
    float r[OUTS];
    for (int p0 = 0; p0 < p.splits; p0 += kJoinChunk) {
        float v[OUTS][kJoinChunk];
        const int nc = p.splits - p0 < kJoinChunk ? p.splits - p0 : kJoinChunk;
#pragma unroll
        for (int o = 0; o < OUTS; o++)
#pragma unroll
            for (int u = 0; u < kJoinChunk; u++)
                v[o][u] = (ok[o] && u < nc)
                              ? __int_as_float(__hip_atomic_load(
                                    reinterpret_cast<const int *>(p.join + (int64_t)(p0 + u) * tile + om[o] * N + on[o]),
                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
                              : 0.0f;
#pragma unroll
        for (int o = 0; o < OUTS; o++) r[o] = tree16(v[o], nc);
        if (p.splits <= kJoinChunk) break;
        bool placed = false;
#pragma unroll
        for (int l = 0; l < 12; l++) {
            if (!placed) {
                if (pending & (1u << l)) {
#pragma unroll
                    for (int o = 0; o < OUTS; o++) r[o] = pend[o][l] + r[o];
                    pending &= ~(1u << l);
                } else {
#pragma unroll
                    for (int o = 0; o < OUTS; o++) pend[o][l] = r[o];
                    pending |= 1u << l;
                    placed = true;
                }
            }
        }
    }
    if (p.splits > kJoinChunk) {
        bool have = false;
#pragma unroll
        for (int l = 0; l < 12; l++)
            if (pending & (1u << l)) {
#pragma unroll
                for (int o = 0; o < OUTS; o++) r[o] = have ? pend[o][l] + r[o] : pend[o][l];
                have = true;
            }
    }
#pragma unroll
    for (int o = 0; o < OUTS; o++)
        if (ok[o]) write_out(o, r[o]);
    if (tid == 0)                                   // ready for the next launch
        __hip_atomic_store(p.counters + blockIdx.x, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (head.W) head_tail();
}

// The head's block of weights for this strip (64 rows x nh <= 1024 floats), requested early so that it
// has arrived long before a finishing workgroup needs it.
template <int COLS = 64, int THREADS = 256>
__device__ __forceinline__ void head_prefetch(const SkinnyHead &head, int64_t N, int64_t n0, int tid,
                                              float (&hw)[(COLS * 16 + THREADS - 1) / THREADS]) {
    constexpr int HWN = (COLS * 16 + THREADS - 1) / THREADS;
#pragma unroll
    for (int q = 0; q < HWN; q++) hw[q] = 0.0f;
    if (head.W) {
        const int cols = N - n0 < COLS ? (int)(N - n0) : COLS;
#pragma unroll
        for (int q = 0; q < HWN; q++) {
            const int e = tid + q * THREADS;
            if (e < cols * head.nh) hw[q] = head.W[n0 * head.nh + e];
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// M <= 8, rows on the 16-byte grid.  A workgroup of THREADS threads owns a strip of COLS columns (COLS / 4
// lanes x float4 per row) and a K range.  Rows are taken in batches of NG * U (NG lane groups): lane group
// g owns the U consecutive rows g * U ... of a batch, so its activations are 16-byte LDS reads (four rows
// at a time) and each of its U weight registers is refilled with the same row of the next batch as soon
// as it has been used: U loads per lane stay in flight through the whole K range.  Addresses are a
// wave-uniform row offset plus one 32-bit lane offset computed once.  A lane past the matrix's last
// column re-reads the strip's first columns: what it computes is never stored, and no load needs a
// column predicate.  Forms: 64 columns x 256 threads (several workgroups per CU, K cut into ranges of at
// most 512 rows), and 32 or 64 columns x 512 threads (one workgroup per CU holding a long K range, so
// that a strip has one or two ranges and the join at the end is a single exchange or none).
template <int MR, bool STREAM, int U, bool PRED, int RB>
__device__ __forceinline__ void stream_batch(float (&acc)[MR][4], v4f (&w)[U], v4f (&xc)[MR], const float *xb, int XP,
                                             const char *bytes, int64_t next_off, int64_t row_bytes, unsigned lane_off, int next_rows,
                                             const char *safe) {
    // xc: this lane group's activations for rows 0..3 of the batch (already read); xb: their place in LDS
#pragma unroll
    for (int u0 = 0; u0 < U; u0 += 4) {
        v4f xn[MR];
        // the activations of the four rows after these (the next batch's first four when u0 is the last)
        const float *xnext = u0 + 4 < U ? xb + u0 + 4 : xb + RB;
#pragma unroll
        for (int m = 0; m < MR; m++) xn[m] = *reinterpret_cast<const v4f *>(xnext + m * XP);
#pragma unroll
        for (int uu = 0; uu < 4; uu++) {
            const int u = u0 + uu;
#pragma unroll
            for (int m = 0; m < MR; m++)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[m][e] = __builtin_fmaf(xc[m][uu], w[u][e], acc[m][e]);
            const float *src = reinterpret_cast<const float *>(bytes + wave_uniform(next_off + u * row_bytes) + lane_off);
            if (!PRED) {
                w[u] = ldw<STREAM>(src);
            } else {
                // a row past the split's end: the load goes to a row that exists and its result is dropped (no branch,
                // so the ring of registers and the wait counts are those of the plain form)
                const bool in = u < next_rows;
                const v4f t = ldw<STREAM>(in ? src : reinterpret_cast<const float *>(safe));
                w[u] = in ? t : v4f{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
#pragma unroll
        for (int m = 0; m < MR; m++) xc[m] = xn[m];
    }
}

template <int MR, bool STREAM, int U, bool PRE, int COLS = 64, int THREADS = 256>
__global__ void __launch_bounds__(THREADS)
k_skinny_stream(const SkinnyArgs p, const SkinnyHead head) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    // sm: [MR][XC] activations of the current chunk of the K range (zero past the range's end); after the
    // range, in the same place, [NPART][MR][COLS] partial sums, then (with a head) [MR][COLS] finished
    // outputs of the strip and the head's [COLS][nh] weights
    static_assert(U % 4 == 0 && MR <= 8, "rows in fours; larger M runs on the matrix cores");
    constexpr int LG = COLS / 4;            // lanes of a lane group
    constexpr int NG = THREADS / LG;        // lane groups
    constexpr int RB = NG * U;              // rows of a batch
    constexpr int XC = 2 * THREADS;         // rows of a chunk: two activations per thread and row of A
    constexpr int BPC = XC / RB;            // batches of a chunk
    constexpr int WAVES = THREADS / 64;
    static_assert(LG == 8 || LG == 16, "strips of 32 or 64 columns");
    static_assert(XC % RB == 0, "whole batches per chunk");
    const int tid = threadIdx.x;
    const int cg = tid % LG;            // column group: columns 4*cg .. 4*cg+3 of the strip
    const int g = tid / LG;             // lane group
    const int64_t n0 = (int64_t)blockIdx.x * COLS;
    const int64_t k_begin = (int64_t)blockIdx.y * p.k_per_split;
    int64_t k_end = k_begin + p.k_per_split;
    if (k_end > p.K) k_end = p.K;
    const int klen = (int)(k_end - k_begin);
    const int64_t col = n0 + 4 * cg;

    // The activations go to LDS a chunk of XC rows of K at a time.  The loads of the first chunk (L2 hits,
    // every workgroup reads the same few rows) are issued first and the first batch of weights right behind
    // them: loads return in issue order, so the staging then waits only for the activations while the
    // weights are on their way.  Later chunks are fetched and written to LDS between two barriers when
    // their turn comes; the ring of weight loads runs on across chunks, and the other workgroups of the
    // CU stream on meanwhile.
    float xr[MR][2];
    auto request_chunk = [&](int first_row) {
#pragma unroll
        for (int m = 0; m < MR; m++)
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const int kk = first_row + tid + c * THREADS;
                xr[m][c] = kk < klen ? p.A[m * p.lda + k_begin + kk] : 0.0f;
            }
    };
    float *xs = sm;
    auto place_chunk = [&]() {
#pragma unroll
        for (int m = 0; m < MR; m++)
#pragma unroll
            for (int c = 0; c < 2; c++) xs[m * XC + tid + c * THREADS] = xr[m][c];
    };
    request_chunk(0);
    const int64_t row_bytes = p.ldb * (int64_t)sizeof(float);
    const unsigned lane_off = (unsigned)((int64_t)g * U * row_bytes + (col < p.N ? col : n0) * (int64_t)sizeof(float));
    const char *bytes = reinterpret_cast<const char *>(p.B);
    const int64_t base = k_begin * row_bytes;                                          // wave-uniform
    const int nbf = klen / RB, nbt = (klen + RB - 1) / RB;
    const int my_first = g * U;                          // this lane group's first row inside a batch
    const char *safe = bytes + base + (col < p.N ? col : n0) * (int64_t)sizeof(float);   // the range's first row, this lane's columns
    v4f w[U];
    if (nbf > 0) {
#pragma unroll
        for (int u = 0; u < U; u++) w[u] = ldw<STREAM>(reinterpret_cast<const float *>(bytes + wave_uniform(base + u * row_bytes) + lane_off));
    } else if (klen > 0) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const bool in = my_first + u < klen;
            const v4f t = ldw<STREAM>(reinterpret_cast<const float *>(in ? bytes + wave_uniform(base + u * row_bytes) + lane_off : safe));
            w[u] = in ? t : v4f{0.0f, 0.0f, 0.0f, 0.0f};
        }
    } else {                                             // K = 0: nothing to read, the sums stay zero
#pragma unroll
        for (int u = 0; u < U; u++) w[u] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }
    float hw[(COLS * 16 + THREADS - 1) / THREADS];
    head_prefetch<COLS, THREADS>(head, p.N, n0, tid, hw);
    place_chunk();
    __syncthreads();

    float acc[MR][4];
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc[m][e] = 0.0f;

    const float *xb = xs + my_first;
    v4f xc[MR];
#pragma unroll
    for (int m = 0; m < MR; m++) xc[m] = *reinterpret_cast<const v4f *>(xb + m * XC);
    int b = 0;
#pragma unroll 1
    for (int c0 = 0; c0 < nbt; c0 += BPC) {
        if (c0 > 0) {
            // the next chunk of activations takes the place of the one every wave has finished with (the rows the
            // last batch read ahead for its successor are read again from the new chunk)
            __syncthreads();
            request_chunk(c0 * RB);
            place_chunk();
            __syncthreads();
            xb = xs + my_first;
#pragma unroll
            for (int m = 0; m < MR; m++) xc[m] = *reinterpret_cast<const v4f *>(xb + m * XC);
        }
        const int b_end = c0 + BPC < nbt ? c0 + BPC : nbt;
        // batches whose successor is a whole batch: the refills need no predicate
#pragma unroll 1
        for (; b + 1 < nbf && b < b_end; b++) {
            stream_batch<MR, STREAM, U, false, RB>(acc, w, xc, xb, XC, bytes, base + (int64_t)(b + 1) * RB * row_bytes, row_bytes, lane_off, U, safe);
            xb += RB;
        }
        // the last whole batch (its successor, if any, is partial) and the partial batch
#pragma unroll 1
        for (; b < b_end; b++) {
            stream_batch<MR, STREAM, U, true, RB>(acc, w, xc, xb, XC, bytes, base + (int64_t)(b + 1) * RB * row_bytes, row_bytes, lane_off,
                                                  klen - (b + 1) * RB - my_first, safe);
            xb += RB;
        }
    }

    // Lane groups are joined through LDS: every lane group writes its own partial tile, or (PRE) the lane
    // groups of a wave (lanes that differ in the bits above the column group hold the same columns) are
    // first added across lanes and one tile per wave goes through LDS.
    // The partial tiles take the place of the activations, which nobody reads any more after the barrier.
    constexpr int NPART = PRE ? WAVES : NG;
    float *red = sm;
    __syncthreads();
#pragma unroll
    for (int m = 0; m < MR; m++) {
        if (PRE) {
            v4f r;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const unsigned u = __builtin_bit_cast(unsigned, acc[m][e]);
                const auto p32 = __builtin_amdgcn_permlane32_swap(u, u, false, false);
                const float h = __builtin_bit_cast(float, (unsigned)p32[0]) + __builtin_bit_cast(float, (unsigned)p32[1]);
                const unsigned u2 = __builtin_bit_cast(unsigned, h);
                const auto p16 = __builtin_amdgcn_permlane16_swap(u2, u2, false, false);
                float q = __builtin_bit_cast(float, (unsigned)p16[0]) + __builtin_bit_cast(float, (unsigned)p16[1]);
                if (LG == 8) q += __shfl_xor(q, 8, 64);
                r[e] = q;
            }
            if ((tid & 63) < LG) *reinterpret_cast<v4f *>(red + ((tid >> 6) * MR + m) * COLS + 4 * cg) = r;
        } else {
            *reinterpret_cast<v4f *>(red + (g * MR + m) * COLS + 4 * cg) = v4f{acc[m][0], acc[m][1], acc[m][2], acc[m][3]};
        }
    }
    __syncthreads();
    strip_finish<MR, NPART, COLS, THREADS>(p, head, red, hw, tid, n0);
}

// ---------------------------------------------------------------------------------------------------
// M = 9..16 on v_mfma_f32_16x16x4_f32, rows on the 16-byte grid.  The 16 lane groups take rows k, k+16, ...
// of the split, so the four lane groups of a wave hold four consecutive k rows, lane cg of a group the
// columns 4*cg .. 4*cg+3: that is the instruction's B operand layout (k = lane / 16, n = lane % 16) for
// the columns 4*i + j with element j of the loaded float4, and the A operand is the activation of row
// m = lane % 16 at the lane group's k: one LDS read and four MFMAs per 16 bytes of weights, against M reads
// and 4 M multiply-adds.  dm[j][v] = C[4 * (lane / 16) + v][4 * cg + j], summed over the wave's k rows.
template <int MR, bool STREAM>
__global__ void __launch_bounds__(256)
k_skinny_mfma(const SkinnyArgs p, const SkinnyHead head) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    const int tid = threadIdx.x, cg = tid & 15, kg = tid >> 4;
    const int64_t n0 = (int64_t)blockIdx.x * COLS;
    const int64_t k_begin = (int64_t)blockIdx.y * p.k_per_split;
    int64_t k_end = k_begin + p.k_per_split;
    if (k_end > p.K) k_end = p.K;
    const int64_t klen = k_end - k_begin, ldb = p.ldb;
    const int XP = p.xp;
    const int64_t col = n0 + 4 * cg;
    const int klen32 = (int)klen;
    float xr[MR][2];
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int kk = tid + c * 256;
            xr[m][c] = kk < klen32 ? p.A[m * p.lda + k_begin + kk] : 0.0f;
        }
    // A lane past the last column reads the strip's first columns instead and a lane whose row m does
    // not exist reads row 0: what they compute lands in columns / rows that are never stored, and the
    // loads of a full batch need no predicate.  Every lane of a wave must reach the MFMAs together, so
    // the first batch is taken when all lane groups have it (the same for the whole workgroup).
    const float *bq = p.B + (col < p.N ? col : n0);
    const bool pre_all = UNROLL * KGROUPS <= klen;
    int64_t k = kg;
    v4f w0[UNROLL];
    if (pre_all) {
#pragma unroll
        for (int u = 0; u < UNROLL; u++) w0[u] = ldw<STREAM>(bq + (k_begin + k + u * KGROUPS) * ldb);
    }
    float hw[4];
    head_prefetch(head, p.N, n0, tid, hw);
    float *xs = sm;
#pragma unroll
    for (int m = 0; m < MR; m++) {
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int kk = tid + c * 256;
            if (kk < klen32) xs[m * XP + kk] = xr[m][c];
        }
        for (int kk = tid + 512; kk < klen32; kk += 256) xs[m * XP + kk] = p.A[m * p.lda + k_begin + kk];
    }
    __syncthreads();

    v4f dm[4];
#pragma unroll
    for (int j = 0; j < 4; j++) dm[j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    const float *xrow = xs + (cg < MR ? cg : 0) * XP;
    if (pre_all) {
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const float xa = xrow[k + u * KGROUPS];
#pragma unroll
            for (int j = 0; j < 4; j++) dm[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(xa, w0[u][j], dm[j], 0, 0, 0);
        }
        k += UNROLL * KGROUPS;
    }
    // every lane makes the same number of rounds: k - kg is the same for the whole workgroup
    int64_t kb = k - kg;
    for (; kb + UNROLL * KGROUPS <= klen; kb += UNROLL * KGROUPS) {
        v4f w[UNROLL];
        float xa[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            w[u] = ldw<STREAM>(bq + (k_begin + kb + u * KGROUPS + kg) * ldb);
            xa[u] = xrow[kb + u * KGROUPS + kg];
        }
#pragma unroll
        for (int u = 0; u < UNROLL; u++)
#pragma unroll
            for (int j = 0; j < 4; j++) dm[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[u], w[u][j], dm[j], 0, 0, 0);
    }
    // the last, partial batch: a lane whose row lies past the split contributes zeros
    for (; kb < klen; kb += KGROUPS) {
        const int64_t row = kb + kg;
        const bool in = row < klen;
        const v4f w = in ? ldw<STREAM>(bq + (k_begin + row) * ldb) : v4f{0.0f, 0.0f, 0.0f, 0.0f};
        const float xa = in ? xrow[row] : 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) dm[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(xa, w[j], dm[j], 0, 0, 0);
    }
    // the wave's sums are complete in dm: one partial tile per wave, rows 4 * (lane / 16) + v
    float *red = sm + MR * XP;
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int m = 4 * ((tid & 63) >> 4) + v;
        if (m < MR)
            *reinterpret_cast<v4f *>(red + ((tid >> 6) * MR + m) * COLS + 4 * cg) = v4f{dm[0][v], dm[1][v], dm[2][v], dm[3][v]};
    }
    __syncthreads();
    strip_finish<MR, 4>(p, head, red, hw, tid, n0);
}

// ---------------------------------------------------------------------------------------------------
// Rows off the 16-byte grid (N or ldb not a multiple of 4, or an unaligned B), any M up to 16: whole column
// groups still take one 16-byte load each, at the alignment the row has; the last, partial group goes by
// element.  All loads of a batch of rows are issued before the first use.
template <int MR>
__global__ void __launch_bounds__(256)
k_skinny_any(const SkinnyArgs p, const SkinnyHead head) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    const int tid = threadIdx.x, cg = tid & 15, kg = tid >> 4;
    const int64_t n0 = (int64_t)blockIdx.x * COLS;
    const int64_t k_begin = (int64_t)blockIdx.y * p.k_per_split;
    int64_t k_end = k_begin + p.k_per_split;
    if (k_end > p.K) k_end = p.K;
    const int64_t klen = k_end - k_begin, ldb = p.ldb, N = p.N;
    const int XP = p.xp;
    const int64_t col = n0 + 4 * cg;
    const float *bp = p.B + col;
    const int klen32 = (int)klen;
    float hw[4];
    head_prefetch(head, N, n0, tid, hw);
    float *xs = sm;
#pragma unroll
    for (int m = 0; m < MR; m++)
        for (int kk = tid; kk < klen32; kk += 256) xs[m * XP + kk] = p.A[m * p.lda + k_begin + kk];
    __syncthreads();

    float acc[MR][4];
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc[m][e] = 0.0f;
    int64_t k = kg;
    for (; k + (UNROLL - 1) * KGROUPS < klen; k += UNROLL * KGROUPS) {
        float w[UNROLL][4];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const float *rp = bp + (k_begin + k + u * KGROUPS) * ldb;
            if (col + 4 <= N) __builtin_memcpy(w[u], rp, 16);      // one load, whatever the row's alignment
            else
#pragma unroll
                for (int e = 0; e < 4; e++) w[u][e] = (col + e < N) ? rp[e] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < UNROLL; u++)
#pragma unroll
            for (int m = 0; m < MR; m++) {
                const float xv = xs[m * XP + k + u * KGROUPS];
#pragma unroll
                for (int e = 0; e < 4; e++) acc[m][e] = __builtin_fmaf(xv, w[u][e], acc[m][e]);
            }
    }
    for (; k < klen; k += KGROUPS) {
        float w[4];
        const float *rp = bp + (k_begin + k) * ldb;
        if (col + 4 <= N) __builtin_memcpy(w, rp, 16);
        else
#pragma unroll
            for (int e = 0; e < 4; e++) w[e] = (col + e < N) ? rp[e] : 0.0f;
#pragma unroll
        for (int m = 0; m < MR; m++) {
            const float xv = xs[m * XP + k];
#pragma unroll
            for (int e = 0; e < 4; e++) acc[m][e] = __builtin_fmaf(xv, w[e], acc[m][e]);
        }
    }

    // From M = 9 on the four lane groups of a wave are first added with the row-swap instructions, so that
    // one partial per wave goes through LDS and the buffer stays small enough for three workgroups per CU.
    constexpr bool PRE = MR > 8;
    constexpr int NPART = PRE ? 4 : KGROUPS;
    float *red = sm + MR * XP;
#pragma unroll
    for (int m = 0; m < MR; m++) {
        if (PRE) {
            v4f r;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const unsigned u = __builtin_bit_cast(unsigned, acc[m][e]);
                const auto p32 = __builtin_amdgcn_permlane32_swap(u, u, false, false);
                const float h = __builtin_bit_cast(float, (unsigned)p32[0]) + __builtin_bit_cast(float, (unsigned)p32[1]);
                const unsigned u2 = __builtin_bit_cast(unsigned, h);
                const auto p16 = __builtin_amdgcn_permlane16_swap(u2, u2, false, false);
                r[e] = __builtin_bit_cast(float, (unsigned)p16[0]) + __builtin_bit_cast(float, (unsigned)p16[1]);
            }
            if ((tid & 63) < 16) *reinterpret_cast<v4f *>(red + ((tid >> 6) * MR + m) * COLS + 4 * cg) = r;
        } else {
            *reinterpret_cast<v4f *>(red + (kg * MR + m) * COLS + 4 * cg) = v4f{acc[m][0], acc[m][1], acc[m][2], acc[m][3]};
        }
    }
    __syncthreads();
    strip_finish<MR, NPART>(p, head, red, hw, tid, n0);
}

// The forms of the M <= 8 kernel (AX_HIP_SKINNY_FORM = position + 1), then the two other kernels.  Measured and
// not kept: strips of 32 columns (128-byte row pieces stream 8 % slower), 16 loads in flight per lane (no faster,
// and beyond 256 registers from M = 3), workgroups of 768 and 1024 threads (level with 512).
struct StreamForm {
    int cols, threads, unroll;
    bool pre;
};
constexpr StreamForm kStreamForms[] = {{64, 256, 8, false}, {64, 256, 8, true}, {64, 512, 8, true}};
constexpr int kStreamFormCount = sizeof(kStreamForms) / sizeof(kStreamForms[0]);
constexpr int kFormMfma = kStreamFormCount, kFormAny = kStreamFormCount + 1;

// What one call launches: grid, split length, kernel form, LDS bytes and the size of the join area.
struct SkinnyPlan {
    int64_t col_blocks, splits, kps, red_floats;
    int xp, form, cols, threads;
    bool nontemporal, tile_join;
    size_t smem, join_bytes;        // join_bytes: (splits - 1) slots of the exchange tree, or `splits` partial tiles
};

int plan_skinny(int64_t M, int64_t N, int64_t K, const float *B, int64_t ldb, int64_t head_width, SkinnyPlan &p) {
    const bool with_head = head_width > 0;
    const bool vec = (N % 4 == 0) && (ldb % 4 == 0) && ((uintptr_t)B % 16 == 0);
    const Tuning &t = tuning();
    // One or two rows: adding the lane groups of a wave across lanes first is ahead (M = 1, 784 x 4096: 6.7 us against
    // 9.8).  Five rows and more against a short K: workgroups of 512 threads, which leave half as many ranges to join
    // (M = 8, 784 x 4096: 8.8 us against 10.3; with K = 4096 they are behind, 17.0 against 16.6).
    const int form = t.skinny_form > 0 ? t.skinny_form - 1 : M <= 2 ? 1 : (M >= 5 && K <= 1024) ? 2 : 0;
    const StreamForm &f = kStreamForms[form];
    // stream form: lane offsets are 32-bit (a batch of rows plus a row must stay below 4 GiB)
    const int64_t stream_rb = (int64_t)(f.threads / (f.cols / 4)) * f.unroll;
    const bool stream_ok = vec && M < kMfmaFromM && stream_rb * ldb * 4 + N * 4 < (int64_t(1) << 32);
    p.form = stream_ok ? form : (vec && M >= kMfmaFromM) ? kFormMfma : kFormAny;
    p.cols = stream_ok ? f.cols : COLS;
    p.threads = stream_ok ? f.threads : 256;
    const bool fat = p.threads > 256;
    p.col_blocks = (N + p.cols - 1) / p.cols;
    const int rb = stream_ok ? (int)stream_rb : KGROUPS;      // rows a workgroup takes at a time
    // Workgroups a launch aims for.  Fewer, longer workgroups leave fewer splits to join.
    const int64_t want_blocks = t.skinny_blocks > 0 ? t.skinny_blocks : fat ? 256 : 512;
    int64_t splits = (want_blocks + p.col_blocks - 1) / p.col_blocks;
    // ranges of at least 192 rows (784 x 4096 at M = 1: 7.5 us with 8 ranges of 98 rows, 6.7 with 4 of 196)
    const int64_t max_splits = K >= 192 ? K / 192 : 1;
    if (splits > max_splits) splits = max_splits;
    // A strip is joined over a tree of its splits: more splits mean more dependent trips to memory at the
    // very end of the launch.  A narrow matrix gets longer workgroups instead of more of them.
    const bool narrow = splits > kJoinChunk;
    if (narrow) splits = kJoinChunk;
    if (splits < 1) splits = 1;
    int64_t kps = (K + splits - 1) / splits;
    kps = (kps + KGROUPS - 1) / KGROUPS * KGROUPS;
    const bool pre = stream_ok ? f.pre : (p.form == kFormMfma || M > 8);
    p.red_floats = (int64_t)(pre ? p.threads / 64 : KGROUPS) * M * p.cols;   // partials per workgroup, as in the kernels
    // k_skinny_mfma / k_skinny_any keep the activations of a whole K range in LDS next to the reduction buffer, within
    // 52 KiB, so that three workgroups share a CU whatever M is (4096 x 11008 at M = 16: 95 us with one 96 KiB workgroup
    // per CU, 60 us this way).  The stream forms stage a chunk of 2 * threads rows at a time and put the reduction buffer
    // in its place afterwards: their K ranges can be as long as the join wants them.
    const int64_t tail_floats = p.red_floats + (with_head ? (M + head_width) * p.cols : 0);
    if (!stream_ok) {
        const int64_t max_kps = ((int64_t)(52 * 1024 / 4) - tail_floats) / M / rb * rb;
        if (kps > max_kps) kps = max_kps;
    }
    // The stream forms take ranges of any length (8192 x 8192 at M = 8: 56.7 us with 16 ranges of 512 rows, 47.4 with 4
    // of 2048 — every range's end costs its workgroup a join while others wait for its place on the CU); the others
    // are bounded by LDS above and keep at most this many rows.
    const int64_t cap = t.skinny_kps > 0 ? t.skinny_kps : stream_ok ? 65536 : narrow ? 2048 : 512;
    if (kps > cap) kps = cap;
    if (kps < KGROUPS) kps = KGROUPS;
    splits = K > 0 ? (K + kps - 1) / kps : 1;
    if (splits > 65535) return fail(AXHIP_ERR_SHAPE, "sgemm_skinny: K=%lld too large", (long long)K);
    if (splits > 1) {                                                                       // ranges of even length
        kps = ((K + splits - 1) / splits + KGROUPS - 1) / KGROUPS * KGROUPS;
        splits = (K + kps - 1) / kps;
    }
    p.splits = splits;
    p.kps = kps;
    p.xp = (int)kps;
    p.nontemporal = vec && K * N * 4 >= (int64_t(32) << 20);
    // stream forms: a chunk, plus the rows a batch reads ahead of itself
    const int64_t x_floats = stream_ok ? M * 2 * p.threads + rb : M * kps;
    p.smem = (size_t)(stream_ok ? (x_floats > tail_floats ? x_floats : tail_floats) : x_floats + tail_floats) * sizeof(float);
    p.tile_join = splits > 1 && (with_head || (M >= 5 && splits > 4));
    p.join_bytes = splits > 1 ? (size_t)(p.tile_join ? splits : splits - 1) * M * N * sizeof(float) : 0;
    return AXHIP_OK;
}

int check_skinny_args(const char *who, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                      const float *B, int64_t ldb, const float *C, int64_t ldc, int act) {
    if (!A || !B || !C) return fail(AXHIP_ERR_NULL_ARG, "%s: NULL matrix", who);
    if (M < 1 || M > 16) return fail(AXHIP_ERR_SHAPE, "%s: M=%lld outside 1..16", who, (long long)M);
    if (N < 0 || K < 0 || lda < K || ldb < N || ldc < N)
        return fail(AXHIP_ERR_SHAPE, "%s: bad dimension or leading dimension", who);
    if (act < AXHIP_ACT_NONE || act > AXHIP_ACT_GELU)
        return fail(AXHIP_ERR_SHAPE, "%s: unknown activation %d", who, act);
    return AXHIP_OK;
}

template <int MR>
void launch_m(const SkinnyPlan &pl, dim3 grid, size_t smem, const SkinnyArgs &a, const SkinnyHead &head) {
    if constexpr (MR < kMfmaFromM) {
        const bool nt = pl.nontemporal;
        switch (pl.form) {
#define AX_STREAM(index, u, pre, cols, threads)                                                                                       \
    case index:                                                                                                                       \
        if (nt) hipLaunchKernelGGL((k_skinny_stream<MR, true, u, pre, cols, threads>), grid, dim3(threads), smem, kStream, a, head);  \
        else hipLaunchKernelGGL((k_skinny_stream<MR, false, u, pre, cols, threads>), grid, dim3(threads), smem, kStream, a, head);    \
        return;
            AX_STREAM(0, 8, false, 64, 256)
            AX_STREAM(1, 8, true, 64, 256)
            AX_STREAM(2, 8, true, 64, 512)
            default: break;
        }
#undef AX_STREAM
    } else if (pl.form == kFormMfma) {
        if (pl.nontemporal) hipLaunchKernelGGL((k_skinny_mfma<MR, true>), grid, dim3(256), smem, kStream, a, head);
        else hipLaunchKernelGGL((k_skinny_mfma<MR, false>), grid, dim3(256), smem, kStream, a, head);
        return;
    }
    hipLaunchKernelGGL((k_skinny_any<MR>), grid, dim3(256), smem, kStream, a, head);
}

// `join` holds plan.join_bytes: for the exchange tree, join slots that are all kEmptySlot (the kernel leaves them
// so); for the tile join, room for the partial tiles, and `counters` plan.col_blocks ints that are zero (the kernel
// leaves them so).  Both unused when the plan has one split.
int run_skinny(const SkinnyPlan &p, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
               const float *B, int64_t ldb, float *C, int64_t ldc, const float *bias, int act,
               float *join, int *counters, const SkinnyHead &head = SkinnyHead{}) {
    SkinnyArgs a;
    a.A = A;
    a.lda = lda;
    a.B = B;
    a.ldb = ldb;
    a.join = join;
    a.N = N;
    a.K = K;
    a.k_per_split = p.kps;
    a.xp = p.xp;
    a.bias = bias;
    a.act = act;
    a.splits = (int)p.splits;
    a.C = C;
    a.ldc = ldc;
    a.counters = counters;
    a.tile_join = p.tile_join;
    dim3 grid((unsigned)p.col_blocks, (unsigned)p.splits);
    const size_t smem = p.smem;
    note_kernel(head.W ? "sgemm_skinny_with_head" : p.form == kFormAny ? "sgemm_skinny_scalar" : "sgemm_skinny_vec4");
    switch (M) {
#define AX_CASE(m) case m: launch_m<m>(p, grid, smem, a, head); break;
        AX_CASE(1) AX_CASE(2) AX_CASE(3) AX_CASE(4) AX_CASE(5) AX_CASE(6) AX_CASE(7) AX_CASE(8)
        AX_CASE(9) AX_CASE(10) AX_CASE(11) AX_CASE(12) AX_CASE(13) AX_CASE(14) AX_CASE(15) AX_CASE(16)
#undef AX_CASE
        default: return AXHIP_ERR_SHAPE;
    }
    return check_launch("sgemm_skinny");
}

// Join slots of the allocating entry point: device memory owned by this file, every word kEmptySlot
// between launches, grown on demand.
unsigned char *g_slots = nullptr;
size_t g_slots_bytes = 0;

float *join_slots(size_t bytes) {
    if (bytes <= g_slots_bytes) return reinterpret_cast<float *>(g_slots);
    if (g_slots) {
        (void)hipDeviceSynchronize();
        (void)hipFree(g_slots);
        g_slots = nullptr;
        g_slots_bytes = 0;
    }
    const size_t want = bytes < (size_t(4) << 20) ? (size_t(4) << 20) : bytes;
    void *ptr = nullptr;
    if (hipMalloc(&ptr, want) != hipSuccess || hipMemset(ptr, 0xFF, want) != hipSuccess) {
        if (ptr) (void)hipFree(ptr);
        (void)hipGetLastError();
        fail(AXHIP_ERR_ALLOC, "skinny join slots of %zu bytes: out of device memory", want);
        return nullptr;
    }
    g_slots = static_cast<unsigned char *>(ptr);
    g_slots_bytes = want;
    return reinterpret_cast<float *>(g_slots);
}

// Scratch of axhip_sgemm_skinny_static: the join slots of the exchange tree (8 MiB, every word kEmptySlot
// between launches), room for the partial tiles of the tile join (8 MiB, contents arbitrary) and its
// per-strip arrival counters (zero between launches).  Every GPU that loads this library holds its own
// copy until the process ends.  In host code the array's name is only a handle for hipGetSymbolAddress;
// the device address is looked up once per device in skinny_setup() and kept in g_scratch_dev, and that
// is also where the slots are first set to kEmptySlot.
constexpr size_t kScratchSlotBytes = size_t(8) << 20, kScratchTileBytes = size_t(8) << 20;
constexpr size_t kScratchCounters = 4096;
constexpr size_t kScratchBytes = kScratchSlotBytes + kScratchTileBytes + kScratchCounters * sizeof(int);
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 16;
unsigned char *g_scratch_dev[kMaxDevices] = {};

template <typename K>
int raise_lds_limit(K kernel, int bytes) {
    AXHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes),
                  "hipFuncSetAttribute");
    return AXHIP_OK;
}

template <int MR>
int raise_stream_limits() {
    constexpr int kSmall = 100 * 1024;
    if (int rc = raise_lds_limit(k_skinny_stream<MR, false, 8, false, 64, 256>, kSmall)) return rc;
    if (int rc = raise_lds_limit(k_skinny_stream<MR, true, 8, false, 64, 256>, kSmall)) return rc;
    if (int rc = raise_lds_limit(k_skinny_stream<MR, false, 8, true, 64, 256>, kSmall)) return rc;
    if (int rc = raise_lds_limit(k_skinny_stream<MR, true, 8, true, 64, 256>, kSmall)) return rc;
    if (int rc = raise_lds_limit(k_skinny_stream<MR, false, 8, true, 64, 512>, kSmall)) return rc;
    if (int rc = raise_lds_limit(k_skinny_stream<MR, true, 8, true, 64, 512>, kSmall)) return rc;
    return AXHIP_OK;
}

template <int MR>
int raise_lds_limits() {
    if constexpr (MR < kMfmaFromM) {
        if (int rc = raise_stream_limits<MR>()) return rc;
    } else {
        if (int rc = raise_lds_limit(k_skinny_mfma<MR, false>, 100 * 1024)) return rc;
        if (int rc = raise_lds_limit(k_skinny_mfma<MR, true>, 100 * 1024)) return rc;
    }
    if (int rc = raise_lds_limit(k_skinny_any<MR>, 100 * 1024)) return rc;
    if constexpr (MR < 16) return raise_lds_limits<MR + 1>();
    return AXHIP_OK;
}

}  // namespace

namespace axhip {
// Once per device, with that device current (called from axhip_init): raises the kernels' dynamic LDS
// limit, looks up where this device keeps the static scratch array and empties its join slots.
int skinny_setup() {
    int dev = 0;
    AXHIP_HIP_TRY(hipGetDevice(&dev), "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(AXHIP_ERR_BACKEND, "device index %d not supported", dev);
    if (int rc = raise_lds_limits<1>()) return rc;
    void *ptr = nullptr;
    AXHIP_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
    if (!ptr) return fail(AXHIP_ERR_BACKEND, "static scratch has no device address");
    AXHIP_HIP_TRY(hipMemset(ptr, 0xFF, kScratchSlotBytes), "hipMemset(scratch slots)");
    AXHIP_HIP_TRY(hipMemset(static_cast<unsigned char *>(ptr) + kScratchSlotBytes + kScratchTileBytes, 0, kScratchCounters * sizeof(int)),
                  "hipMemset(scratch counters)");
    g_scratch_dev[dev] = static_cast<unsigned char *>(ptr);
    if (!join_slots(size_t(4) << 20)) return AXHIP_ERR_ALLOC;
    return AXHIP_OK;
}

// At shutdown: the join slots go back to the driver.
void skinny_teardown() {
    if (g_slots) (void)hipFree(g_slots);
    g_slots = nullptr;
    g_slots_bytes = 0;
}
}  // namespace axhip

extern "C" int axhip_sgemm_skinny(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                                  const float *B, int64_t ldb, float *C, int64_t ldc,
                                  const float *bias, int act) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (int rc = check_skinny_args("sgemm_skinny", M, N, K, A, lda, B, ldb, C, ldc, act)) return rc;
    if (N == 0) return AXHIP_OK;
    SkinnyPlan p;
    if (int rc = plan_skinny(M, N, K, B, ldb, 0, p)) return rc;
    float *join = nullptr;
    int *counters = nullptr;
    if (p.tile_join) {
        join = static_cast<float *>(axhip::workspace(p.join_bytes));
        counters = axhip::strip_counters((size_t)p.col_blocks);
        if (!join || !counters) return AXHIP_ERR_ALLOC;
    } else if (p.splits > 1) {
        join = join_slots(p.join_bytes);
        if (!join) return AXHIP_ERR_ALLOC;
    }
    return run_skinny(p, M, N, K, A, lda, B, ldb, C, ldc, bias, act, join, counters);
}

extern "C" int axhip_sgemm_skinny_static(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                                         const float *B, int64_t ldb, float *C, int64_t ldc,
                                         const float *bias, int act) {
    if (int rc = axhip::ensure_ready()) return rc;      // no-op after axhip_init
    if (int rc = check_skinny_args("sgemm_skinny_static", M, N, K, A, lda, B, ldb, C, ldc, act)) return rc;
    if (N == 0) return AXHIP_OK;
    SkinnyPlan p;
    if (int rc = plan_skinny(M, N, K, B, ldb, 0, p)) return rc;
    int dev = 0;
    AXHIP_HIP_TRY(hipGetDevice(&dev), "hipGetDevice");
    unsigned char *base = (dev >= 0 && dev < kMaxDevices) ? g_scratch_dev[dev] : nullptr;
    if (!base) return fail(AXHIP_ERR_BACKEND, "sgemm_skinny_static: axhip_init has not run on device %d", dev);
    const size_t room = p.tile_join ? kScratchTileBytes : kScratchSlotBytes;
    if (p.join_bytes > room || (p.tile_join && (size_t)p.col_blocks > kScratchCounters))
        return fail(AXHIP_ERR_SHAPE,
                    "sgemm_skinny_static: M=%lld N=%lld K=%lld needs %zu bytes to join its %lld ranges of K over %lld strips; "
                    "the static scratch holds %zu bytes and %zu strip counters (use axhip_sgemm_skinny)",
                    (long long)M, (long long)N, (long long)K, p.join_bytes, (long long)p.splits, (long long)p.col_blocks, room,
                    kScratchCounters);
    // Every slot is kEmptySlot and every counter zero when the library is initialised, and whoever takes a sum
    // out of a slot, or arrives last on a counter, puts that back: nothing needs clearing between calls that
    // run one after another.
    float *join = reinterpret_cast<float *>(p.tile_join ? base + kScratchSlotBytes : base);
    return run_skinny(p, M, N, K, A, lda, B, ldb, C, ldc, bias, act, join,
                      reinterpret_cast<int *>(base + kScratchSlotBytes + kScratchTileBytes));
}

extern "C" int axhip_sgemm_skinny_reset(void) {
    if (int rc = axhip::ensure_ready()) return rc;
    int dev = 0;
    AXHIP_HIP_TRY(hipGetDevice(&dev), "hipGetDevice");
    unsigned char *base = (dev >= 0 && dev < kMaxDevices) ? g_scratch_dev[dev] : nullptr;
    if (!base) return fail(AXHIP_ERR_BACKEND, "sgemm_skinny_reset: axhip_init has not run on device %d", dev);
    AXHIP_HIP_TRY(hipMemsetAsync(base, 0xFF, kScratchSlotBytes, kStream), "hipMemsetAsync(scratch slots)");
    AXHIP_HIP_TRY(hipMemsetAsync(base + kScratchSlotBytes + kScratchTileBytes, 0, kScratchCounters * sizeof(int), kStream),
                  "hipMemsetAsync(scratch counters)");
    if (g_slots) AXHIP_HIP_TRY(hipMemsetAsync(g_slots, 0xFF, g_slots_bytes, kStream), "hipMemsetAsync(join slots)");
    if (int rc = axhip::strip_counters_reset()) return rc;
    return AXHIP_OK;
}

extern "C" int axhip_sgemm_skinny_head(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B,
                                       int64_t ldb, float *C, int64_t ldc, const float *bias, int act, int64_t NH,
                                       const float *W2, const float *bias2, int act2, float *out2) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!W2 || !out2) return fail(AXHIP_ERR_NULL_ARG, "sgemm_skinny_head: NULL head weights or output");
    if (NH < 1 || NH > 16) return fail(AXHIP_ERR_SHAPE, "sgemm_skinny_head: head width %lld outside 1..16", (long long)NH);
    if (act2 < AXHIP_ACT_NONE || act2 > AXHIP_ACT_GELU)
        return fail(AXHIP_ERR_SHAPE, "sgemm_skinny_head: unknown activation %d", act2);
    // C may be NULL (the wide layer's output is then never written); the argument check wants a pointer
    if (int rc = check_skinny_args("sgemm_skinny_head", M, N, K, A, lda, B, ldb, C ? C : out2, C ? ldc : N, act)) return rc;
    if (N < 1) return fail(AXHIP_ERR_SHAPE, "sgemm_skinny_head: the wide layer has no outputs");
    SkinnyPlan p;
    if (int rc = plan_skinny(M, N, K, B, ldb, NH, p)) return rc;
    const size_t main_bytes = (p.join_bytes + 255) / 256 * 256, head_bytes = (size_t)p.col_blocks * M * NH * sizeof(float);
    unsigned char *ws = static_cast<unsigned char *>(axhip::workspace(main_bytes + head_bytes));
    int *counters = axhip::strip_counters((size_t)p.col_blocks + 1);
    if (!ws || !counters) return AXHIP_ERR_ALLOC;
    SkinnyHead head = {};
    head.W = W2;
    head.bias = bias2;
    head.out = out2;
    head.part = reinterpret_cast<float *>(ws + main_bytes);
    head.counter = counters + p.col_blocks;
    head.nh = (int)NH;
    head.act = act2;
    head.strips = (int)p.col_blocks;
    head.keep = C != nullptr;
    return run_skinny(p, M, N, K, A, lda, B, ldb, C ? C : out2, C ? ldc : N, bias, act, reinterpret_cast<float *>(ws), counters, head);
}

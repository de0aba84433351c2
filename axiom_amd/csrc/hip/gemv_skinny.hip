// Skinny-M (1 <= M <= 16) fp32 route: C[M,N] = act(A[M,K] * B[K,N] + bias[n]).
//
// The work is one pass over B (K*N*4 bytes): HBM-bound.  A workgroup of 256 threads owns 64
// columns (16 lanes x float4 = 256 contiguous bytes per B row) and a K range; its 16 lane
// groups take rows k, k+16, ... of that range, so one wave-wide load instruction covers four
// 256-byte row segments and eight of them are kept in flight per lane.  The M activations of
// a k row are wave-uniform only per lane group, so they come from LDS (staged once per
// workgroup); the first batch of weight loads is issued before that staging so HBM latency
// overlaps it.  The 16 lane groups' sums are joined through LDS in a fixed order; from M = 9 on the
// products run on the matrix cores (v_mfma_f32_16x16x4_f32, which sums a wave's four k rows itself;
// rows off the 16-byte grid: vector ALU, the four lane groups of a wave added with row swaps), which
// keeps the LDS buffer at four partial tiles whatever M is.  When K is split over
// several workgroups each writes its partial tile to a workspace and bumps a per-strip
// counter; the workgroup that arrives last adds the partials in split order (not arrival
// order) and applies bias and activation.  The sum order is fixed, so results are
// bit-identical run to run, and there is no second launch.
#include "common.h"

namespace {
using namespace axhip;

// A weight vector.  Every byte of the weights is read once per launch; with STREAM the loads are marked non-temporal,
// which lets large weights that come from HBM arrive 3-6 % faster (4096 x 4096 at M = 1: 16.0 -> 15.6 us, 8192 x 8192
// 50.5 -> 47.7, 11008 x 4096 35.3 -> 33.1) and costs weights small enough to be met again in the caches as much
// (4096 x 784: 7.0 -> 7.5 us), so the launcher sets it from 32 MiB of weights on.
template <bool STREAM>
__device__ __forceinline__ v4f ldw(const float *p) {
    if (STREAM) return __builtin_nontemporal_load(reinterpret_cast<const v4f *>(p));
    return *reinterpret_cast<const v4f *>(p);
}

constexpr int COLS = 64;        // columns per workgroup
constexpr int KGROUPS = 16;     // lane groups per workgroup, each 16 lanes x float4
constexpr int UNROLL = 8;
// workgroups to aim for: enough to cover 256 CUs a few times over; partial-sum traffic grows with M
// Workgroups a launch aims for (M = 1, 2 / M >= 3).  Fewer, longer workgroups leave fewer partial sums to join: with 256
// against 1024 at M = 1, weights from HBM, 4096 x 4096 15.6 -> 14.6 us, 4096 x 2048 11.3 -> 9.9, 2048 x 2048 8.3 -> 7.4, the
// other layer shapes unchanged (their split length is capped either way)
constexpr int64_t kWantBlocksM12 = 256, kWantBlocksM3up = 512;
constexpr int kJoinChunk = 16;              // splits whose partials the finishing workgroup requests at once
constexpr int kMfmaFromM = 9;              // from this M on the products run on the matrix cores (16-byte aligned rows); below, the vector ALU form measured faster (M = 8, 4096 x 32000: 107 us against 117)

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

template <int MR, bool VEC, bool STREAM = false>
__global__ void __launch_bounds__(256)
k_skinny(const float *__restrict__ A, int64_t lda, const float *__restrict__ B, int64_t ldb,
         float *__restrict__ dst, int64_t dst_ld, int64_t dst_split_stride, int64_t N, int64_t K,
         int64_t k_per_split, const float *__restrict__ bias, int act, int splits,
         float *__restrict__ C, int64_t ldc, int *__restrict__ counters, SkinnyHead head) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    __shared__ int head_last;
    // sm: [MR][k_per_split] activations, then [KGROUPS or 4][MR][COLS] partial sums, then (with a head)
    // [MR][COLS] finished outputs of the strip
    const int tid = threadIdx.x;
    const int cg = tid & 15;            // column group: columns 4*cg .. 4*cg+3 of the 64
    const int kg = tid >> 4;            // lane group
    const int64_t n0 = (int64_t)blockIdx.x * COLS;
    const int64_t k_begin = (int64_t)blockIdx.y * k_per_split;
    int64_t k_end = k_begin + k_per_split;
    if (k_end > K) k_end = K;
    const int64_t klen = k_end - k_begin;

    const int64_t col = n0 + 4 * cg;
    const float *bp = B + col;
    int64_t k = kg;
    // Activations of this split go to LDS.  Their loads (L2 hits, every workgroup reads the same
    // few rows) are issued first and the first batch of weights right behind them: loads return
    // in issue order, so the staging then waits only for the activations while the weights are
    // on their way from HBM.
    const int klen32 = (int)klen;
    float xr[MR][2];
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int kk = tid + c * 256;
            xr[m][c] = kk < klen32 ? A[m * lda + k_begin + kk] : 0.0f;
        }
    // first batch of weights (VEC form, full batch available).  From M = 9 on the products run on the
    // matrix cores, whose instructions every lane of a wave must reach together: there the batch is taken
    // when all lane groups have it (pre_all, the same for the whole workgroup).
    constexpr bool MFMA = VEC && MR >= kMfmaFromM;
    const bool pre_all = UNROLL * KGROUPS <= klen;
    const bool pre = MFMA ? pre_all : (VEC && col < N && (UNROLL - 1) * KGROUPS + kg < klen);
    v4f w0[UNROLL];
    if (pre) {
        const float *bf = MFMA && col >= N ? B + n0 : bp;     // MFMA form: see below
#pragma unroll
        for (int u = 0; u < UNROLL; u++)
            w0[u] = ldw<STREAM>(bf + (k_begin + k + u * KGROUPS) * ldb);
    }

    // the head's block of weights for this strip (64 rows x nh <= 1024 floats), requested now so that it
    // is in LDS long before a finishing workgroup needs it
    float hw[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (head.W) {
        const int cols = N - n0 < COLS ? (int)(N - n0) : COLS;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int e = tid + q * 256;
            if (e < cols * head.nh) hw[q] = head.W[n0 * head.nh + e];
        }
    }

    float *xs = sm;
#pragma unroll
    for (int m = 0; m < MR; m++) {
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int kk = tid + c * 256;
            if (kk < klen32) xs[m * (int)k_per_split + kk] = xr[m][c];
        }
        for (int kk = tid + 512; kk < klen32; kk += 256)      // splits longer than 512 rows
            xs[m * (int)k_per_split + kk] = A[m * lda + k_begin + kk];
    }
    __syncthreads();

    float acc[MR][4];
#pragma unroll
    for (int m = 0; m < MR; m++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc[m][e] = 0.0f;

    // M = 9..16 on v_mfma_f32_16x16x4_f32.  The weight layout is already the instruction's: the four lane
    // groups of a wave hold four consecutive k rows, lane cg of a group the columns 4*cg .. 4*cg+3, so
    // element j of the loaded float4 is the B operand (k = lane / 16, n = lane % 16) of the product for
    // columns 4*i + j, and the A operand is the activation of row m = lane % 16 at the lane group's k:
    // one LDS read and four MFMAs per 16 bytes of weights, against M reads and 4 M multiply-adds.
    // dm[j][v] = C[4 * (lane / 16) + v][4 * cg + j], summed over the wave's k rows.
    v4f dm[4];
    if constexpr (MFMA) {
#pragma unroll
        for (int j = 0; j < 4; j++) dm[j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        // A lane past the last column reads the strip's first columns instead and a lane whose row m does
        // not exist reads row 0: what they compute lands in columns / rows that are never stored, and the
        // loads of a full batch need no predicate.
        const float *bq = col < N ? bp : B + n0;
        const float *xrow = xs + (cg < MR ? cg : 0) * k_per_split;
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
    } else if (VEC) {
        if (col < N) {      // N % 4 == 0: a float4 is entirely inside or outside
            if (pre) {
#pragma unroll
                for (int u = 0; u < UNROLL; u++)
#pragma unroll
                    for (int m = 0; m < MR; m++) {
                        const float xv = xs[m * k_per_split + k + u * KGROUPS];
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[m][e] = __builtin_fmaf(xv, w0[u][e], acc[m][e]);
                    }
                k += UNROLL * KGROUPS;
            }
            for (; k + (UNROLL - 1) * KGROUPS < klen; k += UNROLL * KGROUPS) {
                v4f w[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; u++)
                    w[u] = ldw<STREAM>(bp + (k_begin + k + u * KGROUPS) * ldb);
#pragma unroll
                for (int u = 0; u < UNROLL; u++)
#pragma unroll
                    for (int m = 0; m < MR; m++) {
                        const float xv = xs[m * k_per_split + k + u * KGROUPS];
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[m][e] = __builtin_fmaf(xv, w[u][e], acc[m][e]);
                    }
            }
            for (; k < klen; k += KGROUPS) {
                v4f w = ldw<STREAM>(bp + (k_begin + k) * ldb);
#pragma unroll
                for (int m = 0; m < MR; m++) {
                    const float xv = xs[m * k_per_split + k];
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[m][e] = __builtin_fmaf(xv, w[e], acc[m][e]);
                }
            }
        }
    } else {
        // rows off the 16-byte grid (N or ldb not a multiple of 4): whole column groups still take one
        // 16-byte load each, at the alignment the row has; the last, partial group goes by element.
        // All loads of a batch of rows are issued before the first use, as in the vector form.
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
                    const float xv = xs[m * k_per_split + k + u * KGROUPS];
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
                const float xv = xs[m * k_per_split + k];
#pragma unroll
                for (int e = 0; e < 4; e++) acc[m][e] = __builtin_fmaf(xv, w[e], acc[m][e]);
            }
        }
    }

    // Lane groups are joined through LDS.  From M = 9 on the four lane groups of a wave (lanes l,
    // l^16, l^32, l^48 hold the same columns) are first added with the row-swap instructions, so
    // that one partial per wave goes through LDS and the buffer stays small enough for three
    // workgroups per CU; up to M = 8 every lane group writes its own partial (measured faster there).
    constexpr bool PRE = MR > 8 || MFMA;
    constexpr int NPART = PRE ? 4 : KGROUPS;
    float *red = sm + (int64_t)MR * k_per_split;
    if constexpr (MFMA) {
        // the wave's sums are complete in dm: one partial tile per wave, rows 4 * (lane / 16) + v
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int m = 4 * ((tid & 63) >> 4) + v;
            if (m < MR)
                *reinterpret_cast<v4f *>(red + ((tid >> 6) * MR + m) * COLS + 4 * cg) = v4f{dm[0][v], dm[1][v], dm[2][v], dm[3][v]};
        }
    } else
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

    float *hs = red + NPART * MR * COLS;                          // the strip's finished outputs, for the head
    float *hws = hs + MR * COLS;                                  // the head's [64][nh] block of weights
    // The head's share of a finished strip (every thread of the finishing workgroup calls this).
    auto head_tail = [&]() {
        const int nh = head.nh, hm = tid / nh, hj = tid - hm * nh;
#pragma unroll
        for (int q = 0; q < 4; q++)
            if (tid + q * 256 < COLS * nh) hws[tid + q * 256] = hw[q];
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
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (tid == 0) {
            const int arrived = __hip_atomic_fetch_add(head.counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            head_last = (arrived == head.strips - 1);
        }
        __syncthreads();
        if (!head_last) return;
        if (mine) {
            float sum = 0.0f;
            const float *pp = head.part + (int64_t)hm * nh + hj;
            const int64_t step = (int64_t)MR * nh;
            for (int s0 = 0; s0 < head.strips; s0 += 64) {        // strip order; 64 requests in flight at a time
                float v[64];
#pragma unroll
                for (int u = 0; u < 64; u++)
                    v[u] = s0 + u < head.strips
                               ? __int_as_float(__hip_atomic_load(reinterpret_cast<const int *>(pp + (s0 + u) * step),
                                                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
                               : 0.0f;
#pragma unroll
                for (int u = 0; u < 64; u++)
                    if (s0 + u < head.strips) sum += v[u];
            }
            if (head.bias) sum += head.bias[hj];
            head.out[hm * nh + hj] = apply_act(sum, head.act);
        }
        if (tid == 0) __hip_atomic_store(head.counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };

    float *part = dst + (int64_t)blockIdx.y * dst_split_stride;   // == C itself when splits == 1
    for (int i = tid; i < MR * COLS; i += 256) {
        const int m = i / COLS, c = i % COLS;
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < NPART; w++) s += red[(w * MR + m) * COLS + c];
        const int64_t n = n0 + c;
        if (n < N) {
            if (splits == 1) {
                if (bias) s += bias[n];
                s = apply_act(s, act);
                if (!head.W || head.keep) part[m * dst_ld + n] = s;
                if (head.W) hs[i] = s;
            } else {
                // device-scope store: written through to the point all XCDs' L2s agree on
                __hip_atomic_store(reinterpret_cast<int *>(part + m * dst_ld + n), __float_as_int(s),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    if (splits == 1) {
        if (head.W) head_tail();
        return;
    }

    // Publish this partial, then find out whether every split of this column strip is in.
    // Partials, counter and the reads below are all device-scope accesses, so no cache-wide
    // write-back or invalidate is needed (a __threadfence here costs ~150 us per launch: it
    // flushes the XCD's whole L2); the wait makes this thread's stores complete before the
    // barrier, the barrier orders them before thread 0's increment.
    __shared__ int last_flag;
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0) {
        const int arrived = __hip_atomic_fetch_add(counters + blockIdx.x, 1, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
        last_flag = (arrived == splits - 1);
    }
    __syncthreads();
    if (!last_flag) return;
    // Each thread owns up to OUTS outputs.  All partials of a chunk of splits are requested
    // before the first is used (one trip to memory per chunk, not per split); they are added
    // in split order.
    constexpr int OUTS = (MR * COLS + 255) / 256, CHUNK = kJoinChunk;
    const float *pp[OUTS];
    float s[OUTS];
    bool ok[OUTS];
#pragma unroll
    for (int o = 0; o < OUTS; o++) {
        const int i = tid + o * 256, m = i / COLS, c = i % COLS;
        ok[o] = i < MR * COLS && n0 + c < N;
        pp[o] = dst + m * dst_ld + n0 + c;
        s[o] = 0.0f;
    }
    for (int p0 = 0; p0 < splits; p0 += CHUNK) {
        float v[OUTS][CHUNK];
#pragma unroll
        for (int o = 0; o < OUTS; o++)
#pragma unroll
            for (int u = 0; u < CHUNK; u++)
                v[o][u] = (ok[o] && p0 + u < splits)
                              ? __int_as_float(__hip_atomic_load(
                                    reinterpret_cast<const int *>(pp[o] + (int64_t)(p0 + u) * dst_split_stride),
                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
                              : 0.0f;
#pragma unroll
        for (int o = 0; o < OUTS; o++)
#pragma unroll
            for (int u = 0; u < CHUNK; u++)
                if (p0 + u < splits) s[o] += v[o][u];
    }
#pragma unroll
    for (int o = 0; o < OUTS; o++) {
        if (!ok[o]) continue;
        const int i = tid + o * 256, m = i / COLS;
        const int64_t n = n0 + i % COLS;
        float r = s[o];
        if (bias) r += bias[n];
        r = apply_act(r, act);
        if (!head.W || head.keep) C[m * ldc + n] = r;
        if (head.W) hs[i] = r;
    }
    if (tid == 0)                                   // ready for the next launch
        __hip_atomic_store(counters + blockIdx.x, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (head.W) head_tail();
}

template <int MR>
int launch_m(bool vec, dim3 grid, size_t smem, const float *A, int64_t lda, const float *B,
             int64_t ldb, float *dst, int64_t dst_ld, int64_t dst_split, int64_t N, int64_t K,
             int64_t kps, const float *bias, int act, int splits, float *C, int64_t ldc,
             int *counters, const SkinnyHead &head) {
    if (vec && K * N * 4 >= (int64_t(32) << 20))
        hipLaunchKernelGGL((k_skinny<MR, true, true>), grid, dim3(256), smem, kStream, A, lda, B, ldb, dst,
                           dst_ld, dst_split, N, K, kps, bias, act, splits, C, ldc, counters, head);
    else if (vec)
        hipLaunchKernelGGL((k_skinny<MR, true>), grid, dim3(256), smem, kStream, A, lda, B, ldb, dst,
                           dst_ld, dst_split, N, K, kps, bias, act, splits, C, ldc, counters, head);
    else
        hipLaunchKernelGGL((k_skinny<MR, false>), grid, dim3(256), smem, kStream, A, lda, B, ldb,
                           dst, dst_ld, dst_split, N, K, kps, bias, act, splits, C, ldc, counters, head);
    return check_launch("sgemm_skinny");
}


// What one call launches: grid, split length, LDS bytes and the size of the partial-sum area.
struct SkinnyPlan {
    int64_t col_blocks, splits, kps, red_floats;
    bool vec;
    size_t smem, partial_bytes;
};

int plan_skinny(int64_t M, int64_t N, int64_t K, const float *B, int64_t ldb, SkinnyPlan &p) {
    p.col_blocks = (N + COLS - 1) / COLS;
    // enough workgroups to cover 256 CUs a few times over, each with at least 128 k rows
    const int64_t want_blocks = tuning().skinny_blocks > 0 ? tuning().skinny_blocks : M <= 2 ? kWantBlocksM12 : kWantBlocksM3up;
    int64_t splits = (want_blocks + p.col_blocks - 1) / p.col_blocks;
    const int64_t max_splits = K >= 128 ? K / 128 : 1;
    if (splits > max_splits) splits = max_splits;
    // The workgroup that finishes a strip requests the partials of up to 16 splits at once: more splits
    // mean more dependent trips to memory at the very end of the launch (M = 1, 8192 x 1024: 20.7 us with
    // 64 splits, 11.8 with 16).  A narrow matrix gets longer workgroups instead of more of them.
    const bool narrow = splits > kJoinChunk;
    if (narrow) splits = kJoinChunk;
    if (splits < 1) splits = 1;
    int64_t kps = (K + splits - 1) / splits;
    kps = (kps + KGROUPS - 1) / KGROUPS * KGROUPS;
    // the activations of one split must fit LDS next to the reduction buffer
    p.vec = (N % 4 == 0) && (ldb % 4 == 0) && ((uintptr_t)B % 16 == 0);
    p.red_floats = (int64_t)(M > 8 || (p.vec && M >= kMfmaFromM) ? 4 : KGROUPS) * M * COLS;   // partials per workgroup, as in the kernel
    // ... within 52 KiB, so that three workgroups share a CU whatever M is (4096 x 11008 at M = 16: 95 us
    // with one 96 KiB workgroup per CU, 60 us this way)
    const int64_t max_kps = ((int64_t)(52 * 1024 / 4) - p.red_floats) / M / KGROUPS * KGROUPS;
    if (kps > max_kps) kps = max_kps;
    // at most 128 KiB of weights per workgroup: wide matrices get more workgroups, not longer ones
    if (kps > (narrow ? 2048 : 512)) kps = narrow ? 2048 : 512;
    if (kps < KGROUPS) kps = KGROUPS;
    splits = K > 0 ? (K + kps - 1) / kps : 1;
    if (splits > 65535) return fail(AXHIP_ERR_SHAPE, "sgemm_skinny: K=%lld too large", (long long)K);
    p.splits = splits;
    p.kps = kps;
    p.smem = (size_t)(M * kps + p.red_floats) * sizeof(float);
    p.partial_bytes = splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
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

// `partials` holds plan.partial_bytes, `counters` plan.col_blocks ints that are zero (both unused when
// the plan has one split); the kernel leaves the counters at zero.
int run_skinny(const SkinnyPlan &p, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
               const float *B, int64_t ldb, float *C, int64_t ldc, const float *bias, int act,
               float *partials, int *counters, const SkinnyHead &head = SkinnyHead{}) {
    float *dst = C;
    int64_t dst_ld = ldc, dst_split = 0;
    if (p.splits > 1) {
        dst = partials;
        dst_ld = N;
        dst_split = M * N;
    }
    dim3 grid((unsigned)p.col_blocks, (unsigned)p.splits);
    const size_t smem = p.smem + (head.W ? (size_t)(M + head.nh) * COLS * sizeof(float) : 0);
    note_kernel(head.W ? "sgemm_skinny_with_head" : p.vec ? "sgemm_skinny_vec4" : "sgemm_skinny_scalar");
    int rc;
    switch (M) {
#define AX_CASE(m)                                                                                  \
    case m:                                                                                         \
        rc = launch_m<m>(p.vec, grid, smem, A, lda, B, ldb, dst, dst_ld, dst_split, N, K, p.kps,    \
                         bias, act, (int)p.splits, C, ldc, counters, head);                         \
        break;
        AX_CASE(1) AX_CASE(2) AX_CASE(3) AX_CASE(4) AX_CASE(5) AX_CASE(6) AX_CASE(7) AX_CASE(8)
        AX_CASE(9) AX_CASE(10) AX_CASE(11) AX_CASE(12) AX_CASE(13) AX_CASE(14) AX_CASE(15) AX_CASE(16)
#undef AX_CASE
        default: rc = AXHIP_ERR_SHAPE;
    }
    return rc;
}

// Scratch of axhip_sgemm_skinny_static: split-K partial tiles, then the per-strip arrival counters.
// Every GPU that loads this library holds its own copy until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress; the device address is looked up once per
// device in skinny_setup() and kept in g_scratch_dev.
constexpr size_t kScratchPartialBytes = size_t(8) << 20;
constexpr size_t kScratchCounters = 4096;
static __device__ __align__(256) unsigned char scratch[kScratchPartialBytes + kScratchCounters * sizeof(int)];
constexpr int kMaxDevices = 16;
unsigned char *g_scratch_dev[kMaxDevices] = {};

}  // namespace

namespace axhip {
// Once per device, with that device current (called from axhip_init): raises the kernels' dynamic LDS
// limit and looks up where this device keeps the static scratch array.
int skinny_setup() {
    int dev = 0;
    AXHIP_HIP_TRY(hipGetDevice(&dev), "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(AXHIP_ERR_BACKEND, "device index %d not supported", dev);
    const void *ks[] = {
        (const void *)k_skinny<1, true>, (const void *)k_skinny<2, true>, (const void *)k_skinny<3, true>,
        (const void *)k_skinny<4, true>, (const void *)k_skinny<5, true>, (const void *)k_skinny<6, true>,
        (const void *)k_skinny<7, true>, (const void *)k_skinny<8, true>,
        (const void *)k_skinny<1, false>, (const void *)k_skinny<2, false>, (const void *)k_skinny<3, false>,
        (const void *)k_skinny<4, false>, (const void *)k_skinny<5, false>, (const void *)k_skinny<6, false>,
        (const void *)k_skinny<7, false>, (const void *)k_skinny<8, false>,
        (const void *)k_skinny<9, true>, (const void *)k_skinny<10, true>, (const void *)k_skinny<11, true>,
        (const void *)k_skinny<12, true>, (const void *)k_skinny<13, true>, (const void *)k_skinny<14, true>,
        (const void *)k_skinny<15, true>, (const void *)k_skinny<16, true>,
        (const void *)k_skinny<9, false>, (const void *)k_skinny<10, false>, (const void *)k_skinny<11, false>,
        (const void *)k_skinny<12, false>, (const void *)k_skinny<13, false>, (const void *)k_skinny<14, false>,
        (const void *)k_skinny<15, false>, (const void *)k_skinny<16, false>,
        (const void *)k_skinny<1, true, true>, (const void *)k_skinny<2, true, true>, (const void *)k_skinny<3, true, true>,
        (const void *)k_skinny<4, true, true>, (const void *)k_skinny<5, true, true>, (const void *)k_skinny<6, true, true>,
        (const void *)k_skinny<7, true, true>, (const void *)k_skinny<8, true, true>, (const void *)k_skinny<9, true, true>,
        (const void *)k_skinny<10, true, true>, (const void *)k_skinny<11, true, true>, (const void *)k_skinny<12, true, true>,
        (const void *)k_skinny<13, true, true>, (const void *)k_skinny<14, true, true>, (const void *)k_skinny<15, true, true>,
        (const void *)k_skinny<16, true, true>};
    for (const void *k : ks)
        AXHIP_HIP_TRY(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024),
                      "hipFuncSetAttribute");
    void *ptr = nullptr;
    AXHIP_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
    if (!ptr) return fail(AXHIP_ERR_BACKEND, "static scratch has no device address");
    g_scratch_dev[dev] = static_cast<unsigned char *>(ptr);
    return AXHIP_OK;
}
}  // namespace axhip

extern "C" int axhip_sgemm_skinny(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                                  const float *B, int64_t ldb, float *C, int64_t ldc,
                                  const float *bias, int act) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (int rc = check_skinny_args("sgemm_skinny", M, N, K, A, lda, B, ldb, C, ldc, act)) return rc;
    if (N == 0) return AXHIP_OK;
    SkinnyPlan p;
    if (int rc = plan_skinny(M, N, K, B, ldb, p)) return rc;
    float *partials = nullptr;
    int *counters = nullptr;
    if (p.splits > 1) {
        partials = static_cast<float *>(axhip::workspace(p.partial_bytes));
        counters = axhip::strip_counters((size_t)p.col_blocks);
        if (!partials || !counters) return AXHIP_ERR_ALLOC;
    }
    return run_skinny(p, M, N, K, A, lda, B, ldb, C, ldc, bias, act, partials, counters);
}

extern "C" int axhip_sgemm_skinny_static(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                                         const float *B, int64_t ldb, float *C, int64_t ldc,
                                         const float *bias, int act) {
    if (int rc = axhip::ensure_ready()) return rc;      // no-op after axhip_init
    if (int rc = check_skinny_args("sgemm_skinny_static", M, N, K, A, lda, B, ldb, C, ldc, act)) return rc;
    if (N == 0) return AXHIP_OK;
    SkinnyPlan p;
    if (int rc = plan_skinny(M, N, K, B, ldb, p)) return rc;
    int dev = 0;
    AXHIP_HIP_TRY(hipGetDevice(&dev), "hipGetDevice");
    unsigned char *base = (dev >= 0 && dev < kMaxDevices) ? g_scratch_dev[dev] : nullptr;
    if (!base) return fail(AXHIP_ERR_BACKEND, "sgemm_skinny_static: axhip_init has not run on device %d", dev);
    if (p.partial_bytes > kScratchPartialBytes || (size_t)p.col_blocks > kScratchCounters)
        return fail(AXHIP_ERR_SHAPE,
                    "sgemm_skinny_static: M=%lld N=%lld K=%lld needs %zu bytes of partial sums and %lld counters; "
                    "the static scratch holds %zu bytes and %zu counters (use axhip_sgemm_skinny)",
                    (long long)M, (long long)N, (long long)K, p.partial_bytes, (long long)p.col_blocks,
                    kScratchPartialBytes, kScratchCounters);
    // Partials are fully written before they are read.  The counters start at zero when the code object
    // is loaded and every launch's last-arriving workgroups put theirs back to zero, so nothing needs
    // clearing between calls that run one after another.
    return run_skinny(p, M, N, K, A, lda, B, ldb, C, ldc, bias, act, reinterpret_cast<float *>(base),
                      reinterpret_cast<int *>(base + kScratchPartialBytes));
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
    if (int rc = plan_skinny(M, N, K, B, ldb, p)) return rc;
    const size_t main_bytes = (p.partial_bytes + 255) / 256 * 256, head_bytes = (size_t)p.col_blocks * M * NH * sizeof(float);
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

// Scaled dot-product attention forward: O = softmax(scale * Q K^T [+ causal mask]) V per head,
// Q, K, V, O [BH, S, dk] row-major fp32, L [BH, S] = log-sum-exp of each score row (or NULL).
//
// Fused kernel (dk a multiple of 4 up to 128, on the geometry of the next size among 32, 64 and
// 128; any S): the score matrix never leaves the chip.  A
// workgroup of 4 waves owns 128 query rows of one head, a wave 32 of them; keys and values
// stream through LDS in blocks of 64 (direct-to-LDS loads, two stages).  Both products run on
// v_mfma_f32_32x32x2_f32 with the query index on the MFMA's column side, so lane l of a wave
// owns query (l & 31) in the score tile *and* in the output accumulator:
//   S^T tile:  A = K rows (32 keys), B = the wave's Q rows (held in registers for the whole
//              kernel); register v of lane l = score(query l&31, key 8*(v>>2) + 4*(l>>5) + (v&3)).
//   softmax:   running maximum m and sum per query, the online form: the accumulator is
//              rescaled by 2^(m_old - m_new) when the maximum moves.  Row reductions are within
//              a lane plus one exchange with lane l^32.  Scores are kept in base-2 units
//              (scale * log2(e) folded in) so the exponential is the hardware's 2^x.
//   O^T tile:  A = V^T (lane reads V[key][d] with d = l&31), B = the probabilities exactly
//              where the score MFMA left them: key(v, l>>5) above is also a legal pairing of
//              the MFMA's two k indices, and a sum over keys does not care about their order.
// K rows are XOR-swizzled in 16-byte chunks, applied on the global address side of the load, so
// a 16-lane ds_read_b128 touches every bank once; V is laid out per load instruction with a
// pitch (or, for dk = 32, a row order) that puts the two lane halves of a fragment read (keys 4
// apart) on different banks.
//
// Every other head size: scores through a workspace, one batched NT GEMM, a row softmax kernel and
// one batched NN GEMM over as many heads at a time as fit 256 MiB (the structure of
// ax_cuda_sdpa_fwd, cuda/ops_attention.cu:299-392).
#include "common.h"

namespace {
using namespace axhip;

#define AXS_LOAD_LDS(m0val, voff, base)                                                        \
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0val),  \
                 "v"(voff), "s"(base)                                                          \
                 : "memory")
#define AXS_VM0() __builtin_amdgcn_s_waitcnt(0 | (0 << 14) | (7 << 4) | (15 << 8))
// at most n (a constant below 64) vector-memory loads still in flight
#define AXS_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))

constexpr int SD_BQ = 128, SD_BKV = 64;

// LDS geometry for head dimension DK (32, 64 or 128).  A direct-to-LDS load instruction moves
// 1 KiB = RPI whole rows of DK floats.
template <int DK>
struct SdGeom {
    static constexpr int ROWB = DK * 4;                 // bytes per row
    static constexpr int CH = DK / 4;                   // 16-byte chunks per row
    static constexpr int RPI = 1024 / ROWB;             // rows per load instruction
    static constexpr int KSTAGE = SD_BKV * ROWB;        // K block, rows contiguous, chunks swizzled
    // V block: load-instruction groups spaced so that keys k and k+4 (the two lane halves of a
    // fragment read) fall 128 bytes apart modulo 256, i.e. on different halves of the banks
    static constexpr int VGROUP = DK == 64 ? 1152 : DK == 128 ? 1088 : 1024;
    static constexpr int VSTAGE = (SD_BKV / RPI) * VGROUP;
    static constexpr int SMEM = 2 * KSTAGE + 2 * VSTAGE;
    static constexpr int IPW = SD_BKV / RPI / 4;        // load instructions per wave and 64-row block
    static_assert(DK == 32 || DK == 64 || DK == 128, "head dimension");
    static_assert(2 * KSTAGE >= SD_BQ * ROWB, "the Q tile is staged through the two K stages");

    // chunk swizzle key of a K/Q row: the 16 rows a ds_read_b128 serves together (same logical
    // chunk) must land on 16 different 16-byte bank slots
    __device__ static int swz(int row) { return CH >= 16 ? (row & 15) : ((row >> 1) & 7); }
    // which row of its group the lane at group position `slot` fetches (V only; DK = 32 keeps
    // rows k and k+4 next to each other)
    __device__ static int v_row_of_slot(int slot) { return DK == 32 ? ((slot & 1) * 4 + (slot >> 1)) : slot; }
    // byte offset of V row `key` inside a stage
    __device__ static int v_addr(int key) {
        if (DK == 64) return (key >> 2) * VGROUP + (key & 3) * ROWB;
        if (DK == 128) return (key >> 1) * VGROUP + (key & 1) * ROWB;
        return (key >> 3) * VGROUP + (((key & 3) * 2 + ((key >> 2) & 1))) * ROWB;
    }
};

// RAG: S is not a multiple of 128.  Rows past the end of a head are never loaded (the load of such
// a row is redirected to the head's last row, which keeps V finite), keys past the end are masked
// like causal ones, and queries past the end are computed but not stored.
// PAD: the head size dkr is below DK (a multiple of 4).  Lanes whose 16-byte chunk lies past column
// dkr issue no load, so nothing outside a row is read; their places in the K stages are zeroed once
// and never written again, Q's are zeroed in registers, V's feed output columns that are not stored.
// The padded k-blocks and output tiles are multiplied like the others: branching around them
// measured slower than the MFMAs they save (dk 96: 303 us with the branches, 268 without).
template <int DK, bool CAUSAL, bool RAG, bool PAD>
__global__ void __launch_bounds__(256)
k_sdpa(const float *__restrict__ Q, const float *__restrict__ K, const float *__restrict__ V,
       float *__restrict__ O, float *__restrict__ L, int64_t BH, int64_t S, float scale_log2e,
       int64_t H, int64_t ld, int64_t ldo, int dkr, int pair_tiles) {
    using G = SdGeom<DK>;
    constexpr int KB = DK / 8;                   // 8-wide k-blocks of the score product
    constexpr int DT = DK / 32;                  // 32-wide column tiles of the output
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int frow = lane & 31, fhalf = lane >> 5;
    const int64_t nq = (S + SD_BQ - 1) / SD_BQ;
    // Workgroups are handed to the 8 XCDs round-robin by linear index, and inside an XCD to its
    // CUs in a fixed rotation, so every workgroup has to carry the same amount of work.  Eight
    // heads form a group: workgroup r of a group works on head r % 8 (every query tile of a
    // head then runs on the same XCD and shares its L2 copy of K and V) and on unit r / 8.
    // A unit is one query tile, or, causal, the pair of tiles p and nq-1-p, which together
    // visit nq+1 key blocks whatever p is (the middle tile of an odd nq stands alone).  A launch
    // with no more single tiles than CUs keeps them single (pair_tiles = 0): pairing would only
    // halve the CUs at work (64 heads of 256 rows: 33.3 us paired, 22.7 single, 20.7 unmasked).
    const bool paired = CAUSAL && pair_tiles;
    const int64_t units = paired ? (nq + 1) / 2 : nq;
    const int64_t lin = blockIdx.x, group = lin / (8 * units), left = BH - group * 8;
    const int64_t r = lin - group * 8 * units, hpg = left < 8 ? left : 8;
    const int64_t head = group * 8 + r % hpg, unit = r / hpg;
    const int passes = (paired && unit != nq - 1 - unit) ? 2 : 1;
    // head b * H + h starts at row b * S, column h * DK of matrices with row pitch ld (Q, K, V)
    // and ldo (O): H = 1, ld = DK is one matrix per head; H heads side by side in rows of
    // ld >= H * DK floats is the layout a fused projection writes and the output projection reads
    const int64_t hb = head / H, hh = head - hb * H;
    const int64_t in0 = hb * S * ld + hh * (PAD ? dkr : DK);
    const float *Qh = Q + in0, *Kh = K + in0, *Vh = V + in0;
    const unsigned rowb = (unsigned)ld * 4;      // bytes between rows in global memory
    const unsigned lds0 = (unsigned)(uintptr_t)lds;
    if (PAD) {                                   // the K stages' never-loaded chunks must read as zero
        for (int o = tid * 16; o < 2 * G::KSTAGE; o += 256 * 16)
            *reinterpret_cast<v4f *>(lds + o) = v4f{0.f, 0.f, 0.f, 0.f};
        __syncthreads();
    }

    // per-lane byte offsets of the direct-to-LDS loads: instruction i of this wave is number
    // 4*i + wave of a 64-row block and covers rows RPI*(4*i + wave) .. + RPI-1
    unsigned koff[G::IPW], voff[G::IPW];
    bool kact[G::IPW];                           // PAD: does this lane's chunk of a K / Q row exist
    const bool vact = !PAD || (lane % G::CH) * 4 < dkr;
#pragma unroll
    for (int i = 0; i < G::IPW; i++) {
        const int slot = lane / G::CH, c = lane % G::CH;
        const int krow = G::RPI * (4 * i + wave) + slot;
        kact[i] = !PAD || (c ^ G::swz(krow)) * 4 < dkr;
        koff[i] = (unsigned)(krow * rowb + ((c ^ G::swz(krow)) << 4));
        const int vrow = G::RPI * (4 * i + wave) + G::v_row_of_slot(slot);
        voff[i] = (unsigned)(vrow * rowb + (c << 4));
    }
    // the same offsets for a 64-row block of which only the first `valid` (1..63) rows exist: the
    // LDS slot (and so the swizzle) stays that of the nominal row, the source row is the last one
    auto koff_clamped = [&](int i, int valid) {
        const int slot = lane / G::CH, c = lane % G::CH;
        const int krow = G::RPI * (4 * i + wave) + slot;
        return (unsigned)((krow < valid ? krow : valid - 1) * rowb + ((c ^ G::swz(krow)) << 4));
    };
    auto voff_clamped = [&](int i, int valid) {
        const int slot = lane / G::CH, c = lane % G::CH;
        const int vrow = G::RPI * (4 * i + wave) + G::v_row_of_slot(slot);
        return (unsigned)((vrow < valid ? vrow : valid - 1) * rowb + (c << 4));
    };

    for (int pass = 0; pass < passes; pass++) {
        const int64_t q0 = (paired && pass == 0 ? nq - 1 - unit : unit) * SD_BQ;
        if (pass) __syncthreads();                   // the first tile's last key block has been read
        // ---- Q tile (128 rows) through the V area, then into registers; the first key block's
        // K rows stream into their own stage at the same time, so a workgroup pays one load
        // latency, not two, before its first MFMA.  Its V rows follow once Q has left the V area.
        const int64_t all_blocks = (S + SD_BKV - 1) / SD_BKV;
        const int64_t nblocks = CAUSAL && (q0 + SD_BQ) / SD_BKV < all_blocks ? (q0 + SD_BQ) / SD_BKV : all_blocks;
        constexpr unsigned Q_BASE = 2 * G::KSTAGE;   // 2 * KSTAGE bytes of Q fit the two V stages
        static_assert(2 * G::KSTAGE <= 2 * G::VSTAGE, "Q staging area");
        auto issue_k = [&](int64_t blk, int stage) {
            const char *kg = reinterpret_cast<const char *>(Kh + blk * SD_BKV * ld);
            const int64_t valid = S - blk * SD_BKV;
            if (RAG && valid < SD_BKV) {
#pragma unroll
                for (int i = 0; i < G::IPW; i++)
                    if (kact[i]) AXS_LOAD_LDS(lds0 + stage * G::KSTAGE + (4 * i + wave) * 1024, koff_clamped(i, (int)valid), kg);
            } else {
#pragma unroll
                for (int i = 0; i < G::IPW; i++)
                    if (kact[i]) AXS_LOAD_LDS(lds0 + stage * G::KSTAGE + (4 * i + wave) * 1024, koff[i], kg);
            }
        };
        auto issue_v = [&](int64_t blk, int stage) {
            const char *vg = reinterpret_cast<const char *>(Vh + blk * SD_BKV * ld);
            const int64_t valid = S - blk * SD_BKV;
            if (RAG && valid < SD_BKV) {
#pragma unroll
                for (int i = 0; i < G::IPW; i++)
                    if (vact) AXS_LOAD_LDS(lds0 + 2 * G::KSTAGE + stage * G::VSTAGE + (4 * i + wave) * G::VGROUP, voff_clamped(i, (int)valid), vg);
            } else {
#pragma unroll
                for (int i = 0; i < G::IPW; i++)
                    if (vact) AXS_LOAD_LDS(lds0 + 2 * G::KSTAGE + stage * G::VSTAGE + (4 * i + wave) * G::VGROUP, voff[i], vg);
            }
        };
        if (RAG && q0 + SD_BQ > S) {
            // a half with no row inside the head re-reads the first half (its queries are never stored)
            const int64_t valid0 = S - q0 < 64 ? S - q0 : 64, left1 = S - q0 - 64;
            const int64_t base1 = left1 > 0 ? q0 + 64 : q0, valid1 = left1 > 0 ? (left1 < 64 ? left1 : 64) : valid0;
#pragma unroll
            for (int i = 0; i < G::IPW; i++) {
                if (!kact[i]) continue;
                AXS_LOAD_LDS(lds0 + Q_BASE + (4 * i + wave) * 1024, koff_clamped(i, (int)valid0),
                             reinterpret_cast<const char *>(Qh + q0 * ld));
                AXS_LOAD_LDS(lds0 + Q_BASE + G::KSTAGE + (4 * i + wave) * 1024, koff_clamped(i, (int)valid1),
                             reinterpret_cast<const char *>(Qh + base1 * ld));
            }
        } else {
#pragma unroll
            for (int i = 0; i < G::IPW; i++) {
                if (!kact[i]) continue;
                AXS_LOAD_LDS(lds0 + Q_BASE + (4 * i + wave) * 1024, koff[i], reinterpret_cast<const char *>(Qh + q0 * ld));
                AXS_LOAD_LDS(lds0 + Q_BASE + G::KSTAGE + (4 * i + wave) * 1024, koff[i],
                             reinterpret_cast<const char *>(Qh + (q0 + 64) * ld));
            }
        }
        issue_k(0, 0);
        AXS_VM0();
        __syncthreads();
        v4f qf[KB];                                  // k-block kb: dk 8*kb + 4*fhalf .. +3 of this lane's query
        {
            const int r = wave * 32 + frow;          // rows 64..127 sit KSTAGE bytes further on, same swizzle
            const unsigned char *qrow = lds + Q_BASE + (r >> 6) * G::KSTAGE + (r & 63) * G::ROWB;
#pragma unroll
            for (int kb = 0; kb < KB; kb++)      // scale * log2(e) goes into Q once: scores come out in log2 units
            {
                qf[kb] = *reinterpret_cast<const v4f *>(qrow + (((kb * 2 + fhalf) ^ G::swz(r & 63)) << 4)) * scale_log2e;
                if (PAD && kb * 8 + 4 * fhalf >= dkr) qf[kb] = v4f{0.f, 0.f, 0.f, 0.f};   // whatever the unloaded chunk held
            }
        }
        __syncthreads();
        issue_v(0, 0);

        v16f acc_o[DT];
#pragma unroll
        for (int d = 0; d < DT; d++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc_o[d][v] = 0.0f;
        float m_run = -INFINITY, l_run = 0.0f;       // l_run: this lane half's share of the row sum
        const int64_t qg = q0 + wave * 32 + frow;    // this lane's query

        for (int64_t blk = 0; blk < nblocks; blk++) {
            const int stage = (int)(blk & 1);
            if (blk > 0) {
                AXS_VM0();
                __syncthreads();                      // block blk has landed; stage^1 is free again
            }
            if (blk + 1 < nblocks) {
                issue_k(blk + 1, stage ^ 1);
                issue_v(blk + 1, stage ^ 1);
            }
            const unsigned char *ks = lds + stage * G::KSTAGE;
            const unsigned char *vs = lds + 2 * G::KSTAGE + stage * G::VSTAGE;

            // causal: a 32-key tile entirely above this wave's 32 queries is skipped, and only
            // blocks that straddle the diagonal pay for the mask (all wave-uniform decisions)
            const int64_t kb0 = blk * SD_BKV, wq_lo = q0 + wave * 32;
            const bool tile_on[2] = {!CAUSAL || kb0 <= wq_lo + 31,
                                     (!CAUSAL || kb0 + 32 <= wq_lo + 31) && (!RAG || kb0 + 32 < S)};
            const bool need_mask = (CAUSAL && kb0 + SD_BKV - 1 > wq_lo) || (RAG && !CAUSAL && kb0 + SD_BKV > S);
            // keys of this block with index > qrel are masked: those after the query (causal; such a
            // query lies inside the head, so they cover the keys past its end too) or past the end
            const int qrel = (int)((CAUSAL ? qg : S - 1) - kb0);

            // ---- scores of 64 keys ----
            v16f acc_s[2];
            __builtin_amdgcn_s_setprio(1);      // MFMA phases go ahead of the co-resident wave's VALU work
#pragma unroll
            for (int kt = 0; kt < 2; kt++) {
#pragma unroll
                for (int v = 0; v < 16; v++) acc_s[kt][v] = 0.0f;
                if (!tile_on[kt]) continue;
                const int r = kt * 32 + frow;
                const unsigned char *krow = ks + r * G::ROWB;
#pragma unroll
                for (int kb = 0; kb < KB; kb++) {
                    const v4f kf = *reinterpret_cast<const v4f *>(krow + (((kb * 2 + fhalf) ^ G::swz(r)) << 4));
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        acc_s[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[e], qf[kb][e], acc_s[kt], 0, 0, 0);
                }
            }

            __builtin_amdgcn_s_setprio(0);
            // ---- online softmax ----
            // Scores arrive in log2 units (Q was scaled once, above).  The reference point m_run
            // of the exponentials only moves when some query's block maximum exceeds it by more
            // than 2^8: until then p = 2^(s - m_run) <= 256 is safe in fp32 and exact in the
            // quotient O = sum(p v) / sum(p), and the accumulator needs no rescaling pass (which
            // costs as many vector instructions as the exponentials themselves; the fp32 MFMAs
            // run on the same lanes as vector instructions, so every one saved is MFMA time).
            float m_blk = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    float s = acc_s[kt][v];
                    if ((CAUSAL || RAG) && (!tile_on[kt] || (need_mask && kt * 32 + 8 * (v >> 2) + 4 * fhalf + (v & 3) > qrel)))
                        s = -INFINITY;
                    acc_s[kt][v] = s;
                    m_blk = fmaxf(m_blk, s);
                }
            m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32, 64));
            if (__builtin_amdgcn_ballot_w64(m_blk > m_run + 8.0f)) {      // wave-uniform; always taken for block 0
                const float m_new = fmaxf(m_run, m_blk);  // finite: key 0 is visible to every query
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                l_run *= alpha;
                m_run = m_new;
#pragma unroll
                for (int d = 0; d < DT; d++)
#pragma unroll
                    for (int v = 0; v < 16; v++) acc_o[d][v] *= alpha;
            }
            float l_blk = 0.0f;
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const float p = __builtin_amdgcn_exp2f(acc_s[kt][v] - m_run);
                    acc_s[kt][v] = p;
                    l_blk += p;
                }
            l_run += l_blk;

            if (blk == 0) {                           // the first block's V rows were issued last
                if (nblocks > 1) AXS_VM(2 * G::IPW);      // loads return in order: all but block 1's
                else AXS_VM0();
                __syncthreads();
            }
            // ---- O^T += V^T P^T ----
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int kt = 0; kt < 2; kt++) {
                if (!tile_on[kt]) continue;
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int key = kt * 32 + 8 * (v >> 2) + 4 * fhalf + (v & 3);
                    const float *vrow = reinterpret_cast<const float *>(vs + G::v_addr(key));
#pragma unroll
                    for (int d = 0; d < DT; d++)
                        acc_o[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(vrow[d * 32 + frow], acc_s[kt][v], acc_o[d], 0, 0, 0);
                }
            }
            __builtin_amdgcn_s_setprio(0);
        }

        // ---- normalise and write: lane owns query qg, dk columns 32*d + 8*g + 4*fhalf .. +3 ----
        const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
        const float inv = 1.0f / l_tot;
        float *orow = O + (hb * S + qg) * ldo + hh * (PAD ? dkr : DK);
        if (!RAG || qg < S) {
#pragma unroll
            for (int d = 0; d < DT; d++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    v4f r;
#pragma unroll
                    for (int e = 0; e < 4; e++) r[e] = acc_o[d][4 * g + e] * inv;
                    if (!PAD || d * 32 + 8 * g + 4 * fhalf < dkr) *reinterpret_cast<v4f *>(orow + d * 32 + 8 * g + 4 * fhalf) = r;
                }
            if (L && fhalf == 0) L[head * S + qg] = (m_run + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f;
        }
    }
}

template <int DK, bool PAD>
int launch_sdpa_p(const float *Q, const float *K, const float *V, float *O, float *L, int64_t BH, int64_t S,
                  float scale, int causal, int64_t H, int64_t ld, int64_t ldo, int dkr) {
    using G = SdGeom<DK>;
    static bool attr_set = false;
    const void *kernels[4] = {reinterpret_cast<const void *>(k_sdpa<DK, false, false, PAD>),
                              reinterpret_cast<const void *>(k_sdpa<DK, true, false, PAD>),
                              reinterpret_cast<const void *>(k_sdpa<DK, false, true, PAD>),
                              reinterpret_cast<const void *>(k_sdpa<DK, true, true, PAD>)};
    if (!attr_set) {
        for (const void *k : kernels)
            AXHIP_HIP_TRY(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, G::SMEM), "hipFuncSetAttribute");
        attr_set = true;
    }
    const float sl2 = scale * 1.4426950408889634f;
    const int64_t nq = (S + SD_BQ - 1) / SD_BQ;
    // causal tiles p and nq-1-p in one workgroup once there are more tiles than CUs; with a CU for every tile the
    // longest tile sets the time either way and pairing only halves the CUs at work
    const int pair = causal && nq * BH > (int64_t)cu_count();
    dim3 grid((unsigned)((pair ? (nq + 1) / 2 : nq) * BH));
    const bool rag = S % SD_BQ != 0;
#define AXS_GO(C, R)                                                                                              \
    hipLaunchKernelGGL((k_sdpa<DK, C, R, PAD>), grid, dim3(256), G::SMEM, kStream, Q, K, V, O, L, BH, S, sl2, H, ld, \
                       ldo, dkr, pair)
    if (causal && rag) AXS_GO(true, true);
    else if (causal) AXS_GO(true, false);
    else if (rag) AXS_GO(false, true);
    else AXS_GO(false, false);
#undef AXS_GO
    return check_launch("sdpa_fwd");
}

template <int DK>
int launch_sdpa(const float *Q, const float *K, const float *V, float *O, float *L, int64_t BH, int64_t S,
                float scale, int causal, int64_t H, int64_t ld, int64_t ldo, int dkr) {
    return dkr == DK ? launch_sdpa_p<DK, false>(Q, K, V, O, L, BH, S, scale, causal, H, ld, ldo, dkr)
                     : launch_sdpa_p<DK, true>(Q, K, V, O, L, BH, S, scale, causal, H, ld, ldo, dkr);
}

// One workgroup per score row: mask, maximum, exponentials, sum, normalise in place; L = max + log(sum).
__global__ void __launch_bounds__(256)
k_softmax_lse_rows(float *__restrict__ score, float *__restrict__ L, int64_t S, int causal) {
    __shared__ float red[256];
    const int64_t row = blockIdx.x;               // head * S + query
    const int64_t qi = row % S;
    float *p = score + row * S;
    const int64_t n = causal ? qi + 1 : S;        // keys this query sees
    float mx = -INFINITY;
    for (int64_t j = threadIdx.x; j < n; j += 256) mx = fmaxf(mx, p[j]);
    red[threadIdx.x] = mx;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] = fmaxf(red[threadIdx.x], red[threadIdx.x + s]);
        __syncthreads();
    }
    mx = red[0];
    __syncthreads();
    float sum = 0.0f;
    for (int64_t j = threadIdx.x; j < S; j += 256) {
        const float e = j < n ? expf(p[j] - mx) : 0.0f;
        p[j] = e;
        sum += e;
    }
    red[threadIdx.x] = sum;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    sum = red[0];
    const float inv = 1.0f / sum;
    for (int64_t j = threadIdx.x; j < n; j += 256) p[j] *= inv;
    if (L && threadIdx.x == 0) L[row] = mx + logf(sum);
}

int sdpa_unfused(const float *Q, const float *K, const float *V, float *O, float *L, int64_t BH,
                 int64_t S, int64_t dk, float scale, int causal) {
    const size_t per_head = (size_t)S * (size_t)S * sizeof(float);
    int64_t chunk = (int64_t)((size_t(256) << 20) / per_head);
    if (chunk < 1) chunk = 1;
    if (chunk > BH) chunk = BH;
    if (chunk > 65535) chunk = 65535;
    float *score = static_cast<float *>(workspace((size_t)chunk * per_head));
    if (!score) return AXHIP_ERR_ALLOC;
    for (int64_t h0 = 0; h0 < BH; h0 += chunk) {
        const int64_t nb = BH - h0 < chunk ? BH - h0 : chunk;
        const float *q = Q + h0 * S * dk, *k = K + h0 * S * dk, *v = V + h0 * S * dk;
        int rc = axhip_sgemm_strided_batched(0, 1, S, S, dk, scale, q, dk, S * dk, k, dk, S * dk, 0.0f, score, S,
                                             S * S, nb);
        if (rc) return rc;
        if (nb * S > 0x7fffffff) return fail(AXHIP_ERR_SHAPE, "sdpa: too many score rows per chunk");
        hipLaunchKernelGGL(k_softmax_lse_rows, dim3((unsigned)(nb * S)), dim3(256), 0, kStream, score,
                           L ? L + h0 * S : nullptr, S, causal);
        if ((rc = check_launch("sdpa softmax"))) return rc;
        rc = axhip_sgemm_strided_batched(0, 0, S, dk, S, 1.0f, score, S, S * S, v, dk, S * dk, 0.0f,
                                         O + h0 * S * dk, dk, S * dk, nb);
        if (rc) return rc;
    }
    note_kernel("sdpa_unfused");
    return AXHIP_OK;
}

}  // namespace

// shared by both entry points: H heads side by side in rows of ld (Q, K, V) / ldo (O) floats.  A head
// size that is a multiple of 4 up to 128 runs on the kernel of the next size among 32, 64, 128.
static bool sdpa_fusable(int64_t dk) { return dk >= 4 && dk <= 128 && dk % 4 == 0; }

static int sdpa_fused(const float *Q, const float *K, const float *V, float *O, float *L, int64_t BH, int64_t S,
                      int64_t dk, float scale, int causal, int64_t H, int64_t ld, int64_t ldo) {
    int rc;
    if (dk <= 32) {
        rc = launch_sdpa<32>(Q, K, V, O, L, BH, S, scale, causal, H, ld, ldo, (int)dk);
        axhip::note_kernel(causal ? "sdpa_fused_dk32_causal" : "sdpa_fused_dk32");
    } else if (dk <= 64) {
        rc = launch_sdpa<64>(Q, K, V, O, L, BH, S, scale, causal, H, ld, ldo, (int)dk);
        axhip::note_kernel(causal ? "sdpa_fused_dk64_causal" : "sdpa_fused_dk64");
    } else {
        rc = launch_sdpa<128>(Q, K, V, O, L, BH, S, scale, causal, H, ld, ldo, (int)dk);
        axhip::note_kernel(causal ? "sdpa_fused_dk128_causal" : "sdpa_fused_dk128");
    }
    return rc;
}

extern "C" int axhip_sdpa_fwd(const float *Q, const float *K, const float *V, float *O, float *L, int64_t BH,
                              int64_t S, int64_t dk, float scale, int causal) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!Q || !K || !V || !O) return fail(AXHIP_ERR_NULL_ARG, "sdpa_fwd: NULL tensor");
    if (BH < 0 || S < 0 || dk <= 0) return fail(AXHIP_ERR_SHAPE, "sdpa_fwd: bad extent");
    if (BH == 0 || S == 0) return AXHIP_OK;
    const bool aligned = ((((uintptr_t)Q | (uintptr_t)K | (uintptr_t)V | (uintptr_t)O) & 15) == 0);
    if (sdpa_fusable(dk) && aligned && (S + SD_BQ - 1) / SD_BQ * BH <= 0x7fffffff)
        return sdpa_fused(Q, K, V, O, L, BH, S, dk, scale, causal, 1, dk, dk);
    return sdpa_unfused(Q, K, V, O, L, BH, S, dk, scale, causal);
}

extern "C" int axhip_sdpa_fwd_rows(const float *Q, const float *K, const float *V, int64_t ld, float *O, int64_t ldo,
                                   float *L, int64_t B, int64_t H, int64_t S, int64_t dk, float scale, int causal) {
    if (int rc = axhip::ensure_ready()) return rc;
    if (!Q || !K || !V || !O) return fail(AXHIP_ERR_NULL_ARG, "sdpa_fwd_rows: NULL tensor");
    if (B < 0 || H <= 0 || S < 0) return fail(AXHIP_ERR_SHAPE, "sdpa_fwd_rows: bad extent");
    if (!sdpa_fusable(dk))
        return fail(AXHIP_ERR_NOT_IMPLEMENTED, "sdpa_fwd_rows: head size %lld (multiples of 4 up to 128 only)", (long long)dk);
    if (ld < H * dk || ldo < H * dk || ld % 4 != 0 || ldo % 4 != 0 || ld > (1 << 22))
        return fail(AXHIP_ERR_SHAPE, "sdpa_fwd_rows: row pitch must hold H * dk floats and be a multiple of 4");
    if ((((uintptr_t)Q | (uintptr_t)K | (uintptr_t)V | (uintptr_t)O) & 15) != 0)
        return fail(AXHIP_ERR_SHAPE, "sdpa_fwd_rows: tensors must be 16-byte aligned");
    if (B == 0 || S == 0) return AXHIP_OK;
    if (B > 0x7fffffff / H || (S + SD_BQ - 1) / SD_BQ * (B * H) > 0x7fffffff)
        return fail(AXHIP_ERR_SHAPE, "sdpa_fwd_rows: too many tiles");
    return sdpa_fused(Q, K, V, O, L, B * H, S, dk, scale, causal, H, ld, ldo);
}

// Internal helpers shared by the kernel translation units of libaxhip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#include "axhip.h"

namespace axhip {

// Records a failure message for axhip_last_error() and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// 0 when the runtime is initialised on a usable GPU, else an AXHIP_ERR_* code (message set).
int ensure_ready();
// Compute units of the device (valid once ensure_ready() has returned 0).
int cu_count();
// Remembers which kernel variant a GEMM-type entry point chose.
void note_kernel(const char *name);
// Checks the launch that was just issued on the null stream.
int check_launch(const char *what);
// A device workspace of at least `bytes`, owned by the runtime (grown on demand), or NULL.
void *workspace(size_t bytes);
// `n` zero-initialised device ints owned by the runtime.  Kernels that use them as arrival counters
// leave them at zero when they finish.
int *strip_counters(size_t n);
// Queues a fill that puts them back to zero (after a launch that was cut short).
int strip_counters_reset();
// The allocation pool behind axhip_malloc / axhip_free: the size class of a request, and the call
// that hands every cached block back to the driver.
size_t pool_class(size_t bytes);
void pool_release_all();
// At least `n` device floats, all 1.0f, owned by the runtime (grown on demand).
float *ones_vector(size_t n);
// Per-device set-up of the skinny-M kernels (LDS limits, address of the static scratch); the device
// must be current.  Called by axhip_init.
int skinny_setup();
// Frees what skinny_setup allocated (axhip_shutdown).
void skinny_teardown();

// Tile-selection overrides from the environment (0 = choose by shape), read at axhip_init and by
// axhip_tuning_reload; what each one forces is described next to axhip_tuning_reload in axhip.h.
struct Tuning {
    int i8_tile;         // AX_HIP_I8_TILE: 64 (64x64), 642 (64x64 with the k-steps split over two wave sets), 1264 (128x64), 128 or 256
    int i8_splitk;       // AX_HIP_I8_SPLITK: 1..16
    int i8_mfma;         // AX_HIP_I8_MFMA: 32 (v_mfma_i32_32x32x32_i8) or 16 (v_mfma_i32_16x16x64_i8) in the persistent 256x256 kernel
    int f32_tile;        // AX_HIP_F32_TILE: 64 (64x64), 642 (64x64 with the k split over two wave sets), 128 (128x128, eight waves)
    int f32_splitk;      // AX_HIP_F32_SPLITK: 1 = never split K, 2.. = that many ranges where the route applies
    int skinny_blocks;   // AX_HIP_SKINNY_BLOCKS: workgroups the skinny-M route aims for
    int skinny_form;     // AX_HIP_SKINNY_FORM: 1 (64 columns x 256 threads), 2 (the same, the lane groups of a wave added before LDS), 3 (64 columns x 512 threads)
    int skinny_kps;      // AX_HIP_SKINNY_KPS: most rows of K one skinny-M workgroup takes (a multiple of 16)
    int nt_walk;         // AX_HIP_NT_WALK: short-K batched A B^T: 1 = a block of A rows resident, blocks of B walked; 2 = 256 rows of B resident, blocks of A walked
    int w8a32_tile;      // AX_HIP_W8A32_TILE: 1 (128x256), 2 (128x128), 3 (64x128), 4 (32x128), 5 (32x64): W8A32 matrix-core tile for K > 128
};
const Tuning &tuning();

constexpr hipStream_t kStream = nullptr;

typedef int   v4i  __attribute__((ext_vector_type(4)));
typedef int   v16i __attribute__((ext_vector_type(16)));
typedef float v4f  __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

// 0.5 x (1 + tanh(u)) with u = sqrt(2/pi) (x + 0.044715 x^3), evaluated as x / (1 + e^(-2u)):
// the same function (0.5 (1 + tanh u) is the logistic of 2u; the reference's vector path also
// goes through 2*sigmoid(2x) - 1, src/compute/backends/simd_defs.h:308-321) in one hardware
// exponential and one reciprocal instead of a library tanh.  In a fused GEMM write-back every
// vector instruction is time taken from the fp32 MFMAs, which run on the same lanes.
__device__ __forceinline__ float gelu_tanh(float x) {
    const float k0 = 0.7978845608028654f, k1 = 0.044715f;
    const float u = k0 * (x + k1 * x * x * x);
    const float t = __builtin_amdgcn_exp2f(u * -2.8853900817779268f);      // e^(-2u); inf for u << 0
    return x * __builtin_amdgcn_rcpf(1.0f + t);
}

__device__ __forceinline__ float apply_act(float v, int act) {
    if (act == AXHIP_ACT_RELU) return v > 0.0f ? v : 0.0f;
    if (act == AXHIP_ACT_GELU) return gelu_tanh(v);
    return v;
}

// Workgroup id -> output tile.  Consecutive workgroup ids are dealt round-robin to the 8 XCDs,
// each with its own L2; renumbering so that every XCD walks one contiguous run of tiles, in
// bands of 4 tile-rows, keeps the operand panels an XCD re-reads inside that XCD's L2.
// (An integer division by a run-time value costs some thirty vector instructions even when every
// operand is the same for the whole workgroup, and in an fp32 MFMA kernel vector instructions take
// the matrix core's issue slots: the common cases — a power-of-two tile count, full bands and full
// groups — are therefore done with shifts, and the general division is kept for the rest.)
__device__ __forceinline__ unsigned div_by(unsigned n, unsigned d) {
    return (d & (d - 1)) == 0 ? n >> (31 - __builtin_clz(d)) : n / d;
}

__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int &tm, int &tn) {
    const unsigned total = (unsigned)tiles_m * (unsigned)tiles_n;
    unsigned id = (unsigned)bid;
    if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    constexpr unsigned BAND = 4;
    const unsigned per_band = BAND * (unsigned)tiles_n;
    const unsigned band = div_by(id, per_band);
    const unsigned first = band * BAND;
    const unsigned rows = ((unsigned)tiles_m - first) < BAND ? ((unsigned)tiles_m - first) : BAND;
    const unsigned in_band = id - band * per_band;
    const unsigned q = rows == BAND ? in_band >> 2 : in_band / rows;
    tm = (int)(first + (in_band - q * rows));
    tn = (int)q;
}

// The same for a batched launch with grid (tiles, batch): the hardware numbers workgroups x
// fastest, so workgroup lin = x + tiles * y lands on XCD lin % 8.  Eight batch entries form a
// group; inside a group workgroup r works on entry r % 8 and tile r / 8, so every tile of one
// batch entry runs on the same XCD, back to back, and that entry's operands are fetched into one
// L2 only (a partial last group of `left` entries uses r % left, r / left).
__device__ __forceinline__ void tile_of_batched_block(int tiles_m, int tiles_n, int &tm, int &tn, int64_t &batch) {
    const unsigned tiles = (unsigned)tiles_m * (unsigned)tiles_n, entries = gridDim.y;
    // lin = x + tiles * y with x < tiles, so lin / (8 * tiles) = y / 8 and the remainder is x + tiles * (y % 8)
    const unsigned group = blockIdx.y >> 3, r = blockIdx.x + tiles * (blockIdx.y & 7);
    const unsigned left = entries - group * 8;
    unsigned tile;
    if (left >= 8) {
        batch = (int64_t)(group * 8 + (r & 7));
        tile = r >> 3;
    } else {
        tile = r / left;
        batch = (int64_t)(group * 8 + (r - tile * left));
    }
    // consecutive workgroups walk along a tile row: their write-backs fill whole output rows
    const unsigned row = div_by(tile, (unsigned)tiles_n);
    tm = (int)row;
    tn = (int)(tile - row * (unsigned)tiles_n);
}

// Sums NV per-lane values over the 64 lanes of a wave, all NV at once.  A butterfly per value
// would cost 6 cross-lane moves each; here every step also halves the number of values a lane
// carries (lane bit `off` decides which half it keeps, the other half goes to its partner), so NV
// values cost about NV moves in total and end up spread over the lanes: afterwards v[0] of lane l
// holds the wave-wide sum of value number l / (64 / NV).  The first two steps exchange 32- and
// 16-lane rows with the swap instructions of this chip; later ones go through the cross-lane
// network.  The association order is a fixed tree, the same for every value.
template <int NV, typename T>
__device__ __forceinline__ void wave_sum_spread(T (&v)[NV], int lane) {
    static_assert(NV >= 1 && NV <= 64 && (NV & (NV - 1)) == 0 && sizeof(T) == 4, "power of two 32-bit values");
    int n = NV;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        if (n > 1) {
            const int half = n / 2;
#pragma unroll
            for (int i = 0; i < half; i++) {
                if (off >= 16) {
                    const unsigned a = __builtin_bit_cast(unsigned, v[i]), b = __builtin_bit_cast(unsigned, v[i + half]);
                    const auto r = off == 32 ? __builtin_amdgcn_permlane32_swap(a, b, false, false)
                                             : __builtin_amdgcn_permlane16_swap(a, b, false, false);
                    v[i] = __builtin_bit_cast(T, (unsigned)r[0]) + __builtin_bit_cast(T, (unsigned)r[1]);
                } else {
                    const bool up = (lane & off) != 0;
                    const T keep = up ? v[i + half] : v[i], send = up ? v[i] : v[i + half];
                    v[i] = keep + __shfl_xor(send, off, 64);
                }
            }
            n = half;
        } else {
            v[0] += __shfl_xor(v[0], off, 64);
        }
    }
}

// Write-back of one 32x32 MFMA result tile held in the layout "lane l owns row (l & 31), and
// for g = 0..3 the four consecutive columns 8*g + 4*(l >> 5) + e": the wave turns the tile
// through 4 KiB of LDS private to it so that each store instruction writes 8 rows of 128
// contiguous bytes (whole cache lines) instead of 32 rows of 32 bytes.  LDS rows are 128 bytes
// with 16-byte chunk c of row r kept at chunk c ^ ((r >> 1) & 7): both the write (16 rows, one
// chunk column per 16-lane group) and the read (2 rows, all chunks) touch every bank once.
// V4 is a 16-byte vector; dst points at the tile's element (0, 0), ld in elements.
template <typename V4, typename T>
__device__ __forceinline__ void turn_tile_and_store(unsigned char *turn, int lane, const V4 (&r)[4],
                                                    T *dst, int64_t ld) {
    static_assert(sizeof(V4) == 16 && sizeof(T) == 4, "32-bit elements in 16-byte vectors");
    const int frow = lane & 31, fhalf = lane >> 5;
#pragma unroll
    for (int g = 0; g < 4; g++)
        *reinterpret_cast<V4 *>(turn + frow * 128 + (((2 * g + fhalf) ^ ((frow >> 1) & 7)) << 4)) = r[g];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    V4 o[4];
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const int row = p * 8 + (lane >> 3);
        o[p] = *reinterpret_cast<const V4 *>(turn + row * 128 + (((lane & 7) ^ ((row >> 1) & 7)) << 4));
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int p = 0; p < 4; p++)
        *reinterpret_cast<V4 *>(dst + (int64_t)(p * 8 + (lane >> 3)) * ld + (lane & 7) * 4) = o[p];
}

// The same write-back for a tile that may hang over the matrix edge: only rows below `rows` and
// 4-column groups that begin below `cols` (a multiple of 4) are stored.
template <typename V4, typename T>
__device__ __forceinline__ void turn_tile_and_store_edge(unsigned char *turn, int lane, const V4 (&r)[4],
                                                         T *dst, int64_t ld, int64_t rows, int64_t cols) {
    static_assert(sizeof(V4) == 16 && sizeof(T) == 4, "32-bit elements in 16-byte vectors");
    const int frow = lane & 31, fhalf = lane >> 5;
#pragma unroll
    for (int g = 0; g < 4; g++)
        *reinterpret_cast<V4 *>(turn + frow * 128 + (((2 * g + fhalf) ^ ((frow >> 1) & 7)) << 4)) = r[g];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    V4 o[4];
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const int row = p * 8 + (lane >> 3);
        o[p] = *reinterpret_cast<const V4 *>(turn + row * 128 + (((lane & 7) ^ ((row >> 1) & 7)) << 4));
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int p = 0; p < 4; p++)
        if (p * 8 + (lane >> 3) < rows && (lane & 7) * 4 < cols)
            *reinterpret_cast<V4 *>(dst + (int64_t)(p * 8 + (lane >> 3)) * ld + (lane & 7) * 4) = o[p];
}

}  // namespace axhip

#define AXHIP_HIP_TRY(expr, what)                                                         \
    do {                                                                                  \
        hipError_t e_ = (expr);                                                           \
        if (e_ != hipSuccess)                                                             \
            return axhip::fail(AXHIP_ERR_BACKEND, "%s: %s", what, hipGetErrorString(e_)); \
    } while (0)

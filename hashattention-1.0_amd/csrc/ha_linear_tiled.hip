// y = x W^T for up to 16 rows of x (one new token per sequence of a batch of 9 to 16) on the matrix cores, with W stored in
// tiles of 16 rows x 32 inputs in the order the matrix instruction takes its operand: every wave load is one contiguous KiB
// and lands in the registers it is multiplied from.
//
//   ha_weight_tiles_elems / ha_pack_weight_tiles   the tiled copy of a [N, K] bf16 matrix
//   ha_linear_tiled                                the product, residual or SwiGLU behind
//
// The projections of the reference's decoding harness (efficiency/model.py:236-262, 304-305) with the elementwise steps next
// to them (:308-319 RMSNorm, :190-191 residuals), roundings as those modules round.
#include "ha_common.h"
#include <cstdlib>

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 16, kTileK = 32, kTileElems = kTileRows * kTileK;  // 512 bf16 = 1 KiB

// Tile (nt, s) holds W[16 nt + r][32 s + 8 g + e] at element (lane * 8 + e) with lane = 16 g + r: lane (r, g) of a wave reads
// its eight inputs of row r as one 128-bit load, which is the A operand of v_mfma_f32_16x16x32_bf16.  `glu`: the matrix is
// [gate rows; up rows] (N = 2 F) and tile nt holds gate rows 8 nt .. 8 nt + 7 followed by the up rows of the same columns, so
// that a tile's 16 sums are 8 activated outputs.  Rows beyond N are zero.
__global__ __launch_bounds__(256) void pack_tiles_kernel(const uint16_t *__restrict__ w, int64_t w_sn, int N, int K, int glu,
                                                         uint16_t *__restrict__ tiles) {
    const int ksteps = K / kTileK;
    const int64_t piece = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one 16-byte piece per thread
    const int64_t n_pieces = (int64_t)((N + kTileRows - 1) / kTileRows) * ksteps * 64;
    if (piece >= n_pieces) return;
    const int lane = (int)(piece % 64);
    const int64_t tile = piece / 64;
    const int s = (int)(tile % ksteps), nt = (int)(tile / ksteps), r = lane & 15, g = lane >> 4;
    int64_t row;
    if (glu) {
        const int F = N / 2, col = 8 * nt + (r & 7);
        row = col < F ? (r < 8 ? col : F + col) : -1;
    } else {
        row = 16 * nt + r < N ? 16 * nt + r : -1;
    }
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (row >= 0) v = *reinterpret_cast<const uint4 *>(w + row * w_sn + 32 * s + 8 * g);
    reinterpret_cast<uint4 *>(tiles)[piece] = v;
}

// grid: workgroups walk the row tiles blockIdx.x, blockIdx.x + gridDim.x, ...  The NWAVE waves of a workgroup cut K into
// slices of XS k-steps; a wave keeps its slice of x in registers as the B operand (lane (m, g): row m of x, inputs 8 g .. 8 g + 7
// of each k-step), streams its slice of the tile row - XS consecutive KiB - and leaves one 16 x 16 partial per tile row, summed
// across the waves through LDS.
// GLU: SwiGLU behind (tiles packed with `glu`): out [M, F] = bf16(bf16(silu(bf16 gate)) * bf16 up).
// (An RMSNorm in front, as the row-streaming kernel has it, would keep a second copy of the slice alive while it is applied:
// 241 registers at 16 k-steps per wave.  Batches of this size run ha_rmsnorm as a launch of its own.)
// MB: blocks of 16 rows of x (1 or 2): with 17 to 32 rows every weight operand is multiplied twice.
template <int NWAVE, int XS, bool GLU, int MB>
__global__ __launch_bounds__(NWAVE * 64) void tiled_linear_kernel(const uint16_t *__restrict__ x, int64_t x_sm,
                                                                  const uint16_t *__restrict__ tiles,
                                                                  const uint16_t *__restrict__ res, int64_t res_sm,
                                                                  uint16_t *__restrict__ out, int64_t out_sm, int M, int N, int K) {
    constexpr int PF = 4;  // k-steps requested together
    constexpr bool kGlu = GLU;
    static_assert(XS % PF == 0, "a wave's slice is whole groups of k-steps");
    __shared__ float s_c[NWAVE][16][16 * MB + 1];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, m = lane & 15, g = lane >> 4;
    const int ksteps = K / kTileK;
    const int s_beg = wave * XS;  // this wave's k-steps [s_beg, s_beg + XS); those beyond ksteps are zero
    const int n_tiles = kGlu ? (N / 2 + 7) / 8 : (N + kTileRows - 1) / kTileRows;

    auto fetch = [&](int nt, int j0, uint4 (&wv)[PF]) {
        const uint4 *tp = reinterpret_cast<const uint4 *>(tiles) + ((int64_t)nt * ksteps + s_beg + j0) * 64 + lane;
#pragma unroll
        for (int i = 0; i < PF; ++i) {
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (nt < n_tiles && s_beg + j0 + i < ksteps) v = ha_load16_stream(tp + (int64_t)i * 64);
            wv[i] = v;
        }
    };
    uint4 wc[PF], wn[PF];
    int nt = blockIdx.x;
    fetch(nt, 0, wc);  // the first weights are on their way before x is set up

    uint4 xr[MB][XS];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int j = 0; j < XS; ++j) {
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (16 * mb + m < M && s_beg + j < ksteps)
                v = *reinterpret_cast<const uint4 *>(x + (int64_t)(16 * mb + m) * x_sm + (s_beg + j) * kTileK + 8 * g);
            xr[mb][j] = v;
        }

    while (nt < n_tiles) {
        const int nt_next = nt + gridDim.x;
        f32x4 acc[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j0 = 0; j0 < XS; j0 += PF) {
            if (j0 + PF < XS) fetch(nt, j0 + PF, wn);
            else fetch(nt_next, 0, wn);  // nothing is requested past the last tile row
#pragma unroll
            for (int i = 0; i < PF; ++i)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wc[i]),
                                                                      __builtin_bit_cast(bf16x8, xr[mb][j0 + i]), acc[mb], 0, 0, 0);
#pragma unroll
            for (int i = 0; i < PF; ++i) wc[i] = wn[i];
        }
        // acc[mb][i] = sum for tile row 4 g + i and row 16 mb + m of x
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) s_c[wave][4 * g + i][16 * mb + m] = acc[mb][i];
        __syncthreads();
        if constexpr (kGlu) {
            const int F = N / 2;
            for (int t = tid; t < 8 * M; t += NWAVE * 64) {
                const int mm = t >> 3, c = t & 7, col = 8 * nt + c;
                if (col >= F) continue;
                float gt = 0.f, up = 0.f;
#pragma unroll
                for (int wv = 0; wv < NWAVE; ++wv) {
                    gt += s_c[wv][c][mm];
                    up += s_c[wv][8 + c][mm];
                }
                gt = ha_round_bf16(gt);
                const float y = ha_round_bf16(gt / (1.0f + __expf(-gt))) * ha_round_bf16(up);
                out[(int64_t)mm * out_sm + col] = (uint16_t)ha_f32_to_bf16_bits(y);
            }
        } else {
            for (int t = tid; t < 16 * M; t += NWAVE * 64) {
                const int mm = t >> 4, r = t & 15, n = 16 * nt + r;
                if (n >= N) continue;
                float y = 0.f;
#pragma unroll
                for (int wv = 0; wv < NWAVE; ++wv) y += s_c[wv][r][mm];
                if (res) y = ha_round_bf16(y) + ha_bf16_lo((uint32_t)res[(int64_t)mm * res_sm + n]);  // the projection's rounding, then the addition's
                out[(int64_t)mm * out_sm + n] = (uint16_t)ha_f32_to_bf16_bits(y);
            }
        }
        nt = nt_next;
        if (nt < n_tiles) __syncthreads();  // the partials are read: the next tile row may overwrite them
    }
}

// The same product for rows of W too long for x to stay in registers (the down projection: 14336 inputs): every wave requests
// its slices of x next to the weight tiles they meet.  x is then read once per tile row - from L2, it is a few hundred KiB - so
// this form is for matrices of few tile rows per workgroup, where keeping x would not save anything either.  Up to 16 rows of x.
template <int NWAVE>
__global__ __launch_bounds__(NWAVE * 64) void tiled_linear_stream_kernel(const uint16_t *__restrict__ x, int64_t x_sm,
                                                                         const uint16_t *__restrict__ tiles,
                                                                         const uint16_t *__restrict__ res, int64_t res_sm,
                                                                         uint16_t *__restrict__ out, int64_t out_sm, int M, int N, int K) {
    constexpr int PF = 4;
    __shared__ float s_c[NWAVE][16][17];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, m = lane & 15, g = lane >> 4;
    const int ksteps = K / kTileK;
    const int per = ((ksteps + NWAVE - 1) / NWAVE + PF - 1) / PF * PF;  // k-steps per wave, whole groups of PF
    const int s_beg = wave * per, s_end = min(s_beg + per, ksteps);
    const int n_tiles = (N + kTileRows - 1) / kTileRows;
    const uint16_t *xrow = x + (int64_t)min(m, M - 1) * x_sm + 8 * g;
    const bool x_ok = m < M;
    auto fetch = [&](int nt, int s0, uint4 (&wv)[PF], uint4 (&xv)[PF]) {
        const uint4 *tp = reinterpret_cast<const uint4 *>(tiles) + ((int64_t)nt * ksteps + s0) * 64 + lane;
#pragma unroll
        for (int i = 0; i < PF; ++i) {
            const bool ok = nt < n_tiles && s0 + i < s_end;
            uint4 wq = make_uint4(0u, 0u, 0u, 0u), xq = make_uint4(0u, 0u, 0u, 0u);
            if (ok) wq = ha_load16_stream(tp + (int64_t)i * 64);
            if (ok && x_ok) xq = *reinterpret_cast<const uint4 *>(xrow + (int64_t)(s0 + i) * kTileK);
            wv[i] = wq;
            xv[i] = xq;
        }
    };
    uint4 wc[PF], xc[PF], wn[PF], xn[PF];
    int nt = blockIdx.x;
    fetch(nt, s_beg, wc, xc);
    while (nt < n_tiles) {
        const int nt_next = nt + gridDim.x;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int s0 = s_beg; s0 < s_end; s0 += PF) {
            if (s0 + PF < s_end) fetch(nt, s0 + PF, wn, xn);
            else fetch(nt_next, s_beg, wn, xn);
#pragma unroll
            for (int i = 0; i < PF; ++i)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wc[i]), __builtin_bit_cast(bf16x8, xc[i]), acc, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < PF; ++i) {
                wc[i] = wn[i];
                xc[i] = xn[i];
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) s_c[wave][4 * g + i][m] = acc[i];
        __syncthreads();
        for (int t = tid; t < 16 * M; t += NWAVE * 64) {
            const int mm = t >> 4, r = t & 15, n = 16 * nt + r;
            if (n >= N) continue;
            float y = 0.f;
#pragma unroll
            for (int wv = 0; wv < NWAVE; ++wv) y += s_c[wv][r][mm];
            if (res) y = ha_round_bf16(y) + ha_bf16_lo((uint32_t)res[(int64_t)mm * res_sm + n]);  // the projection's rounding, then the addition's
            out[(int64_t)mm * out_sm + n] = (uint16_t)ha_f32_to_bf16_bits(y);
        }
        nt = nt_next;
        if (nt < n_tiles) __syncthreads();
    }
}

}  // namespace

extern "C" {

int64_t ha_weight_tiles_elems(int N, int K, int glu) {
    if (N <= 0 || K <= 0 || K % kTileK != 0 || (glu && N % 2 != 0)) return 0;
    const int64_t n_tiles = glu ? (N / 2 + 7) / 8 : (N + kTileRows - 1) / kTileRows;
    return n_tiles * (K / kTileK) * kTileElems;
}

int ha_pack_weight_tiles(const void *w, int64_t w_stride_n, int N, int K, int glu, void *tiles, void *stream) {
    HA_REQUIRE(w && tiles, HA_ERR_NULL_POINTER, "w/tiles is NULL");
    HA_REQUIRE(N > 0 && K > 0 && K % kTileK == 0 && w_stride_n >= K && (glu == 0 || (glu == 1 && N % 2 == 0)), HA_ERR_BAD_SHAPE,
               "need N > 0, K a multiple of 32, an even N for the gate/up form");
    HA_REQUIRE(ha_aligned(w, 16) && ha_aligned(tiles, 16) && w_stride_n % 8 == 0, HA_ERR_MISALIGNED, "w rows and tiles must be 16-byte aligned");
    int st = ha_require_device();
    if (st) return st;
    const int64_t pieces = ha_weight_tiles_elems(N, K, glu) / 8;
    HA_REQUIRE((pieces + 255) / 256 <= 2147483647LL, HA_ERR_BAD_SHAPE, "matrix too large for one launch");
    hipLaunchKernelGGL(pack_tiles_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, (hipStream_t)stream, (const uint16_t *)w,
                       w_stride_n, N, K, glu, (uint16_t *)tiles);
    HA_CHECK_LAUNCH("pack_tiles_kernel");
    return HA_OK;
}

int ha_linear_tiled(const void *x, int64_t x_stride_m, const void *tiles, const void *residual, int64_t residual_stride_m, int act,
                    void *out, int64_t out_stride_m, int M, int N, int K, void *stream) {
    HA_REQUIRE(x && tiles && out, HA_ERR_NULL_POINTER, "x/tiles/out is NULL");
    HA_REQUIRE(M >= 1 && M <= 32 && N >= 1 && K >= 32 && K % kTileK == 0, HA_ERR_BAD_SHAPE, "need 1 <= M <= 32, N >= 1, K a multiple of 32");
    HA_REQUIRE(act == 0 || act == 1, HA_ERR_BAD_SHAPE, "unknown activation %d", act);
    // longer rows than a workgroup keeps of x in registers: the form that requests x next to the tiles (16 rows, no activation)
    const bool stream_x = K > (M <= 16 ? 8192 : 4096);
    HA_REQUIRE(!stream_x || (M <= 16 && !act), HA_ERR_BAD_SHAPE,
               "K=%d: x stays in registers up to 8192 inputs of 16 rows or 4096 of 32; longer rows take up to 16 rows of x and no activation", K);
    const int n_out = act ? N / 2 : N;
    HA_REQUIRE(!act || (N % 2 == 0 && !residual), HA_ERR_BAD_SHAPE, "SwiGLU needs an even number of weight rows and no residual");
    HA_REQUIRE(x_stride_m >= K && out_stride_m >= n_out && (!residual || residual_stride_m >= N), HA_ERR_BAD_SHAPE,
               "strides smaller than the rows they span");
    HA_REQUIRE(ha_aligned(x, 16) && ha_aligned(tiles, 16) && x_stride_m % 8 == 0, HA_ERR_MISALIGNED,
               "x rows and tiles must be 16-byte aligned");
    int st = ha_require_device();
    if (st) return st;
    const int ksteps = K / kTileK;
    const int n_tiles = act ? (N / 2 + 7) / 8 : (N + kTileRows - 1) / kTileRows;
    // One workgroup per CU, walking the tile rows: with two 512-thread workgroups resident per CU, grids between 256 and 512
    // leave some CUs twice the rows of others (QKV 6144 x 4096, 16 rows of x: 384 workgroups 15.4 us, 192 or 256 13.1 us;
    // gate/up 28672 x 4096: 512 workgroups 41.3 us, 256 40.7 us, 1792 47.4 us)
    int grid = n_tiles < 256 ? n_tiles : 256;
#ifdef HASHATTN_TUNING_ENV
    if (const char *e = getenv("HA_TILED_GRID")) grid = atoi(e) < n_tiles ? atoi(e) : n_tiles;
#endif
    const uint16_t *xp = (const uint16_t *)x, *tp = (const uint16_t *)tiles, *rp = (const uint16_t *)residual;
    uint16_t *op = (uint16_t *)out;
    hipStream_t s = (hipStream_t)stream;
    if (stream_x) {
        hipLaunchKernelGGL(tiled_linear_stream_kernel<16>, dim3(grid), dim3(1024), 0, s, xp, x_stride_m, tp, rp, residual_stride_m, op,
                           out_stride_m, M, N, K);
        HA_CHECK_LAUNCH("tiled_linear_stream_kernel");
        return HA_OK;
    }
#define HA_TILED_LAUNCH(NW_, XS_, G_, MB_)                                                                                    \
    hipLaunchKernelGGL((tiled_linear_kernel<NW_, XS_, G_, MB_>), dim3(grid), dim3(NW_ * 64), 0, s, xp, x_stride_m, tp, rp,    \
                       residual_stride_m, op, out_stride_m, M, N, K)
#define HA_TILED_FUSE(NW_, XS_, MB_)                   \
    do {                                               \
        if (act) HA_TILED_LAUNCH(NW_, XS_, true, MB_); \
        else HA_TILED_LAUNCH(NW_, XS_, false, MB_);    \
    } while (0)
    if (M <= 16) {
        if (ksteps <= 32) HA_TILED_FUSE(8, 4, 1);
        else if (ksteps <= 64) HA_TILED_FUSE(8, 8, 1);
        else if (ksteps <= 128) HA_TILED_FUSE(8, 16, 1);
        else HA_TILED_FUSE(16, 16, 1);
    } else {  // 17 to 32 rows: twice the registers per k-step
        if (ksteps <= 32) HA_TILED_FUSE(8, 4, 2);
        else if (ksteps <= 64) HA_TILED_FUSE(8, 8, 2);
        else HA_TILED_FUSE(16, 8, 2);
    }
#undef HA_TILED_FUSE
#undef HA_TILED_LAUNCH
    HA_CHECK_LAUNCH("tiled_linear_kernel");
    return HA_OK;
}

}  // extern "C"

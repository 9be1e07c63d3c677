// Products of 17 to 64 rows of x with a matrix packed for the matrix cores (pack_for_mfma):
// out[M, N] = x[M, K] . w[N, K]^T, bfloat16 in, float32 sums.
//
// At this many rows the weights are still the traffic from memory (a step of 64 sequences reads every
// weight once for 64 tokens), but every kilobyte of them meets RT kilobytes of x (RT tiles of 16 rows).  A
// wavefront that fetches those for itself from the L2 cache asks that cache for four times what memory
// delivers.  Here the W wavefronts of a workgroup (three or four) work on W neighbouring row tiles of the
// matrix over the same stretch of K and share the tiles of x through LDS: a slice of WD_SLICE steps (of 32 k) is copied
// in once for all of them, in two buffers that take turns, so that there is one barrier a slice and the
// copy of the next slice is in registers while this one is multiplied.  A wavefront keeps WD_SLICE weight
// fragments in flight as a ring: a register asks for its step of the next slice as soon as the matrix
// cores have taken the one it held.
//
// A compute unit streams from memory at a rate of its own (about 30 GB/s here, an eighth of a thousandth of
// the machine's), so the product is as fast as the fullest compute unit: the workgroups should be a multiple
// of the compute units, all alike.  Three wavefronts instead of four do that for a matrix whose row tiles are
// a multiple of three times the compute units (768 pairs of gate|up tiles: 256 workgroups of three, where
// groups of four make 192 and leave a quarter of the machine idle), five to eight for gate|up matrices of more
// than four pairs of row tiles a compute unit.  A matrix of a few thousand rows has too
// few groups of row tiles to give every compute unit work, so K is cut into `parts` stretches (blockIdx.y) whose float32 sums go to out[part][M][N] for a reader
// that adds them in order (the residual stream's norm, or ri_sum_parts below).  A row's result does not
// depend on the number of rows: rows beyond M are zero columns, every tile of x has accumulators of its own.
//
// 65 to 128 rows (PAIR): five to eight tiles of x, and every wavefront takes two neighbouring row tiles of the
// matrix, so that a fragment of x read from LDS meets two weight fragments (with one, the LDS reads of eight tiles
// of x for every kilobyte of weights come close to what LDS delivers) and a workgroup's copy of x serves twice the
// weights.  A slice of x is then up to 64 KB and the two buffers all of a compute unit's LDS that one workgroup
// may have: one workgroup a compute unit, K in stretches, float32 sums for a reader that adds them.
#include "api.h"
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

union FragW {
    bf16x8 v;
    uint4 u;
};

#define WD_SLICE 8        // MFMA steps (of 32 k) per slice of x in LDS

__device__ __forceinline__ float silu_wd(float z) { return z / (1.0f + expf(-z)); }

// W: wavefronts of a workgroup, one row tile of the matrix each (with SWIGLU a gate tile and its up tile, with
// PAIR two neighbouring tiles)
template <int RT, bool SWIGLU, typename TO, int NS, int W, bool PAIR = false>
__global__ void __launch_bounds__(W * 64)
gemm_wide_packed_kernel(TO* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ wpacked, int M,
                        int N, int K, int k_tiles, int part_tiles, int row_tiles, int tiled, long part_stride) {
    constexpr int FRAGS = RT * WD_SLICE;                     // fragments of x (64 pieces of 16 bytes) in a slice
    constexpr int PER_THREAD = (FRAGS + W - 1) / W;          // of which a wavefront copies this many
    __shared__ uint4 xs[2][RT][WD_SLICE][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    static_assert(!(SWIGLU && PAIR), "the second stream of weights is the up tile or the next row tile");
    constexpr bool TWO = SWIGLU || PAIR;
    const int nt = (blockIdx.x * W + wave) * (PAIR ? 2 : 1);
    const bool live_tile = nt < row_tiles;                    // past the edge: works on tile 0 again and stores nothing
    const int kt_begin = blockIdx.y * part_tiles, kt_end = min(k_tiles, kt_begin + part_tiles);
    const int slices = (kt_end - kt_begin + WD_SLICE - 1) / WD_SLICE;
    const int ntc = live_tile ? nt : 0;
    const bf16_t* wp = wpacked + ((size_t)ntc * k_tiles * 64 + lane) * 8;
    // the second stream: the up tile of the pair, or the next row tile (past the edge: this one again, not stored)
    const int nt2 = SWIGLU ? row_tiles + ntc : min(ntc + 1, row_tiles - 1);
    const bf16_t* up = TWO ? wpacked + ((size_t)nt2 * k_tiles * 64 + lane) * 8 : nullptr;
    const bool x_tiled = tiled & TILED_X;
    const int jg = lane >> 4;

    // Every load below is issued whatever the indices are: what lies outside x is read from a kilobyte of zeros
    // instead, and weights past the stretch's end (pulled back to its last tile) meet a slice of x that is zero
    // there.  A load inside a branch would end the pipelining: the compiler cannot
    // count the loads in flight across a branch that may not have issued one, and waits for all of them.
    // piece j of this thread's share of a slice: (tile of x, step) = q / WD_SLICE, q % WD_SLICE with
    // q = wave + j * W; the 64 lanes of a wavefront copy one fragment (64 x 16 bytes).  Where the fragments do
    // not divide among the wavefronts, the last one is copied twice (the same values to the same place).
    auto fetch = [&](int j, int slice) -> uint4 {
        const int q = min(wave + j * W, FRAGS - 1);
        const int step = q % WD_SLICE, rt = q / WD_SLICE;
        const int row = rt * 16 + (lane & 15);
        const int kt = kt_begin + slice * WD_SLICE + step;
        const int ktc = min(kt, k_tiles - 1);
        // rows beyond M and columns beyond K are zero (the packed matrix is zero beyond K too)
        const bool ok = row < M && kt < kt_end && kt * 32 + jg * 8 < K;
        const bf16_t* p = x_tiled ? x + (((size_t)rt * k_tiles + ktc) * 64 + lane) * 8
                                  : x + (size_t)min(row, M - 1) * K + min(ktc * 32 + jg * 8, K - 8);
        return *reinterpret_cast<const uint4*>(ok ? p : ri_zero_fragment + lane * 8);
    };
    auto stash = [&](int j, int buf, const uint4& v) {
        const int q = min(wave + j * W, FRAGS - 1);
        xs[buf][q / WD_SLICE][q % WD_SLICE][lane] = v;
    };

    floatx4 acc[RT], accu[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) acc[rt] = accu[rt] = floatx4{0.f, 0.f, 0.f, 0.f};

    // the weights of the first NS slices are asked for before anything else: a ring of NS * WD_SLICE registers
    const int kt_last = kt_end - 1;
    FragW wf[NS][WD_SLICE], uf[NS][WD_SLICE];
#pragma unroll
    for (int ss = 0; ss < NS; ++ss)
#pragma unroll
        for (int c = 0; c < WD_SLICE; ++c) {
            const int kt = min(kt_begin + ss * WD_SLICE + c, kt_last);
            wf[ss][c].u = load_stream16(wp + (size_t)kt * 512);
            if (TWO) uf[ss][c].u = load_stream16(up + (size_t)kt * 512);
        }
    uint4 stage[PER_THREAD];
#pragma unroll
    for (int j = 0; j < PER_THREAD; ++j) stage[j] = fetch(j, 0);
#pragma unroll
    for (int j = 0; j < PER_THREAD; ++j) stash(j, 0, stage[j]);
    __syncthreads();

    // (the number of slices is rounded up to a multiple of NS: a slice past the end is zeros of x against the
    // stretch's last weights again)
    const int rounds = (slices + NS - 1) / NS;
    for (int round = 0; round < rounds; ++round) {
#pragma unroll
        for (int ss = 0; ss < NS; ++ss) {
            const int s = round * NS + ss;
            const int buf = s & 1;
#pragma unroll
            for (int j = 0; j < PER_THREAD; ++j) stage[j] = fetch(j, s + 1);   // past the last slice: zeros
            const int kt0 = kt_begin + s * WD_SLICE;
#pragma unroll
            for (int c = 0; c < WD_SLICE; ++c) {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    FragW xf;
                    xf.u = xs[buf][rt][c][lane];
                    acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[ss][c].v, xf.v, acc[rt], 0, 0, 0);
                    if (TWO) accu[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[ss][c].v, xf.v, accu[rt], 0, 0, 0);
                }
                // this register's step NS slices on (past the end: the stretch's last tile again, which then
                // meets zeros of x)
                const int next = min(kt0 + NS * WD_SLICE + c, kt_last);
                wf[ss][c].u = load_stream16(wp + (size_t)next * 512);
                if (TWO) uf[ss][c].u = load_stream16(up + (size_t)next * 512);
            }
#pragma unroll
            for (int j = 0; j < PER_THREAD; ++j) stash(j, buf ^ 1, stage[j]);
            __syncthreads();       // the next slice is in place; this one may be overwritten after the next
        }
    }

    if (!live_tile) return;
    // D[row n, column m] of a tile: register r of lane l holds n = 4 * (l / 16) + r, m = l % 16.
    // A product in parts stores its sums as they are; with the activation still to come, the gate sums fill
    // columns 0..N-1 and the up sums N..2N-1 of rows 2 N wide.
    const bool raw = gridDim.y > 1;
    const int width = (SWIGLU && raw) ? 2 * N : N;
    out += (size_t)blockIdx.y * part_stride;          // (M * width, or more where the rows are a slice of a taller result)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int m = rt * 16 + (lane & 15);
        if (m >= M) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int n = nt * 16 + 4 * jg + r;
            if (n >= N) continue;
            if (PAIR) {                                      // the sums of both row tiles as they are
                from_f32(out + (size_t)m * width + n, acc[rt][r]);
                if (n + 16 < N) from_f32(out + (size_t)m * width + n + 16, accu[rt][r]);
                continue;
            }
            if (SWIGLU && raw) {
                from_f32(out + (size_t)m * width + n, acc[rt][r]);
                from_f32(out + (size_t)m * width + N + n, accu[rt][r]);
                continue;
            }
            const float v = SWIGLU ? silu_wd(acc[rt][r]) * accu[rt][r] : acc[rt][r];
            from_f32(out + ((tiled & TILED_OUT) ? tiled_at(m, n, (N + 31) / 32) : (size_t)m * N + n), v);
        }
    }
}

// How many wavefronts a workgroup has (row tiles it takes) and into how many stretches K is cut: of three and
// four wavefronts the choice whose workgroups fill the compute units more evenly (four on a tie), with K cut
// until every compute unit has a workgroup, whole slices each, and not at all with the activation (its parts
// would have to be added by a kernel of their own).
// (Measured on 4096 x 12288 at 64 rows with four wavefronts: 66, 38, 26 and 26 us with 1, 2, 4 and 8 stretches;
// every stretch more is another float32 copy of the result for the reader to add.)
static int wide_parts(int groups, int k_tiles, bool swiglu, int cus) {
    int parts = 1;
    while (!swiglu && parts < 16 && groups * parts < cus && k_tiles / (parts * 2) >= 2 * WD_SLICE) parts *= 2;
    return parts;
}

extern "C" int ri_gemm_wide_packed_bf16_plan(int n, int k, int swiglu, int* waves, int* parts) {
    const int row_tiles = (n + 15) / 16, k_tiles = (k + 31) / 32;
    const int cus = ri_compute_units();
    if (swiglu && row_tiles > 4 * cus && row_tiles <= 8 * cus) {
        // With the activation K stays whole, and pairs of row tiles for more than four wavefronts a compute unit
        // would be a second round on some of them (groups of three or four: two workgroups on some compute units,
        // one on others, and the product takes what the fuller ones take).  Up to eight wavefronts a workgroup
        // bring the groups within the compute units' number again: 1,088 pairs (17408 x 5120) in 218 groups of
        // five take 61 to 71 us at 24 to 64 rows where 363 groups of three take 74 to 93; 1,600 pairs (25600 x
        // 5120) in 229 groups of seven 87 to 95 us where 400 groups of four take 97 to 113.
        *waves = (row_tiles + cus - 1) / cus;
        *parts = 1;
        return 0;
    }
    double best = -1.0;
    for (int w = 4; w >= 3; --w) {
        const int groups = (row_tiles + w - 1) / w;
        const int p = wide_parts(groups, k_tiles, swiglu != 0, cus);
        const long wgs = (long)groups * p;
        const double fill = (double)wgs / (double)((wgs + cus - 1) / cus * cus);
        if (fill > best + 1e-9) {
            best = fill;
            *waves = w;
            *parts = p;
        }
    }
    return 0;
}

// The plan for a product without the activation by the rows of x too.  Up to 16 rows it is the one above: x is
// small, and twice the workgroups, two to a compute unit, keep more loads in flight.  From 17 rows on a
// workgroup's copy of x weighs as much as its weights, and the product is about as fast as a compute unit fetches
// its workgroups' bytes (some 30 GB/s, from memory or from the L2 cache alike): the rows of x and the weight rows
// over one stretch, and its share of the float32 stretches that are written here and read again by whoever adds
// them.  K is cut only while the workgroups stay within the compute units' number (65 to 128 rows, two row tiles
// a wavefront: a compute unit holds one workgroup then, its two buffers of x are most of the LDS, and more are a
// second round; 4096 x 12288 at 96 rows takes 33 us in 8 stretches, 256 workgroups, 45 in 4 and 44 in 16; at 64
// rows 26.5 us in 4 stretches and 29 in 8).  Of three and four wavefronts and every number of stretches, a power
// of two or not, the plan takes the one with the fewest bytes.  5120 x 17408 at 64 rows: 80 groups of four
// wavefronts in 3 stretches 43 us, 107 groups of three in 4 stretches, what the plan above says, 56; 2560 x 9728:
// 40 groups in 6 stretches 17 us, 54 in 8 stretches 21.5; at 128 rows 5120 x 17408 as 40 groups in 6 stretches 66 us,
// as 54 in 4 stretches 88.  At 4 and 16 rows the same choice makes a decode step at Qwen3-14B and 32B sizes 1.3 to
// 2.6% longer.
// (Eight wavefronts, 256 weight rows to a copy of x, were timed too at 65 to 128 rows: 4 to 6% ahead at 128 rows of
// x on the matrices of many long rows, 5120 x 17408 and x 25600 in 12 stretches, 5 to 8% behind at 80 rows, and 13%
// behind on 4096 x 12288, whose stretches get short.)
extern "C" int ri_gemm_wide_stretch_plan(int m, int n, int k, int* waves, int* parts) {
    if (m <= 16) return ri_gemm_wide_packed_bf16_plan(n, k, 0, waves, parts);
    if (m > 128) {                                            // two passes: the plan for the taller one
        const int tiles = (m + 15) / 16, passes = (tiles + 7) / 8;
        m = (tiles + passes - 1) / passes * 16;
    }
    const int row_tiles = (n + 15) / 16, k_tiles = (k + 31) / 32;
    const int cus = ri_compute_units();
    const int x_rows = (m + 15) / 16 * 16;
    double best = -1.0;
    *waves = 4;
    *parts = 1;
    const int tiles_a_wave = m > 64 ? 2 : 1;
    for (int w = 4; w >= 3; --w) {
        const int groups = (row_tiles + tiles_a_wave * w - 1) / (tiles_a_wave * w);
        const int most = max(1, min(16, cus / groups));
        const long rounds = (groups + cus - 1) / cus;                   // (more than one only where K stays whole)
        for (int p = 1; p <= most; ++p) {
            const int stretch = ((k_tiles + p - 1) / p + WD_SLICE - 1) / WD_SLICE * WD_SLICE;
            if (p > 1 && stretch < 2 * WD_SLICE) break;
            const int used = (k_tiles + stretch - 1) / stretch;          // stretches that hold any of K
            if (used != p) continue;
            const double bytes = (double)rounds * (x_rows + 16 * tiles_a_wave * w) * stretch * 64.0 +
                                 (double)used * m * n * 8.0 / cus;
            if (best < 0 || bytes < best * (1.0 - 1e-9)) {
                best = bytes;
                *waves = w;
                *parts = used;
            }
        }
    }
    return 0;
}

template <int RT, int W>
static void launch_wide_pairs(float* out, const bf16_t* x, const bf16_t* w, int m, int n, int k, int parts, long part_stride,
                              hipStream_t s) {
    const int k_tiles = (k + 31) / 32, row_tiles = (n + 15) / 16;
    const int part_tiles = ((k_tiles + parts - 1) / parts + WD_SLICE - 1) / WD_SLICE * WD_SLICE;
    dim3 grid((row_tiles + 2 * W - 1) / (2 * W), parts);
    gemm_wide_packed_kernel<RT, false, float, 1, W, true><<<grid, W * 64, 0, s>>>(out, x, w, m, n, k, k_tiles, part_tiles,
                                                                                 row_tiles, 0, part_stride);
}

template <int RT, bool SWIGLU, int NS, int W>
static void launch_wide(void* out, int out_dtype, const bf16_t* x, const bf16_t* w, int m, int n, int k, int parts,
                        int tiled, hipStream_t s) {
    const int k_tiles = (k + 31) / 32, row_tiles = (n + 15) / 16;
    const int part_tiles = ((k_tiles + parts - 1) / parts + WD_SLICE - 1) / WD_SLICE * WD_SLICE;
    dim3 grid((row_tiles + W - 1) / W, parts);
    if (out_dtype == RI_F32)
        gemm_wide_packed_kernel<RT, SWIGLU, float, NS, W><<<grid, W * 64, 0, s>>>(
            (float*)out, x, w, m, n, k, k_tiles, part_tiles, row_tiles, tiled, (long)m * (SWIGLU && parts > 1 ? 2 * n : n));
    else
        gemm_wide_packed_kernel<RT, SWIGLU, bf16_t, NS, W><<<grid, W * 64, 0, s>>>(
            (bf16_t*)out, x, w, m, n, k, k_tiles, part_tiles, row_tiles, tiled, (long)m * n);
}

// depth: slices of weights a wavefront keeps in flight (1 or 2); waves: wavefronts (row tiles) a workgroup (3 or 4;
// with the activation and depth 1 up to 8).
// (Eight wavefronts on eight row tiles, with K in twice the stretches so that the workgroups stay as many and each
// fetches half the rows of x, were timed at 17 to 64 rows: at 4096 x 4096 and 4096 x 12288 level or behind, 14.1
// against 13.6 us and 24.8 against 24.2 us at 64 rows, and the reading norm then adds twice the stretches.)
extern "C" int ri_gemm_wide_packed_bf16(void* out, int out_dtype, const void* x, const void* wpacked, int m, int n,
                                        int k, int swiglu, int parts, int tiled, int depth, int waves, void* stream) {
    RI_REQUIRE(m > 0 && m <= 256, "gemm_wide_packed_bf16: %d rows of x, this kernel takes 1 to 256", m);
    if (m > 64 && m <= 128 && swiglu) {
        // 65 to 128 rows with the activation, for the matrices that take five to eight wavefronts a workgroup: five to
        // eight tiles of x, K whole, a gate tile and its up tile a wavefront (17408 x 5120 pairs at 65 / 96 / 128 rows:
        // 76 / 88 / 98 us against the library's and its activation kernel's 102 / 103 / 108; 25600 x 5120: 95 / 103 / 121
        // against 113 / 116 / 125; with three or four wavefronts, 12288 x 4096 and 9728 x 2560, it is ahead up to 80
        // rows only, 54 and 32 us against 56 to 58 and 34, and loses beyond: 74 and 50 against 57 and 35 at 128)
        RI_REQUIRE(depth == 1 && parts == 1 && !tiled && waves >= 5 && waves <= 8,
                   "gemm_wide_packed_bf16: %d rows with the activation: depth 1, K whole, plain rows, 5 to 8 wavefronts", m);
        hipStream_t s2 = (hipStream_t)stream;
        const bf16_t* xb2 = (const bf16_t*)x;
        const bf16_t* wb2 = (const bf16_t*)wpacked;
#define RI_WIDE_TALL_W(RT, W) launch_wide<RT, true, 1, W>(out, out_dtype, xb2, wb2, m, n, k, 1, 0, s2)
#define RI_WIDE_TALL(RT)                                                                           \
    do {                                                                                           \
        switch (waves) {                                                                           \
            case 5: RI_WIDE_TALL_W(RT, 5); break;                                                  \
            case 6: RI_WIDE_TALL_W(RT, 6); break;                                                  \
            case 7: RI_WIDE_TALL_W(RT, 7); break;                                                  \
            default: RI_WIDE_TALL_W(RT, 8); break;                                                 \
        }                                                                                          \
    } while (0)
        if (m <= 80) RI_WIDE_TALL(5); else if (m <= 96) RI_WIDE_TALL(6); else if (m <= 112) RI_WIDE_TALL(7); else RI_WIDE_TALL(8);
#undef RI_WIDE_TALL
#undef RI_WIDE_TALL_W
        RI_LAUNCH_CHECK("gemm_wide_packed_bf16");
        return 0;
    }
    RI_REQUIRE(m <= 64 || (!swiglu && out_dtype == RI_F32 && !tiled && depth == 1),
               "gemm_wide_packed_bf16: %d rows of x: more than 64 give float32 sums in plain rows from plain rows, "
               "without the activation, one slice of weights in flight", m);
    RI_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_wide_packed_bf16: n %d, k %d (k must be a multiple of 8)", n, k);
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "gemm_wide_packed_bf16: out dtype %d", out_dtype);
    RI_REQUIRE(parts >= 1 && parts <= 64 && (parts == 1 || out_dtype == RI_F32),
               "gemm_wide_packed_bf16: %d parts of K (more than one needs float32 sums)", parts);
    RI_REQUIRE(!(tiled & ~(TILED_X | TILED_OUT)) && (!(tiled & TILED_OUT) || (out_dtype == RI_BF16 && parts == 1)),
               "gemm_wide_packed_bf16: layout flags %d (a tiled result is bfloat16 and whole)", tiled);
    RI_REQUIRE(depth == 1 || depth == 2, "gemm_wide_packed_bf16: depth %d", depth);
    RI_REQUIRE(waves == 3 || waves == 4 || (waves >= 5 && waves <= 8 && swiglu && depth == 1 && m <= 64),
               "gemm_wide_packed_bf16: %d wavefronts a workgroup (3 or 4; 5 to 8 too with the activation at depth 1)", waves);
    hipStream_t s = (hipStream_t)stream;
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)wpacked;
#define RI_WIDE_GO(RT, SG, NS)                                                                       \
    do {                                                                                             \
        if (waves == 3) launch_wide<RT, SG, NS, 3>(out, out_dtype, xb, wb, m, n, k, parts, tiled, s); \
        else            launch_wide<RT, SG, NS, 4>(out, out_dtype, xb, wb, m, n, k, parts, tiled, s); \
    } while (0)
#define RI_WIDE_CASE(RT)                                                                  \
    if (swiglu) { if (depth == 2) RI_WIDE_GO(RT, true, 2); else RI_WIDE_GO(RT, true, 1); } \
    else        { if (depth == 2) RI_WIDE_GO(RT, false, 2); else RI_WIDE_GO(RT, false, 1); }
#define RI_WIDE_PAIRS(RT)                                                                                  \
    do {                                                                                                    \
        if (waves == 3) launch_wide_pairs<RT, 3>(po, px, wb, rows, n, k, parts, (long)m * n, s);            \
        else            launch_wide_pairs<RT, 4>(po, px, wb, rows, n, k, parts, (long)m * n, s);            \
    } while (0)
#define RI_WIDE_MANY(RT)                                                                                     \
    do {                                                                                                     \
        if (waves == 5)      launch_wide<RT, true, 1, 5>(out, out_dtype, xb, wb, m, n, k, parts, tiled, s);  \
        else if (waves == 6) launch_wide<RT, true, 1, 6>(out, out_dtype, xb, wb, m, n, k, parts, tiled, s);  \
        else if (waves == 7) launch_wide<RT, true, 1, 7>(out, out_dtype, xb, wb, m, n, k, parts, tiled, s);  \
        else                 launch_wide<RT, true, 1, 8>(out, out_dtype, xb, wb, m, n, k, parts, tiled, s);  \
    } while (0)
    if (waves > 4) {
        if (m <= 16)      RI_WIDE_MANY(1);
        else if (m <= 32) RI_WIDE_MANY(2);
        else if (m <= 48) RI_WIDE_MANY(3);
        else              RI_WIDE_MANY(4);
    }
    else if (m <= 16)  { RI_WIDE_CASE(1) }
    else if (m <= 32)  { RI_WIDE_CASE(2) }
    else if (m <= 48)  { RI_WIDE_CASE(3) }
    else if (m <= 64)  { RI_WIDE_CASE(4) }
    else {
        // 65 to 128 rows in one pass, up to 256 in two of as many tiles of 16 rows each as can be (the second may
        // have one less): each pass reads the weights once and writes its rows of every stretch's float32 sums
        const int tiles = (m + 15) / 16, passes = (tiles + 7) / 8;
        int r0 = 0;
        for (int pass = 0; pass < passes; ++pass) {
            const int pass_tiles = tiles / passes + (pass < tiles % passes ? 1 : 0);
            const int rows = min(pass_tiles * 16, m - r0);
            float* po = (float*)out + (size_t)r0 * n;
            const bf16_t* px = xb + (size_t)r0 * k;
            switch (pass_tiles) {
                case 4: RI_WIDE_PAIRS(4); break;
                case 5: RI_WIDE_PAIRS(5); break;
                case 6: RI_WIDE_PAIRS(6); break;
                case 7: RI_WIDE_PAIRS(7); break;
                default: RI_WIDE_PAIRS(8); break;
            }
            r0 += rows;
        }
    }
#undef RI_WIDE_PAIRS
#undef RI_WIDE_MANY
#undef RI_WIDE_CASE
#undef RI_WIDE_GO
    RI_LAUNCH_CHECK("gemm_wide_packed_bf16");
    return 0;
}

// ------------------------------------------------------------------ adding the parts of a split product
// out[m, i] = sum over p, in order, of parts[p][m][i], for a reader that cannot add them itself; with swiglu the
// rows of the parts are gate sums then up sums (2 x width) and out[m, i] = silu(sum gate) * (sum up).
template <typename TO>
__global__ void sum_parts_kernel(TO* __restrict__ out, const float* __restrict__ parts, int n_parts, long part_stride,
                                 int width, int swiglu, int tiled, long total) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const int m = (int)(e / width), i = (int)(e - (long)m * width);
    const float* p = parts + (long)m * (swiglu ? 2 * width : width) + i;
    float g = 0.f, u = 0.f;
    for (int q = 0; q < n_parts; ++q) {
        g += p[q * part_stride];
        if (swiglu) u += p[q * part_stride + width];
    }
    from_f32(out + (tiled ? tiled_at(m, i, (width + 31) / 32) : e), swiglu ? silu_wd(g) * u : g);
}

extern "C" int ri_sum_parts(void* out, int out_dtype, const float* parts, int n_parts, int rows, int width, int swiglu,
                            int tiled, void* stream) {
    RI_REQUIRE(n_parts > 0 && rows > 0 && width > 0, "sum_parts: %d parts of %d x %d", n_parts, rows, width);
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "sum_parts: out dtype %d", out_dtype);
    RI_REQUIRE(!tiled || (out_dtype == RI_BF16 && rows <= 64), "sum_parts: a tiled result is bfloat16 and at most 64 rows");
    const long total = (long)rows * width;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    const long stride = total * (swiglu ? 2 : 1);
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == RI_F32)
        sum_parts_kernel<float><<<blocks, 256, 0, s>>>((float*)out, parts, n_parts, stride, width, swiglu, tiled, total);
    else
        sum_parts_kernel<bf16_t><<<blocks, 256, 0, s>>>((bf16_t*)out, parts, n_parts, stride, width, swiglu, tiled, total);
    RI_LAUNCH_CHECK("sum_parts");
    return 0;
}

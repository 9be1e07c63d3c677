// Decode-size products on the matrix cores: out[M, N] = x[M, K] . w[N, K]^T for bfloat16 with up to
// 16 rows of x per tile of MFMA 16x16x32 columns.  The weights are the traffic and are read once:
// a workgroup of four or eight wavefronts owns 16 rows of w, each wavefront its share of K; the weight
// fragments go from global memory straight into the A operand (lane l: row l % 16, eight
// consecutive k at 8 * (l / 16)), the rows of x into the B operand the same way (they come from
// the L2 cache), and the partial sums are added through LDS in wavefront order.  Rows of x
// beyond M are zero columns, so a row's result does not depend on how many rows there are.
// Optional SwiGLU epilogue for the fused gate|up matrix: out = silu(x . gate^T) * (x . up^T).
// The weights are packed for the matrix cores ahead of time: the matrix is cut into tiles of 16 rows by
// 32 k, each tile stored as the 1 KB that one MFMA A operand is (lane l's 16 bytes: row l % 16,
// k 8 * (l / 16) ..+8), tiles of one row block consecutive in k.  A wavefront's loads are then whole
// contiguous kilobytes, which is what the memory system streams fastest.
// packed: [row_tiles][k_tiles][64 lanes][8]; for SwiGLU the up matrix's tiles follow the gate's.
#include "api.h"
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

union Frag {
    bf16x8 v;
    uint4 u;
};

// MFMA steps (of 32 k) whose loads are in flight together.  Measured on the decode products of three model
// sizes: 4 steps are 2 to 10% slower than 8 (more wavefronts fit, but each has half the bytes under way),
// and two sets of 4 that take turns, one loading while the other multiplies, 1 to 5% slower; 16 steps, with
// the ring below keeping all of them in flight, 0.5% slower at Qwen3-8B sizes, and eight wavefronts instead
// of four on the matrices of 4,096 and 6,144 rows no faster either.
#define SK_CHUNK 8

__device__ __forceinline__ float silu_sk(float z) { return z / (1.0f + expf(-z)); }

#define SK_ROWS (16 / SK_WAVES)   // rows of x whose sums of squares one wavefront adds up
#define SK_PRE 4                  // partial sums of squares a lane fetches ahead of the weights

// A wavefront's sum over its share of K is kept in two halves, the steps of the same parity as its first one
// and the others, each added up in order and the two added at the end.  That makes two chains of matrix
// instructions that do not wait for one another, and it is the order in which PAIRED gets its sums:
// PAIRED (up to 8 rows of x, the ring's conditions): a lane's piece of x is a row's 8 elements of one step for
// lanes 0-7 of every 16 and of the next step for lanes 8-15, so one load of x serves two steps of K (the rows
// of x that a workgroup pulls from the L2 cache count against what its compute unit can pull like the weights
// do).  The fragment goes through the matrix cores with either step's weights: columns 0-7 of the first
// product and columns 8-15 of the second are the rows' sums over the even and over the odd steps, the other
// columns pair one step's weights with the other step's x and are dropped.  The same bits as without.
template <int SK_WAVES, bool SWIGLU, typename TO, bool PAIRED>
__global__ void __launch_bounds__(SK_WAVES * 64)
gemm_skinny_packed_kernel(TO* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ wpacked,
                          int M, int N, int K, int k_tiles, int tiles_per_wave, int up_tile_offset, NormLink link, int tiled) {
    __shared__ float red[SWIGLU ? 2 : 1][PAIRED ? 2 : 1][SK_WAVES][4][64];
    __shared__ float inv_lds[16];
    __shared__ float sq_lds[16][17];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, jg = lane >> 4;
    const int nt = blockIdx.x;
    const bool x_ok = i < M;
    // blockIdx.y cuts K into gridDim.y parts whose sums go to separate outputs out[part][M][N]
    const int part_tiles = (k_tiles + gridDim.y - 1) / gridDim.y;
    const int part_begin = blockIdx.y * part_tiles, part_end = min(k_tiles, part_begin + part_tiles);
    const int kt_begin = part_begin + wave * tiles_per_wave, kt_end = min(part_end, kt_begin + tiles_per_wave);
    out += (size_t)blockIdx.y * M * N;
    const bf16_t* wp = wpacked + ((size_t)nt * k_tiles * 64 + lane) * 8;
    const bf16_t* up = SWIGLU ? wpacked + ((size_t)(up_tile_offset + nt) * k_tiles * 64 + lane) * 8 : nullptr;
    const bool x_tiled = tiled & TILED_X;
    // the same in every wavefront of the launch
    const bool ring = K % 32 == 0 && tiles_per_wave % SK_CHUNK == 0 && part_tiles == tiles_per_wave * SK_WAVES &&
                      k_tiles % part_tiles == 0;
    const bf16_t* xp = x_tiled ? x + (size_t)lane * 8 : x + (size_t)(x_ok ? i : 0) * K + jg * 8;
    const int x_step = x_tiled ? 512 : 32;                   // elements from one step's fragment to the next
    const uint4 zero = make_uint4(0, 0, 0, 0);

    // Loads whose values are wanted only after the weights have streamed are issued here, so that their
    // latency hides behind the stream.  Partial sums of squares: wavefront w has the rows w, w + SK_WAVES, ...,
    // each lane SK_PRE of a row's partial sums (more are fetched afterwards).  And the element of the
    // residual stream and the gain that this thread's result meets.
    // (None of these loads sits in a branch either: each is issued from an address inside its array, or inside
    // the weights where there is no such array, and a value from outside is dropped.  In branches the compiler
    // had every row's first load wait for the one before it: four trips to the L2 cache in turn before the
    // first weight was asked for.)
    float pre[SK_ROWS][SK_PRE];
    {
        const float* sp = link.ssq_in ? link.ssq_in : reinterpret_cast<const float*>(wpacked);
#pragma unroll
        for (int j = 0; j < SK_ROWS; ++j)
#pragma unroll
            for (int q = 0; q < SK_PRE; ++q) {
                const int m = wave + j * SK_WAVES, p = lane + q * 64;
                const bool have = link.ssq_in && m < M && p < link.n_in;
                const float v = sp[have ? (size_t)m * link.n_in + p : 0];
                pre[j][q] = have ? v : 0.f;
            }
    }
    const int t = threadIdx.x;
    const int ln = t & 63, r = (t >> 6) & 3;
    const int nl = 4 * (ln >> 4) + r, n = nt * 16 + nl, m = ln & 15;      // D[row n, column m]
    const bool ok = m < M && n < N;
    float res_pre = 0.f, gain_pre = 0.f;
    {
        const bool have = link.residual && t < 256 && ok;
        const float* rp = link.residual ? link.residual : reinterpret_cast<const float*>(wpacked);
        const float* gp = link.residual ? link.next_gain : reinterpret_cast<const float*>(wpacked);
        res_pre = rp[have ? (size_t)m * N + n : 0];
        gain_pre = gp[have ? n : 0];
    }

    floatx4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}}, accu[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    if (PAIRED) {
        // (the host launches this form only where the ring's conditions hold, or where every wavefront's share is a
        // whole number of pairs of steps)
        constexpr int PC = SK_CHUNK / 2;                     // pairs of steps in flight: as many weights as the ring below
        const int sub = i >> 3;                              // which step of a pair this lane's piece of x belongs to
        const bf16_t* xq = x_tiled ? x + (size_t)(jg * 16 + (i & 7)) * 8 + (size_t)sub * 512
                                   : x + (size_t)((i & 7) < M ? (i & 7) : 0) * K + jg * 8 + sub * 32;
        Frag wa[PC], wb[PC], ua[PC], ub[PC], xf[PC];
        if (!ring) {
            // A share that is a whole number of pairs but no whole number of rounds (the host sees to the pairs):
            // loads for pairs past the share's end come from its last pair, and in the last round zeros go to the
            // matrix cores in their place, as in the ring for such shares below.
            const int last = max(kt_end - 2, 0);
#pragma unroll
            for (int c = 0; c < PC; ++c) {
                const size_t at = (size_t)min(kt_begin + 2 * c, last);
                wa[c].u = load_stream16(wp + at * 512);
                wb[c].u = load_stream16(wp + (at + 1) * 512);
                if (SWIGLU) {
                    ua[c].u = load_stream16(up + at * 512);
                    ub[c].u = load_stream16(up + (at + 1) * 512);
                }
                xf[c].u = *reinterpret_cast<const uint4*>(xq + at * x_step);
            }
            int kt = kt_begin;
            for (; kt + SK_CHUNK < kt_end; kt += SK_CHUNK) {
#pragma unroll
                for (int c = 0; c < PC; ++c) {
                    acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[c].v, xf[c].v, acc[0], 0, 0, 0);
                    acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[c].v, xf[c].v, acc[1], 0, 0, 0);
                    if (SWIGLU) {
                        accu[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ua[c].v, xf[c].v, accu[0], 0, 0, 0);
                        accu[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ub[c].v, xf[c].v, accu[1], 0, 0, 0);
                    }
                    const size_t next = (size_t)min(kt + 2 * c + SK_CHUNK, last);
                    wa[c].u = load_stream16(wp + next * 512);
                    wb[c].u = load_stream16(wp + (next + 1) * 512);
                    if (SWIGLU) {
                        ua[c].u = load_stream16(up + next * 512);
                        ub[c].u = load_stream16(up + (next + 1) * 512);
                    }
                    xf[c].u = *reinterpret_cast<const uint4*>(xq + next * x_step);
                }
            }
#pragma unroll
            for (int c = 0; c < PC; ++c) {
                const bool live = kt + 2 * c < kt_end;
                Frag a, b, xv;
                a.u = live ? wa[c].u : zero;
                b.u = live ? wb[c].u : zero;
                xv.u = live ? xf[c].u : zero;
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, xv.v, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b.v, xv.v, acc[1], 0, 0, 0);
                if (SWIGLU) {
                    a.u = live ? ua[c].u : zero;
                    b.u = live ? ub[c].u : zero;
                    accu[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, xv.v, accu[0], 0, 0, 0);
                    accu[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b.v, xv.v, accu[1], 0, 0, 0);
                }
            }
        } else {
#pragma unroll
        for (int c = 0; c < PC; ++c) {
            const size_t at = (size_t)(kt_begin + 2 * c);
            wa[c].u = load_stream16(wp + at * 512);
            wb[c].u = load_stream16(wp + (at + 1) * 512);
            if (SWIGLU) {
                ua[c].u = load_stream16(up + at * 512);
                ub[c].u = load_stream16(up + (at + 1) * 512);
            }
            xf[c].u = *reinterpret_cast<const uint4*>(xq + at * x_step);
        }
        int kt = kt_begin;
        for (; kt + SK_CHUNK < kt_end; kt += SK_CHUNK) {
#pragma unroll
            for (int c = 0; c < PC; ++c) {
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[c].v, xf[c].v, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[c].v, xf[c].v, acc[1], 0, 0, 0);
                if (SWIGLU) {
                    accu[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ua[c].v, xf[c].v, accu[0], 0, 0, 0);
                    accu[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ub[c].v, xf[c].v, accu[1], 0, 0, 0);
                }
                const size_t next = (size_t)(kt + 2 * c + SK_CHUNK);
                wa[c].u = load_stream16(wp + next * 512);
                wb[c].u = load_stream16(wp + (next + 1) * 512);
                if (SWIGLU) {
                    ua[c].u = load_stream16(up + next * 512);
                    ub[c].u = load_stream16(up + (next + 1) * 512);
                }
                xf[c].u = *reinterpret_cast<const uint4*>(xq + next * x_step);
            }
        }
#pragma unroll
        for (int c = 0; c < PC; ++c) {
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[c].v, xf[c].v, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[c].v, xf[c].v, acc[1], 0, 0, 0);
            if (SWIGLU) {
                accu[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ua[c].v, xf[c].v, accu[0], 0, 0, 0);
                accu[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ub[c].v, xf[c].v, accu[1], 0, 0, 0);
            }
        }
        }
    } else if (ring) {
        // Every wavefront's share is a whole number of rounds of SK_CHUNK steps and K a multiple of 32: the
        // fragments are a ring, and a register asks for the step SK_CHUNK further on as soon as the matrix
        // cores have taken the one it held, so that SK_CHUNK steps' loads stay in flight all the way instead
        // of draining at the end of every round.  The sums are the same ones in the same order.
        // (No load here sits in a branch: the compiler keeps count of loads in flight only across code without
        // branches, and waits for all of them otherwise.  The columns of rows beyond M therefore hold what row 0,
        // or the unused rows of a tile, hold: they are never stored.)
        Frag wf[SK_CHUNK], uf[SK_CHUNK], xf[SK_CHUNK];
#pragma unroll
        for (int c = 0; c < SK_CHUNK; ++c) {
            wf[c].u = load_stream16(wp + (size_t)(kt_begin + c) * 512);
            if (SWIGLU) uf[c].u = load_stream16(up + (size_t)(kt_begin + c) * 512);
            xf[c].u = *reinterpret_cast<const uint4*>(xp + (size_t)(kt_begin + c) * x_step);
        }
        int kt = kt_begin;
        for (; kt + SK_CHUNK < kt_end; kt += SK_CHUNK) {
#pragma unroll
            for (int c = 0; c < SK_CHUNK; ++c) {
                acc[c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[c].v, xf[c].v, acc[c & 1], 0, 0, 0);
                if (SWIGLU) accu[c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[c].v, xf[c].v, accu[c & 1], 0, 0, 0);
                const size_t next = (size_t)(kt + c + SK_CHUNK);
                wf[c].u = load_stream16(wp + next * 512);
                if (SWIGLU) uf[c].u = load_stream16(up + next * 512);
                xf[c].u = *reinterpret_cast<const uint4*>(xp + next * x_step);
            }
        }
#pragma unroll
        for (int c = 0; c < SK_CHUNK; ++c) {
            acc[c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[c].v, xf[c].v, acc[c & 1], 0, 0, 0);
            if (SWIGLU) accu[c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[c].v, xf[c].v, accu[c & 1], 0, 0, 0);
        }
    } else if (K % 32 == 0) {
        // A share that is no whole number of rounds (K = 2,560 or 9,728 over four wavefronts): the same ring.  A
        // load for a step past the share's end is issued all the same, from the share's last step (no load in a
        // branch), and in the last round, the only one that holds such steps, zeros go to the matrix cores in
        // their place (chosen where the fragment is used: choosing where it is loaded would wait for every load
        // in turn).  The same sums in the same order as the loop below.
        Frag wf[SK_CHUNK], uf[SK_CHUNK], xf[SK_CHUNK];
        const int last = max(min(kt_end, k_tiles) - 1, 0);
#pragma unroll
        for (int c = 0; c < SK_CHUNK; ++c) {
            const size_t from = (size_t)min(kt_begin + c, last);
            wf[c].u = load_stream16(wp + from * 512);
            if (SWIGLU) uf[c].u = load_stream16(up + from * 512);
            xf[c].u = *reinterpret_cast<const uint4*>(xp + from * x_step);
        }
        int kt = kt_begin;
        for (; kt + SK_CHUNK < kt_end; kt += SK_CHUNK) {      // every step of these rounds lies inside the share
#pragma unroll
            for (int c = 0; c < SK_CHUNK; ++c) {
                acc[c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[c].v, xf[c].v, acc[c & 1], 0, 0, 0);
                if (SWIGLU) accu[c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[c].v, xf[c].v, accu[c & 1], 0, 0, 0);
                const size_t from = (size_t)min(kt + c + SK_CHUNK, last);
                wf[c].u = load_stream16(wp + from * 512);
                if (SWIGLU) uf[c].u = load_stream16(up + from * 512);
                xf[c].u = *reinterpret_cast<const uint4*>(xp + from * x_step);
            }
        }
#pragma unroll
        for (int c = 0; c < SK_CHUNK; ++c) {
            const bool live = kt + c < kt_end;
            Frag w, u, xv;
            w.u = live ? wf[c].u : zero;
            xv.u = live ? xf[c].u : zero;
            acc[c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w.v, xv.v, acc[c & 1], 0, 0, 0);
            if (SWIGLU) {
                u.u = live ? uf[c].u : zero;
                accu[c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(u.v, xv.v, accu[c & 1], 0, 0, 0);
            }
        }
    } else
    for (int kt = kt_begin; kt < kt_end; kt += SK_CHUNK) {
        Frag wf[SK_CHUNK], uf[SK_CHUNK], xf[SK_CHUNK];
#pragma unroll
        for (int c = 0; c < SK_CHUNK; ++c) {
            const bool live = kt + c < kt_end;
            wf[c].u = live ? load_stream16(wp + (size_t)(kt + c) * 512) : zero;
            if (SWIGLU) uf[c].u = live ? load_stream16(up + (size_t)(kt + c) * 512) : zero;
            // the packed matrix is zero beyond K; x is not padded
            xf[c].u = (live && x_ok && (kt + c) * 32 + jg * 8 < K)
                          ? *reinterpret_cast<const uint4*>(xp + (size_t)(kt + c) * x_step) : zero;
        }
#pragma unroll
        for (int c = 0; c < SK_CHUNK; ++c) {               // SK_CHUNK is even: c's parity is the step's, counted from kt_begin
            acc[c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[c].v, xf[c].v, acc[c & 1], 0, 0, 0);
            if (SWIGLU) accu[c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[c].v, xf[c].v, accu[c & 1], 0, 0, 0);
        }
    }
    if (PAIRED) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                red[0][PAIRED ? h : 0][wave][e][lane] = acc[h][e];
                if (SWIGLU) red[SWIGLU ? 1 : 0][PAIRED ? h : 0][wave][e][lane] = accu[h][e];
            }
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            red[0][0][wave][e][lane] = acc[0][e] + acc[1][e];
            if (SWIGLU) red[SWIGLU ? 1 : 0][0][wave][e][lane] = accu[0][e] + accu[1][e];
        }
    }
    // rows of x that still want their 1 / rms: the lanes' shares in the order of wave_sum, the same in every
    // workgroup
    if (link.ssq_in) {
#pragma unroll
        for (int j = 0; j < SK_ROWS; ++j) {
            const int mr = wave + j * SK_WAVES;
            if (mr < M) {
                float sq = 0.f;
#pragma unroll
                for (int q = 0; q < SK_PRE; ++q) sq += pre[j][q];
                for (int p = lane + SK_PRE * 64; p < link.n_in; p += 64) sq += link.ssq_in[(size_t)mr * link.n_in + p];
                sq = wave_sum(sq);
                if (lane == 0) inv_lds[mr] = 1.0f / sqrtf(sq / (float)link.dim + link.eps);
            }
        }
    }
    __syncthreads();
    if (t < 256) {
        float g = 0.f, u = 0.f;
#pragma unroll
        for (int wv = 0; wv < SK_WAVES; ++wv) {
            // PAIRED: column m of the even steps' product plus column m + 8 of the odd steps' (m < 8 is all that is stored)
            g += PAIRED ? red[0][0][wv][r][ln] + red[0][PAIRED ? 1 : 0][wv][r][(ln + 8) & 63] : red[0][0][wv][r][ln];
            if (SWIGLU) u += PAIRED ? red[SWIGLU ? 1 : 0][0][wv][r][ln] + red[SWIGLU ? 1 : 0][PAIRED ? 1 : 0][wv][r][(ln + 8) & 63] : red[SWIGLU ? 1 : 0][0][wv][r][ln];
        }
        if (link.ssq_in && m < M) {
            g *= inv_lds[m];
            u *= inv_lds[m];
        }
        float v = SWIGLU ? silu_sk(g) * u : g;
        if (link.residual) {
            if (ok) {
                const size_t at = (size_t)m * N + n;
                v += res_pre;
                link.residual[at] = v;                   // this element belongs to this thread alone
                link.xg_out[(tiled & TILED_OUT) ? tiled_at(m, n, (N + 31) / 32) : at] = f32_to_bf16(v * gain_pre);
            }
            sq_lds[m][nl] = ok ? v * v : 0.f;
        } else if (ok) {
            from_f32(out + ((tiled & TILED_OUT) ? tiled_at(m, n, (N + 31) / 32) : (size_t)m * N + n), v);
        }
    }
    if (link.residual) {                                 // the workgroup's share of every row's sum of squares
        __syncthreads();
        if (t < M) {
            float total = 0.f;
            for (int c = 0; c < 16; ++c) total += sq_lds[t][c];
            link.ssq_out[(size_t)t * gridDim.x + blockIdx.x] = total;
        }
    }
}

// Four wavefronts a workgroup stream fastest when there are many row tiles (5.0 TB/s on the 24576 x 4096
// gate|up matrix against 4.6 with eight); a long K with few row tiles wants the eight (K = 12288, 256 tiles).
// (Two wavefronts for that gate|up pair are 5% faster alone at 8 and 16 rows of x and 1 to 2% slower inside
// the model, where each wavefront then adds up eight rows' sums of squares for the norm before it.)
// (A matrix of 384 row tiles leaves half of 256 compute units with two workgroups and the others with one, and a
// compute unit streams at a rate of its own: the launch takes as long as 512 tiles would.  Workgroups of three
// half tiles (8 rows, two wavefronts each on half of K, a load fetching the rows for two steps of K at once) make
// 256 equal workgroups of it and were slower all the same, 15.0 against 13.7 us at 8 rows: every step of K then
// needs its rows of x for 8 rows of weights instead of 16, and a compute unit's vector memory path counts those
// bytes from the L2 cache like the ones from memory.)
static int skinny_waves(int n, int k) { return k >= 8192 ? 8 : 4; }

template <int WAVES, bool SWIGLU>
static void launch_packed(void* out, int out_dtype, const bf16_t* x, const bf16_t* w, int m, int n, int k, int parts,
                          const NormLink& link, int tiled, hipStream_t s) {
    const int k_tiles = (k + 31) / 32, row_tiles = (n + 15) / 16;
    const int part_tiles = (k_tiles + parts - 1) / parts;
    const int tiles_per_wave = (part_tiles + WAVES - 1) / WAVES;
    dim3 grid(row_tiles, parts);
    // at most 8 rows and every wavefront's share a whole number of pairs of steps: two steps to a load of x (the
    // kernel works out for itself whether the share is whole rounds of the ring too)
    const bool paired = m <= 8 && k % 32 == 0 && tiles_per_wave % 2 == 0 && part_tiles == tiles_per_wave * WAVES &&
                        k_tiles % part_tiles == 0;
#define RI_SKINNY_GO(TO, PAIRED)                                                        \
    gemm_skinny_packed_kernel<WAVES, SWIGLU, TO, PAIRED><<<grid, WAVES * 64, 0, s>>>(   \
        (TO*)out, x, w, m, n, k, k_tiles, tiles_per_wave, row_tiles, link, tiled)
    if (out_dtype == RI_F32) {
        if (paired) RI_SKINNY_GO(float, true); else RI_SKINNY_GO(float, false);
    } else {
        if (paired) RI_SKINNY_GO(bf16_t, true); else RI_SKINNY_GO(bf16_t, false);
    }
#undef RI_SKINNY_GO
}

static int packed_run(void* out, int out_dtype, const void* x, const void* wpacked, int m, int n, int k, int swiglu,
                      int parts, const NormLink& link, int tiled, hipStream_t s) {
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)wpacked;
    const bool eight = skinny_waves(n, (k + parts - 1) / parts) == 8;
    if (swiglu) {
        if (eight) launch_packed<8, true>(out, out_dtype, xb, wb, m, n, k, parts, link, tiled, s);
        else       launch_packed<4, true>(out, out_dtype, xb, wb, m, n, k, parts, link, tiled, s);
    } else {
        if (eight) launch_packed<8, false>(out, out_dtype, xb, wb, m, n, k, parts, link, tiled, s);
        else       launch_packed<4, false>(out, out_dtype, xb, wb, m, n, k, parts, link, tiled, s);
    }
    RI_LAUNCH_CHECK("gemm_skinny_packed_bf16");
    return 0;
}

extern "C" int ri_gemm_skinny_packed_bf16(void* out, int out_dtype, const void* x, const void* wpacked, int m, int n,
                                          int k, int swiglu, int parts, int tiled, void* stream) {
    RI_REQUIRE(m > 0 && m <= 16, "gemm_skinny_packed_bf16: %d rows of x, this kernel takes 1 to 16", m);
    RI_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_skinny_packed_bf16: n %d, k %d (k must be a multiple of 8)", n, k);
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "gemm_skinny_packed_bf16: out dtype %d", out_dtype);
    RI_REQUIRE(parts >= 1 && parts <= 64 && (parts == 1 || (!swiglu && out_dtype == RI_F32)),
               "gemm_skinny_packed_bf16: %d parts of K (more than one needs float32 sums and no activation)", parts);
    RI_REQUIRE(!(tiled & ~(TILED_X | TILED_OUT)) && (!(tiled & TILED_OUT) || (out_dtype == RI_BF16 && parts == 1)),
               "gemm_skinny_packed_bf16: layout flags %d (a tiled result is bfloat16 and whole)", tiled);
    NormLink link = {};
    return packed_run(out, out_dtype, x, wpacked, m, n, k, swiglu, parts, link, tiled, (hipStream_t)stream);
}

// Number of workgroups (and so of partial sums of squares per row) of a linked product with n output columns.
extern "C" int ri_gemm_skinny_packed_bf16_partials(int n) { return (n + 15) / 16; }

extern "C" int ri_gemm_skinny_packed_bf16_linked(void* out, int out_dtype, const void* x, const void* wpacked, int m,
                                                 int n, int k, int swiglu, const float* ssq_in, int n_in, float eps,
                                                 int dim, float* residual, const float* next_gain, void* xg_out,
                                                 float* ssq_out, int tiled, void* stream) {
    RI_REQUIRE(m > 0 && m <= 16, "gemm_skinny_packed_bf16_linked: %d rows of x, this kernel takes 1 to 16", m);
    RI_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_skinny_packed_bf16_linked: n %d, k %d (k must be a multiple of 8)", n,
               k);
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "gemm_skinny_packed_bf16_linked: out dtype %d", out_dtype);
    RI_REQUIRE(!ssq_in || (n_in > 0 && dim > 0), "gemm_skinny_packed_bf16_linked: %d partial sums over %d elements", n_in,
               dim);
    RI_REQUIRE(!residual || (next_gain && xg_out && ssq_out && !swiglu),
               "gemm_skinny_packed_bf16_linked: a product that feeds the residual stream needs the next gain and both "
               "outputs");
    RI_REQUIRE(residual || out, "gemm_skinny_packed_bf16_linked: no output");
    RI_REQUIRE(!(tiled & ~(TILED_X | TILED_OUT)) && (!(tiled & TILED_OUT) || residual || out_dtype == RI_BF16),
               "gemm_skinny_packed_bf16_linked: layout flags %d (a tiled result is bfloat16)", tiled);
    NormLink link = {ssq_in, n_in, eps, dim, residual, next_gain, (bf16_t*)xg_out, ssq_out};
    return packed_run(out, out_dtype, x, wpacked, m, n, k, swiglu, 1, link, tiled, (hipStream_t)stream);
}

// ------------------------------------------------------------------ 17 to 64 rows of x
// The packed matrix against RT tiles of 16 rows of x: every weight fragment, read once from memory, meets
// RT fragments of x from the L2 cache (the weights stream past that cache without settling in it, so the
// few hundred kilobytes of x stay there).  Otherwise as the kernel above, without the norm links: steps of
// this size keep their norm kernels.  A row's result does not depend on the number of rows: rows beyond M
// are zero columns, and every row tile has accumulators of its own.
template <int SK_WAVES, bool SWIGLU, typename TO, int RT>
__global__ void __launch_bounds__(SK_WAVES * 64)
gemm_mid_packed_kernel(TO* __restrict__ out, const bf16_t* __restrict__ x, const bf16_t* __restrict__ wpacked, int M,
                       int N, int K, int k_tiles, int tiles_per_wave, int up_tile_offset, int tiled) {
    constexpr int CH = RT <= 2 ? 8 : 4;                      // MFMA steps whose loads are in flight together
    __shared__ float red[SWIGLU ? 2 : 1][SK_WAVES][RT * 4][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, jg = lane >> 4;
    const int nt = blockIdx.x;
    const int kt_begin = wave * tiles_per_wave, kt_end = min(k_tiles, kt_begin + tiles_per_wave);
    const bf16_t* wp = wpacked + ((size_t)nt * k_tiles * 64 + lane) * 8;
    const bf16_t* up = SWIGLU ? wpacked + ((size_t)(up_tile_offset + nt) * k_tiles * 64 + lane) * 8 : nullptr;
    const bf16_t* xp[RT];
    bool x_ok[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        x_ok[rt] = rt * 16 + i < M;
        // (RT may be more tiles than x has: up to 16 rows are one tile and run with RT = 2.  A tile beyond the
        // last is never read: the loop that asks for every fragment reads the last tile again instead.)
        xp[rt] = (tiled & TILED_X) ? x + ((size_t)min(rt, (M - 1) >> 4) * k_tiles * 64 + lane) * 8
                                   : x + (size_t)(x_ok[rt] ? rt * 16 + i : 0) * K + jg * 8;
    }
    const int x_step = (tiled & TILED_X) ? 512 : 32;         // elements from one step's fragment to the next
    // two halves of every sum, by the parity of the step counted from the wavefront's first, added at the end:
    // the order of the kernel above, so that a row's bits are the same from either
    floatx4 acc[RT][2], accu[RT][2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) acc[rt][0] = acc[rt][1] = accu[rt][0] = accu[rt][1] = floatx4{0.f, 0.f, 0.f, 0.f};
    // the same in every wavefront of the launch: K in whole steps, every wavefront's share whole rounds of CH
    const bool ring = K % 32 == 0 && tiles_per_wave % CH == 0 && k_tiles == tiles_per_wave * SK_WAVES;
    if (ring) {
        // The fragments are a ring: a register asks for the step CH further on as soon as the matrix cores have
        // taken the one it held, and no load sits in a branch (see the kernel above).  Rows of x beyond M read
        // row 0, the unused rows of a tile or the last tile once more: their columns are never stored.
        Frag wf[CH], uf[CH], xf[RT][CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            wf[c].u = load_stream16(wp + (size_t)(kt_begin + c) * 512);
            if (SWIGLU) uf[c].u = load_stream16(up + (size_t)(kt_begin + c) * 512);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
                xf[rt][c].u = *reinterpret_cast<const uint4*>(xp[rt] + (size_t)(kt_begin + c) * x_step);
        }
        int kt = kt_begin;
        for (; kt + CH < kt_end; kt += CH) {
#pragma unroll
            for (int c = 0; c < CH; ++c) {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    acc[rt][c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[c].v, xf[rt][c].v, acc[rt][c & 1], 0, 0, 0);
                    if (SWIGLU) accu[rt][c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[c].v, xf[rt][c].v, accu[rt][c & 1], 0, 0, 0);
                }
                const size_t next = (size_t)(kt + c + CH);
                wf[c].u = load_stream16(wp + next * 512);
                if (SWIGLU) uf[c].u = load_stream16(up + next * 512);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) xf[rt][c].u = *reinterpret_cast<const uint4*>(xp[rt] + next * x_step);
            }
        }
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                acc[rt][c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[c].v, xf[rt][c].v, acc[rt][c & 1], 0, 0, 0);
                if (SWIGLU) accu[rt][c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[c].v, xf[rt][c].v, accu[rt][c & 1], 0, 0, 0);
            }
    } else
    for (int kt = kt_begin; kt < kt_end; kt += CH) {
        const uint4 zero = make_uint4(0, 0, 0, 0);
        Frag wf[CH], uf[CH], xf[RT][CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const bool live = kt + c < kt_end;
            wf[c].u = live ? load_stream16(wp + (size_t)(kt + c) * 512) : zero;
            if (SWIGLU) uf[c].u = live ? load_stream16(up + (size_t)(kt + c) * 512) : zero;
            const bool k_ok = live && (kt + c) * 32 + jg * 8 < K;            // the packed matrix is zero beyond K; x is not padded
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
                xf[rt][c].u = (k_ok && x_ok[rt]) ? *reinterpret_cast<const uint4*>(xp[rt] + (size_t)(kt + c) * x_step) : zero;
        }
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                acc[rt][c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[c].v, xf[rt][c].v, acc[rt][c & 1], 0, 0, 0);
                if (SWIGLU) accu[rt][c & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[c].v, xf[rt][c].v, accu[rt][c & 1], 0, 0, 0);
            }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            red[0][wave][rt * 4 + e][lane] = acc[rt][0][e] + acc[rt][1][e];
            if (SWIGLU) red[1][wave][rt * 4 + e][lane] = accu[rt][0][e] + accu[rt][1][e];
        }
    __syncthreads();
    // D[row n, column m] of a tile: lane ln of register r holds n = 4 * (ln / 16) + r, m = ln % 16
    for (int t = threadIdx.x; t < RT * 256; t += SK_WAVES * 64) {
        const int rt = t >> 8, ln = t & 63, r = (t >> 6) & 3;
        const int n = nt * 16 + 4 * (ln >> 4) + r, m = rt * 16 + (ln & 15);
        float g = 0.f, u = 0.f;
#pragma unroll
        for (int wv = 0; wv < SK_WAVES; ++wv) {
            g += red[0][wv][rt * 4 + r][ln];
            if (SWIGLU) u += red[1][wv][rt * 4 + r][ln];
        }
        if (m < M && n < N)
            from_f32(out + ((tiled & TILED_OUT) ? tiled_at(m, n, (N + 31) / 32) : (size_t)m * N + n), SWIGLU ? silu_sk(g) * u : g);
    }
}

template <int WAVES, bool SWIGLU, int RT>
static void launch_mid(void* out, int out_dtype, const bf16_t* x, const bf16_t* w, int m, int n, int k, int tiled,
                       hipStream_t s) {
    const int k_tiles = (k + 31) / 32, row_tiles = (n + 15) / 16;
    const int tiles_per_wave = (k_tiles + WAVES - 1) / WAVES;
    if (out_dtype == RI_F32)
        gemm_mid_packed_kernel<WAVES, SWIGLU, float, RT><<<row_tiles, WAVES * 64, 0, s>>>(
            (float*)out, x, w, m, n, k, k_tiles, tiles_per_wave, row_tiles, tiled);
    else
        gemm_mid_packed_kernel<WAVES, SWIGLU, bf16_t, RT><<<row_tiles, WAVES * 64, 0, s>>>(
            (bf16_t*)out, x, w, m, n, k, k_tiles, tiles_per_wave, row_tiles, tiled);
}

extern "C" int ri_gemm_mid_packed_bf16(void* out, int out_dtype, const void* x, const void* wpacked, int m, int n, int k,
                                       int swiglu, int tiled, void* stream) {
    RI_REQUIRE(m > 0 && m <= 64, "gemm_mid_packed_bf16: %d rows of x, this kernel takes 1 to 64", m);
    RI_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_mid_packed_bf16: n %d, k %d (k must be a multiple of 8)", n, k);
    RI_REQUIRE(out_dtype == RI_F32 || out_dtype == RI_BF16, "gemm_mid_packed_bf16: out dtype %d", out_dtype);
    RI_REQUIRE(!(tiled & ~(TILED_X | TILED_OUT)) && (!(tiled & TILED_OUT) || out_dtype == RI_BF16),
               "gemm_mid_packed_bf16: layout flags %d (a tiled result is bfloat16)", tiled);
    hipStream_t s = (hipStream_t)stream;
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)wpacked;
    const bool eight = skinny_waves(n, k) == 8;
#define RI_MID_CASE(W, SG, RT) launch_mid<W, SG, RT>(out, out_dtype, xb, wb, m, n, k, tiled, s)
    if (m <= 32) {
        if (swiglu) { if (eight) RI_MID_CASE(8, true, 2); else RI_MID_CASE(4, true, 2); }
        else        { if (eight) RI_MID_CASE(8, false, 2); else RI_MID_CASE(4, false, 2); }
    } else if (m <= 48) {
        if (swiglu) { if (eight) RI_MID_CASE(8, true, 3); else RI_MID_CASE(4, true, 3); }
        else        { if (eight) RI_MID_CASE(8, false, 3); else RI_MID_CASE(4, false, 3); }
    } else {
        if (swiglu) { if (eight) RI_MID_CASE(8, true, 4); else RI_MID_CASE(4, true, 4); }
        else        { if (eight) RI_MID_CASE(8, false, 4); else RI_MID_CASE(4, false, 4); }
    }
#undef RI_MID_CASE
    RI_LAUNCH_CHECK("gemm_mid_packed_bf16");
    return 0;
}

// Q4G128 GEMM for a decode batch over PREPARED activations; x lives in registers, the
// weights stream through a ring in LDS:
//   part[j][b][n] = sum over K part j of x[b][k] * w[n][k]   (fp32)
//
// The streaming kernel of qgemm_q4_stream.hip keeps a 1024-column part of x in LDS, reads
// it back as the MFMA A operand for every weight tile and holds the weights in flight in
// registers, one tile ahead.  Timelines of that kernel show its waves waiting: a wave can
// only ask for the next tile once registers are free, every request of 16 rows x 64 bytes
// touches 16 half cache lines, and nothing is in flight while the x part is staged.  Here
// the roles are turned round.
//
// * A wave owns a slice of GS groups (128 * GS columns) of K for the whole launch and holds
//   that slice of x, for all batch rows, in registers (16 * GS * BT dwords per lane) together
//   with the slice's per-group sums of x.  The eight waves of a workgroup sit side by side
//   on K, so the workgroup covers 1024 * GS columns — all of K = 4096 at GS = 4 — and walks
//   down its share of the 16-row weight tiles.
// * Weights, scales and zeros go from global memory straight into a per-wave ring of R
//   tiles in LDS (global_load_lds), so a wave has up to R tiles in flight without holding a
//   register for them, and asks for the first R before it loads its x.  One request covers
//   64 / (4 * GS) rows end to end (256 or 128 contiguous bytes per row).  Which 16-byte
//   piece a lane fetches is rotated by the row index, so that the later ds_read_b128 of the
//   MFMA B operand (lane = 16 rows x 4 pieces of one group) touches every bank once.
// * Per tile a wave reads its 16 rows from the ring, multiplies, applies the per-group scale
//   and zero, and the eight waves' partial sums meet in LDS: one 1 KiB * BT store per wave,
//   one barrier, one conflict-free read of eight floats per thread.
//
// The compiler orders LDS accesses it can see behind every outstanding global_load_lds, so
// inside the tile loop LDS is only touched through inline assembly, with explicit counts:
// a wave's memory operations retire in issue order, and the count to wait for is the number
// of ring requests issued after the tile that is needed (stores are left out of the count,
// which can only make the wait longer).
//
// With all of K inside the workgroup there is one part (K = 4096) or three (K = 12288)
// instead of four or twelve: less fp32 written here and fewer loads in the consumers.
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "q4_common.hpp"

#include <hip/hip_fp16.h>

namespace lg {

constexpr int kRegxWaves = 8;
constexpr int kRegxMaxRing = 8;

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* glb_ptr_t;

// Waits until at most m * REQ of this wave's vector memory operations are outstanding.
template <int REQ>
__device__ __forceinline__ void regx_wait_tiles(int m) {
#define LG_VMCNT_CASE(M) \
    case M: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(M * REQ > 63 ? 63 : M * REQ) : "memory"); break;
    switch (m) {
        LG_VMCNT_CASE(1) LG_VMCNT_CASE(2) LG_VMCNT_CASE(3) LG_VMCNT_CASE(4)
        LG_VMCNT_CASE(5) LG_VMCNT_CASE(6) LG_VMCNT_CASE(7)
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
#undef LG_VMCNT_CASE
}

// LDS bytes: per wave a ring of R tiles (GS KiB of weights + 256 bytes of scales and zeros
// each), then the exchange buffers of the partial sums (half a batch of tiles).
__host__ __device__ constexpr int regx_tile_bytes(int gs) { return gs * 1024 + 256; }
__host__ __device__ constexpr int regx_batch_tiles(int gs) { return gs == 4 ? 6 : 8; }
__host__ __device__ constexpr int regx_lds_bytes(int bt, int gs, int ring) {
    return kRegxWaves * ring * regx_tile_bytes(gs) + (regx_batch_tiles(gs) / 2) * kRegxWaves * bt * 1024;
}

template <int BT, int GS, bool PLAIN>
__global__ __launch_bounds__(64 * kRegxWaves) void qgemm_q4g128_regx_kernel(
    const uint4_t* __restrict__ xprep, const uint8_t* __restrict__ qw,
    const __half* __restrict__ scale, const __half* __restrict__ zero, float* __restrict__ part,
    int b, int n, int k, int tiles_per_worker, int ring, const float* __restrict__ bias) {
    static_assert(GS == 2 || GS == 4, "slices of 2 or 4 groups");
    constexpr int BP = BT * 16;
    constexpr int W = kRegxWaves;
    constexpr int GW = W * GS;           // groups per workgroup
    constexpr int PIECES = 4 * GS;       // 16-byte pieces of a row's slice
    constexpr int RPD = 64 / PIECES;     // rows per weight request
    constexpr int TB = regx_tile_bytes(GS);
    constexpr int TM = regx_batch_tiles(GS);  // tiles between exchanges
    constexpr int CH = TM / 2;                // tiles per exchange (TM even)
    extern __shared__ uint4_t lds[];

    const int groups = k >> 7;
    const int j = blockIdx.y;
    const int tiles = (n + 15) >> 4;
    const int t_begin = blockIdx.x * tiles_per_worker;
    if (t_begin >= tiles) return;
    const int t_end = min(tiles, t_begin + tiles_per_worker);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col = lane & 15;
    const int kc = lane >> 4;
    const int g0 = j * GW + wave * GS;  // this wave's first group

    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));

    const unsigned lds_base = (unsigned)(uintptr_t)(lds_ptr_t)lds;
    const unsigned ring_base = lds_base + (unsigned)(wave * ring * TB);
    const unsigned red_base = lds_base + (unsigned)(W * ring * TB);
    char* const ring_ptr = reinterpret_cast<char*>(lds) + wave * ring * TB;

    // ---- ring requests.  Weight request a of a tile: lane -> row a * RPD + lane / PIECES,
    // position lane % PIECES of that row, which holds piece (position - rotation) of the
    // slice.  Scale / zero request: lanes 0..31 the scales, 32..63 the zeros, one dword each.
    const uint8_t* wbase = qw + (int64_t)g0 * 64;  // uniform; lane offsets fit 32 bits (N*K < 2^31)
    const unsigned khalf = (unsigned)(k >> 1);
    const int dr = lane / PIECES;  // row of this lane inside a request
    unsigned piece_off[GS];
#pragma unroll
    for (int a = 0; a < GS; ++a) {
        const int rot = GS == 4 ? a * RPD + dr : dr + a;
        piece_off[a] = (unsigned)(((lane % PIECES) - rot) & (PIECES - 1)) * 16u;
    }
    const __half* szbase = ((lane & 32) ? zero : scale) + g0;
    const int sz_row = GS == 4 ? (lane & 31) >> 1 : lane & 15;
    const int sz_col = GS == 4 ? 2 * (lane & 1) : 0;
    auto request_tile = [&](int t, int slot) {
        char* dst = ring_ptr + slot * TB;
#pragma unroll
        for (int a = 0; a < GS; ++a) {
            const int row = min(t * 16 + a * RPD + dr, n - 1);
            const uint8_t* src = wbase + ((unsigned)row * khalf + piece_off[a]);
            __builtin_amdgcn_global_load_lds((glb_ptr_t)src, (lds_ptr_t)(dst + a * 1024), 16, 0, 0);
        }
        const int row = min(t * 16 + sz_row, n - 1);
        const __half* src = szbase + ((unsigned)row * (unsigned)groups + (unsigned)sz_col);
        __builtin_amdgcn_global_load_lds((glb_ptr_t)src, (lds_ptr_t)(dst + GS * 1024), 4, 0, 0);
    };
    constexpr int kReq = GS + 1;  // requests per tile

    const int my_tiles = t_end - t_begin;
    const int ahead = min(ring, my_tiles);
    // the first tile ahead of x, the rest of the ring behind it: a wave's loads come back in
    // the order they were issued, and nothing can start before x is here
    request_tile(t_begin, 0);

    // ---- this wave's slice of x (kept for the whole launch).  The group sums of x, for
    // the zero-point term, are the A operand of one fp32 MFMA per tile (K = 4 = groups).
    uint4_t xr[GS][4][BT];
    float xs[BT];
    if constexpr (PLAIN) {
        // x as a plain bf16 [b][K] matrix: the 16 bytes of a chunk are contiguous there
        const uint16_t* xp = reinterpret_cast<const uint16_t*>(xprep);
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) {
            const int row = bt * 16 + col;
            const uint16_t* xrow = xp + (int64_t)min(row, b - 1) * k;
#pragma unroll
            for (int i = 0; i < GS; ++i)
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) {
                    const uint4_t v = *reinterpret_cast<const uint4_t*>(xrow + 8 * (16 * (g0 + i) + 4 * kc + s4));
                    xr[i][s4][bt] = row < b ? v : uint4_t{0u, 0u, 0u, 0u};
                }
        }
    } else {
#pragma unroll
        for (int i = 0; i < GS; ++i)
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
                for (int bt = 0; bt < BT; ++bt)
                    xr[i][s4][bt] = xprep[(16 * (g0 + i) + 4 * kc + s4) * BP + bt * 16 + col];
        const float* xg_src = reinterpret_cast<const float*>(
            reinterpret_cast<const char*>(xprep) + xprep_xg_offset(b, k));
#pragma unroll
        for (int bt = 0; bt < BT; ++bt)
            xs[bt] = kc < GS ? xg_src[(g0 + kc) * BP + bt * 16 + col] : 0.0f;
    }
    // the wait for x belongs here, before the loop: left to the compiler it would sit at the
    // first use inside the loop body and drain the ring on every tile
#pragma unroll
    for (int i = 0; i < GS; ++i)
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) asm volatile("" : "+v"(xr[i][s4][bt]));
    if constexpr (PLAIN) {
        // group sums: a lane holds a quarter of each group's chunks of its batch row, the
        // lanes 16, 32 and 48 further on the rest; then pair order for the MFMA operand
#pragma unroll
        for (int bt = 0; bt < BT; ++bt) {
            float mine = 0.0f;
#pragma unroll
            for (int i = 0; i < GS; ++i) {
                float part_sum = 0.0f;
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) part_sum += sum8_bf16(xr[i][s4][bt]);
                part_sum += __shfl_xor(part_sum, 16);
                part_sum += __shfl_xor(part_sum, 32);
                if (kc == i) mine = part_sum;
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) xr[i][s4][bt] = pair_order(xr[i][s4][bt]);
            }
            xs[bt] = mine;
        }
    }
#pragma unroll
    for (int bt = 0; bt < BT; ++bt) asm volatile("" : "+v"(xs[bt]));
    for (int s = 1; s < ahead; ++s) request_tile(t_begin + s, s);

    // ---- ring reads: B operand of group i = 16 bytes of row `col`, piece 4 * i + kc
    unsigned rd_off[GS];
#pragma unroll
    for (int i = 0; i < GS; ++i) {
        const int p = 4 * i + kc;
        if constexpr (GS == 4)
            rd_off[i] = (unsigned)((col >> 2) * 1024 + ((col & 3) * 16 + ((p + col) & 15)) * 16);
        else
            rd_off[i] = (unsigned)((col >> 3) * 1024 + ((col & 7) * 8 + ((p + (col & 7) + (col >> 3)) & 7)) * 16);
    }
    const unsigned sz_rd = (unsigned)(GS * 1024 + col * (GS == 4 ? 8 : 4));

    // exchange of a chunk of CH tiles: this wave's partial sums at red[u][wave][bt][lane];
    // thread -> (batch row bi = 4 * wave + lane / 16, weight row lane % 16) sums the waves
    const unsigned red_wr = red_base + (unsigned)(wave * BT * 1024 + lane * 16);
    const int bi = 4 * wave + kc;
    const unsigned red_rd = red_base + (unsigned)((bi >> 4) * 1024 + (((bi >> 2) & 3) * 16 + col) * 16 + (bi & 3) * 4);
    const bool reducer = BT == 2 || wave < 4;
    constexpr unsigned kRedTile = W * BT * 1024;

    float* pbase = part + (int64_t)j * b * n;  // uniform

    // The waves of a workgroup run on their own through a batch of TM tiles (their x
    // arrives at different times) and keep the tiles' partial sums in registers; only then
    // do they meet, CH tiles at a time.
    int slot = 0;
    for (int s0 = 0; s0 < my_tiles; s0 += TM) {
        float4_t ykeep[TM - CH][BT];  // second half of the batch; the first goes to LDS at once
#pragma unroll
        for (int u = 0; u < TM; ++u) {
            float4_t y[BT];
#pragma unroll
            for (int bt = 0; bt < BT; ++bt) y[bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
            if (u >= CH) {
#pragma unroll
                for (int bt = 0; bt < BT; ++bt) ykeep[u >= CH ? u - CH : 0][bt] = y[bt];
            }
            const int s = s0 + u;
            if (s >= my_tiles) continue;  // uniform
            // requests issued after tile s's: the tiles s+1 .. min(s + ring, my_tiles) - 1
            regx_wait_tiles<kReq>(min(s + ring, my_tiles) - 1 - s);
            uint4_t w[GS];
            unsigned sw[GS / 2], zw[GS / 2];
            const unsigned slot_addr = ring_base + (unsigned)(slot * TB);
            if constexpr (GS == 4) {
                uint2_t s2, z2;
                asm volatile(
                    "ds_read_b128 %0, %6\n\tds_read_b128 %1, %7\n\tds_read_b128 %2, %8\n\t"
                    "ds_read_b128 %3, %9\n\tds_read_b64 %4, %10\n\tds_read_b64 %5, %10 offset:128\n\t"
                    "s_waitcnt lgkmcnt(0)"
                    : "=&v"(w[0]), "=&v"(w[1]), "=&v"(w[2]), "=&v"(w[3]), "=&v"(s2), "=&v"(z2)
                    : "v"(slot_addr + rd_off[0]), "v"(slot_addr + rd_off[1]),
                      "v"(slot_addr + rd_off[2]), "v"(slot_addr + rd_off[3]), "v"(slot_addr + sz_rd)
                    : "memory");
                sw[0] = s2[0], sw[1] = s2[1], zw[0] = z2[0], zw[1] = z2[1];
            } else {
                asm volatile(
                    "ds_read_b128 %0, %4\n\tds_read_b128 %1, %5\n\tds_read_b32 %2, %6\n\t"
                    "ds_read_b32 %3, %6 offset:128\n\ts_waitcnt lgkmcnt(0)"
                    : "=&v"(w[0]), "=&v"(w[1]), "=&v"(sw[0]), "=&v"(zw[0])
                    : "v"(slot_addr + rd_off[0]), "v"(slot_addr + rd_off[1]), "v"(slot_addr + sz_rd)
                    : "memory");
            }
            // the slot is free again: ask for the tile `ring` steps on
            if (s + ring < my_tiles) request_tile(t_begin + s + ring, slot);
            slot = slot + 1 == ring ? 0 : slot + 1;

            // zero-point term: -scale * (128 + zero) of group kc, times the group's sum of x
            {
                const unsigned swk = (GS == 4 && (kc & 2)) ? sw[GS / 2 - 1] : sw[0];
                const unsigned zwk = (GS == 4 && (kc & 2)) ? zw[GS / 2 - 1] : zw[0];
                const unsigned short sh = (unsigned short)((kc & 1) ? (swk >> 16) : (swk & 0xffffu));
                const unsigned short zh = (unsigned short)((kc & 1) ? (zwk >> 16) : (zwk & 0xffffu));
                const float bneg = -__half2float(__builtin_bit_cast(__half, sh)) *
                                   (128.0f + __half2float(__builtin_bit_cast(__half, zh)));
#pragma unroll
                for (int bt = 0; bt < BT; ++bt)
                    y[bt] = __builtin_amdgcn_mfma_f32_16x16x4f32(xs[bt], bneg, y[bt], 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < GS; ++i) {
                const unsigned short sh = (unsigned short)((i & 1) ? (sw[i >> 1] >> 16) : (sw[i >> 1] & 0xffffu));
                const float sf = __half2float(__builtin_bit_cast(__half, sh));
                float4_t acc[BT];
#pragma unroll
                for (int bt = 0; bt < BT; ++bt) acc[bt] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) {
                    const unsigned wd = w[i][s4];
                    uint4_t h;
#pragma unroll
                    for (int sft = 0; sft < 4; ++sft) h[sft] = ((wd >> (4 * sft)) & kNibMask) | magic;
                    const bf16x8_t bop = __builtin_bit_cast(bf16x8_t, h);
#pragma unroll
                    for (int bt = 0; bt < BT; ++bt)
                        acc[bt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8_t, xr[i][s4][bt]), bop, acc[bt], 0, 0, 0);
                }
#pragma unroll
                for (int bt = 0; bt < BT; ++bt)
#pragma unroll
                    for (int e = 0; e < 4; ++e) y[bt][e] = fmaf(sf, acc[bt][e], y[bt][e]);
            }
            if (u < CH) {
                const unsigned dst = red_wr + (unsigned)u * kRedTile;
                if constexpr (BT == 2)
                    asm volatile("ds_write_b128 %0, %1\n\tds_write_b128 %0, %2 offset:1024"
                                 :: "v"(dst), "v"(y[0]), "v"(y[1]) : "memory");
                else
                    asm volatile("ds_write_b128 %0, %1" :: "v"(dst), "v"(y[0]) : "memory");
            } else {
#pragma unroll
                for (int bt = 0; bt < BT; ++bt) ykeep[u >= CH ? u - CH : 0][bt] = y[bt];
            }
        }

        // ---- the eight K slices meet in LDS, CH tiles per exchange
#pragma unroll
        for (int c0 = 0; c0 < TM; c0 += CH) {
            if (s0 + c0 >= my_tiles) break;  // uniform
            if (c0 > 0) {
#pragma unroll
                for (int c = 0; c < TM - CH; ++c) {
                    const unsigned dst = red_wr + (unsigned)c * kRedTile;
                    if constexpr (BT == 2)
                        asm volatile("ds_write_b128 %0, %1\n\tds_write_b128 %0, %2 offset:1024"
                                     :: "v"(dst), "v"(ykeep[c][0]), "v"(ykeep[c][1]) : "memory");
                    else
                        asm volatile("ds_write_b128 %0, %1" :: "v"(dst), "v"(ykeep[c][0]) : "memory");
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            if (reducer) {
#pragma unroll
                for (int c = 0; c < CH; ++c) {
                    const int s = s0 + c0 + c;
                    if (c0 + c >= TM || s >= my_tiles) continue;  // uniform
                    float v0, v1, v2, v3, v4, v5, v6, v7;
                    const unsigned src = red_rd + (unsigned)c * kRedTile;
                    if constexpr (BT == 2)
                        asm volatile(
                            "ds_read_b32 %0, %8\n\tds_read_b32 %1, %8 offset:2048\n\t"
                            "ds_read_b32 %2, %8 offset:4096\n\tds_read_b32 %3, %8 offset:6144\n\t"
                            "ds_read_b32 %4, %8 offset:8192\n\tds_read_b32 %5, %8 offset:10240\n\t"
                            "ds_read_b32 %6, %8 offset:12288\n\tds_read_b32 %7, %8 offset:14336\n\t"
                            "s_waitcnt lgkmcnt(0)"
                            : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3), "=&v"(v4), "=&v"(v5),
                              "=&v"(v6), "=&v"(v7)
                            : "v"(src)
                            : "memory");
                    else
                        asm volatile(
                            "ds_read_b32 %0, %8\n\tds_read_b32 %1, %8 offset:1024\n\t"
                            "ds_read_b32 %2, %8 offset:2048\n\tds_read_b32 %3, %8 offset:3072\n\t"
                            "ds_read_b32 %4, %8 offset:4096\n\tds_read_b32 %5, %8 offset:5120\n\t"
                            "ds_read_b32 %6, %8 offset:6144\n\tds_read_b32 %7, %8 offset:7168\n\t"
                            "s_waitcnt lgkmcnt(0)"
                            : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3), "=&v"(v4), "=&v"(v5),
                              "=&v"(v6), "=&v"(v7)
                            : "v"(src)
                            : "memory");
                    const float sum = ((((((v0 + v1) + v2) + v3) + v4) + v5) + v6) + v7;
                    const int row = (t_begin + s) * 16 + col;
                    if (row < n && bi < b) {
                        if constexpr (PLAIN)
                            reinterpret_cast<unsigned short*>(part)[(unsigned)bi * (unsigned)n + (unsigned)row] =
                                f32_to_bf16_rne(bias ? sum + bias[row] : sum);
                        else
                            pbase[(unsigned)bi * (unsigned)n + (unsigned)row] = sum;
                    }
                }
            }
            // the next exchange writes the same buffers
            __builtin_amdgcn_s_barrier();
        }
    }
}

// The same for 17 .. 32 batch rows on the 32 x 32 x 16 MFMA, which does twice the
// arithmetic of the 16 x 16 x 32 one in the same number of passes: a tile is 32 weight rows,
// lane = (k half, row), and a lane's 16-byte piece feeds four MFMAs.  Per tile and wave:
// 2 * GS ring reads, 8 * GS MFMAs into one 16-register accumulator per group, GS / 2 fp32
// MFMAs (32 x 32 x 2) for the zero-point term.  The first two tiles of a batch of three go to
// the exchange buffers at once, the third waits in registers.
__host__ __device__ constexpr int regx32_tile_bytes(int gs) { return 32 * gs * 64 + 32 * gs * 4; }
__host__ __device__ constexpr int regx32_lds_bytes(int gs, int ring) {
    return kRegxWaves * ring * regx32_tile_bytes(gs) + 2 * kRegxWaves * 4096;
}

typedef float float2_t __attribute__((ext_vector_type(2)));

template <int GS, bool PLAIN>
__global__ __launch_bounds__(64 * kRegxWaves) void qgemm_q4g128_regx32_kernel(
    const uint4_t* __restrict__ xprep, const uint8_t* __restrict__ qw,
    const __half* __restrict__ scale, const __half* __restrict__ zero, float* __restrict__ part,
    int b, int n, int k, int tiles_per_worker, int ring, const float* __restrict__ bias) {
    static_assert(GS == 2 || GS == 4, "slices of 2 or 4 groups");
    constexpr int BP = 32;
    constexpr int W = kRegxWaves;
    constexpr int GW = W * GS;
    constexpr int PIECES = 4 * GS;
    constexpr int RPD = 64 / PIECES;   // rows per weight request
    constexpr int NWR = 32 / RPD;      // weight requests per tile
    constexpr int NSZ = GS / 2;        // scale / zero requests per tile
    constexpr int kReq = NWR + NSZ;
    constexpr int TB = regx32_tile_bytes(GS);
    constexpr int SZ = 32 * GS * 64;   // offset of the scales inside a ring slot
    constexpr int TM = 3, CH = 2;
    constexpr unsigned kRedTile = W * 4096;
    extern __shared__ uint4_t lds[];

    const int groups = k >> 7;
    const int j = blockIdx.y;
    const int tiles = (n + 31) >> 5;
    const int t_begin = blockIdx.x * tiles_per_worker;
    if (t_begin >= tiles) return;
    const int my_tiles = min(tiles, t_begin + tiles_per_worker) - t_begin;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r32 = lane & 31;
    const int kh = lane >> 5;
    const int g0 = j * GW + wave * GS;

    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));

    const unsigned lds_base = (unsigned)(uintptr_t)(lds_ptr_t)lds;
    const unsigned ring_base = lds_base + (unsigned)(wave * ring * TB);
    const unsigned red_base = lds_base + (unsigned)(W * ring * TB);
    char* const ring_ptr = reinterpret_cast<char*>(lds) + wave * ring * TB;

    // ---- ring requests (see the 16-row kernel): request a covers rows a * RPD .. + RPD - 1
    const uint8_t* wbase = qw + (int64_t)g0 * 64;
    const unsigned khalf = (unsigned)(k >> 1);
    const int dr = lane / PIECES;
    const int pos = lane % PIECES;
    auto request_tile = [&](int t, int slot) {
        char* dst = ring_ptr + slot * TB;
#pragma unroll
        for (int a = 0; a < NWR; ++a) {
            const int trow = a * RPD + dr;
            const int rot = GS == 4 ? (trow & 15) : ((dr + (a & 1)) & 7);
            const unsigned poff = (unsigned)((pos - rot) & (PIECES - 1)) * 16u;
            const int row = min(t * 32 + trow, n - 1);
            const uint8_t* src = wbase + ((unsigned)row * khalf + poff);
            __builtin_amdgcn_global_load_lds((glb_ptr_t)src, (lds_ptr_t)(dst + a * 1024), 16, 0, 0);
        }
        if constexpr (GS == 4) {
            // lanes -> (row lane / 2, groups 2 * (lane % 2) ..): scales, then zeros
            const int row = min(t * 32 + (lane >> 1), n - 1);
            const unsigned off = (unsigned)row * (unsigned)groups + (unsigned)(g0 + 2 * (lane & 1));
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(scale + off), (lds_ptr_t)(dst + SZ), 4, 0, 0);
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(zero + off), (lds_ptr_t)(dst + SZ + 256), 4, 0, 0);
        } else {
            const int row = min(t * 32 + r32, n - 1);
            const __half* src = (kh ? zero : scale) + ((unsigned)row * (unsigned)groups + (unsigned)g0);
            __builtin_amdgcn_global_load_lds((glb_ptr_t)src, (lds_ptr_t)(dst + SZ), 4, 0, 0);
        }
    };

    const int ahead = min(ring, my_tiles);
    request_tile(t_begin, 0);

    // ---- x: A operand of MFMA (group i, half h2, dword d) = chunk 16 (g0 + i) + 8 h2 + 4 kh + d
    uint4_t xr[GS][2][4];
    float xs[GS / 2];
    if constexpr (PLAIN) {
        const uint16_t* xrow = reinterpret_cast<const uint16_t*>(xprep) + (int64_t)min(r32, b - 1) * k;
#pragma unroll
        for (int i = 0; i < GS; ++i)
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const uint4_t v = *reinterpret_cast<const uint4_t*>(xrow + 8 * (16 * (g0 + i) + 8 * h2 + 4 * kh + d));
                    xr[i][h2][d] = r32 < b ? v : uint4_t{0u, 0u, 0u, 0u};
                }
    } else {
#pragma unroll
        for (int i = 0; i < GS; ++i)
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
                for (int d = 0; d < 4; ++d)
                    xr[i][h2][d] = xprep[(16 * (g0 + i) + 8 * h2 + 4 * kh + d) * BP + r32];
        const float* xg_src = reinterpret_cast<const float*>(
            reinterpret_cast<const char*>(xprep) + xprep_xg_offset(b, k));
#pragma unroll
        for (int e = 0; e < GS / 2; ++e) xs[e] = xg_src[(g0 + 2 * e + kh) * BP + r32];
    }
#pragma unroll
    for (int i = 0; i < GS; ++i)
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
            for (int d = 0; d < 4; ++d) asm volatile("" : "+v"(xr[i][h2][d]));
    if constexpr (PLAIN) {
        // group sums: this lane holds half of each group's chunks, the lane 32 on the rest
#pragma unroll
        for (int i = 0; i < GS; ++i) {
            float part_sum = 0.0f;
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
                for (int d = 0; d < 4; ++d) part_sum += sum8_bf16(xr[i][h2][d]);
            part_sum += __shfl_xor(part_sum, 32);
            if ((i & 1) == kh) xs[i >> 1] = part_sum;
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
                for (int d = 0; d < 4; ++d) xr[i][h2][d] = pair_order(xr[i][h2][d]);
        }
    }
#pragma unroll
    for (int e = 0; e < GS / 2; ++e) asm volatile("" : "+v"(xs[e]));
    for (int s = 1; s < ahead; ++s) request_tile(t_begin + s, s);

    // ---- ring reads: piece 4 i + 2 h2 + kh of row r32
    unsigned rd_off[GS][2];
#pragma unroll
    for (int i = 0; i < GS; ++i)
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
            const int p = 4 * i + 2 * h2 + kh;
            if constexpr (GS == 4)
                rd_off[i][h2] = (unsigned)((r32 >> 2) * 1024 + ((r32 & 3) * 16 + ((p + (r32 & 15)) & 15)) * 16);
            else
                rd_off[i][h2] = (unsigned)((r32 >> 3) * 1024 + ((r32 & 7) * 8 + ((p + (r32 & 7) + ((r32 >> 3) & 1)) & 7)) * 16);
        }
    const unsigned sz_rd = (unsigned)(SZ + r32 * (GS == 4 ? 8 : 4));

    // exchange: partial sums at red[u][wave][g][lane] (float4: batch rows 8 g + 4 kh + 0..3 of
    // weight row r32); thread -> weight row r32, batch rows 2 * (2 * wave + kh) + 0..1
    const unsigned red_wr = red_base + (unsigned)(wave * 4096 + lane * 16);
    const int m0 = 2 * (2 * wave + kh);
    const unsigned red_rd = red_base + (unsigned)((m0 >> 3) * 1024 + (((m0 >> 2) & 1) * 32 + r32) * 16 + (m0 & 3) * 4);

    float* pbase = part + (int64_t)j * b * n;

    int slot = 0;
    for (int s0 = 0; s0 < my_tiles; s0 += TM) {
        float16_t ykeep;
#pragma unroll
        for (int v = 0; v < 16; ++v) ykeep[v] = 0.0f;
#pragma unroll
        for (int u = 0; u < TM; ++u) {
            const int s = s0 + u;
            if (s >= my_tiles) continue;  // uniform
            regx_wait_tiles<kReq>(min(s + ring, my_tiles) - 1 - s);
            uint4_t w[GS][2];
            unsigned sw[GS / 2], zw[GS / 2];
            const unsigned slot_addr = ring_base + (unsigned)(slot * TB);
            if constexpr (GS == 4) {
                uint2_t s2, z2;
                asm volatile(
                    "ds_read_b128 %0, %10\n\tds_read_b128 %1, %11\n\tds_read_b128 %2, %12\n\t"
                    "ds_read_b128 %3, %13\n\tds_read_b128 %4, %14\n\tds_read_b128 %5, %15\n\t"
                    "ds_read_b128 %6, %16\n\tds_read_b128 %7, %17\n\tds_read_b64 %8, %18\n\t"
                    "ds_read_b64 %9, %18 offset:256\n\ts_waitcnt lgkmcnt(0)"
                    : "=&v"(w[0][0]), "=&v"(w[0][1]), "=&v"(w[1][0]), "=&v"(w[1][1]), "=&v"(w[2][0]),
                      "=&v"(w[2][1]), "=&v"(w[3][0]), "=&v"(w[3][1]), "=&v"(s2), "=&v"(z2)
                    : "v"(slot_addr + rd_off[0][0]), "v"(slot_addr + rd_off[0][1]),
                      "v"(slot_addr + rd_off[1][0]), "v"(slot_addr + rd_off[1][1]),
                      "v"(slot_addr + rd_off[2][0]), "v"(slot_addr + rd_off[2][1]),
                      "v"(slot_addr + rd_off[3][0]), "v"(slot_addr + rd_off[3][1]),
                      "v"(slot_addr + sz_rd)
                    : "memory");
                sw[0] = s2[0], sw[1] = s2[1], zw[0] = z2[0], zw[1] = z2[1];
            } else {
                asm volatile(
                    "ds_read_b128 %0, %6\n\tds_read_b128 %1, %7\n\tds_read_b128 %2, %8\n\t"
                    "ds_read_b128 %3, %9\n\tds_read_b32 %4, %10\n\tds_read_b32 %5, %10 offset:128\n\t"
                    "s_waitcnt lgkmcnt(0)"
                    : "=&v"(w[0][0]), "=&v"(w[0][1]), "=&v"(w[1][0]), "=&v"(w[1][1]), "=&v"(sw[0]),
                      "=&v"(zw[0])
                    : "v"(slot_addr + rd_off[0][0]), "v"(slot_addr + rd_off[0][1]),
                      "v"(slot_addr + rd_off[1][0]), "v"(slot_addr + rd_off[1][1]),
                      "v"(slot_addr + sz_rd)
                    : "memory");
            }
            if (s + ring < my_tiles) request_tile(t_begin + s + ring, slot);
            slot = slot + 1 == ring ? 0 : slot + 1;

            float16_t y;
#pragma unroll
            for (int v = 0; v < 16; ++v) y[v] = 0.0f;
            // zero-point term: groups 2 e + kh
#pragma unroll
            for (int e = 0; e < GS / 2; ++e) {
                const unsigned short sh = (unsigned short)(kh ? (sw[e] >> 16) : (sw[e] & 0xffffu));
                const unsigned short zh = (unsigned short)(kh ? (zw[e] >> 16) : (zw[e] & 0xffffu));
                const float bneg = -__half2float(__builtin_bit_cast(__half, sh)) *
                                   (128.0f + __half2float(__builtin_bit_cast(__half, zh)));
                y = __builtin_amdgcn_mfma_f32_32x32x2f32(xs[e], bneg, y, 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < GS; ++i) {
                const unsigned short sh = (unsigned short)((i & 1) ? (sw[i >> 1] >> 16) : (sw[i >> 1] & 0xffffu));
                const float sf = __half2float(__builtin_bit_cast(__half, sh));
                float16_t acc;
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
#pragma unroll
                for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        const unsigned wd = w[i][h2][d];
                        uint4_t h;
#pragma unroll
                        for (int sft = 0; sft < 4; ++sft) h[sft] = ((wd >> (4 * sft)) & kNibMask) | magic;
                        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(bf16x8_t, xr[i][h2][d]), __builtin_bit_cast(bf16x8_t, h),
                            acc, 0, 0, 0);
                    }
#pragma unroll
                for (int v = 0; v < 16; ++v) y[v] = fmaf(sf, acc[v], y[v]);
            }
            if (u < CH) {
                const unsigned dst = red_wr + (unsigned)u * kRedTile;
                asm volatile(
                    "ds_write_b128 %0, %1\n\tds_write_b128 %0, %2 offset:1024\n\t"
                    "ds_write_b128 %0, %3 offset:2048\n\tds_write_b128 %0, %4 offset:3072"
                    :: "v"(dst), "v"(__builtin_shufflevector(y, y, 0, 1, 2, 3)),
                       "v"(__builtin_shufflevector(y, y, 4, 5, 6, 7)),
                       "v"(__builtin_shufflevector(y, y, 8, 9, 10, 11)),
                       "v"(__builtin_shufflevector(y, y, 12, 13, 14, 15))
                    : "memory");
            } else {
                ykeep = y;
            }
        }

        // ---- the eight K slices meet in LDS: tiles 0, 1 of the batch, then tile 2
#pragma unroll
        for (int c0 = 0; c0 < TM; c0 += CH) {
            if (s0 + c0 >= my_tiles) break;  // uniform
            if (c0 > 0)
                asm volatile(
                    "ds_write_b128 %0, %1\n\tds_write_b128 %0, %2 offset:1024\n\t"
                    "ds_write_b128 %0, %3 offset:2048\n\tds_write_b128 %0, %4 offset:3072"
                    :: "v"(red_wr), "v"(__builtin_shufflevector(ykeep, ykeep, 0, 1, 2, 3)),
                       "v"(__builtin_shufflevector(ykeep, ykeep, 4, 5, 6, 7)),
                       "v"(__builtin_shufflevector(ykeep, ykeep, 8, 9, 10, 11)),
                       "v"(__builtin_shufflevector(ykeep, ykeep, 12, 13, 14, 15))
                    : "memory");
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const int s = s0 + c0 + c;
                if (c0 + c >= TM || s >= my_tiles) continue;  // uniform
                float2_t v0, v1, v2, v3, v4, v5, v6, v7;
                asm volatile(
                    "ds_read_b64 %0, %8\n\tds_read_b64 %1, %8 offset:4096\n\t"
                    "ds_read_b64 %2, %8 offset:8192\n\tds_read_b64 %3, %8 offset:12288\n\t"
                    "ds_read_b64 %4, %8 offset:16384\n\tds_read_b64 %5, %8 offset:20480\n\t"
                    "ds_read_b64 %6, %8 offset:24576\n\tds_read_b64 %7, %8 offset:28672\n\t"
                    "s_waitcnt lgkmcnt(0)"
                    : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3), "=&v"(v4), "=&v"(v5), "=&v"(v6),
                      "=&v"(v7)
                    : "v"(red_rd + (unsigned)c * kRedTile)
                    : "memory");
                const float2_t sum = ((((((v0 + v1) + v2) + v3) + v4) + v5) + v6) + v7;
                const int row = (t_begin + s) * 32 + r32;
                if (row < n) {
                    if constexpr (PLAIN) {
                        unsigned short* y = reinterpret_cast<unsigned short*>(part);
                        const float bv = bias ? bias[row] : 0.0f;
                        if (m0 < b)
                            y[(unsigned)m0 * (unsigned)n + (unsigned)row] = f32_to_bf16_rne(sum[0] + bv);
                        if (m0 + 1 < b)
                            y[(unsigned)(m0 + 1) * (unsigned)n + (unsigned)row] =
                                f32_to_bf16_rne(sum[1] + bv);
                    } else {
                        if (m0 < b) pbase[(unsigned)m0 * (unsigned)n + (unsigned)row] = sum[0];
                        if (m0 + 1 < b) pbase[(unsigned)(m0 + 1) * (unsigned)n + (unsigned)row] = sum[1];
                    }
                }
            }
            // the next exchange writes the same buffers
            __builtin_amdgcn_s_barrier();
        }
    }
}

template <int GS, bool PLAIN>
static hipError_t launch_regx32(const void* xprep, const void* qw, const void* scale,
                                const void* zero, void* part, const float* bias, int b, int n, int k,
                                int tpw, int ring, hipStream_t stream) {
    const int tiles = (n + 31) / 32;
    const size_t lds = (size_t)regx32_lds_bytes(GS, ring);
    auto kern = qgemm_q4g128_regx32_kernel<GS, PLAIN>;
    static const hipError_t opt = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
        160 * 1024);
    if (opt != hipSuccess) return opt;
    dim3 grid((tiles + tpw - 1) / tpw, (k / 128) / (kRegxWaves * GS));
    kern<<<grid, dim3(64 * kRegxWaves), lds, stream>>>(
        static_cast<const uint4_t*>(xprep), static_cast<const uint8_t*>(qw),
        static_cast<const __half*>(scale), static_cast<const __half*>(zero),
        static_cast<float*>(part), b, n, k, tpw, ring, bias);
    return hipGetLastError();
}

static hipError_t qgemm_q4_regx32_launch(const void* xprep, const void* qw, const void* scale,
                                         const void* zero, void* part, const float* bias, int b, int n,
                                         int k, int gs, int tpw, int ring, bool plain,
                                         hipStream_t stream) {
    if (gs != 2 && gs != 4) return hipErrorInvalidValue;
    if (b <= 16 || b > 32) return hipErrorInvalidValue;
    if ((k / 128) % (kRegxWaves * gs) != 0 || tpw < 1 || ring < 1 || ring > kRegxMaxRing)
        return hipErrorInvalidValue;
    if (regx32_lds_bytes(gs, ring) > 160 * 1024) return hipErrorInvalidValue;
    if (plain) {
        if (gs == 2) return launch_regx32<2, true>(xprep, qw, scale, zero, part, bias, b, n, k, tpw, ring, stream);
        return launch_regx32<4, true>(xprep, qw, scale, zero, part, bias, b, n, k, tpw, ring, stream);
    }
    if (gs == 2) return launch_regx32<2, false>(xprep, qw, scale, zero, part, bias, b, n, k, tpw, ring, stream);
    return launch_regx32<4, false>(xprep, qw, scale, zero, part, bias, b, n, k, tpw, ring, stream);
}

template <int BT, int GS, bool PLAIN>
static hipError_t launch_regx(const void* xprep, const void* qw, const void* scale,
                              const void* zero, void* part, const float* bias, int b, int n, int k,
                              int tpw, int ring, hipStream_t stream) {
    const int tiles = (n + 15) / 16;
    const size_t lds = (size_t)regx_lds_bytes(BT, GS, ring);
    auto kern = qgemm_q4g128_regx_kernel<BT, GS, PLAIN>;
    static const hipError_t opt = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
        160 * 1024);
    if (opt != hipSuccess) return opt;
    dim3 grid((tiles + tpw - 1) / tpw, (k / 128) / (kRegxWaves * GS));
    kern<<<grid, dim3(64 * kRegxWaves), lds, stream>>>(
        static_cast<const uint4_t*>(xprep), static_cast<const uint8_t*>(qw),
        static_cast<const __half*>(scale), static_cast<const __half*>(zero),
        static_cast<float*>(part), b, n, k, tpw, ring, bias);
    return hipGetLastError();
}

static hipError_t qgemm_q4_regx16_launch(const void* xprep, const void* qw, const void* scale,
                                         const void* zero, void* part, const float* bias, int b, int n,
                                         int k, int gs, int tpw, int ring, bool plain,
                                         hipStream_t stream) {
    if (gs != 2 && gs != 4) return hipErrorInvalidValue;
    if (b < 1 || b > 16) return hipErrorInvalidValue;
    if ((k / 128) % (kRegxWaves * gs) != 0 || tpw < 1 || ring < 1 || ring > kRegxMaxRing)
        return hipErrorInvalidValue;
    if (regx_lds_bytes(1, gs, ring) > 160 * 1024) return hipErrorInvalidValue;
    if (plain) {
        if (gs == 2) return launch_regx<1, 2, true>(xprep, qw, scale, zero, part, bias, b, n, k, tpw, ring, stream);
        return launch_regx<1, 4, true>(xprep, qw, scale, zero, part, bias, b, n, k, tpw, ring, stream);
    }
    if (gs == 2) return launch_regx<1, 2, false>(xprep, qw, scale, zero, part, bias, b, n, k, tpw, ring, stream);
    return launch_regx<1, 4, false>(xprep, qw, scale, zero, part, bias, b, n, k, tpw, ring, stream);
}

// Shapes the kernels above take, and how: K a multiple of 2048 (slices of two groups, two
// parts per 4096 columns) or, for longer rows, of 4096 (slices of four groups); batches
// from 3 rows (below that the split-K kernel's VALU path is the faster one) and matrices
// of at least 1024 rows.  Measured at batch 32 on 24576 x 4096, 4096 x 12288, 6144 x 4096
// and 4096 x 4096: slices of two groups win up to K = 4096, four beyond; a ring deeper than
// one tile (two for the 16-row kernel's short slices) gains nothing.
RegxPlan regx_plan(int b, int n, int k) {
    RegxPlan p{0, 0, 0, 0, 0};
    const int groups = k / 128;
    if (b < 3 || b > 32 || n < 1024 || k % 128 != 0) return p;
    int gs = 0;
    if (k <= 4096 && groups % (kRegxWaves * 2) == 0) gs = 2;
    else if (groups % (kRegxWaves * 4) == 0) gs = 4;
    else if (groups % (kRegxWaves * 2) == 0) gs = 2;
    if (gs == 0) return p;
    p.gs = gs;
    p.parts = groups / (kRegxWaves * gs);
    p.rows = b <= 16 ? 16 : 32;
    p.ring = (p.rows == 16 && gs == 2) ? 2 : 1;
    const int tiles = (n + p.rows - 1) / p.rows;
    const int columns = device_cu_count() / p.parts > 0 ? device_cu_count() / p.parts : 1;
    p.tpw = (tiles + columns - 1) / columns;
    return p;
}

// The same kernels reading x as a plain bf16 matrix and writing the bf16 product: possible
// where one workgroup covers all of K (K = 2048 or 4096), so that there is a single part.
RegxPlan regx_plain_plan(int b, int n, int k) {
    RegxPlan p{0, 0, 0, 0, 0};
    if (k != 2048 && k != 4096) return p;
    if (b < 2 || b > 32 || n < 1024) return p;
    // batch 2: the VALU GEMV stays ahead on small matrices (4096 x 4096: 5.5 vs 6.2 us), this
    // kernel on large ones (12288 x 4096: 8.6 vs 9.6 us, 24576 x 4096: 13.0 vs 16.3 us)
    if (b == 2 && (int64_t)n * k < 40000000) return p;
    p.gs = k / 1024;
    p.parts = 1;
    p.rows = b <= 16 ? 16 : 32;
    p.ring = (p.rows == 16 && p.gs == 2) ? 2 : 1;
    const int tiles = (n + p.rows - 1) / p.rows;
    const int columns = device_cu_count();
    p.tpw = (tiles + columns - 1) / columns;
    return p;
}

hipError_t qgemm_q4_regx_launch(const RegxPlan& p, const void* xprep, const void* qw,
                                const void* scale, const void* zero, void* part, int b, int n,
                                int k, hipStream_t stream) {
    if (p.rows == 32)
        return qgemm_q4_regx32_launch(xprep, qw, scale, zero, part, nullptr, b, n, k, p.gs, p.tpw,
                                      p.ring, false, stream);
    return qgemm_q4_regx16_launch(xprep, qw, scale, zero, part, nullptr, b, n, k, p.gs, p.tpw, p.ring,
                                  false, stream);
}

hipError_t qgemm_q4_regx_plain_launch(const RegxPlan& p, const void* x_bf16, const void* qw,
                                      const void* scale, const void* zero, void* y_bf16,
                                      const float* bias, int b, int n, int k,
                                      hipStream_t stream) {
    if (p.parts != 1) return hipErrorInvalidValue;
    if (p.rows == 32)
        return qgemm_q4_regx32_launch(x_bf16, qw, scale, zero, y_bf16, bias, b, n, k, p.gs, p.tpw,
                                      p.ring, true, stream);
    return qgemm_q4_regx16_launch(x_bf16, qw, scale, zero, y_bf16, bias, b, n, k, p.gs, p.tpw, p.ring,
                                  true, stream);
}

}  // namespace lg

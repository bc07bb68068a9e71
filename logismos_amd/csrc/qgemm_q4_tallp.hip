// Q4G128 GEMM for a tall x over a workspace: the tiled kernel of qgemm_q4_tall.hip with the
// work that does not belong in its inner loop taken out of it.
//   y[m][n] = sum_k x[m][k] * (q[n][k] - zero[n][k/128]) * scale[n][k/128] (+ bias[n])
// `cpu_f32::linear_t` (crates/kernels/src/cpu_f32/mod.rs:271-345) at m = hundreds to thousands
// of rows over the dequantised matrix.
//
// Counters of the workspace-less kernel show its vector pipe, not its matrix pipe, setting the
// pace: per 32 MFMAs a wave issues ~500 vector instructions -- the nibble unpack (112), the
// staging of x through registers into LDS with the pair-order permute and the group sums
// (~130), and two multiply-adds per result and group for scale and zero point (128).  Here:
//
// * a first pass (`q4_tall_prepare_kernel`, x read once, ~1 % of the product's time) writes x
//   in the order the nibble unpack produces ("pair order": (x0,x4)(x1,x5)(x2,x6)(x3,x7) per
//   16-byte chunk), rows padded with zeros to a multiple of 128, and every row's sum over each
//   group of 128 columns;
// * the product kernel (128 x 256 tiles, eight waves of 64 x 64, one workgroup per CU) moves
//   a group's 128 x 128 slab of that copy and its 256 x 128 tile of nibbles from global
//   memory STRAIGHT into LDS (global_load_lds, 16 bytes per lane, no registers, no vector
//   instructions) into a ring of three buffers, requested two groups ahead, one barrier per
//   group.  A request writes 1 KiB of consecutive LDS, so instead of padding rows the
//   16-byte chunks of a row are stored XOR-swizzled by the row index and the ds_read_b128 of
//   the MFMA operands stay conflict-free;
// * scales, zeros and the group sums of x reach a lane's registers for four (or two) pairs
//   of groups per load where K allows: a lane's row of scales is 64 bytes apart from the
//   next lane's, so each such load costs the address path a cache line per lane -- one per
//   pair and array, they took it twice as long as the tiles themselves and held every wave
//   up behind each barrier.  The first pass writes the group sums in the layout these loads
//   want ([row tile][block of pairs][group's place in its pair][row][pair]);
// * the zero-point term -scale * (128 + zero) * sum_x is a rank-(K/128) product of its own:
//   one v_mfma_f32_32x32x2_f32 per output tile and PAIR of groups, accumulating into the same
//   registers, in place of a multiply-add per result and group;
// * what is left per group and wave: the unpack (a lane of the v_mfma_f32_32x32x16_bf16 B
//   operand is one weight row and one dword of nibbles, made bf16 `128 + q` with an and-or per
//   pair, exact), one multiply-add per result for the group's scale, 32 MFMAs.
//
// * workgroups all take the same time and a CU holds one, so a launch whose tile count is not
//   a multiple of the CU count ends on a round that leaves most CUs idle (config 4's o and
//   down projections: 1040 tiles on 256 CUs, a fifth round for 16 tiles).  The tiles of that
//   last partial round are split over K into parts, one workgroup each, that write fp32
//   partial tiles into the workspace; `q4_tall_reduce_kernel` sums a tile's parts in part
//   order (deterministic), adds the bias and writes y.  A launch of fewer tiles than CUs is
//   all "last round": the split also fills the device at a few hundred rows.
//
// LDS is only touched through inline assembly inside the loop: the compiler would order
// every LDS access it can see behind all outstanding global_load_lds.
#include "device_utils.hpp"
#include "launch_common.hpp"
#include "q4_common.hpp"

#include <hip/hip_fp16.h>

namespace lg {

typedef __attribute__((address_space(3))) void* tp_lds_ptr_t;
typedef const __attribute__((address_space(1))) void* tp_glb_ptr_t;

constexpr int kTpTileM = 128;             // rows of x per workgroup
constexpr int kTpTileN = 256;             // weight rows per workgroup
constexpr int kTpSlabBytes = 128 * 256;   // one group's slab of x: 128 rows x 128 bf16
constexpr int kTpWBytes = 256 * 64;       // one group's tile of weights: 256 rows x 128 nibbles
constexpr int kTpBufBytes = kTpSlabBytes + kTpWBytes;
constexpr int kTpBufs = 3;                // groups in LDS: one in use, two on their way

constexpr int kTpTileElems = kTpTileM * kTpTileN;
constexpr int kTpMaxParts = 512;          // partial tiles the workspace holds (fp32, 128 KiB each)
constexpr int kTpMinGroupsPerPart = 4;    // a part of a tile takes at least four groups of K

static_assert(kTpTileM == kTallTileRows, "the layout helpers of q4_common.hpp are for this tile");
__host__ __device__ inline int tp_padded_rows(int m) { return tall_padded_rows(m); }
__host__ __device__ inline size_t tp_sums_offset(int m, int k) { return tall_sums_offset(m, k); }
__host__ __device__ inline size_t tp_partials_offset(int m, int k) {
    return (tp_sums_offset(m, k) + (size_t)tp_padded_rows(m) * (k / 128) * 4 + 255) & ~(size_t)255;
}

// How a launch of `tiles` workgroup tiles is laid over `cus` CUs: the first `full` tiles whole,
// the other `tiles - full` (the last, partial round) in `split` parts over K each.
struct TpPlan {
    int full, split;
};
inline TpPlan tp_plan(int tiles, int groups, int block_groups, int cus) {
    const int rem = tiles % cus;
    TpPlan p{tiles, 1};
    if (rem == 0) return p;
    int split = cus / rem;
    // parts are whole blocks of the kernel's small loads and at least four groups
    const int most = groups / (block_groups > kTpMinGroupsPerPart ? block_groups : kTpMinGroupsPerPart);
    if (split > most) split = most;
    if (split > 1 && rem * split <= kTpMaxParts) p = TpPlan{tiles - rem, split};
    return p;
}

// x [m][k] bf16 -> xp [m_pad][k] bf16 in pair order (rows >= m: zeros), xs: the fp32 sum of the
// bf16 values of every row and group, laid out for the product kernel's loads as
// [row tile of 128][block of w pairs of groups][group's place in its pair][row][pair].
// One thread per 16-byte chunk; the 16 lanes of a row of lanes hold one group of one row.
__global__ __launch_bounds__(256) void q4_tall_prepare_kernel(const uint16_t* __restrict__ x,
                                                             uint16_t* __restrict__ xp,
                                                             float* __restrict__ xs, int m,
                                                             int m_pad, int k, int w) {
    const int64_t chunks_per_row = k >> 3;
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= (int64_t)m_pad * chunks_per_row) return;  // (whole rows of 16 lanes: k % 128 == 0)
    const int64_t row = id / chunks_per_row;
    const int64_t c = id - row * chunks_per_row;
    uint4_t v = {0u, 0u, 0u, 0u};
    if (row < m) v = *reinterpret_cast<const uint4_t*>(x + row * k + c * 8);
    const float gs = row16_sum(sum8_bf16(v));
    *reinterpret_cast<uint4_t*>(xp + row * k + c * 8) = pair_order(v);
    if ((threadIdx.x & 15) == 0) xs[tall_sum_index(row, (int)(c >> 4), k, w)] = gs;
}

// W values a lane loads at once, as one register operand of an assembly statement: a vector
// of W, or the plain value for W = 1 (a vector of one is no register operand).
template <typename T, int W>
struct TpRegs {
    typedef T raw_t __attribute__((ext_vector_type(W)));
    raw_t raw;
    __device__ __forceinline__ T operator[](int i) const { return raw[i]; }
};
template <typename T>
struct TpRegs<T, 1> {
    typedef T raw_t;
    raw_t raw;
    __device__ __forceinline__ T operator[](int) const { return raw; }
};

// What a launch writes.  kTpOutSwiglu: the weights are a gate/up pair [gate rows | up rows]
// (2 n rows) and y [m][n] is bf16 silu(gate) * up -- a workgroup tile takes 128 gate rows and
// the 128 up rows of the same outputs, a wave's first 32 columns the gate and its other 32 the
// up values of the same 32 outputs, so a lane holds both products of a result and the fp32
// gate/up products (a gigabyte at 8240 rows of a 12288-wide MLP) never go to memory.
// kTpOutSwigluOperand: the same product, written as the operand of a following launch of this
// kernel over K = n (n a multiple of 256): y is that launch's workspace -- the bf16 values in
// pair order, rows up to the padded count (the padding rows of x are zeros, and so are their
// activations), and the group sums (a tile's 128 outputs are one group), added up in the order
// of the first pass (`q4_tall_prepare_kernel`), so that the workspace is bit for bit what that
// pass makes of the bf16 activations.
constexpr int kTpOutBf16 = 0, kTpOutF32 = 1, kTpOutSwiglu = 2, kTpOutSwigluOperand = 3;
__host__ __device__ constexpr bool tp_is_swiglu(int out) { return out >= kTpOutSwiglu; }

// 16-bit slot of element j of a 16-byte chunk in pair order ((x0,x4)(x1,x5)(x2,x6)(x3,x7))
__device__ __forceinline__ int tp_pair_slot(int j) { return 2 * (j & 3) + (j >> 2); }

// The sum of a chunk's eight values as `sum8_bf16` adds them, for values that sit one per lane
// in eight consecutive lanes (x_j in lane 8 c + j): the chunk's first lane gets
// (((0 + (x0 + x1)) + (x2 + x3)) + (x4 + x5)) + (x6 + x7).
__device__ __forceinline__ float tp_chunk_sum_across_lanes(float v) {
    const float p = v + __shfl_down(v, 1, 64);  // x_j + x_(j+1): even j count
    float s = 0.0f + p;
    s += __shfl_down(p, 2, 64);
    s += __shfl_down(p, 4, 64);
    s += __shfl_down(p, 6, 64);
    return s;
}
// ... and of a row's 16 chunk sums as `row16_sum` adds them (chunk c with c + 8, those with
// the pair of c + 4, then c + 2, then c + 1), from sums[wave column wq = c / 4][c % 4]
__device__ __forceinline__ float tp_group_sum(const float (&cs)[4][4]) {
    float quad[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) quad[q] = (cs[0][q] + cs[2][q]) + (cs[1][q] + cs[3][q]);
    return (quad[0] + quad[2]) + (quad[1] + quad[3]);
}

// W: pairs of groups whose scales, zeros and group sums a lane loads at once (1, 2 or 4: a
// dword, two or four per load; K a multiple of 256 W).
template <int OUT, int W>
__global__ __launch_bounds__(512) void qgemm_q4g128_tallp_kernel(
    const uint16_t* __restrict__ xp, const float* __restrict__ xs, const uint8_t* __restrict__ qw,
    const __half* __restrict__ scale, const __half* __restrict__ zero,
    const float* __restrict__ bias, void* __restrict__ y_out, float* __restrict__ partials, int m,
    int n, int k, int tiles_n, int full_tiles, int split, int out_pairs) {
    extern __shared__ uint4_t tp_lds[];  // kTpBufs x {slab of x, tile of weights}
    constexpr int BL = 2 * W;            // groups per block of small loads
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31;
    const int h = lane >> 5;
    // workgroup -> tile (columns fastest) and, past the whole tiles, part of a tile: groups
    // [g_begin, groups) of K, both multiples of BL
    int tile = blockIdx.x, part = -1;
    int g_begin = 0, groups = k >> 7;
    if (tile >= full_tiles) {
        const int p = tile - full_tiles;
        tile = full_tiles + p / split;
        part = p;
        const int blocks = groups / BL, q = p % split;
        g_begin = BL * (int)((int64_t)blocks * q / split);
        groups = BL * (int)((int64_t)blocks * (q + 1) / split);
    }
    const int row_tile = tile / tiles_n;
    const int row0 = row_tile * kTpTileM;
    // (SwiGLU: a tile is 128 outputs wide -- 128 gate and 128 up rows of the weights)
    constexpr int kTileOutputs = tp_is_swiglu(OUT) ? kTpTileN / 2 : kTpTileN;
    const int col0 = (tile % tiles_n) * kTileOutputs;
    // weight row behind row L of the tile in LDS (a wave's B operand rows are L = wc + 32 j + r)
    auto weight_row = [&](int L) {
        if constexpr (tp_is_swiglu(OUT)) {
            const int out_col = min(col0 + (L >> 6) * 32 + (L & 31), n - 1);
            return ((L >> 5) & 1) ? n + out_col : out_col;
        } else {
            return min(col0 + L, n - 1);  // a row past n re-reads the last row
        }
    };
    const int wr = (wave >> 2) * 64;  // this wave's 64 x 64 part of the 128 x 256 tile
    const int wc = (wave & 3) * 64;
    const int groups_row = k >> 7;    // scales and zeros: groups per weight row
    unsigned magic;
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));
    const unsigned lds_base = (unsigned)(uintptr_t)(tp_lds_ptr_t)tp_lds;

    // ---- requests of a group, straight into LDS (a request writes 1 KiB of consecutive LDS).
    // x: request q of this wave covers rows 16 wave + 4 q .. + 3, lane -> row + lane / 16, LDS
    // position lane % 16 of that row, which holds the row's chunk (position ^ row % 16).
    // weights: request q covers rows 32 wave + 16 q .. + 15 of the tile, lane -> row + lane / 4,
    // position lane % 4 of the row's 64 bytes, which holds piece (position ^ (row / 4) % 4).
    // Byte offsets fit 32 bits (m_pad * K * 2 and N * K < 2^31 are checked on the host).
    unsigned xoff[4], woff[2];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int row = 16 * wave + 4 * q + (lane >> 4);
        const int c = (lane & 15) ^ (row & 15);
        xoff[q] = ((unsigned)(row0 + row) * (unsigned)k + (unsigned)c * 8u) * 2u;
    }
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const int row = 32 * wave + 16 * q + (lane >> 2);
        const int piece = (lane & 3) ^ ((row >> 2) & 3);
        woff[q] = (unsigned)weight_row(row) * (unsigned)(k >> 1) + (unsigned)piece * 16u;
    }
    // As assembly: the 32-bit offsets above with a scalar base (the builtin widens each to a
    // 64-bit address in two more registers); M0 holds the LDS address of lane 0's 16 bytes and
    // nothing else in this kernel uses M0.
    auto request_group = [&](int g, int buf_off) {
        const char* xsrc = reinterpret_cast<const char*>(xp) + (size_t)g * 256;
        const char* wsrc = reinterpret_cast<const char*>(qw) + (size_t)g * 64;
        // (scalar registers for sure: a value the compiler takes for lane-dependent would be
        // handed to the statement in vector registers)
        const unsigned xdst = __builtin_amdgcn_readfirstlane(lds_base + (unsigned)buf_off +
                                                             (unsigned)wave * 4096u);
        const unsigned wdst = xdst + kTpSlabBytes - (unsigned)wave * 2048u;
        asm volatile(
            "s_mov_b32 m0, %8\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %6\n\t"
            "s_add_u32 m0, %8, 0x400\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %6\n\t"
            "s_add_u32 m0, %8, 0x800\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %6\n\t"
            "s_add_u32 m0, %8, 0xc00\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %3, %6\n\t"
            "s_mov_b32 m0, %9\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %7\n\t"
            "s_add_u32 m0, %9, 0x400\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %5, %7"
            :
            : "v"(xoff[0]), "v"(xoff[1]), "v"(xoff[2]), "v"(xoff[3]), "v"(woff[0]), "v"(woff[1]),
              "s"(xsrc), "s"(wsrc), "s"(xdst), "s"(wdst)
            : "memory", "scc");
    };
    constexpr int kReq = 6;  // requests per group and wave
    // ---- A operand reads: lane (r, h) at step s8 wants chunk 8 h + s8 of row wr + 32 i + r,
    // stored at position (8 h + s8) ^ (r % 16): a0 ^ (s8 << 4), the i-tile as an immediate
    // (a buffer's offset in the ring is a multiple of 16 KiB: adding it commutes with the XOR)
    const unsigned a0 = lds_base + (unsigned)(wr + r) * 256u +
                        (unsigned)(((8 * h) ^ (r & 8)) | (r & 7)) * 16u;
    // ---- B operand reads: lane (r, h) of n-tile j wants the pieces 2 h, 2 h + 1 of row
    // wc + 32 j + r (dword s8 % 4 of piece 2 h + s8 / 4 feeds step s8); j as an immediate
    unsigned b_addr[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
        b_addr[t] = lds_base + kTpSlabBytes + (unsigned)(wc + r) * 64u +
                    (unsigned)((2 * h + t) ^ ((r >> 2) & 3)) * 16u;

    // ---- The small loads of a block of W pairs of groups, from global memory into registers:
    // scales and zeros of this lane's two weight rows (a lane's 16 results of a tile belong to
    // one weight row; pair p in dword p: group 2 p in the low half), and the group sums of x
    // for the zero-point product (lane (r, h) holds row wr + 32 i + r, group 2 p + h of pair
    // p; the first pass wrote them as [row tile][block][h][row][p], so a wave reads 512
    // consecutive bytes x W).  Six loads per block and wave, written as assembly with the
    // wait for them spelled out below, once per block: for loads it can see the compiler
    // waits with vmcnt(0) wherever a value is used, in every group, which also waits for
    // every request of the groups ahead and takes the ring's depth away.  A register loaded
    // here must not be touched before `small_loads_landed` has named it.
    struct Small {
        TpRegs<unsigned, W> s[2], z[2];
        TpRegs<float, W> xs[2];
    };
    unsigned soff[2], xsoff[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
        soff[j] = (unsigned)weight_row(wc + 32 * j + r) * (unsigned)groups_row * 2u;
#pragma unroll
    for (int i = 0; i < 2; ++i) xsoff[i] = (unsigned)((h * kTpTileM + wr + 32 * i + r) * W) * 4u;
    auto gload_small = [&](int g, Small& v) {
        const __half* sb = scale + g;
        const __half* zb = zero + g;
        const float* xb = xs + ((size_t)row_tile * (groups_row / BL) + g / BL) * (2 * kTpTileM * W);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if constexpr (W == 1) {
                asm volatile("global_load_dword %0, %1, %2" : "=&v"(v.s[j].raw) : "v"(soff[j]), "s"(sb) : "memory");
                asm volatile("global_load_dword %0, %1, %2" : "=&v"(v.z[j].raw) : "v"(soff[j]), "s"(zb) : "memory");
            } else if constexpr (W == 2) {
                asm volatile("global_load_dwordx2 %0, %1, %2" : "=&v"(v.s[j].raw) : "v"(soff[j]), "s"(sb) : "memory");
                asm volatile("global_load_dwordx2 %0, %1, %2" : "=&v"(v.z[j].raw) : "v"(soff[j]), "s"(zb) : "memory");
            } else {
                asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(v.s[j].raw) : "v"(soff[j]), "s"(sb) : "memory");
                asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(v.z[j].raw) : "v"(soff[j]), "s"(zb) : "memory");
            }
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if constexpr (W == 1)
                asm volatile("global_load_dword %0, %1, %2" : "=&v"(v.xs[i].raw) : "v"(xsoff[i]), "s"(xb) : "memory");
            else if constexpr (W == 2)
                asm volatile("global_load_dwordx2 %0, %1, %2" : "=&v"(v.xs[i].raw) : "v"(xsoff[i]), "s"(xb) : "memory");
            else
                asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(v.xs[i].raw) : "v"(xsoff[i]), "s"(xb) : "memory");
        }
    };
    // Waits for everything this wave has outstanding and hands the registers over.  (Not
    // "at most the requests issued behind them": whether loads into registers and requests
    // into LDS complete in order with each other is not relied on.  The requests of the group
    // after next, issued most of a group ago, are waited for with them -- once per block.)
    auto small_loads_landed = [&](Small& v) {
        asm volatile("s_waitcnt vmcnt(0)"
                     : "+v"(v.s[0].raw), "+v"(v.s[1].raw), "+v"(v.z[0].raw), "+v"(v.z[1].raw),
                       "+v"(v.xs[0].raw), "+v"(v.xs[1].raw)
                     :
                     : "memory");
    };
    // One block's values are in use while the next one's are on their way (W = 1), or the
    // next block's are loaded over them behind their last use (W > 1: a block lasts four or
    // eight groups, and a load issued at the end of one group has landed by the end of the
    // next).
    Small cur;
    Small nxt;  // W == 1 only

    float16_t yacc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) yacc[i][j][e] = 0.0f;

    gload_small(g_begin, cur);
    request_group(g_begin, 0);
    request_group(g_begin + 1, kTpBufBytes);  // (a range holds at least one pair)
    small_loads_landed(cur);

    // The requests of the group after next go into the buffer everybody stopped reading before
    // this group's barrier.  (Measured and not kept: the two waves of a SIMD issuing theirs at
    // different times -- behind the barrier and in the middle of the group -- so that one
    // feeds the matrix pipe while the other is held up by its burst of requests; no change.)
    auto issue_requests = [&](int g, int buf_off) {
        if (g + 2 < groups) {
            int dst = buf_off + 2 * kTpBufBytes;
            if (dst >= kTpBufs * kTpBufBytes) dst -= kTpBufs * kTpBufBytes;
            request_group(g + 2, dst);
        }
    };

    // One group of 128 columns out of the buffer at byte `buf_off` of the ring; U: the group's
    // place in its block.  A wave's requests complete in the order they were issued, so "at
    // most the six youngest outstanding" names what has landed.
    auto group = [&](auto u_c, int g, int buf_off) {
        constexpr int U = decltype(u_c)::value;
        constexpr int PAR = U & 1;
        // this wave's requests of the group, issued two groups ago, have landed; those of
        // the next group may be on their way.  (Requests complete in the order they were
        // issued.  Behind a block's small loads the count is not raised by their number:
        // whether they complete in order with the requests is not relied on.)
        if (g + 1 >= groups) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kReq) : "memory");
        // after the barrier everybody's requests for this group have landed, and everybody is
        // done reading the buffer of the group before it, which the group after next reuses
        __builtin_amdgcn_s_barrier();
        if constexpr (W == 1) {
            if (U == 1 && g + 1 < groups) gload_small(g + 1, nxt);
        }
        issue_requests(g, buf_off);
        float16_t acc[2][2];
        bf16x8_t av[2][2];  // [step parity][i]
        bf16x8_t bv[2][2];  // [step parity][j]
        uint4_t wq[2][2];   // [j][half of the group]: the group's nibbles of this lane's rows
        // (the buffer's offset is added here: LDS offsets of up to 144 KiB do not fit the
        // 16-bit immediate of a read)
        unsigned t0, t1;
        asm volatile("v_add_u32 %4, %8, %6\n\tv_add_u32 %5, %8, %7\n\t"
                     "ds_read_b128 %0, %4\n\tds_read_b128 %1, %5\n\t"
                     "ds_read_b128 %2, %4 offset:2048\n\tds_read_b128 %3, %5 offset:2048"
                     : "=&v"(wq[0][0]), "=&v"(wq[0][1]), "=&v"(wq[1][0]), "=&v"(wq[1][1]),
                       "=&v"(t0), "=&v"(t1)
                     : "v"(b_addr[0]), "v"(b_addr[1]), "s"(buf_off)
                     : "memory");
        const unsigned a_buf = a0 + (unsigned)buf_off;
        asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %2 offset:8192"
                     : "=&v"(av[0][0]), "=&v"(av[0][1])
                     : "v"(a_buf)
                     : "memory");
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(wq[0][0]), "+v"(wq[0][1]), "+v"(wq[1][0]), "+v"(wq[1][1]),
                       "+v"(av[0][0]), "+v"(av[0][1])::"memory");
        auto unpack = [&](auto s8c, bf16x8_t (&b)[2]) {
            constexpr int s8 = decltype(s8c)::value;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const unsigned wd = wq[j][s8 >> 2][s8 & 3];
                uint4_t e4;
#pragma unroll
                for (int sft = 0; sft < 4; ++sft) e4[sft] = ((wd >> (4 * sft)) & kNibMask) | magic;
                b[j] = __builtin_bit_cast(bf16x8_t, e4);
            }
        };
        unpack(ic<0>{}, bv[0]);
        // Step s8 issues the reads of step s8 + 1, then its four MFMAs with the unpack of step
        // s8 + 1 between them (the matrix pipe takes 32 cycles per MFMA, eight issue slots of
        // the vector pipe), and only then waits for the reads.  The order is pinned: left
        // alone the scheduler sinks the MFMAs below the wait, which then sits right behind the
        // reads it waits for.
        static_for<8>([&](auto s8c) {
            constexpr int s8 = decltype(s8c)::value;
            constexpr int cur_p = s8 & 1;
            if constexpr (s8 < 7) {
                unsigned ta;
                asm volatile("v_xor_b32 %2, %c4, %3\n\t"
                             "ds_read_b128 %0, %2\n\tds_read_b128 %1, %2 offset:8192"
                             : "=&v"(av[cur_p ^ 1][0]), "=&v"(av[cur_p ^ 1][1]), "=&v"(ta)
                             : "v"(a_buf), "n"((s8 + 1) << 4)
                             : "memory");
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (s8 < 7) unpack(ic<(s8 < 7 ? s8 + 1 : 7)>{}, bv[cur_p ^ 1]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if constexpr (s8 == 0) {
                        float16_t z16;
#pragma unroll
                        for (int e = 0; e < 16; ++e) z16[e] = 0.0f;
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            av[cur_p][i], bv[cur_p][j], z16, 0, 0, 0);
                    } else {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            av[cur_p][i], bv[cur_p][j], acc[i][j], 0, 0, 0);
                    }
                }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // four vector instructions
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (s8 < 7)
                asm volatile("s_waitcnt lgkmcnt(0)"
                             : "+v"(av[cur_p ^ 1][0]), "+v"(av[cur_p ^ 1][1])::"memory");
        });
        if constexpr (W > 1 && U == 0) {
            // the block's values, requested at the end of the group before this one
            if (g > g_begin) small_loads_landed(cur);
        }
        // y += scale * acc  (measured and not kept: the last two steps tile by tile with a
        // tile's multiply-adds between the MFMAs of the tiles after it; no change)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const unsigned sd = cur.s[j][U >> 1];
            const unsigned short sb = (unsigned short)(PAR ? (sd >> 16) : sd);
            const float sf = __half2float(__builtin_bit_cast(__half, sb));
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) yacc[i][j][e] = fmaf(sf, acc[i][j][e], yacc[i][j][e]);
        }
        if constexpr (PAR == 1) {
            // zero-point term of the groups g - 1 (lanes h = 0) and g (h = 1):
            // y[m][n] += sum_x[m][g'] * (-scale[n][g'] * (128 + zero[n][g']))
            float cv[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const unsigned sd = cur.s[j][U >> 1], zd = cur.z[j][U >> 1];
                const unsigned short sb = (unsigned short)(h ? (sd >> 16) : sd);
                const unsigned short zb = (unsigned short)(h ? (zd >> 16) : zd);
                cv[j] = -__half2float(__builtin_bit_cast(__half, sb)) *
                        (128.0f + __half2float(__builtin_bit_cast(__half, zb)));
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    yacc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(cur.xs[i][U >> 1], cv[j],
                                                                      yacc[i][j], 0, 0, 0);
            if constexpr (W == 1) {
                if (g + 1 < groups) {
                    small_loads_landed(nxt);
                    cur = nxt;
                }
            } else if constexpr (U == BL - 1) {
                if (g + 1 < groups) gload_small(g + 1, cur);
            }
        }
    };
    // ranges are whole blocks (K is a multiple of 256 W); buffers go round in threes
    int buf_off = 0;
    for (int g0 = g_begin; g0 < groups; g0 += BL) {
        static_for<BL>([&](auto uc) {
            group(uc, g0 + decltype(uc)::value, buf_off);
            buf_off = buf_off + kTpBufBytes == kTpBufs * kTpBufBytes ? 0 : buf_off + kTpBufBytes;
        });
    }

    if (part >= 0) {
        // a part of a tile: the wave's 64 x 64 results as they lie in registers, lane fastest
        float* dst = partials + (size_t)part * kTpTileElems + (size_t)wave * 4096 + lane;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) dst[((i * 2 + j) * 16 + e) * 64] = yacc[i][j][e];
        return;
    }
    if constexpr (OUT == kTpOutSwigluOperand) {
        // (n is a multiple of 128 here: every column of the tile is a result)
        const int gn = col0 + (wc >> 1) + r;
        uint16_t* const xo = static_cast<uint16_t*>(y_out);
        float* const so = reinterpret_cast<float*>(static_cast<char*>(y_out) + tall_sums_offset(m, n));
        // the ring is done with once every wave has read its last operands
        __syncthreads();
        float* const red = reinterpret_cast<float*>(tp_lds);  // [wave column][chunk of it][row]
        const int wq = wave & 3, cq = r >> 3;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = wr + 32 * i + 8 * (e >> 2) + 4 * h + (e & 3);
                const float g = yacc[i][0][e], u = yacc[i][1][e];
                const uint16_t b = f32_to_bf16_rne(g / (1.0f + expf(-g)) * u);
                xo[(int64_t)(row0 + row) * n + (gn & ~7) + tp_pair_slot(gn & 7)] = b;
                const float cs = tp_chunk_sum_across_lanes(__uint_as_float((unsigned)b << 16));
                if ((r & 7) == 0) red[(wq * 4 + cq) * kTpTileM + row] = cs;
            }
        __syncthreads();
        if (tid < kTpTileM) {
            float cs[4][4];
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int c = 0; c < 4; ++c) cs[a][c] = red[(a * 4 + c) * kTpTileM + tid];
            so[tall_sum_index(row0 + tid, col0 >> 7, n, out_pairs)] = tp_group_sum(cs);
        }
        return;
    }
    if constexpr (OUT == kTpOutSwiglu) {
        const int gn = col0 + (wc >> 1) + r;
        if (gn >= n) return;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int gr = row0 + wr + 32 * i + 8 * (e >> 2) + 4 * h + (e & 3);
                if (gr < m) {
                    const float g = yacc[i][0][e], u = yacc[i][1][e];
                    static_cast<uint16_t*>(y_out)[(int64_t)gr * n + gn] =
                        f32_to_bf16_rne(g / (1.0f + expf(-g)) * u);
                }
            }
        return;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int gn = col0 + wc + 32 * j + r;
        if (gn >= n) continue;
        const float bv = bias ? bias[gn] : 0.0f;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int gr = row0 + wr + 32 * i + 8 * (e >> 2) + 4 * h + (e & 3);
                if (gr < m) {
                    if constexpr (OUT == kTpOutF32)
                        static_cast<float*>(y_out)[(int64_t)gr * n + gn] = yacc[i][j][e] + bv;
                    else
                        static_cast<uint16_t*>(y_out)[(int64_t)gr * n + gn] =
                            f32_to_bf16_rne(yacc[i][j][e] + bv);
                }
            }
    }
}

// Sums the `split` fp32 parts of each tile of the last round, in part order, adds the bias and
// writes y.  One thread per result; a part's element index is (wave, i, j, e, lane) as the
// product kernel left it.  (SwiGLU: j = 0 is the gate and j = 1 the up product of the same
// result; one thread takes both.)
template <int OUT>
__global__ __launch_bounds__(256) void q4_tall_reduce_kernel(const float* __restrict__ partials,
                                                            const float* __restrict__ bias,
                                                            void* __restrict__ y_out, int m, int n,
                                                            int tiles_n, int full_tiles,
                                                            int split) {
    static_assert(OUT != kTpOutSwigluOperand, "q4_tall_reduce_operand_kernel");
    constexpr int kPerTile = OUT == kTpOutSwiglu ? kTpTileElems / 2 : kTpTileElems;
    const int t = blockIdx.x / (kPerTile / 256);
    int idx = (blockIdx.x % (kPerTile / 256)) * 256 + threadIdx.x;
    if constexpr (OUT == kTpOutSwiglu) idx = ((idx >> 10) << 11) | (idx & 1023);  // j = 0
    const int lane = idx & 63, e = (idx >> 6) & 15, j = (idx >> 10) & 1, i = (idx >> 11) & 1;
    const int wave = idx >> 12;
    const int tile = full_tiles + t;
    const int gr = (tile / tiles_n) * kTpTileM + (wave >> 2) * 64 + 32 * i + 8 * (e >> 2) +
                   4 * (lane >> 5) + (e & 3);
    const float* src = partials + (size_t)t * split * kTpTileElems + idx;
    if constexpr (OUT == kTpOutSwiglu) {
        const int gn = (tile % tiles_n) * (kTpTileN / 2) + (wave & 3) * 32 + (lane & 31);
        if (gr >= m || gn >= n) return;
        float g = 0.0f, u = 0.0f;
        for (int q = 0; q < split; ++q) {
            g += src[(size_t)q * kTpTileElems];
            u += src[(size_t)q * kTpTileElems + 1024];
        }
        static_cast<uint16_t*>(y_out)[(int64_t)gr * n + gn] =
            f32_to_bf16_rne(g / (1.0f + expf(-g)) * u);
    } else {
        const int gn = (tile % tiles_n) * kTpTileN + (wave & 3) * 64 + 32 * j + (lane & 31);
        if (gr >= m || gn >= n) return;
        float acc = 0.0f;
        for (int q = 0; q < split; ++q) acc += src[(size_t)q * kTpTileElems];
        if (bias) acc += bias[gn];
        if constexpr (OUT == kTpOutF32) static_cast<float*>(y_out)[(int64_t)gr * n + gn] = acc;
        else static_cast<uint16_t*>(y_out)[(int64_t)gr * n + gn] = f32_to_bf16_rne(acc);
    }
}

// The same for kTpOutSwigluOperand: a workgroup takes four rows-of-registers (e = 4 eq .. + 3)
// of one (row half, i) of a tile across all four wave columns, i.e. eight rows of the tile with
// all their 128 outputs, so that it can add up their group sums: thread (wave column wq, lane)
// sums the parts of the gate and the up product of its result in part order, applies the
// activation and writes the bf16 value in pair order; chunk and group sums as in the product
// kernel.  grid: 16 workgroups per tile.
__global__ __launch_bounds__(256) void q4_tall_reduce_operand_kernel(
    const float* __restrict__ partials, void* __restrict__ y_out, int m, int n, int tiles_n,
    int full_tiles, int split, int out_pairs) {
    __shared__ float red[4][4][8];  // [wave column][chunk of it][row of the eight]
    const int t = blockIdx.x >> 4;
    const int half = (blockIdx.x >> 3) & 1, i = (blockIdx.x >> 2) & 1, eq = blockIdx.x & 3;
    const int wq = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 31, h = lane >> 5;
    const int tile = full_tiles + t;
    const int row0 = (tile / tiles_n) * kTpTileM, col0 = (tile % tiles_n) * (kTpTileN / 2);
    const int gn = col0 + 32 * wq + r;
    uint16_t* const xo = static_cast<uint16_t*>(y_out);
    float* const so = reinterpret_cast<float*>(static_cast<char*>(y_out) + tall_sums_offset(m, n));
    const float* src = partials + (size_t)t * split * kTpTileElems +
                       (size_t)(half * 4 + wq) * 4096 + (size_t)i * 2048 + lane;
#pragma unroll
    for (int el = 0; el < 4; ++el) {
        const int e = 4 * eq + el;
        float g = 0.0f, u = 0.0f;
        for (int q = 0; q < split; ++q) {
            g += src[(size_t)q * kTpTileElems + e * 64];
            u += src[(size_t)q * kTpTileElems + 1024 + e * 64];
        }
        const int row = 64 * half + 32 * i + 8 * (e >> 2) + 4 * h + (e & 3);
        const uint16_t b = f32_to_bf16_rne(g / (1.0f + expf(-g)) * u);
        xo[(int64_t)(row0 + row) * n + (gn & ~7) + tp_pair_slot(gn & 7)] = b;
        const float cs = tp_chunk_sum_across_lanes(__uint_as_float((unsigned)b << 16));
        if ((r & 7) == 0) red[wq][r >> 3][2 * el + h] = cs;
    }
    __syncthreads();
    if (threadIdx.x < 8) {
        const int el = threadIdx.x >> 1, hh = threadIdx.x & 1, e = 4 * eq + el;
        float cs[4][4];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int c = 0; c < 4; ++c) cs[a][c] = red[a][c][threadIdx.x];
        const int row = 64 * half + 32 * i + 8 * (e >> 2) + 4 * hh + (e & 3);
        so[tall_sum_index(row0 + row, col0 >> 7, n, out_pairs)] = tp_group_sum(cs);
    }
}

inline int tp_pairs_per_load(int k, const void* scale, const void* zero) {
    return tall_pairs_per_load(k, scale, zero);
}

template <int OUT, int W>
static hipError_t tallp_launch(const uint16_t* xp, const float* xs, float* partials,
                               const uint8_t* qw, const __half* scale, const __half* zero,
                               const float* bias, void* y, int m, int n, int k, hipStream_t st,
                               int out_pairs = 0) {
    constexpr size_t lds = (size_t)kTpBufs * kTpBufBytes;
    static const hipError_t opt = hipFuncSetAttribute(
        reinterpret_cast<const void*>(qgemm_q4g128_tallp_kernel<OUT, W>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (opt != hipSuccess) return opt;
    constexpr int tile_outputs = tp_is_swiglu(OUT) ? kTpTileN / 2 : kTpTileN;
    const int tiles_n = (n + tile_outputs - 1) / tile_outputs;
    const int tiles = tiles_n * (tp_padded_rows(m) / kTpTileM);
    const int cus = device_cu_count();
    if (cus <= 0) return hipErrorInvalidDevice;
    const TpPlan plan = tp_plan(tiles, k >> 7, 2 * W, cus);
    const int parts = (tiles - plan.full) * plan.split;
    qgemm_q4g128_tallp_kernel<OUT, W>
        <<<dim3(plan.full + (plan.split > 1 ? parts : 0)), dim3(512), lds, st>>>(
            xp, xs, qw, scale, zero, bias, y, partials, m, n, k, tiles_n, plan.full, plan.split,
            out_pairs);
    if (plan.split > 1) {
        if constexpr (OUT == kTpOutSwigluOperand) {
            q4_tall_reduce_operand_kernel<<<dim3((tiles - plan.full) * 16), dim3(256), 0, st>>>(
                partials, y, m, n, tiles_n, plan.full, plan.split, out_pairs);
        } else {
            constexpr int per_tile = OUT == kTpOutSwiglu ? kTpTileElems / 2 : kTpTileElems;
            q4_tall_reduce_kernel<OUT>
                <<<dim3((tiles - plan.full) * (per_tile / 256)), dim3(256), 0, st>>>(
                    partials, bias, y, m, n, tiles_n, plan.full, plan.split);
        }
    }
    return hipGetLastError();
}

template <int OUT>
static hipError_t tallp_launch_w(int w, const uint16_t* xp, const float* xs, float* partials,
                                 const uint8_t* qw, const __half* scale, const __half* zero,
                                 const float* bias, void* y, int m, int n, int k, hipStream_t st,
                                 int out_pairs = 0) {
    switch (w) {
        case 4:
            return tallp_launch<OUT, 4>(xp, xs, partials, qw, scale, zero, bias, y, m, n, k, st,
                                        out_pairs);
        case 2:
            return tallp_launch<OUT, 2>(xp, xs, partials, qw, scale, zero, bias, y, m, n, k, st,
                                        out_pairs);
        default:
            return tallp_launch<OUT, 1>(xp, xs, partials, qw, scale, zero, bias, y, m, n, k, st,
                                        out_pairs);
    }
}

}  // namespace lg

extern "C" logismos_status_t logismos_check_qgemm_q4g128_tall_shape(int m, int n, int k, char* msg,
                                                                    size_t msg_cap) {
    const char* kn = "qgemm_q4g128_tall";
    if (m <= 0) return lg::reject(msg, msg_cap, "%s: rows must be positive, got %d", kn, m);
    if (n <= 0) return lg::reject(msg, msg_cap, "%s: N must be positive, got %d", kn, n);
    if (k <= 0 || k % 256 != 0)
        return lg::reject(msg, msg_cap,
                          "%s: K = %d is not a positive multiple of 256 (pairs of groups of 128)",
                          kn, k);
    const int64_t lim = INT32_MAX;
    if ((int64_t)n * k > lim)
        return lg::reject(msg, msg_cap, "%s: N*K = %lld exceeds i32::MAX", kn,
                          (long long)((int64_t)n * k));
    if ((int64_t)lg::tp_padded_rows(m) * k * 2 > lim || (int64_t)m * n > lim)
        return lg::reject(msg, msg_cap, "%s: rows*K*2 or rows*N exceeds i32::MAX", kn);
    return 0;
}

extern "C" size_t logismos_qgemm_q4g128_tall_workspace_bytes(int m, int k) {
    if (m <= 0 || k <= 0 || k % 128 != 0) return 0;
    return lg::tp_partials_offset(m, k) + (size_t)lg::kTpMaxParts * lg::kTpTileElems * 4;
}

static logismos_status_t tall_args_ok(const void* qw_u8, const void* scale_f16,
                                      const void* zero_f16, const void* y, const void* workspace,
                                      int m, int n, int k) {
    if (logismos_check_qgemm_q4g128_tall_shape(m, n, k, nullptr, 0) != 0)
        return hipErrorInvalidValue;
    if (!qw_u8 || !scale_f16 || !zero_f16 || !y || !workspace) return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(qw_u8) | reinterpret_cast<uintptr_t>(workspace)) & 15u)
        return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(scale_f16) | reinterpret_cast<uintptr_t>(zero_f16)) & 3u)
        return hipErrorInvalidValue;
    return hipSuccess;
}

extern "C" int logismos_qgemm_q4g128_tall_pairs_per_load(int k, const void* scale_f16,
                                                         const void* zero_f16) {
    return lg::tall_pairs_per_load(k, scale_f16, zero_f16);
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g128_tall_prepared(
    const void* qw_u8, const void* scale_f16, const void* zero_f16, const void* bias_f32, void* y,
    int y_is_f32, void* workspace, int m, int n, int k, logismos_stream_t stream) {
    if (const logismos_status_t e = tall_args_ok(qw_u8, scale_f16, zero_f16, y, workspace, m, n, k))
        return e;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t* xp = static_cast<const uint16_t*>(workspace);
    const float* xs =
        reinterpret_cast<const float*>(static_cast<char*>(workspace) + lg::tp_sums_offset(m, k));
    float* partials = reinterpret_cast<float*>(static_cast<char*>(workspace) +
                                               lg::tp_partials_offset(m, k));
    const int w = lg::tp_pairs_per_load(k, scale_f16, zero_f16);
    if (y_is_f32)
        return lg::tallp_launch_w<lg::kTpOutF32>(w, xp, xs, partials, static_cast<const uint8_t*>(qw_u8),
                                        static_cast<const __half*>(scale_f16),
                                        static_cast<const __half*>(zero_f16),
                                        static_cast<const float*>(bias_f32), y, m, n, k, st);
    return lg::tallp_launch_w<lg::kTpOutBf16>(w, xp, xs, partials, static_cast<const uint8_t*>(qw_u8),
                                     static_cast<const __half*>(scale_f16),
                                     static_cast<const __half*>(zero_f16),
                                     static_cast<const float*>(bias_f32), y, m, n, k, st);
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g128_tall_swiglu_prepared(
    const void* gate_up_qw_u8, const void* scale_f16, const void* zero_f16, void* act_bf16,
    void* workspace, int m, int inter, int k, logismos_stream_t stream) {
    // the weights are 2 * inter rows (gate, then up); the output is m x inter
    if (inter <= 0 || inter > INT32_MAX / 2) return hipErrorInvalidValue;
    if (const logismos_status_t e = tall_args_ok(gate_up_qw_u8, scale_f16, zero_f16, act_bf16,
                                                 workspace, m, 2 * inter, k))
        return e;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t* xp = static_cast<const uint16_t*>(workspace);
    const float* xs =
        reinterpret_cast<const float*>(static_cast<char*>(workspace) + lg::tp_sums_offset(m, k));
    float* partials = reinterpret_cast<float*>(static_cast<char*>(workspace) +
                                               lg::tp_partials_offset(m, k));
    const int w = lg::tp_pairs_per_load(k, scale_f16, zero_f16);
    return lg::tallp_launch_w<lg::kTpOutSwiglu>(
        w, xp, xs, partials, static_cast<const uint8_t*>(gate_up_qw_u8),
        static_cast<const __half*>(scale_f16), static_cast<const __half*>(zero_f16), nullptr,
        act_bf16, m, inter, k, st);
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g128_tall_swiglu_operand(
    const void* gate_up_qw_u8, const void* scale_f16, const void* zero_f16, void* next_workspace,
    int next_pairs_per_load, void* workspace, int m, int inter, int k, logismos_stream_t stream) {
    // the output is the operand of a product over K = inter: whole pairs of groups, and as many
    // pairs per load as the caller's next launch will ask for (whole blocks of them)
    if (inter <= 0 || inter > INT32_MAX / 2 || inter % 256 != 0) return hipErrorInvalidValue;
    if (next_pairs_per_load != 1 && next_pairs_per_load != 2 && next_pairs_per_load != 4)
        return hipErrorInvalidValue;
    if (inter % (256 * next_pairs_per_load) != 0) return hipErrorInvalidValue;
    if (const logismos_status_t e = tall_args_ok(gate_up_qw_u8, scale_f16, zero_f16,
                                                 next_workspace, workspace, m, 2 * inter, k))
        return e;
    // (the next launch's own shape: rows * inter * 2 within 32 bits)
    if (logismos_check_qgemm_q4g128_tall_shape(m, 1, inter, nullptr, 0) != 0)
        return hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(next_workspace) & 15u) || next_workspace == workspace)
        return hipErrorInvalidValue;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t* xp = static_cast<const uint16_t*>(workspace);
    const float* xs =
        reinterpret_cast<const float*>(static_cast<char*>(workspace) + lg::tp_sums_offset(m, k));
    float* partials = reinterpret_cast<float*>(static_cast<char*>(workspace) +
                                               lg::tp_partials_offset(m, k));
    const int w = lg::tp_pairs_per_load(k, scale_f16, zero_f16);
    return lg::tallp_launch_w<lg::kTpOutSwigluOperand>(
        w, xp, xs, partials, static_cast<const uint8_t*>(gate_up_qw_u8),
        static_cast<const __half*>(scale_f16), static_cast<const __half*>(zero_f16), nullptr,
        next_workspace, m, inter, k, st, next_pairs_per_load);
}

extern "C" logismos_status_t logismos_launch_qgemm_q4g128_tall(
    const void* x_bf16, const void* qw_u8, const void* scale_f16, const void* zero_f16,
    const void* bias_f32, void* y, int y_is_f32, void* workspace, int m, int n, int k,
    logismos_stream_t stream) {
    if (const logismos_status_t e = tall_args_ok(qw_u8, scale_f16, zero_f16, y, workspace, m, n, k))
        return e;
    if (!x_bf16 || (reinterpret_cast<uintptr_t>(x_bf16) & 15u)) return hipErrorInvalidValue;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int m_pad = lg::tp_padded_rows(m);
    uint16_t* xp = static_cast<uint16_t*>(workspace);
    float* xs = reinterpret_cast<float*>(static_cast<char*>(workspace) + lg::tp_sums_offset(m, k));
    const int64_t chunks = (int64_t)m_pad * (k / 8);
    const int w = lg::tp_pairs_per_load(k, scale_f16, zero_f16);
    lg::q4_tall_prepare_kernel<<<dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, st>>>(
        static_cast<const uint16_t*>(x_bf16), xp, xs, m, m_pad, k, w);
    if (const hipError_t e = hipGetLastError()) return e;
    return logismos_launch_qgemm_q4g128_tall_prepared(qw_u8, scale_f16, zero_f16, bias_f32, y,
                                                      y_is_f32, workspace, m, n, k, stream);
}

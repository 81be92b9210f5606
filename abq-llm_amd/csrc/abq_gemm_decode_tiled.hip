// GEMM core for decode-sized M on prepared operands: both operands in the K-tiled field-packed layout
// (abq_bits.h), widths of a single field (2, 4 or 8 bits).
//
// Replaces AqBMMAKernel::mainLoop + ::epilogue of the reference
// (engine/mma_any/aq_bmma_kernel.h:109-271, :485-580) for one (x_bits, w_bits) pair per
// translation unit: compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>.
//
// A decode GEMM streams 4 to 11 MB of weights once; at 8 TB/s that takes 0.5 to 1.4 us, the same order as
// one memory round trip and as a kernel launch, and every kernel starts with cold caches.  What decides
// the time is therefore the length of the dependent chain from the first instruction to the last store and
// the number of vector instructions on it (with sixteen waves on a compute unit an instruction of every
// wave costs sixteen issue cycles per SIMD quad), not the byte count.  Hence:
//   * prepared operands: a lane's 16-byte weight load is what it feeds the matrix core after a shift and a
//     mask per four elements (no bit-matrix transpose), activations are int8-ready records (nothing to
//     expand, no bytes more than the planes have);
//   * a workgroup is T tiles of 16 weight rows over the whole K; wave w takes K steps w, w + NW, ...
//     (a step = one 16-byte load per lane = 512 / P elements of K over the four lane groups);
//   * the activations of the workgroup's rows go from global memory straight into LDS
//     (global_load_lds_dwordx4: no registers, nothing to wait for before the weight loads are issued);
//     chunk c of a row lands at c ^ (row & (Q - 1)) so that the sixteen rows a lane group reads hit
//     different banks (the permutation is applied to the source address, the destination is linear);
//   * the first D steps' weight loads of every wave are issued right behind them, all before the first
//     wait; one counted wait (the activation loads are older than the weight loads) and one barrier
//     later every wave reads its A operands with ds_read_b128;
//   * the loads are issued from inline assembly: the compiler would sink plain loads below the barrier,
//     next to their first use.  Values loaded that way are consumed through `landed()` after a counted
//     wait, in the loop iteration that issued them (no register of theirs lives across the back edge,
//     where a compiler-inserted copy could read it before it has landed);
//   * per-wave partial tiles meet in LDS and are summed by the threads that store them (integer adds:
//     any order gives the same bits).
// K longer than NW * D steps runs further rounds of the same loop (their latency is exposed).
#include <type_traits>

#include "abq_kernels.h"
#include "abq_bits.h"
#include "abq_quant.h"

#ifndef ABQ_Q
#error "compile with -DABQ_Q=<x_bits> -DABQ_P=<w_bits>"
#endif

namespace abq {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

constexpr bool decode_tiled_width(int b) { return b == 2 || b == 4 || b == 8; }
// single-field widths, activations at least as wide as the weights
constexpr bool decode_tiled_built(int q, int p) { return decode_tiled_width(q) && decode_tiled_width(p) && q >= p; }

__device__ __forceinline__ void dt_load_to_lds(const void *src, unsigned lds_addr)
{
    // lane l of the wave lands at lds_addr + 16 * l.  (M0 cannot be named as clobbered: the compiler reserves it and
    // sets it up itself right before each of its own uses, it keeps no value there across other instructions.)
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(src)
                 : "memory");
}

__device__ __forceinline__ v4u dt_load16(const char *base, uint32_t off)
{
    v4u v;
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(v) : "v"(off), "s"(base) : "memory");
    return v;
}
// the same for weight records.  once: nothing reads the record a second time (the grid has one block of rows), and the
// load is marked non-temporal, so that the lines do not displace what the workgroups share in the L2; with several
// blocks of rows the other blocks' workgroups read the record again and it is loaded like anything else.  (wave-uniform)
// (One statement with a scalar branch inside, not two statements under an if: the destination is then one register
// whichever way the load is issued, and no copy of a register still in flight can come between load and wait.)
__device__ __forceinline__ v4u dt_load16_weights(const char *base, uint32_t off, int once)
{
    v4u v;
    asm volatile("s_cmp_lg_u32 %3, 0\n\t"
                 "s_cbranch_scc1 .Ldt_once_%=\n\t"
                 "global_load_dwordx4 %0, %1, %2\n\t"
                 "s_branch .Ldt_issued_%=\n"
                 ".Ldt_once_%=:\n\t"
                 "global_load_dwordx4 %0, %1, %2 nt\n"
                 ".Ldt_issued_%=:"
                 : "=&v"(v)
                 : "v"(off), "s"(base), "s"(__builtin_amdgcn_readfirstlane(once))
                 : "memory", "scc");
    return v;
}

template <int N> __device__ __forceinline__ void dt_wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// the same with a count that is constant only after unrolling
__device__ __forceinline__ void dt_wait_loads_n(int n)
{
    switch (n) {
    case 0: dt_wait_loads<0>(); break;
    case 1: dt_wait_loads<1>(); break;
    case 2: dt_wait_loads<2>(); break;
    case 3: dt_wait_loads<3>(); break;
    case 4: dt_wait_loads<4>(); break;
    case 5: dt_wait_loads<5>(); break;
    case 6: dt_wait_loads<6>(); break;
    case 8: dt_wait_loads<8>(); break;
    case 10: dt_wait_loads<10>(); break;
    case 12: dt_wait_loads<12>(); break;
    case 16: dt_wait_loads<16>(); break;
    case 20: dt_wait_loads<20>(); break;
    default: dt_wait_loads<0>(); break;
    }
}
// ties a register filled by dt_load16 to the wait in front of it: every use comes after
__device__ __forceinline__ void dt_landed(v4u &v) { asm volatile("" : "+v"(v)); }

// One 16-byte unit of a BITS-wide single-field record -> 8 / BITS MFMA operands of four dwords.
// Signed: value * 2^(8 - BITS) (the field at the top of the byte); unsigned: the value.
template <int BITS, bool SIGNED> __device__ __forceinline__ void dt_unpack(const v4u &u, v4i (&out)[8 / BITS])
{
    if (BITS == 8) {
        out[0] = v4i{ (int)u[0], (int)u[1], (int)u[2], (int)u[3] };
    } else if (BITS == 4) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint32_t a = u[2 * i], b = u[2 * i + 1];
            if (SIGNED)
                out[i] = v4i{ (int)((a << 4) & 0xF0F0F0F0u), (int)(a & 0xF0F0F0F0u), (int)((b << 4) & 0xF0F0F0F0u), (int)(b & 0xF0F0F0F0u) };
            else
                out[i] = v4i{ (int)(a & 0x0F0F0F0Fu), (int)((a >> 4) & 0x0F0F0F0Fu), (int)(b & 0x0F0F0F0Fu), (int)((b >> 4) & 0x0F0F0F0Fu) };
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = u[i];
            if (SIGNED)
                out[i] = v4i{ (int)((w << 6) & 0xC0C0C0C0u), (int)((w << 4) & 0xC0C0C0C0u), (int)((w << 2) & 0xC0C0C0C0u), (int)(w & 0xC0C0C0C0u) };
            else
                out[i] = v4i{ (int)(w & 0x03030303u), (int)((w >> 2) & 0x03030303u), (int)((w >> 4) & 0x03030303u), (int)((w >> 6) & 0x03030303u) };
        }
    }
}

// XF16: the activations arrive as fp16 [M][K] and are quantised here with one static scale, value =
// (int)(half(x) * half(scale)) as pack_half of the reference does (abq_gemm_wrapper.cu:29-54), straight into the
// int8 records in LDS: the pack kernel and its launch in front of every decode GEMM of the FT wrapper fall away.
// Every workgroup converts the rows it multiplies (M x K halves, from L2 after the first).  8-bit activations.
// XF16 is the number of 16-byte units of eight halves a thread holds per pass (0: the activations arrive packed; 1, 2
// or 4, the launcher takes the fewest that cover the rows in one pass, at most 4: eight rows of 4096 with sixteen waves;
// more spills, and with four the instances need 95 - 104 registers against 52 - 67, which costs workgroups per unit).
// FLIP (unsigned pairs): the 8-bit records hold codes up to 255, which the signed matrix cores take as value - 128
// (bit 7 flipped: one xor per dword after the load); the result is put right with 128 x the other operand's row
// sums (GemmArgs::x_row_sums / w_row_sums, abq_row_sums) and, when both operands are 8 bits wide, - 2^14 K.  Without
// FLIP the bytes of an unsigned 8-bit record are fed as they are: padded records of narrower codes (below 128).
template <int Q, int P, bool SIGNED, int NW, int D, int T, int XF16 = 0, bool FLIP = false>
__global__ __launch_bounds__(64 * NW) void gemm_decode_tiled(const GemmArgs a, int mrows)
{
    static_assert(!XF16 || Q == 8, "in-kernel quantisation writes 8-bit records");
    static_assert(!FLIP || (!SIGNED && Q == 8 && !XF16), "flipping is for unsigned 8-bit records");
    constexpr bool FLIP_X = FLIP && Q == 8, FLIP_W = FLIP && P == 8;
    static_assert(XF16 == 0 || XF16 == 1 || XF16 == 2 || XF16 == 4, "units per thread and pass");
    constexpr int XP = XF16 > 0 ? XF16 : 1;
    constexpr int NXL = Q / P;   // activation chunks (16 bytes) per weight unit
    constexpr int NM = 8 / P;    // MFMAs per weight unit
    constexpr int MX = 8 / Q;    // MFMAs per activation chunk
    constexpr int NT = 64 * NW;
    constexpr int QLOG = Q == 8 ? 3 : Q == 4 ? 2 : 1;
    constexpr int XC = 6;        // activation wave loads per wave that are unrolled
    extern __shared__ __align__(16) unsigned char smem[];
    int *red = reinterpret_cast<int *>(smem);   // [NW][T][16][16]
    unsigned char *xs = smem + NW * T * 1024;   // [kt][row][Q chunks], chunks permuted within a row

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int M = a.M, N = a.N;
    const int KT = a.K >> 7;
    const int U = KT * P;            // 16-byte units per weight row
    const int S = (U + 3) >> 2;      // steps
    const int tile0 = blockIdx.x * T;
    const int m0 = blockIdx.y * mrows;
    const int once = gridDim.y == 1; // no other workgroup reads this one's weight records
    const int Mb = min(mrows, M - m0);
    const char *Xt = reinterpret_cast<const char *>(a.X);
    const char *Wt = reinterpret_cast<const char *>(a.W);
    const unsigned xs_addr = (unsigned)(size_t)xs;
    const int xchunks = KT * Mb * Q;

    // ---- activations: LDS chunk p <- chunk p ^ ((p / Q) & (Q - 1)) of the workgroup's rows -----------
    // (XF16: loaded, quantised and written inside the first round below)
    const int upr = a.K >> 3;     // XF16: units of eight halves per row
    const int nunits = Mb * upr;
    const char *Xh = Xt + (size_t)m0 * a.K * 2;
    uint32_t sel_pair = 0, sel_half = 0;
    if constexpr (XF16)
        quad_transpose_selectors(tid & 3, sel_pair, sel_half);
    // eight halves of unit p (row p / upr, elements 8 u .. 8 u + 7) -> their bytes of the row's int8 record: the
    // quad's four units are one word-set, whose expanded dword s, byte c is element 7 - s of lane 3 - c
    auto quantise_unit = [&](const v4u &raw, int p, _Float16 hs) {
        union {
            v4u q;
            _Float16 h[8];
        } r;
        r.q = raw;
        int v[8];
#pragma unroll
        for (int c = 0; c < 8; ++c)
            v[c] = (int)(_Float16)(r.h[c] * hs); // fp16 product rounded to nearest even, conversion truncating
        const uint32_t e_even = quad_transpose_bytes(pack_low_bytes(v[7], v[5], v[3], v[1]), sel_pair, sel_half);
        const uint32_t e_odd = quad_transpose_bytes(pack_low_bytes(v[6], v[4], v[2], v[0]), sel_pair, sel_half);
        if (p < nunits) {
            const int row = p / upr, u = p - row * upr;
            const int rowi = (u >> 4) * Mb + row;                        // K tile * rows + row
            const int dw = 8 * ((u >> 2) & 3) + 2 * (u & 3);             // first of the lane's two dwords in the record
            const int chunk = (dw >> 2) ^ (rowi & 7);
            *reinterpret_cast<uint2 *>(xs + ((uint32_t)rowi * 8 + chunk) * 16u + (dw & 3) * 4u) = make_uint2(e_even, e_odd);
        }
    };
    if constexpr (XF16) {
    } else if (Mb == M) { // the rows of all K tiles are one contiguous block
#pragma unroll
        for (int i = 0; i < XC; ++i) {
            const int pb = wid * 64 + i * NT; // wave-uniform
            if (pb < xchunks) {
                const int p = pb + lane;
                const int src = min(p ^ ((p >> QLOG) & (Q - 1)), xchunks - 1);
                dt_load_to_lds(Xt + (uint32_t)src * 16u, xs_addr + (unsigned)pb * 16u);
            }
        }
        for (int pb = wid * 64 + XC * NT; pb < xchunks; pb += NT) {
            const int p = pb + lane;
            const int src = min(p ^ ((p >> QLOG) & (Q - 1)), xchunks - 1);
            dt_load_to_lds(Xt + (uint32_t)src * 16u, xs_addr + (unsigned)pb * 16u);
        }
    } else { // several blocks of rows: a K tile's rows are Mb * Q chunks out of M * Q
        const int per = Mb * Q;
        for (int pb = wid * 64; pb < xchunks; pb += NT) {
            const int p = min(pb + lane, xchunks - 1);
            const int q = p ^ ((p >> QLOG) & (Q - 1));
            const int kt = q / per, rem = q - kt * per;
            dt_load_to_lds(Xt + ((size_t)(kt * M + m0) * Q + rem) * 16u, xs_addr + (unsigned)pb * 16u);
        }
    }

    // ---- weights: byte offset of (lane, step s, tile t) = step_w(s) + woff[t] ------------------------
    uint32_t woff[T], back;
    {
        const int n = min(tile0 * 16 + r, N - 1);
        const uint32_t lane_w = P == 2 ? ((uint32_t)(g >> 1) * N + n) * 32u + (g & 1) * 16u : (uint32_t)n * (P * 16u) + g * 16u;
        back = lane_w - (uint32_t)n * (P * 16u); // distance to the first unit of the step in the same row
#pragma unroll
        for (int t = 0; t < T; ++t)
            woff[t] = lane_w + ((T > 1 && (tile0 + t) * 16 + r < N) ? t * (16u * P * 16u) : 0u);
    }
    const uint32_t step_bytes = (uint32_t)N * 64u; // a step covers 4 units of every row: 64 bytes times N rows
    auto step_w = [&](int s) -> uint32_t {
        return P == 8 ? (uint32_t)(s >> 1) * (2u * step_bytes) + (s & 1) * 64u : (uint32_t)s * step_bytes;
    };
    const bool ragged = (U & 3) != 0; // the last step has fewer than four units

    v4i acc[T][2];
#pragma unroll
    for (int t = 0; t < T; ++t)
        acc[t][0] = acc[t][1] = v4i{ 0, 0, 0, 0 };
    const int ml = min(r, Mb - 1);

    int round = 0;
    do {
        // this round's steps of the wave: wid + (round * D + d) * NW.  Every wave issues D * T loads (steps past
        // the end repeat the last one), so that the waits below can count.
        v4u wb[D][T];
        v4u xr[XF16 ? XP : 1];
        if (XF16 && round == 0) {
            // every pass is loaded, past the rows' end the last unit once more: a load under a condition would leave the
            // compiler a register to merge with an undefined one, and a copy it inserts for that reads before the data lands
#pragma unroll
            for (int i = 0; i < XP; ++i)
                xr[i] = dt_load16(Xh, (uint32_t)min(tid + i * NT, nunits - 1) * 16u);
        }
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int s = min(wid + (round * D + d) * NW, S - 1);
            const char *wp = Wt + step_w(s);
            // lanes past the end of K (last step only) read the step's first unit of their row instead
            const uint32_t bk = (ragged && s == S - 1 && 4 * s + g >= U) ? back : 0u;
#pragma unroll
            for (int t = 0; t < T; ++t)
                wb[d][t] = dt_load16_weights(wp, woff[t] - bk, once);
        }
        if (round == 0) {
            dt_wait_loads<D * T>(); // the activation loads are older than these
            if constexpr (XF16) {
                const _Float16 hs = (_Float16)a.x_pack_scale[0];
#pragma unroll
                for (int i = 0; i < XP; ++i)
                    dt_landed(xr[i]);
#pragma unroll
                for (int i = 0; i < XP; ++i) {
                    if (i * NT < nunits) // the quads of a wave are whole
                        quantise_unit(xr[i], tid + i * NT, hs);
                }
                // rows too long for one pass: further passes, their latency exposed
                for (int base = XP * NT; base < nunits; base += XP * NT) {
                    v4u more[XP];
#pragma unroll
                    for (int i = 0; i < XP; ++i)
                        more[i] = dt_load16(Xh, (uint32_t)min(base + tid + i * NT, nunits - 1) * 16u);
                    dt_wait_loads<0>(); // these are the youngest loads
#pragma unroll
                    for (int i = 0; i < XP; ++i) {
                        dt_landed(more[i]);
                        if (base + i * NT < nunits)
                            quantise_unit(more[i], base + tid + i * NT, hs);
                    }
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int cs = wid + (round * D + d) * NW;
            const bool have = cs < S; // wave-uniform
            v4i av[NM];
            if (have) {
                const int u0 = (4 * cs + g) * NXL;           // first activation chunk of lane group and step along K
                const int rowi = (u0 >> QLOG) * Mb + ml;      // row index in LDS: K tile * rows + row
#pragma unroll
                for (int i = 0; i < NXL; ++i) {
                    const int part = ((u0 + i) & (Q - 1)) ^ (rowi & (Q - 1));
                    const v4u xv = *reinterpret_cast<const v4u *>(xs + ((uint32_t)rowi * Q + part) * 16u);
                    v4i tt[MX];
                    dt_unpack<Q, SIGNED>(xv, tt);
                    if constexpr (FLIP_X)
                        tt[0] = v4i{ tt[0][0] ^ (int)0x80808080u, tt[0][1] ^ (int)0x80808080u, tt[0][2] ^ (int)0x80808080u,
                                     tt[0][3] ^ (int)0x80808080u };
#pragma unroll
                    for (int k = 0; k < MX; ++k)
                        av[i * MX + k] = tt[k];
                }
            }
            // Waited for and marked as landed on every path: a register with a load still in flight must not
            // look free to the compiler (it would reuse it, and the late data would land on the new value).
            dt_wait_loads_n((D - 1 - d) * T);
#pragma unroll
            for (int t = 0; t < T; ++t)
                dt_landed(wb[d][t]);
            if (have) {
                const bool ok = 4 * cs + g < U;
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    // (lanes past the end of K feed zeros, also where the weights are flipped)
                    constexpr unsigned kFlipW = FLIP_W ? 0x80808080u : 0u;
                    const v4u wv = ok ? v4u{ wb[d][t][0] ^ kFlipW, wb[d][t][1] ^ kFlipW, wb[d][t][2] ^ kFlipW, wb[d][t][3] ^ kFlipW }
                                      : v4u{ 0u, 0u, 0u, 0u };
                    v4i bv[NM];
                    dt_unpack<P, SIGNED>(wv, bv);
#pragma unroll
                    for (int i = 0; i < NM; ++i)
                        acc[t][i & 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[i], bv[i], acc[t][i & 1], 0, 0, 0);
                }
            }
        }
        ++round;
    } while (wid + round * D * NW < S);

    // ---- the waves' partial tiles meet in LDS ----------------------------------------------------------
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (4 * g + e < Mb)
                red[((wid * T + t) * 16 + 4 * g + e) * 16 + r] = acc[t][0][e] + acc[t][1][e];
    __syncthreads();
    for (int o = tid; o < T * 256; o += NT) {
        const int t = o >> 8, rem = o & 255;
        const int n = (tile0 + t) * 16 + (rem & 15);
        if ((rem >> 4) < Mb && n < N) {
            int part[NW];
#pragma unroll
            for (int w = 0; w < NW; ++w)
                part[w] = red[(w * T + t) * 256 + rem];
            int v = 0;
#pragma unroll
            for (int w = 0; w < NW; ++w)
                v += part[w];
            if (SIGNED)
                v >>= 16 - Q - P; // both operands were fed at the top of the byte
            if constexpr (FLIP_X)
                v = (int)((unsigned)v + 128u * (unsigned)a.w_row_sums[n]);
            if constexpr (FLIP_W)
                v = (int)((unsigned)v + 128u * (unsigned)a.x_row_sums[m0 + (rem >> 4)]);
            if constexpr (FLIP_X && FLIP_W)
                v = (int)((unsigned)v - 16384u * (unsigned)a.K);
            store_result(a, m0 + (rem >> 4), n, v);
        }
    }
}

// ---- weights of several fields ------------------------------------------------------------------
//
// Widths of 3, 5, 6 and 7 bits are records of a 4-bit, a 2-bit and a 1-bit field (abq_bits.h: a row's K tile is
// P * 16 bytes, the field of width F the F units of 16 bytes at byte 16 * (P & ~(2F - 1))).  Inside its region a
// field is laid out exactly as a single-field record of that width, so the plan above carries over field by field:
// a step of field F is one 16-byte load per lane, lane group g taking unit 4 cs + g of the field's units along K
// (K tile (4 cs + g) / F, unit (4 cs + g) % F of it), 8 / F MFMAs against the 128 / F activations the unit covers.
// A field is fed at the place its bits have in the code (signed: in the code moved to the top of the byte, so that
// the widest field carries the sign and the others are non-negative), all fields into one accumulator: the sum is
// the dot product times 2^(16 - QP - P) as for a single field.  The steps of all fields form one list (4-bit
// field first), wave w takes steps w, w + NW, ...; which field a step belongs to is the same for the whole wave.
// The weights are the records the prefill kernels read (abq_relayout_planes): one copy serves both.  The
// activations are records of a single field of QP bits: their own width, or for 3, 5, 6 and 7 bits the next such
// width with the codes extended (abq_relayout_planes_padded); activation bytes are small at decode.
template <int F, int POS, bool TOP> __device__ __forceinline__ void dt_unpack_field(const v4u &u, v4i (&out)[8 / F])
{
    // word j of the unit carries in byte c, at bits [F s, F s + F), the field of expanded dword (8 / F) j + s;
    // operand i = expanded dwords 4 i .. 4 i + 3.  The field goes to bits [POS, POS + F) of the byte.
    constexpr uint32_t mask = field_mask(F) << POS;
    constexpr int per = 8 / F; // expanded dwords per word
#pragma unroll
    for (int i = 0; i < 8 / F; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int d = 4 * i + c, j = d / per, sft = POS - F * (d % per);
            const uint32_t w = u[j];
            out[i][c] = (int)((sft >= 0 ? w << (sft >= 0 ? sft : 0) : w >> (sft < 0 ? -sft : 0)) & mask);
        }
    (void)TOP;
}

constexpr int dt_field_steps(int kt, int p, int f) { return (p & f) ? (kt * f + 3) / 4 : 0; }

template <int QP, int P, bool SIGNED, int NW, int D, bool FLIP_X = false>
__global__ __launch_bounds__(64 * NW) void gemm_decode_fields(const GemmArgs a, int mrows)
{
    static_assert(QP == 4 || QP == 8, "activations as records of one field");
    static_assert(P == 3 || P == 5 || P == 6 || P == 7, "weights of several fields");
    static_assert(!FLIP_X || (!SIGNED && QP == 8), "flipping is for unsigned 8-bit records");
    constexpr int MX = 8 / QP; // MFMAs per activation chunk
    constexpr int NT = 64 * NW;
    constexpr int QLOG = QP == 8 ? 3 : 2;
    constexpr int XC = 6;
    constexpr int WPOS = SIGNED ? 8 - P : 0; // place of the code's lowest bit in the byte
    extern __shared__ __align__(16) unsigned char smem[];
    int *red = reinterpret_cast<int *>(smem); // [NW][16][16]
    unsigned char *xs = smem + NW * 1024;     // [kt][row][QP chunks], chunks permuted within a row

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int M = a.M, N = a.N;
    const int KT = a.K >> 7;
    const int S4 = dt_field_steps(KT, P, 4), S2 = dt_field_steps(KT, P, 2), S1 = dt_field_steps(KT, P, 1);
    const int S = S4 + S2 + S1;
    const int tile0 = blockIdx.x;
    const int m0 = blockIdx.y * mrows;
    const int once = gridDim.y == 1;
    const int Mb = min(mrows, M - m0);
    const char *Xt = reinterpret_cast<const char *>(a.X);
    const char *Wt = reinterpret_cast<const char *>(a.W);
    const unsigned xs_addr = (unsigned)(size_t)xs;
    const int xchunks = KT * Mb * QP;

    // ---- activations: as in gemm_decode_tiled ---------------------------------------------------------
    if (Mb == M) {
#pragma unroll
        for (int i = 0; i < XC; ++i) {
            const int pb = wid * 64 + i * NT;
            if (pb < xchunks) {
                const int p = pb + lane;
                const int src = min(p ^ ((p >> QLOG) & (QP - 1)), xchunks - 1);
                dt_load_to_lds(Xt + (uint32_t)src * 16u, xs_addr + (unsigned)pb * 16u);
            }
        }
        for (int pb = wid * 64 + XC * NT; pb < xchunks; pb += NT) {
            const int p = pb + lane;
            const int src = min(p ^ ((p >> QLOG) & (QP - 1)), xchunks - 1);
            dt_load_to_lds(Xt + (uint32_t)src * 16u, xs_addr + (unsigned)pb * 16u);
        }
    } else {
        const int per = Mb * QP;
        for (int pb = wid * 64; pb < xchunks; pb += NT) {
            const int p = min(pb + lane, xchunks - 1);
            const int q = p ^ ((p >> QLOG) & (QP - 1));
            const int kt = q / per, rem = q - kt * per;
            dt_load_to_lds(Xt + ((size_t)(kt * M + m0) * QP + rem) * 16u, xs_addr + (unsigned)pb * 16u);
        }
    }

    // ---- weights: byte offset of (lane, field F, step cs) = K tile * tile_bytes + row_off + field_off[F] ----
    const uint32_t tile_bytes = (uint32_t)N * (P * 16u);
    const uint32_t row_off = (uint32_t)min(tile0 * 16 + r, N - 1) * (P * 16u);
    // flat step t -> field (4: t < S4; 2: t < S4 + S2; else 1) and the field's own step; wave-uniform
    auto weight_offset = [&](int t) -> uint32_t {
        int kt;
        uint32_t fo;
        if (t < S4) {
            kt = t;
            fo = 16u * field_list_index(P, 4) + 16u * g;
        } else if (t < S4 + S2) {
            kt = 2 * (t - S4) + (g >> 1);
            fo = 16u * field_list_index(P, 2) + 16u * (g & 1);
        } else {
            kt = 4 * (t - S4 - S2) + g;
            fo = 16u * field_list_index(P, 1);
        }
        return (uint32_t)min(kt, KT - 1) * tile_bytes + row_off + fo; // lanes past the end of K repeat the last K tile
    };

    v4i acc[2];
    acc[0] = acc[1] = v4i{ 0, 0, 0, 0 };
    const int ml = min(r, Mb - 1);

    // the activations of the unit (field F, step cs) of this lane group -> 8 / F MFMA operands
    auto read_x = [&](auto fc, int cs, v4i(&av)[8]) {
        constexpr int F = decltype(fc)::value;
        constexpr int NXL = QP >= F ? QP / F : 1; // activation chunks per weight unit
        const int uu = min(4 * cs + g, KT * F - 1);
        const int u0 = uu * NXL;
        const int rowi = (u0 >> QLOG) * Mb + ml;
#pragma unroll
        for (int i = 0; i < NXL; ++i) {
            const int part = ((u0 + i) & (QP - 1)) ^ (rowi & (QP - 1));
            const v4u xv = *reinterpret_cast<const v4u *>(xs + ((uint32_t)rowi * QP + part) * 16u);
            v4i tt[MX];
            dt_unpack<QP, SIGNED>(xv, tt);
            if constexpr (FLIP_X)
                tt[0] = v4i{ tt[0][0] ^ (int)0x80808080u, tt[0][1] ^ (int)0x80808080u, tt[0][2] ^ (int)0x80808080u,
                             tt[0][3] ^ (int)0x80808080u };
#pragma unroll
            for (int k = 0; k < MX; ++k)
                av[i * MX + k] = tt[k];
        }
    };
    auto multiply = [&](auto fc, int cs, const v4u &wraw, const v4i(&av)[8]) {
        constexpr int F = decltype(fc)::value;
        const bool ok = 4 * cs + g < KT * F;
        const v4u wv = ok ? wraw : v4u{ 0u, 0u, 0u, 0u };
        v4i bv[8 / F];
        dt_unpack_field<F, WPOS + field_base(P, F), SIGNED>(wv, bv);
#pragma unroll
        for (int i = 0; i < 8 / F; ++i)
            acc[i & 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[i], bv[i], acc[i & 1], 0, 0, 0);
    };

    int round = 0;
    do {
        v4u wb[D];
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int t = min(wid + (round * D + d) * NW, S - 1);
            wb[d] = dt_load16_weights(Wt, weight_offset(t), once);
        }
        if (round == 0) {
            dt_wait_loads<D>(); // the activation loads are older than these
            __syncthreads();
        }
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int t = wid + (round * D + d) * NW;
            const bool have = t < S; // wave-uniform
            v4i av[8];
            if (have) {
                if ((P & 4) && t < S4)
                    read_x(std::integral_constant<int, 4>{}, t, av);
                else if ((P & 2) && t < S4 + S2)
                    read_x(std::integral_constant<int, 2>{}, t - S4, av);
                else if (P & 1)
                    read_x(std::integral_constant<int, 1>{}, t - S4 - S2, av);
            }
            dt_wait_loads_n(D - 1 - d);
            dt_landed(wb[d]);
            if (have) {
                if ((P & 4) && t < S4)
                    multiply(std::integral_constant<int, 4>{}, t, wb[d], av);
                else if ((P & 2) && t < S4 + S2)
                    multiply(std::integral_constant<int, 2>{}, t - S4, wb[d], av);
                else if (P & 1)
                    multiply(std::integral_constant<int, 1>{}, t - S4 - S2, wb[d], av);
            }
        }
        ++round;
    } while (wid + round * D * NW < S);

    // ---- the waves' partial tiles meet in LDS ----------------------------------------------------------
#pragma unroll
    for (int e = 0; e < 4; ++e)
        if (4 * g + e < Mb)
            red[(wid * 16 + 4 * g + e) * 16 + r] = acc[0][e] + acc[1][e];
    __syncthreads();
    for (int o = tid; o < 256; o += NT) {
        const int n = tile0 * 16 + (o & 15);
        if ((o >> 4) < Mb && n < N) {
            int part[NW];
#pragma unroll
            for (int w = 0; w < NW; ++w)
                part[w] = red[w * 256 + o];
            int v = 0;
#pragma unroll
            for (int w = 0; w < NW; ++w)
                v += part[w];
            if (SIGNED)
                v >>= 16 - QP - P;
            if constexpr (FLIP_X)
                v = (int)((unsigned)v + 128u * (unsigned)a.w_row_sums[n]);
            store_result(a, m0 + (o >> 4), n, v);
        }
    }
}

template <int QP, int P, bool SIGNED, int NW, int D, bool MAY_FLIP>
static hipError_t launch_decode_fields(const GemmArgs &a, hipStream_t stream)
{
    const int mrows = decode_tiled_rows(NW, 1, a.M, a.K, QP);
    if (mrows == 0 || (size_t)a.N * a.K * P / 8 >= (1ull << 32) || (size_t)a.M * a.K * QP / 8 >= (1ull << 32))
        return hipErrorInvalidValue;
    const size_t lds = decode_tiled_lds(NW, 1, mrows, a.K, QP);
    const int tiles = (a.N + 15) / 16;
    const dim3 grid(tiles, (a.M + mrows - 1) / mrows);
    auto go = [&](auto kernel) -> hipError_t {
        const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (attr != hipSuccess)
            return attr;
        hipLaunchKernelGGL(kernel, grid, dim3(64 * NW), lds, stream, a, mrows);
        return hipGetLastError();
    };
    if constexpr (!SIGNED && QP == 8 && MAY_FLIP) {
        if (a.flip_x) { // true 8-bit codes (fed as value - 128); padded narrower codes go as they are
            if (!a.w_row_sums)
                return hipErrorInvalidValue;
            return go(&gemm_decode_fields<QP, P, SIGNED, NW, D, true>);
        }
    }
    return go(&gemm_decode_fields<QP, P, SIGNED, NW, D, false>);
}

template <int Q, int P, bool SIGNED, int NW, int D, int T, int XU, bool FLIP = false>
static hipError_t launch_decode_tiled_instance(const GemmArgs &a, int mrows, hipStream_t stream)
{
    const size_t lds = decode_tiled_lds(NW, T, mrows, a.K, Q);
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_decode_tiled<Q, P, SIGNED, NW, D, T, XU, FLIP>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr != hipSuccess)
        return attr;
    const int tiles = (a.N + 15) / 16;
    const dim3 grid((tiles + T - 1) / T, (a.M + mrows - 1) / mrows);
    hipLaunchKernelGGL((gemm_decode_tiled<Q, P, SIGNED, NW, D, T, XU, FLIP>), grid, dim3(64 * NW), lds, stream, a, mrows);
    return hipGetLastError();
}

template <int Q, int P, bool SIGNED, int NW, int D, int T, bool XF16 = false>
static hipError_t launch_decode_tiled(const GemmArgs &a, hipStream_t stream)
{
    const int mrows = decode_tiled_rows(NW, T, a.M, a.K, Q);
    if (mrows == 0 || (size_t)a.N * a.K * P / 8 >= (1ull << 32) || (size_t)a.M * a.K * (XF16 ? 16 : Q) / 8 >= (1ull << 32))
        return hipErrorInvalidValue;
    if (XF16 && !a.x_pack_scale)
        return hipErrorInvalidValue;
    if constexpr (XF16) {
        const int need = (int)(((size_t)mrows * a.K / 8 + 64 * NW - 1) / (64 * NW)); // units per thread for one pass
        if (need <= 1)
            return launch_decode_tiled_instance<Q, P, SIGNED, NW, D, T, 1>(a, mrows, stream);
        if (need <= 2)
            return launch_decode_tiled_instance<Q, P, SIGNED, NW, D, T, 2>(a, mrows, stream);
        return launch_decode_tiled_instance<Q, P, SIGNED, NW, D, T, 4>(a, mrows, stream);
    } else if constexpr (!SIGNED && Q == 8) {
        // unsigned 8-bit records: codes up to 255 in every 8-bit operand (flipped, row sums needed), or padded
        // narrower codes in every one (fed as they are); a mix of the two has no instance
        const bool flip_x = a.flip_x != 0, flip_w = P == 8 && a.flip_w != 0;
        if (!flip_x && !flip_w)
            return launch_decode_tiled_instance<Q, P, SIGNED, NW, D, T, 0>(a, mrows, stream);
        if (!flip_x || (P == 8 && !flip_w) || !a.w_row_sums || (P == 8 && !a.x_row_sums))
            return hipErrorInvalidValue;
        return launch_decode_tiled_instance<Q, P, SIGNED, NW, D, T, 0, true>(a, mrows, stream);
    } else {
        return launch_decode_tiled_instance<Q, P, SIGNED, NW, D, T, 0>(a, mrows, stream);
    }
}

// ---- the same plan with group-wise weight scales -------------------------------------------------
//
// D[m][n] = x_scale[m] * ( sum_g w_scale[n][g] * (acc_g - w_zero[n][g] * Sx[m][g]) - x_zero[m] * T[n] ),
// acc_g the integer dot product over scale group g; semantics of algorithm/quantize/quantizer.py:111-179 of the
// reference, groups of 128, fp16 output, optionally the fused SiLU gate (tile pairs: 16 gate rows, their 16 up rows).
//
// A matrix-core instruction sums over its four lane groups, so all four must hold elements of the same scale
// group: a step is ONE K tile (= one group of 128) here, lane group g holds 32 of its elements (4 P bytes of the
// weight record: an 8-, 16- or 32-byte load; the two 16-byte pieces 2g, 2g + 1 of an 8-bit activation record), and
// the step's two instructions leave acc_g itself, which is folded into fp32 with the group's scale right away.  For
// 2-bit weights the sixteen records of a tile's K tile are 512 contiguous bytes: one wave load covers them exactly.
// The scales, zero points and activation group sums of the workgroup's rows are staged in LDS as [group][16 rows]
// by four-byte DMA loads issued with the activations (no register, no wait before the weight loads; issuing them
// behind the weight loads and waiting for everything was 0.2 to 0.5 us slower), so the fold reads them with
// conflict-free ds_reads instead of a gather per step.  All the waves of a
// compute unit share one LDS pipeline, so bank conflicts on these reads cost real time here: with the rows stored
// as they lie in memory ([16 rows][groups], a column read is 8-way conflicted at 32 groups) the zero-point variant
// took 0.5 to 1 us longer.
typedef unsigned v2u __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void dt_dma_dword(const void *src, unsigned lds_addr)
{
    // lane l of the wave lands at lds_addr + 4 * l
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(src)
                 : "memory");
}

// a lane's share of one weight record (32 elements): P dwords
template <int P> struct DtgShare {
    v4u v[P / 4];
    static constexpr int kLoads = P / 4;
    __device__ __forceinline__ void issue(const char *base, uint32_t off, int once)
    {
#pragma unroll
        for (int i = 0; i < P / 4; ++i)
            v[i] = dt_load16_weights(base, off + 16u * i, once);
    }
    __device__ __forceinline__ void landed()
    {
#pragma unroll
        for (int i = 0; i < P / 4; ++i)
            dt_landed(v[i]);
    }
};
template <> struct DtgShare<2> {
    v2u v;
    static constexpr int kLoads = 1;
    __device__ __forceinline__ void issue(const char *base, uint32_t off, int once)
    {
        asm volatile("s_cmp_lg_u32 %3, 0\n\t"
                     "s_cbranch_scc1 .Ldt_once_%=\n\t"
                     "global_load_dwordx2 %0, %1, %2\n\t"
                     "s_branch .Ldt_issued_%=\n"
                     ".Ldt_once_%=:\n\t"
                     "global_load_dwordx2 %0, %1, %2 nt\n"
                     ".Ldt_issued_%=:"
                     : "=&v"(v)
                     : "v"(off), "s"(base), "s"(__builtin_amdgcn_readfirstlane(once))
                     : "memory", "scc");
    }
    __device__ __forceinline__ void landed() { asm volatile("" : "+v"(v)); }
};

// one dword of a 2-bit record -> one MFMA operand
template <bool SIGNED> __device__ __forceinline__ v4i dtg_unpack2(uint32_t w)
{
    if (SIGNED)
        return v4i{ (int)((w << 6) & 0xC0C0C0C0u), (int)((w << 4) & 0xC0C0C0C0u), (int)((w << 2) & 0xC0C0C0C0u), (int)(w & 0xC0C0C0C0u) };
    return v4i{ (int)(w & 0x03030303u), (int)((w >> 2) & 0x03030303u), (int)((w >> 4) & 0x03030303u), (int)((w >> 6) & 0x03030303u) };
}

template <int P, bool SIGNED> __device__ __forceinline__ void dtg_operands(const DtgShare<P> &w, v4i (&bv)[2])
{
    if constexpr (P == 2) {
        bv[0] = dtg_unpack2<SIGNED>(w.v[0]);
        bv[1] = dtg_unpack2<SIGNED>(w.v[1]);
    } else if constexpr (P == 4) {
        dt_unpack<4, SIGNED>(w.v[0], bv);
    } else {
        bv[0] = v4i{ (int)w.v[0][0], (int)w.v[0][1], (int)w.v[0][2], (int)w.v[0][3] };
        bv[1] = v4i{ (int)w.v[1][0], (int)w.v[1][1], (int)w.v[1][2], (int)w.v[1][3] };
    }
}

// XDYN: the activations arrive as fp16 [M][K] and are quantised here per token, symmetric or with a zero point
// (a.x_dynamic = 1 or 2), exactly as the quantise-and-pack kernel does it (abq_quant.h): every workgroup loads the
// rows it multiplies (at most XP * 64 NW units of eight halves), takes their extrema through LDS, writes the int8
// records and the group sums into LDS and keeps the rows' scales and zero points there for the epilogue.  The
// quantising launch in front of every decode GEMM, and the memory round trip between the two, fall away.
// XDYN is the number of units a thread holds (0: the activations arrive packed): 1, 2 or, with eight waves, 4, i.e. up
// to 16384 elements per workgroup; the launcher takes the smallest that covers the rows (a row of 4096 needs one unit
// per thread of eight waves: 52 + 25 registers instead of 52 + 49, three workgroups per compute unit instead of two).
// G64: groups of 64, two to a K tile: lane groups 0, 1 hold the elements of the first, 2, 3 those of the second, and
// the matrix core sums over all four, so a step runs its two instructions twice: once on all lanes and once with
// the activations of lane groups 2, 3 zeroed; the difference is the second group's dot product.  Scales, zero
// points and group sums are staged as [2 K tiles' worth of groups][16] and folded per half.
template <int Q, int P, bool SIGNED, int NW, int D, int T, int XDYN = 0, bool G64 = false>
__global__ __launch_bounds__(64 * NW) void gemm_decode_tiled_grouped(const GemmArgs a, int mrows)
{
    static_assert(!XDYN || (Q == 8 && SIGNED), "in-kernel quantisation writes signed 8-bit records");
    static_assert(!(XDYN && G64), "in-kernel quantisation takes group sums over 128 elements");
    constexpr int GPT = G64 ? 2 : 1; // scale groups per K tile
    static_assert(XDYN == 0 || XDYN == 1 || XDYN == 2 || (XDYN == 4 && NW == 8), "units per thread");
    constexpr int XP = XDYN > 0 ? XDYN : 1; // XDYN: units per thread
    constexpr int NT = 64 * NW;
    constexpr int QLOG = Q == 8 ? 3 : Q == 4 ? 2 : 1;
    constexpr int LPS = DtgShare<P>::kLoads; // loads per step and tile
    extern __shared__ __align__(16) unsigned char smem[];
    float *red = reinterpret_cast<float *>(smem); // [NW][T][16][16]
    unsigned char *xs = smem + NW * T * 1024;     // [kt][row][Q chunks], chunks permuted within a row

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int M = a.M, N = a.N;
    const int KT = a.K >> 7; // K tiles = scale groups = steps
    const int tile0 = blockIdx.x * T;
    const int m0 = blockIdx.y * mrows;
    const int once = gridDim.y == 1; // no other workgroup reads this one's weight records
    const int Mb = min(mrows, M - m0);
    const char *Xt = reinterpret_cast<const char *>(a.X);
    const char *Wt = reinterpret_cast<const char *>(a.W);
    const unsigned xs_addr = (unsigned)(size_t)xs;
    const int xchunks = KT * Mb * Q;
    const int NG = KT * GPT;                   // scale groups along K
    const int per_arr = (NG * 16 + 63) & ~63;  // floats of one [group][16] array, in whole wave loads
    float *sws = reinterpret_cast<float *>(xs + (size_t)mrows * (KT + 1) * Q * 16 + 1024); // [T][group][16]
    float *zws = sws + T * per_arr;                                                       // [T][group][16]
    int *sxs = reinterpret_cast<int *>(zws + T * per_arr);                                // [group][16]
    // XDYN: the rows' extrema (as integers that order like the floats), then their scales and zero points
    int *row_ext = sxs + per_arr;                                                         // [2][16]
    float *row_par = reinterpret_cast<float *>(row_ext + 32);                             // [2][16]
    const bool zp = a.w_zero != nullptr;
    const int upr = a.K >> 3; // XDYN: units of eight halves per row
    const int nunits = Mb * upr;
    const char *Xh = Xt + (size_t)m0 * a.K * 2;
    if constexpr (XDYN) {
        if (tid < 16) {
            row_ext[tid] = INT_MIN;      // maxima
            row_ext[16 + tid] = INT_MAX; // minima
        }
        __syncthreads(); // the extrema are initialised before any wave updates them
    }

    // ---- activations: LDS chunk p <- chunk p ^ ((p / Q) & (Q - 1)) of the workgroup's rows -----------
    if constexpr (!XDYN) {
        const int per = Mb * Q;
        for (int pb = wid * 64; pb < xchunks; pb += NT) {
            const int p = min(pb + lane, xchunks - 1);
            const int q = p ^ ((p >> QLOG) & (Q - 1));
            size_t src = (size_t)q;
            if (Mb != M) { // several blocks of rows: a K tile's rows are Mb * Q chunks out of M * Q
                const int kt = q / per, rem = q - kt * per;
                src = (size_t)(kt * M + m0) * Q + rem;
            }
            dt_load_to_lds(Xt + src * 16u, xs_addr + (unsigned)pb * 16u);
        }
    }
    // ---- scales, zero points of the tiles' rows and group sums of the activation rows: [group][16] ----
    {
        const int nfl = NG * 16;
#pragma unroll
        for (int t = 0; t < T; ++t) {
            for (int pb = wid * 64; pb < nfl; pb += NT) {
                const int p = min(pb + lane, nfl - 1);
                const int n = min((tile0 + t) * 16 + (p & 15), N - 1);
                const size_t src = (size_t)n * NG + (p >> 4);
                dt_dma_dword(a.w_scale + src, (unsigned)(size_t)(sws + t * per_arr + pb));
                if (zp)
                    dt_dma_dword(a.w_zero + src, (unsigned)(size_t)(zws + t * per_arr + pb));
            }
        }
        if (zp && !XDYN) {
            for (int pb = wid * 64; pb < nfl; pb += NT) {
                const int p = min(pb + lane, nfl - 1);
                const int m = m0 + min(p & 15, Mb - 1);
                dt_dma_dword(a.x_group_sums + (size_t)m * NG + (p >> 4), (unsigned)(size_t)(sxs + pb));
            }
        }
    }

    // ---- weights: byte offset of (lane, step s, tile t) = s * N * 16 P + woff[t] ----------------------
    uint32_t woff[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        const int n = min((tile0 + t) * 16 + r, N - 1);
        woff[t] = (uint32_t)n * (P * 16u) + (uint32_t)g * (4u * P);
    }
    const uint32_t step_bytes = (uint32_t)N * (P * 16u);

    float facc[T][4];
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e)
            facc[t][e] = 0.f;
    const int ml = min(r, Mb - 1);
    // the signed route feeds value * 2^(8 - bits): the exact power of two that undoes it rides on the scale
    const float unshift = SIGNED ? 1.0f / (float)(1 << (16 - Q - P)) : 1.0f;

    int round = 0;
    do {
        DtgShare<P> wb[D][T];
        v4u xr[XDYN ? XP : 1]; // (declared and loaded inside the round that uses them, like the weight registers)
        if (XDYN && round == 0) {
            // every pass is loaded, past the rows' end the last unit once more: a load under a condition would leave the
            // compiler a register to merge with an undefined one, and a copy it inserts for that reads before the data lands
#pragma unroll
            for (int i = 0; i < XP; ++i)
                xr[i] = dt_load16(Xh, (uint32_t)min(tid + i * NT, nunits - 1) * 16u);
        }
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int s = min(wid + (round * D + d) * NW, KT - 1); // steps past the end repeat the last one
            const char *wp = Wt + (size_t)s * step_bytes;
#pragma unroll
            for (int t = 0; t < T; ++t)
                wb[d][t].issue(wp, woff[t], once);
        }
        if (round == 0) {
            dt_wait_loads<D * T * LPS>(); // the DMA loads (and the rows' fp16 units) are older than these
            if constexpr (XDYN) {
                // extrema of the rows: per unit on the fp16 pairs, per wave across the lanes where the wave's units
                // of this pass belong to one row, then one LDS update per wave (per lane where rows meet in a wave)
                typedef _Float16 h2 __attribute__((ext_vector_type(2)));
#pragma unroll
                for (int i = 0; i < XP; ++i)
                    dt_landed(xr[i]);
#pragma unroll
                for (int i = 0; i < XP; ++i) {
                    if (i * NT < nunits) {
                        const int p = tid + i * NT;
                        union {
                            v4u q;
                            h2 h[4];
                        } raw;
                        raw.q = xr[i];
                        h2 mx2 = __builtin_elementwise_max(__builtin_elementwise_max(raw.h[0], raw.h[1]), __builtin_elementwise_max(raw.h[2], raw.h[3]));
                        h2 mn2 = __builtin_elementwise_min(__builtin_elementwise_min(raw.h[0], raw.h[1]), __builtin_elementwise_min(raw.h[2], raw.h[3]));
                        float mx = fmaxf((float)mx2.x, (float)mx2.y), mn = fminf((float)mn2.x, (float)mn2.y);
                        const int pc = min(p, nunits - 1);
                        const int row = pc / upr;
                        const int first = __builtin_amdgcn_readfirstlane(min(p - lane, nunits - 1) / upr);
                        const int last = __builtin_amdgcn_readfirstlane(min(p - lane + 63, nunits - 1) / upr);
                        auto ordered = [](float f) { const int k = __builtin_bit_cast(int, f); return k ^ ((k >> 31) & 0x7FFFFFFF); };
                        if (first == last) {
                            // across the wave with lane permutations inside the vector ALU (a shuffle through the LDS
                            // crossbar per step would be six dependent round trips): quads, halves of a row of 16, the
                            // row, then the rows' last lanes handed on; lane 63 ends up with the wave's extrema
                            auto dpp = [](float v, auto ctrl, auto row_mask) {
                                return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v),
                                                                                             decltype(ctrl)::value, decltype(row_mask)::value, 0xF, false));
                            };
                            using std::integral_constant;
                            mx = fmaxf(mx, dpp(mx, integral_constant<int, 0xB1>{}, integral_constant<int, 0xF>{}));  // quad_perm [1,0,3,2]
                            mn = fminf(mn, dpp(mn, integral_constant<int, 0xB1>{}, integral_constant<int, 0xF>{}));
                            mx = fmaxf(mx, dpp(mx, integral_constant<int, 0x4E>{}, integral_constant<int, 0xF>{}));  // quad_perm [2,3,0,1]
                            mn = fminf(mn, dpp(mn, integral_constant<int, 0x4E>{}, integral_constant<int, 0xF>{}));
                            mx = fmaxf(mx, dpp(mx, integral_constant<int, 0x141>{}, integral_constant<int, 0xF>{})); // row_half_mirror
                            mn = fminf(mn, dpp(mn, integral_constant<int, 0x141>{}, integral_constant<int, 0xF>{}));
                            mx = fmaxf(mx, dpp(mx, integral_constant<int, 0x140>{}, integral_constant<int, 0xF>{})); // row_mirror
                            mn = fminf(mn, dpp(mn, integral_constant<int, 0x140>{}, integral_constant<int, 0xF>{}));
                            mx = fmaxf(mx, dpp(mx, integral_constant<int, 0x142>{}, integral_constant<int, 0xA>{})); // row_bcast 15 into rows 1, 3
                            mn = fminf(mn, dpp(mn, integral_constant<int, 0x142>{}, integral_constant<int, 0xA>{}));
                            mx = fmaxf(mx, dpp(mx, integral_constant<int, 0x143>{}, integral_constant<int, 0xC>{})); // row_bcast 31 into rows 2, 3
                            mn = fminf(mn, dpp(mn, integral_constant<int, 0x143>{}, integral_constant<int, 0xC>{}));
                            if (lane == 63) {
                                atomicMax(&row_ext[row], ordered(mx));
                                atomicMin(&row_ext[16 + row], ordered(mn));
                            }
                        } else if (p < nunits) {
                            atomicMax(&row_ext[row], ordered(mx));
                            atomicMin(&row_ext[16 + row], ordered(mn));
                        }
                    }
                }
                __syncthreads();
                uint32_t sel_pair, sel_half;
                quad_transpose_selectors(tid & 3, sel_pair, sel_half);
                auto unordered = [](int k) { return __builtin_bit_cast(float, k ^ ((k >> 31) & 0x7FFFFFFF)); };
#pragma unroll
                for (int i = 0; i < XP; ++i) {
                    if (i * NT < nunits) { // quads and scale groups of a wave are whole: K is a multiple of 128
                        const int p = tid + i * NT;
                        const int pc = min(p, nunits - 1);
                        const int row = pc / upr, u = pc - row * upr;
                        const QuantRow qr = quant_row_params(unordered(row_ext[row]), unordered(row_ext[16 + row]), 8, a.x_dynamic == 1);
                        union {
                            v4u q;
                            _Float16 h[8];
                        } raw;
                        raw.q = xr[i];
                        int v[8], sum = 0;
#pragma unroll
                        for (int c = 0; c < 8; ++c) {
                            v[c] = quant_code((float)raw.h[c], qr);
                            sum += v[c];
                        }
                        // the sixteen units of a scale group sit in sixteen consecutive lanes
                        sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
                        sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
                        sum += __builtin_amdgcn_update_dpp(0, sum, 0x141, 0xF, 0xF, true); // row_half_mirror
                        sum += __builtin_amdgcn_update_dpp(0, sum, 0x140, 0xF, 0xF, true); // row_mirror
                        const uint32_t e_even = quad_transpose_bytes(pack_low_bytes(v[7], v[5], v[3], v[1]), sel_pair, sel_half);
                        const uint32_t e_odd = quad_transpose_bytes(pack_low_bytes(v[6], v[4], v[2], v[0]), sel_pair, sel_half);
                        if (p < nunits) {
                            const int rowi = (u >> 4) * Mb + row;            // K tile * rows + row
                            const int dw = 8 * ((u >> 2) & 3) + 2 * (u & 3); // first of the lane's two dwords in the record
                            const int chunk = (dw >> 2) ^ (rowi & 7);
                            *reinterpret_cast<uint2 *>(xs + ((uint32_t)rowi * 8 + chunk) * 16u + (dw & 3) * 4u) = make_uint2(e_even, e_odd);
                            if ((u & 15) == 0)
                                sxs[(u >> 4) * 16 + row] = sum;
                            if (u == 0) {
                                row_par[row] = qr.scale;
                                row_par[16 + row] = qr.zero_out;
                            }
                        }
                    }
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int cs = wid + (round * D + d) * NW;
            const bool have = cs < KT; // wave-uniform
            v4i av[2];
            float sw[T], zs[T], sxf[4];
            float sw2[G64 ? T : 1], zs2[G64 ? T : 1], sxf2[4]; // G64: the K tile's second group
            if (have) {
                const int rowi = cs * Mb + ml; // row index in LDS: K tile * rows + row
                const unsigned char *xrow = xs + (uint32_t)rowi * (Q * 16u);
                if (Q == 8) {
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        const v4u xv = *reinterpret_cast<const v4u *>(xrow + (((2 * g + i) ^ (rowi & 7)) * 16u));
                        av[i] = v4i{ (int)xv[0], (int)xv[1], (int)xv[2], (int)xv[3] };
                    }
                } else if (Q == 4) {
                    const v4u xv = *reinterpret_cast<const v4u *>(xrow + ((g ^ (rowi & 3)) * 16u));
                    dt_unpack<4, SIGNED>(xv, av);
                } else {
                    const v4u xv = *reinterpret_cast<const v4u *>(xrow + (((g >> 1) ^ (rowi & 1)) * 16u));
                    av[0] = dtg_unpack2<SIGNED>((g & 1) ? xv[2] : xv[0]);
                    av[1] = dtg_unpack2<SIGNED>((g & 1) ? xv[3] : xv[1]);
                }
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    sw[t] = sws[t * per_arr + (GPT * cs) * 16 + r];
                    zs[t] = zp ? sw[t] * zws[t * per_arr + (GPT * cs) * 16 + r] : 0.f;
                    sw[t] *= unshift;
                    if constexpr (G64) {
                        sw2[t] = sws[t * per_arr + (2 * cs + 1) * 16 + r];
                        zs2[t] = zp ? sw2[t] * zws[t * per_arr + (2 * cs + 1) * 16 + r] : 0.f;
                        sw2[t] *= unshift;
                    }
                }
                if (zp) {
                    const v4i sx = *reinterpret_cast<const v4i *>(sxs + (GPT * cs) * 16 + 4 * g);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        sxf[e] = (float)sx[e];
                    if constexpr (G64) {
                        const v4i sx2 = *reinterpret_cast<const v4i *>(sxs + (2 * cs + 1) * 16 + 4 * g);
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            sxf2[e] = (float)sx2[e];
                    }
                } else {
                    sxf[0] = sxf[1] = sxf[2] = sxf[3] = 0.f;
                    sxf2[0] = sxf2[1] = sxf2[2] = sxf2[3] = 0.f;
                }
            }
            // Waited for and marked as landed on every path: a register with a load still in flight must not
            // look free to the compiler.
            dt_wait_loads_n((D - 1 - d) * T * LPS);
#pragma unroll
            for (int t = 0; t < T; ++t)
                wb[d][t].landed();
            if (have) {
#pragma unroll
                for (int t = 0; t < T; ++t) {
                    v4i bv[2];
                    dtg_operands<P, SIGNED>(wb[d][t], bv);
                    v4i acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[0], bv[0], v4i{ 0, 0, 0, 0 }, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[1], bv[1], acc, 0, 0, 0);
                    if constexpr (G64) {
                        // the first group alone: the activations of lane groups 2, 3 zeroed
                        const v4i zero = v4i{ 0, 0, 0, 0 };
                        const v4i a0 = g < 2 ? av[0] : zero, a1 = g < 2 ? av[1] : zero;
                        v4i lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, bv[0], zero, 0, 0, 0);
                        lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, bv[1], lo, 0, 0, 0);
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            facc[t][e] += sw[t] * (float)lo[e] - zs[t] * sxf[e] + sw2[t] * (float)(acc[e] - lo[e]) - zs2[t] * sxf2[e];
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            facc[t][e] += sw[t] * (float)acc[e] - zs[t] * sxf[e];
                    }
                }
            }
        }
        ++round;
    } while (wid + round * D * NW < KT);

    // ---- the waves' partial tiles meet in LDS, summed in a fixed order ---------------------------------
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e)
            red[((wid * T + t) * 16 + 4 * g + e) * 16 + r] = facc[t][e];
    __syncthreads();
    for (int o = tid; o < T * 256; o += NT) {
        const int t = o >> 8, rem = o & 255, i = rem >> 4, c = rem & 15;
        const int n = (tile0 + t) * 16 + c;
        if (i < Mb && n < N && !(a.act && (t & 1))) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w)
                v += red[(w * T + t) * 256 + rem];
            const bool row_zero = XDYN ? a.x_dynamic == 2 : a.x_zero != nullptr;
            const float xz = !row_zero ? 0.f : XDYN ? row_par[16 + i] : a.x_zero[m0 + i];
            const float xsc = XDYN ? row_par[i] : a.x_scale[m0 + i];
            if (row_zero)
                v -= xz * a.w_zero_term[n];
            v *= xsc;
            if (T > 1 && a.act) { // this tile holds gate rows, the next one their up rows
                float up = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w)
                    up += red[(w * T + (T > 1 ? t + 1 : t)) * 256 + rem];
                if (row_zero)
                    up -= xz * a.w_zero_term[n + 16];
                up *= xsc;
                reinterpret_cast<_Float16 *>(a.D)[(size_t)(m0 + i) * (N / 2) + (n >> 5) * 16 + c] = (_Float16)(silu(v) * up);
            } else {
                reinterpret_cast<_Float16 *>(a.D)[(size_t)(m0 + i) * N + n] = (_Float16)v;
            }
        }
    }
}

template <int Q, int P, bool SIGNED, int NW, int D, int T, int XD, bool G64 = false>
static hipError_t launch_decode_tiled_grouped_instance(const GemmArgs &a, int mrows, hipStream_t stream)
{
    const size_t lds = decode_tiled_grouped_lds(NW, T, mrows, a.K, Q, G64 ? 64 : 128);
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_decode_tiled_grouped<Q, P, SIGNED, NW, D, T, XD, G64>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr != hipSuccess)
        return attr;
    const int tiles = (a.N + 15) / 16;
    const dim3 grid((tiles + T - 1) / T, (a.M + mrows - 1) / mrows);
    hipLaunchKernelGGL((gemm_decode_tiled_grouped<Q, P, SIGNED, NW, D, T, XD, G64>), grid, dim3(64 * NW), lds, stream, a, mrows);
    return hipGetLastError();
}

// (waves, loads in flight per wave, tiles) by shape; the fused gate needs a tile pair per workgroup.
template <int Q, int P, bool SIGNED, int NW, int D, int T, bool XDYN = false>
static hipError_t launch_decode_tiled_grouped_as(const GemmArgs &a, hipStream_t stream)
{
    const int mrows = decode_tiled_grouped_rows(NW, T, a.M, a.K, Q, a.group_size);
    if (mrows == 0)
        return hipErrorInvalidValue;
    // in-kernel quantisation: a workgroup's rows fit its threads' registers (two or four units of eight halves each)
    if (XDYN && (size_t)mrows * a.K > 16384)
        return hipErrorInvalidValue;
    if (a.group_size == 64) {
        if constexpr (XDYN)
            return hipErrorInvalidValue;
        else
            return launch_decode_tiled_grouped_instance<Q, P, SIGNED, NW, D, T, 0, true>(a, mrows, stream);
    }
    if constexpr (XDYN) {
        // the fewest units per thread that cover the workgroup's rows
        const int need = (int)(((size_t)mrows * a.K / 8 + 64 * NW - 1) / (64 * NW));
        if (need <= 1)
            return launch_decode_tiled_grouped_instance<Q, P, SIGNED, NW, D, T, 1>(a, mrows, stream);
        if (need <= 2 || NW == 16)
            return launch_decode_tiled_grouped_instance<Q, P, SIGNED, NW, D, T, 2>(a, mrows, stream);
        return launch_decode_tiled_grouped_instance<Q, P, SIGNED, NW, D, T, NW == 8 ? 4 : 2>(a, mrows, stream);
    } else {
        return launch_decode_tiled_grouped_instance<Q, P, SIGNED, NW, D, T, 0>(a, mrows, stream);
    }
}

template <int Q, int P, bool SIGNED, int T, bool XDYN = false>
static hipError_t launch_decode_tiled_grouped_t(const GemmArgs &a, hipStream_t stream)
{
    // loads in flight per wave, in units of 8 bytes per lane: 2 or 6 (1 or 3 steps of 8-bit weights)
    constexpr int DS = P == 8 ? 1 : 2, DL = P == 8 ? 3 : 6, DM = P == 8 ? 2 : 4;
    const int KT = a.K / 128;
    const int wgs = ((a.N + 15) / 16 + T - 1) / T;
    // (the quantising variant on tile pairs has no registers left for the long instances: more rounds instead)
    constexpr bool kLong = !(XDYN && T == 2);
    if (wgs > 512) // twice the workgroups fit a compute unit with eight waves
        return kLong && (KT + 7) / 8 > DM ? launch_decode_tiled_grouped_as<Q, P, SIGNED, 8, kLong ? DL : DM, T, XDYN>(a, stream)
                                          : launch_decode_tiled_grouped_as<Q, P, SIGNED, 8, DM, T, XDYN>(a, stream);
    return kLong && (KT + 15) / 16 > DS ? launch_decode_tiled_grouped_as<Q, P, SIGNED, 16, kLong ? DL : DS, T, XDYN>(a, stream)
                                        : launch_decode_tiled_grouped_as<Q, P, SIGNED, 16, DS, T, XDYN>(a, stream);
}

template <int Q, int P, bool SIGNED, bool XDYN = false> static hipError_t launch_decode_tiled_grouped(const GemmArgs &a, hipStream_t stream)
{
    if ((a.group_size != 128 && !(a.group_size == 64 && !XDYN)) || !a.w_scale || (!XDYN && !a.x_scale) || (size_t)a.N * a.K * P / 8 >= (1ull << 32) ||
        (size_t)a.M * a.K * Q / 8 >= (1ull << 32) || (XDYN && (a.x_dynamic < 1 || a.x_dynamic > 2 || (a.x_dynamic == 2 && !a.w_zero_term))))
        return hipErrorInvalidValue;
    if (a.act) {
        if (a.N % 32 != 0)
            return hipErrorInvalidValue;
        return launch_decode_tiled_grouped_t<Q, P, SIGNED, 2, XDYN>(a, stream);
    }
    // More than 8 rows on wide outputs: two tiles per workgroup as well, so that the rows a workgroup stages (64 KB at
    // 16 x 4096 8-bit activations, five times the weights of one tile) serve twice the weights; W2A8 16 x 12288 x 4096
    // 9.9 against 11.1 us, 16 x 11008 x 4096 9.7 against 11.0 (at 8 rows 7.2 against 6.8: not taken).  Only where the
    // rows of a block stay the same, and not for shapes the variant that quantises in the kernel takes (at most 16384
    // elements), whose output has to stay that of this one bit for bit.
    if (!XDYN && a.M > 8 && (size_t)a.M * a.K > 16384 && (a.N + 15) / 16 >= 512 && a.N % 32 == 0 &&
        decode_tiled_grouped_rows(16, 2, a.M, a.K, Q, a.group_size) == decode_tiled_grouped_rows(16, 1, a.M, a.K, Q, a.group_size))
        return launch_decode_tiled_grouped_t<Q, P, SIGNED, 2, XDYN>(a, stream);
    return launch_decode_tiled_grouped_t<Q, P, SIGNED, 1, XDYN>(a, stream);
}

// Native tile space of this kernel: (waves, weight loads in flight per wave, tiles per workgroup).  Entries name
// MFMA 16x16x64 with NSTAGE = 6; wk = waves, tn = tiles, kb = K elements a wave has in flight (D steps).
#define ABQ_DT_VARIANTS(V) V(16, 1, 1) V(16, 3, 1) V(8, 2, 1) V(16, 1, 3) V(8, 1, 2) V(8, 2, 2) V(16, 1, 2)

#define ABQ_DT_ENTRY_T(NW, D, T) { 16, 1, T, 1, 1, NW, 6, &launch_decode_tiled<ABQ_Q, ABQ_P, true, NW, D, T>, (512 / ABQ_P) * D },
#define ABQ_DT_ENTRY_F(NW, D, T) { 16, 1, T, 1, 1, NW, 6, &launch_decode_tiled<ABQ_Q, ABQ_P, false, NW, D, T>, (512 / ABQ_P) * D },

// activations of 3, 5, 6 or 7 bits reach these kernels as records of the next single-field width
#define ABQ_QP (ABQ_Q == 3 ? 4 : (ABQ_Q >= 5 && ABQ_Q <= 7) ? 8 : ABQ_Q)
#define ABQ_P_ONE_FIELD (ABQ_P == 2 || ABQ_P == 4 || ABQ_P == 8)
#define ABQ_Q_ONE_FIELD (ABQ_Q == 2 || ABQ_Q == 4 || ABQ_Q == 8)

#if ABQ_Q_ONE_FIELD && ABQ_P_ONE_FIELD
static const KernelEntry kSigned[] = { ABQ_DT_VARIANTS(ABQ_DT_ENTRY_T) };
// the single-tile instances with in-kernel quantisation of fp16 activations (8-bit activations, signed), same order
#if ABQ_Q == 8
#define ABQ_DT_ENTRY_X(NW, D, T) { 16, 1, T, 1, 1, NW, 6, &launch_decode_tiled<ABQ_Q, ABQ_P, true, NW, D, T, true>, (512 / ABQ_P) * D },
static const KernelEntry kSignedF16[] = { ABQ_DT_ENTRY_X(16, 1, 1) ABQ_DT_ENTRY_X(16, 3, 1) ABQ_DT_ENTRY_X(8, 2, 1) };
#define ABQ_DT_NF16 3
#else
static const KernelEntry *const kSignedF16 = nullptr;
#define ABQ_DT_NF16 0
#endif
// one entry: the launcher picks waves, loads in flight and tiles by shape
static const KernelEntry kSignedGrouped[] = { { 16, 1, 1, 1, 1, 16, 6, &launch_decode_tiled_grouped<ABQ_Q, ABQ_P, true>, 128 } };
// ... and the same quantising fp16 activations per token itself (8-bit activations)
#if ABQ_Q == 8
static const KernelEntry kSignedGroupedDyn[] = { { 16, 1, 1, 1, 1, 16, 6, &launch_decode_tiled_grouped<ABQ_Q, ABQ_P, true, true>, 128 } };
#define ABQ_DT_NDYN 1
#else
static const KernelEntry *const kSignedGroupedDyn = nullptr;
#define ABQ_DT_NDYN 0
#endif
#if ABQ_Q < 8
static const KernelEntry kUnsignedGrouped[] = { { 16, 1, 1, 1, 1, 16, 6, &launch_decode_tiled_grouped<ABQ_Q, ABQ_P, false>, 128 } };
#else
static const KernelEntry *const kUnsignedGrouped = nullptr;
#endif
static const KernelEntry kUnsigned[] = { ABQ_DT_VARIANTS(ABQ_DT_ENTRY_F) };
#define ABQ_DT_NUNSIGNED ((int)(sizeof(kUnsigned) / sizeof(kUnsigned[0])))
#define ABQ_DT_NSIGNED ((int)(sizeof(kSigned) / sizeof(kSigned[0])))
#else
static const KernelEntry *const kSignedGrouped = nullptr;
static const KernelEntry *const kUnsignedGrouped = nullptr;
static const KernelEntry *const kSignedGroupedDyn = nullptr;
#define ABQ_DT_NDYN 0
static const KernelEntry *const kSignedF16 = nullptr;
#define ABQ_DT_NF16 0
#if ABQ_P_ONE_FIELD
// activations of several fields over weights of one (W2A6): the kernel above on activation records padded to ABQ_QP bits
#define ABQ_DT_ENTRY_PT(NW, D, T) { 16, 1, T, 1, 1, NW, 6, &launch_decode_tiled<ABQ_QP, ABQ_P, true, NW, D, T>, (512 / ABQ_P) * D },
#define ABQ_DT_ENTRY_PF(NW, D, T) { 16, 1, T, 1, 1, NW, 6, &launch_decode_tiled<ABQ_QP, ABQ_P, false, NW, D, T>, (512 / ABQ_P) * D },
static const KernelEntry kSigned[] = { ABQ_DT_VARIANTS(ABQ_DT_ENTRY_PT) };
static const KernelEntry kUnsigned[] = { ABQ_DT_VARIANTS(ABQ_DT_ENTRY_PF) };
#else
// weights of several fields: (waves, weight loads in flight per wave); warp K in the tile's name = 128 D
#define ABQ_DF_VARIANTS(V) V(16, 2) V(16, 4) V(8, 4)
#define ABQ_DF_ENTRY_T(NW, D) { 16, 1, 1, 1, 1, NW, 6, &launch_decode_fields<ABQ_QP, ABQ_P, true, NW, D, false>, 128 * D },
#define ABQ_DF_ENTRY_F(NW, D) { 16, 1, 1, 1, 1, NW, 6, &launch_decode_fields<ABQ_QP, ABQ_P, false, NW, D, ABQ_Q == 8>, 128 * D },
static const KernelEntry kSigned[] = { ABQ_DF_VARIANTS(ABQ_DF_ENTRY_T) };
static const KernelEntry kUnsigned[] = { ABQ_DF_VARIANTS(ABQ_DF_ENTRY_F) };
#endif
#define ABQ_DT_NUNSIGNED ((int)(sizeof(kUnsigned) / sizeof(kUnsigned[0])))
#define ABQ_DT_NSIGNED ((int)(sizeof(kSigned) / sizeof(kSigned[0])))
#endif

#define ABQ_CAT_(a, b, c, d) a##b##c##d
#define ABQ_CAT(a, b, c, d) ABQ_CAT_(a, b, c, d)

void ABQ_CAT(abq_decode_tiled_register_, ABQ_Q, _, ABQ_P)(KernelTable *out)
{
    out[0] = KernelTable{ ABQ_Q, ABQ_P, 1, kSigned, ABQ_DT_NSIGNED };
    out[1] = KernelTable{ ABQ_Q, ABQ_P, 0, kUnsigned, ABQ_DT_NUNSIGNED };
}

void ABQ_CAT(abq_decode_tiled_f16_register_, ABQ_Q, _, ABQ_P)(KernelTable *out)
{
    out[0] = KernelTable{ ABQ_Q, ABQ_P, 1, kSignedF16, ABQ_DT_NF16 };
    out[1] = KernelTable{ ABQ_Q, ABQ_P, 0, nullptr, 0 };
}

void ABQ_CAT(abq_decode_tiled_grouped_register_, ABQ_Q, _, ABQ_P)(KernelTable *out)
{
    out[0] = KernelTable{ ABQ_Q, ABQ_P, 1, kSignedGrouped, kSignedGrouped ? 1 : 0 };
    out[1] = KernelTable{ ABQ_Q, ABQ_P, 0, kUnsignedGrouped, kUnsignedGrouped ? 1 : 0 };
}

void ABQ_CAT(abq_decode_tiled_grouped_dyn_register_, ABQ_Q, _, ABQ_P)(KernelTable *out)
{
    out[0] = KernelTable{ ABQ_Q, ABQ_P, 1, kSignedGroupedDyn, ABQ_DT_NDYN };
    out[1] = KernelTable{ ABQ_Q, ABQ_P, 0, nullptr, 0 };
}

} // namespace abq

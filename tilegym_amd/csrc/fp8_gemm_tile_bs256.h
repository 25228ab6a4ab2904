// 256x256 block-scaled tile, persistent, three weight slabs: C[m,n] = sum_kb As[m,kb] * Bs[n/128,kb] * sum_{k in kb} A[m,k] * B[n,k].
//
// Same slab layout, swizzles, fragment addressing, per-accumulator arithmetic (one fused multiply-add of every K
// block's 16x16 product with As * Bs, K blocks in ascending order) and epilogue as
// fp8_gemm_tile_kernel<256, 256, 4, 2, true, GROUP, false>: identical results.  What differs is the schedule, which is
// the one of fp8_gemm_tile256_kernel carried over to eight waves (the scale-and-add is VALU work on the accumulators,
// so they have to live in ordinary registers: 128 per lane, i.e. a 64 x 128 part of the tile per wave):
//   * All 160 KiB of LDS hold operand slabs -- two activation slabs and THREE weight slabs -- so that a step can
//     request the weights of step k+2 between its first MFMAs and needs one barrier: the weights, which stream from
//     HBM, get 1.25 - 2 steps to land instead of one.  No scale tables and no row maps in LDS:
//       - the scales travel in registers in chunks of four K steps: lane (row li, K group lg) of a wave holds, for
//         each of the wave's four 16-row groups, As[row li][4c + lg] * Bs[wave's column block][4c + lg] (one 4-byte load
//         per row group and chunk, 16 rows x 16 contiguous bytes per instruction, plus one for the weight scales; the
//         product is formed once per chunk); the value a step needs is fetched from the lane that holds it with one
//         ds_bpermute per row group (the LDS crossbar, no LDS memory); chunk c+1 is requested during the first step of
//         chunk c.  The loop is bound by VALU issue (an MFMA holds the issue port for about as long as its four
//         scale-and-add instructions, together exactly the MFMA's time in the matrix pipe), so the scale path costs
//         one VALU instruction per step and wave.
//   * Persistent: one workgroup per compute unit walks its tiles, and the slab rings run on across tiles: the last
//     two K steps of a tile request steps 0 and 1 of the workgroup's next tile, so set-up and first-load latency of a
//     tile (8 - 11 k clocks of a 16-step MoE tile) are hidden behind the previous tile's last steps and epilogue.
//   * All waves load, one 1 KiB direct load behind each group of MFMAs (weights behind column tiles 0 - 3, activations
//     behind the row groups of column tile 7), never in bursts.
// The activation-scale loads write registers from inline assembly (the compiler's own wait-count insertion cannot see
// the direct loads and would drain them all in front of the first use of an ordinary load's result).  Their
// completion is covered by the step's vmcnt wait: a chunk is used two steps or more after it was requested, and
// every step waits for all but its own four most recent weight loads.
// K must be at least two steps (256).
#pragma once

#include "fp8_gemm_tile.h"
#include "tg_host.h"

namespace tg {

// Raw buffer descriptor over [base, base + bytes): reads past the end return zero.
__device__ __forceinline__ v4i make_rsrc_sized(const void* base, uint32_t bytes) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(base);
    const int lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    const int hi = __builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xFFFFu));
    return v4i{lo, hi, __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000};
}

// 4 bytes per lane from a buffer into a register.  The caller orders its use behind a vmcnt wait by hand.
// (s_nop 4: five wait states between a vector instruction that wrote the scalar offset and this read of it,
// which the compiler does not insert in front of inline assembly.)
__device__ __forceinline__ int buffer_load_b32_raw(v4i rsrc, uint32_t voffset, int soffset) {
    int r;
    soffset = __builtin_amdgcn_readfirstlane(soffset);
    asm volatile("s_nop 4\n\tbuffer_load_dword %0, %1, %2, %3 offen" : "=v"(r) : "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
    return r;
}

// One float at a wave-uniform address: a scalar load.
__device__ __forceinline__ float uniform_load_f32(const float* p) {
    return *(const __attribute__((address_space(4))) float*)(uintptr_t)p;
}
__device__ __forceinline__ int uniform_load_i32(const int* p) {
    return *(const __attribute__((address_space(4))) int*)(uintptr_t)p;
}

// TAIL: the number of K steps need not be a multiple of four (one select per row group and step more; K % 512 == 128,
// a tile whose last chunk of scales is a single step, stays with the generic kernel)
template <int GROUP, bool TAIL>
__global__ void __launch_bounds__(512, 1) fp8_gemm_bs256_kernel(const GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    static_assert(GROUP == GROUP_DENSE || GROUP == GROUP_RAGGED, "row modes of this kernel");
    constexpr int BM = 256, BN = 256, WGM = 4, WGN = 2, NW = 8;
    constexpr int WTN = BN / WGN;                 // 128 columns per wave: one weight-block scale per wave and K step
    constexpr int TM = 4, TN = WTN / 16;          // 4 row groups x 8 column tiles per wave
    constexpr int SLAB = 256 * kKBlock;           // 32 KiB
    constexpr int A_STAGES = 2, B_STAGES = 3;
    constexpr int IT = 256 / (8 * NW);            // 4 loads per wave, slab and step
    constexpr int QUAD = 4;                       // K steps per chunk of activation scales
    static_assert(TN == 8 && IT == 4 && TM == 4, "the schedule below is written for 4 x 8 MFMA tiles and 4 + 4 loads per wave");

    __shared__ __align__(1024) uint8_t sA[A_STAGES * SLAB];
    __shared__ __align__(1024) uint8_t sB[B_STAGES * SLAB];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;
    const int K = p.K, kblocks = p.kblocks;
    // The once-per-tile code (tile lookup, hand-over, epilogue) reads the kernel arguments again from the argument segment
    // through a pointer the compiler cannot see through: kept in scalar registers across the K loop, with the loop's own
    // state, they are more than the scalar register file holds, and what does not fit is spilled to vector lanes.
    typedef const __attribute__((address_space(4))) GemmParams* ParamPtr;
    auto args = [&]() __attribute__((always_inline)) {
        ParamPtr q = (ParamPtr)__builtin_amdgcn_kernarg_segment_ptr();
        asm volatile("" : "+s"(q));
        return q;
    };
    const int tiles_n = (args()->N + BN - 1) / BN;
    const int nsteps = kblocks, last = nsteps - 1;
    const int stride = (int)gridDim.x;

    // ---------------------------------------------------------------- the tile sequence
    // Workgroup b computes positions b, b + grid, b + 2 grid, ... of the sequence; xcd_remap gives each XCD (own L2) a
    // contiguous range of it.  A position is a (row tile, column tile) pair: dense row tiles in groups of eight with the
    // column tile varying slowest inside a group; ragged row tiles (the 256-row pieces of the experts' segments, counted
    // on the device from m_indptr) with the column tile varying fastest, so that the row tiles of an expert run on one XCD
    // at about the same time and share its weights there.
    struct Tile {
        int m0, n0, rows, expert;  // first row (of A and C), first column, valid rows (<= 256), expert (ragged)
    };
    int total;
    if constexpr (GROUP == GROUP_DENSE) total = ((args()->M + BM - 1) / BM) * tiles_n;
    else total = ragged_count_tiles(args()->m_indptr, args()->E, BM, lane) * tiles_n;
    total = __builtin_amdgcn_readfirstlane(total);
    auto locate = [&](int v) -> Tile {
        Tile t{0, 0, 0, 0};
        ParamPtr q = args();
        const int pid = xcd_remap(v, total);
        if constexpr (GROUP == GROUP_DENSE) {
            const int tiles_m = (q->M + BM - 1) / BM;
            constexpr int GM = 8;
            const int width = GM * tiles_n;
            const int group = pid / width, first_m = group * GM;
            const int gsz = min(tiles_m - first_m, GM);
            t.m0 = (first_m + (pid % width) % gsz) * BM;
            t.n0 = ((pid % width) / gsz) * BN;
            t.rows = min(BM, q->M - t.m0);
        } else {
            const int tile_m = pid / tiles_n;
            t.n0 = (pid % tiles_n) * BN;
            int e, t_in_e;
            ragged_find(q->m_indptr, q->E, BM, lane, tile_m, e, t_in_e);
            e = __builtin_amdgcn_readfirstlane(e);
            t_in_e = __builtin_amdgcn_readfirstlane(t_in_e);
            e = max(e, 0);
            const int lo = uniform_load_i32(q->m_indptr + e), hi = min(uniform_load_i32(q->m_indptr + e + 1), q->M);
            // (the clamps only matter for a malformed m_indptr: it costs wrong rows, never an access out of range)
            t.m0 = min(max(lo + t_in_e * BM, 0), q->M - 1);
            t.rows = max(min(min(BM, hi - t.m0), q->M - t.m0), 1);
            t.expert = e;
        }
        t.m0 = __builtin_amdgcn_readfirstlane(t.m0);
        t.n0 = __builtin_amdgcn_readfirstlane(t.n0);
        t.rows = __builtin_amdgcn_readfirstlane(t.rows);
        return t;
    };
    int vt = (int)blockIdx.x;
    if (vt >= total) return;
    Tile cur_t = locate(vt);

    // ---------------------------------------------------------------- direct loads
    // pass i of wave w fills slab rows 8*(i*8 + w) .. +7 (lane l: row + l/8, chunk position l%8)
    const int lrow = lane >> 3;
    const int lj = (lane & 7) ^ swz16(lrow);
    const int ljb = (lane & 7) ^ swz_w(((wave & 1) << 3) | lrow);
    const int li = lane & 15, lg = lane >> 4;
    // (the rows of a pass are 64 rows below those of the pass before: one per-lane offset per operand, the pass in the
    // scalar offset; rows past the end of an operand read zeros through the sized descriptors, and rows of the tensor
    // that are not rows of this tile are computed and never stored)
    // (one descriptor over the weights of all experts, the expert in the per-lane offset: the whole weight tensor is below
    // 4 GiB, the host checks; a descriptor per expert would be loop-carried scalar state the register file has no room for)
    uint32_t a_off, b_off;
    auto set_offsets = [&](const Tile& t) {
        a_off = (uint32_t)(t.m0 + wave * 8 + lrow) * (uint32_t)K + lj * 16;
        uint32_t brow = (uint32_t)(t.n0 + wave * 8 + lrow);
        if constexpr (GROUP != GROUP_DENSE) brow += (uint32_t)t.expert * (uint32_t)p.N;
        b_off = brow * (uint32_t)K + ljb * 16;
    };
    set_offsets(cur_t);
    const v4i rsrc_b = make_rsrc_sized(p.B, (uint32_t)(GROUP == GROUP_DENSE ? 1 : p.E) * (uint32_t)p.N * (uint32_t)K);
    const v4i rsrc_a = make_rsrc_sized(p.A, (uint32_t)p.M * (uint32_t)K);
    const v4i rsrc_s = make_rsrc_sized(p.As, (uint32_t)p.M * (uint32_t)kblocks * 4u);
    const uint32_t ldsA = lds_address(sA) + wave * 1024, ldsB = lds_address(sB) + wave * 1024;
    // (address arithmetic on scalars that the compiler must redo at every use: hoisted out of the loops as loop
    // invariants, these few dozen values are more than the scalar register file holds next to the loop's own state)
    auto fresh = [](int x) __attribute__((always_inline)) {
        asm volatile("" : "+s"(x));
        return x;
    };
    auto load_a = [&](int i, int kstep, int stage) {
        direct_load_b128(rsrc_a, fresh(ldsA) + stage * SLAB + i * NW * 1024, a_off, kstep * kKBlock + i * 64 * fresh(K));
    };
    auto load_b = [&](int i, int kstep, int stage) {
        direct_load_b128(rsrc_b, fresh(ldsB) + stage * SLAB + i * NW * 1024, b_off, kstep * kKBlock + i * 64 * fresh(K));
    };

    // ---------------------------------------------------------------- fragment addresses (see fp8_gemm_tile.h)
    const uint32_t frag0 = wm * 16 * kKBlock + li * kKBlock + ((lg ^ swz16(li)) << 4), frag1 = frag0 ^ 64;
    const int wrow = ((li >> 2) << 3) | (li & 3);
    const uint32_t wfrag0 = wn * WTN * kKBlock + wrow * kKBlock + ((lg ^ swz_w(wrow)) << 4), wfrag1 = wfrag0 ^ 64;
    auto read_a = [&](int tm, const uint8_t* cA) {
        const uint8_t* base = cA + tm * (WGM * 16 * kKBlock);
        return join(*reinterpret_cast<const v4i*>(base + frag0), *reinterpret_cast<const v4i*>(base + frag1));
    };
    auto read_w = [&](int tn, const uint8_t* cB) {
        const uint8_t* base = cB + ((tn >> 1) * 32 + (tn & 1) * 4) * kKBlock;
        return join(*reinterpret_cast<const v4i*>(base + wfrag0), *reinterpret_cast<const v4i*>(base + wfrag1));
    };
    auto tile_row = [&](int tm) { return (tm * WGM + wm) * 16; };

    // ---------------------------------------------------------------- scales
    // Chunk q (K steps 4q .. 4q+3) of a tile: lane (li, lg) loads As[row(tm, li)][4q + lg] for tm = 0 .. 3 and
    // Bs[column block of the wave][4q + lg].  Steps past the end of a row read what follows in memory (zero past the end
    // of the tensor): those lanes' values are never used.
    const v4i rsrc_bs = make_rsrc_sized(p.Bs, (uint32_t)(GROUP == GROUP_DENSE ? 1 : p.E) * (uint32_t)p.nblocks * (uint32_t)kblocks * 4u);
    uint32_t roff;       // byte offset of As[row(0, li)][lg] for the tile whose scales are requested next (row group tm: 64 rows on)
    int bs_soff;         // byte offset of the first weight scale of that tile for this wave
    auto set_scale_rows = [&](const Tile& t) {
        roff = ((uint32_t)(t.m0 + tile_row(0) + li) * (uint32_t)kblocks + (uint32_t)lg) * 4u;
        const int nblocks = p.nblocks;
        int brow = min(t.n0 / 128 + wn, nblocks - 1);
        if constexpr (GROUP != GROUP_DENSE) brow += t.expert * nblocks;
        bs_soff = brow * kblocks * 4;
    };
    const uint32_t lg4 = lg * 4;
    int s_nxt[TM], bs_nxt;   // the chunk after the current one: raw scales as requested, then (form_products) As * Bs
    float s_cur[TM];         // As * Bs of the current chunk
    auto request_scales = [&](int first_step) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) s_nxt[tm] = buffer_load_b32_raw(rsrc_s, roff, (first_step + tm * (WGM * 16) * fresh(kblocks)) * 4);
        bs_nxt = buffer_load_b32_raw(rsrc_bs, lg4, bs_soff + first_step * 4);
    };
    // As * Bs of the requested chunk, in place.  (The loaded registers count as written here, not where the loads were
    // issued: the compiler must not move the products up to a place where the data may still be in flight.)
    auto form_products = [&]() {
        asm volatile("" : "+v"(s_nxt[0]), "+v"(s_nxt[1]), "+v"(s_nxt[2]), "+v"(s_nxt[3]), "+v"(bs_nxt));
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) s_nxt[tm] = __float_as_int(__int_as_float(s_nxt[tm]) * __int_as_float(bs_nxt));
    };
    const int bp_base = li * 4;  // ds_bpermute address of lane (li, 0)

    v4f acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = v4f{0.f, 0.f, 0.f, 0.f};

    constexpr int kWaitBut8 = 0x0F70 | 8, kWaitBut4 = 0x0F70 | 4, kWaitAll = 0x0F70;
    constexpr int kWaitLds = 0xC07F;  // lgkmcnt(0)
#define TG_FENCE() __builtin_amdgcn_sched_barrier(0)

    // ---------------------------------------------------------------- prologue
    // requests in order: scales(chunk 0) x5, A(0) x4, B(0) x4, B(1) x4, A(1) x4; all but the last eight must have landed
    set_scale_rows(cur_t);
    request_scales(0);
#pragma unroll
    for (int i = 0; i < IT; ++i) load_a(i, 0, 0);
#pragma unroll
    for (int i = 0; i < IT; ++i) load_b(i, 0, 0);
#pragma unroll
    for (int i = 0; i < IT; ++i) load_b(i, min(1, last), 1);
#pragma unroll
    for (int i = 0; i < IT; ++i) load_a(i, min(1, last), 1);
    __builtin_amdgcn_s_waitcnt(kWaitBut8);
    __builtin_amdgcn_s_barrier();
    TG_FENCE();
    v8i af[TM], wf[2];
    float sc_n[TM];  // scales of the coming step (row group tm, this lane's row)
    wf[0] = read_w(0, sB);
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) af[tm] = read_a(tm, sA);
    form_products();
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
        s_cur[tm] = 0.f;
        sc_n[tm] = __int_as_float(__builtin_amdgcn_ds_bpermute(bp_base, s_nxt[tm]));
    }

    // ---------------------------------------------------------------- main loop
    // On entry to step k: A(k) and B(k) are in LDS and visible to every wave; the reads of af (fragments of A(k)) and
    // wf[0] (column tile 0 of B(k)) and the bpermutes of sc_n (scales of step k) are issued; B(k+1) and A(k+1) are
    // requested.
    // Requests of a wave in order: ... B(k+1) x4 | [scales x5] A(k+1) x4 | B(k+2) x4 |: the wait of step k lets the last
    // four be in flight, so B(k+1), A(k+1) and any scale chunk requested before them have landed.  (The stores of a
    // tile's results sit in that sequence like loads.)
    int sa = 0, sb = 0;  // slabs that hold A(k) and B(k)
    for (;;) {           // tiles of this workgroup
        const Tile this_t = cur_t;
        const bool more = vt + stride < total;
        Tile next_t = cur_t;
        if (more) next_t = locate(vt + stride);
        bool switched = false;

        // One K step.  PH = k % 4 (position in the chunk of scales).  The step has no branch around VALU work: a branch
        // between the scale-and-add instructions lets the compiler collect them behind it, with every product alive until then.
        // NTM: row groups of this wave that hold valid rows of the tile (the others cost no MFMAs and no scale-and-add; every
        // wave issues the same loads and barriers whatever its NTM).
        auto step = [&](auto ntm_tag, auto ph_tag, const int k) __attribute__((always_inline)) {
            constexpr int NTM = decltype(ntm_tag)::value;
            constexpr int PH = decltype(ph_tag)::value;
            if (k == nsteps - 2 && more) {  // from here on the requests are for the next tile
                set_offsets(next_t);
                switched = true;
            }
            int k2 = k + 2;  // step the requests of this step are for
            if (k2 >= nsteps) k2 = more ? k2 - nsteps : last;
            const int sa1 = sa ^ 1;
            const int sb1 = sb == B_STAGES - 1 ? 0 : sb + 1;
            const int sb2 = sb1 == B_STAGES - 1 ? 0 : sb1 + 1;
            const uint8_t* cB = sB + sb * SLAB;
            const uint8_t* nA = sA + sa1 * SLAB;
            const uint8_t* nB = sB + sb1 * SLAB;
            float sc[TM];
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) sc[tm] = sc_n[tm];
            if constexpr (PH == 0) {
#pragma unroll
                for (int tm = 0; tm < TM; ++tm) s_cur[tm] = __int_as_float(s_nxt[tm]);
            }
            TG_FENCE();
            // 32 MFMAs, each into a fresh 16x16 product; the product issued two MFMAs earlier is scaled and added behind each
            v4f part[3];
            constexpr int NJ = TN * NTM;  // MFMAs of this wave and step, numbered column tile by column tile
            auto fma_of = [&](int j) __attribute__((always_inline)) {
                if constexpr (NTM > 0) {
                    if (j < 0) return;
                    const int tn = j / NTM, tm = j % NTM;
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[tn][tm][r] = __builtin_fmaf(part[j % 3][r], sc[tm], acc[tn][tm][r]);
                }
            };
            // column tiles 0 .. 5; behind each of the first four one weight load (B(k+2) goes to the slab B(k-1) had)
#pragma unroll
            for (int tn = 0; tn < 6; ++tn) {
#pragma unroll
                for (int tm = 0; tm < NTM; ++tm) {
                    const int j = tn * NTM + tm;
                    part[j % 3] = mfma_e4m3(wf[tn & 1], af[tm], v4f{0.f, 0.f, 0.f, 0.f});
                    if (tm == 0) wf[(tn + 1) & 1] = read_w(tn + 1, cB);
                    fma_of(j - 2);
                    TG_FENCE();
                }
                asm volatile("" : : "v"(wf[tn & 1]));
                if (tn < IT) {
                    load_b(tn, k2, sb2);
                    TG_FENCE();
                }
            }
            // B(k+1) and A(k+1) have landed (all but the four requests of B(k+2)); all my reads of A(k) are done
            __builtin_amdgcn_s_waitcnt(kWaitBut4);
            __builtin_amdgcn_s_waitcnt(kWaitLds);
            __builtin_amdgcn_s_barrier();
            TG_FENCE();
            // column tile 6, then the first weight fragment of step k+1
#pragma unroll
            for (int tm = 0; tm < NTM; ++tm) {
                const int j = 6 * NTM + tm;
                part[j % 3] = mfma_e4m3(wf[0], af[tm], v4f{0.f, 0.f, 0.f, 0.f});
                if (tm == 0) wf[1] = read_w(7, cB);
                fma_of(j - 2);
                TG_FENCE();
            }
            asm volatile("" : : "v"(wf[0]));
            wf[0] = read_w(0, nB);  // (whatever NTM: the next tile may need it)
            // Scales.  The chunk after this one (of this tile, or the first of the next tile, whose rows the offsets then
            // move to) is requested in a chunk's first step; the step after, whose wait has covered the request, forms its
            // products; the current chunk is replaced by it at the top of the next chunk's first step.  The scales of step
            // k+1 come from the lanes that hold them: the next position of this chunk, or -- after a chunk's last step, and
            // after a tile's last step -- the first position of the next.
            if constexpr (PH == 0) {
                const bool within = k + QUAD < nsteps;
                if (!within) set_scale_rows(next_t);
                request_scales(within ? k + QUAD : 0);
                TG_FENCE();
            }
            if constexpr (PH == 1) form_products();
            {
                // (a chunk's first step is never a tile's last: the host gives this kernel no K with a last chunk of one
                // step, and nothing that was requested in this step is read in it)
                const bool from_next = PH == QUAD - 1 || (TAIL && PH != 0 && k == last);
                const int src_lane_off = from_next ? 0 : (PH + 1) * 64;
#pragma unroll
                for (int tm = 0; tm < TM; ++tm) {
                    int v;
                    if constexpr (PH == QUAD - 1) v = s_nxt[tm];
                    else if constexpr (TAIL && PH != 0) v = from_next ? s_nxt[tm] : __float_as_int(s_cur[tm]);
                    else v = __float_as_int(s_cur[tm]);
                    sc_n[tm] = __int_as_float(__builtin_amdgcn_ds_bpermute(bp_base + src_lane_off, v));
                }
            }
            TG_FENCE();
            // column tile 7 by row group: each MFMA releases one activation fragment, which is refilled from A(k+1) at once;
            // A(k)'s slab is free (every wave read its fragments before the barrier) and receives A(k+2)
            // (all four fragments are refilled and all four scales fetched whatever NTM: the next step may be the first of a
            // tile in which this wave has more row groups)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
                if (tm < NTM) {
                    const int j = 7 * NTM + tm;
                    part[j % 3] = mfma_e4m3(wf[1], af[tm], v4f{0.f, 0.f, 0.f, 0.f});
                    fma_of(j - 2);
                    TG_FENCE();
                }
                af[tm] = read_a(tm, nA);
                load_a(tm, k2, sa);
                TG_FENCE();
            }
            asm volatile("" : : "v"(wf[1]));
            fma_of(NJ - 2);
            fma_of(NJ - 1);
            // keep the scale-and-add chain inside this step (see fp8_gemm_tile.h)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int tm = 0; tm < NTM; ++tm) asm volatile("" : "+v"(acc[tn][tm]));
            sa = sa1;
            sb = sb1;
        };
        auto k_loop = [&](auto ntm_tag) __attribute__((always_inline)) {
            for (int k0 = 0; k0 < nsteps; k0 += QUAD) {
                step(ntm_tag, std::integral_constant<int, 0>{}, k0);
                if constexpr (TAIL) {
                    // (k0 + 1 < nsteps always holds: the launcher gives this kernel no K whose last chunk is a single step.
                    // Written as a test all the same: run unconditionally, or as a loop over whole chunks with the last chunk
                    // apart, the step costs 126 - 216 spilled registers.  check_hazards.py therefore sees a path on which a
                    // chunk's scale requests meet no wait -- the one-step chunk -- and lists these two instantiations as known.)
                    if (k0 + 1 < nsteps) step(ntm_tag, std::integral_constant<int, 1>{}, k0 + 1);
                    if (k0 + 2 < nsteps) step(ntm_tag, std::integral_constant<int, 2>{}, k0 + 2);
                    if (k0 + 3 < nsteps) step(ntm_tag, std::integral_constant<int, 3>{}, k0 + 3);
                } else {
                    step(ntm_tag, std::integral_constant<int, 1>{}, k0 + 1);
                    step(ntm_tag, std::integral_constant<int, 2>{}, k0 + 2);
                    step(ntm_tag, std::integral_constant<int, 3>{}, k0 + 3);
                }
            }
        };
        // (Every wave computes all four of its row groups, also those without a valid row: a second copy of the loop
        // for tiles of at most 128 rows measured no faster, and one copy per number of row groups, as
        // fp8_gemm_tile_kernel has, spills; the step keeps NTM as a parameter.)
        k_loop(std::integral_constant<int, TM>{});

        // ---------------------------------------------------------------- epilogue, straight from the accumulators
        ParamPtr q = args();
        const float scale = q->alpha, beta = q->beta;
        const int N = q->N, ldc = q->ldc, out_type = q->out_type;
        void* const C = q->C;
        const bool vec_ok = q->vec_store != 0 && (N % 8) == 0;
        int dsts[TM];
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const int rt = tile_row(tm) + li;
            dsts[tm] = rt < this_t.rows ? this_t.m0 + rt : -1;
        }
        auto emit = [&](auto type_tag) __attribute__((always_inline)) {
            constexpr int OT = decltype(type_tag)::value;
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
                for (int tp = 0; tp < TN / 2; ++tp) {
                    const int col = this_t.n0 + wn * WTN + tp * 32 + lg * 8;
                    if (dsts[tm] < 0 || col >= N) continue;
                    store8(C, OT, dsts[tm], col, N, ldc, acc[2 * tp][tm] * scale, acc[2 * tp + 1][tm] * scale, beta, vec_ok);
                }
            }
        };
        if (out_type == OUT_BF16) emit(std::integral_constant<int, OUT_BF16>{});
        else if (out_type == OUT_F32) emit(std::integral_constant<int, OUT_F32>{});
        else if (out_type == OUT_F8) emit(std::integral_constant<int, OUT_F8>{});
        else emit(std::integral_constant<int, OUT_F16>{});
        if (!more) break;
        vt += stride;
        cur_t = next_t;
        if (!switched) set_offsets(cur_t);  // (cannot happen with nsteps >= 2; keeps the offsets right whatever the step count)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = v4f{0.f, 0.f, 0.f, 0.f};
    }
#undef TG_FENCE
    __builtin_amdgcn_s_waitcnt(kWaitAll);  // the re-fetches past the end must land before the workgroup's LDS is released
#endif
}

// `grid` = min(upper bound of the tile count, compute units)


template <int GROUP>
inline hipError_t launch_bs256(const GemmParams& p, int tiles_bound, int max_workgroups, hipStream_t stream) {
    if (!bs256_takes_k(p.kblocks) || !p.As || !p.Bs) return hipErrorInvalidValue;
    const int grid = tiles_bound < max_workgroups ? tiles_bound : max_workgroups;
    if (p.kblocks % 4 == 0) hipLaunchKernelGGL((fp8_gemm_bs256_kernel<GROUP, false>), dim3(grid, 1, 1), dim3(512, 1, 1), 0, stream, p);
    else hipLaunchKernelGGL((fp8_gemm_bs256_kernel<GROUP, true>), dim3(grid, 1, 1), dim3(512, 1, 1), 0, stream, p);
    return hipGetLastError();
}

}  // namespace tg

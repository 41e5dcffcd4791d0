// Skinny-M GEMM for gfx950: M <= 128 rows against a long, narrow strip of B, the K split done inside the
// workgroup.  The "split-K variant for skinny M" of the reference's plan (README.md:28; the unused split_k of
// src/gemm/sm89_gemm_kernel_v5.cu:319), built for a part where such a shape is bound by how many bytes are in
// flight, not by arithmetic: B is read exactly once, straight from HBM.
//
// A workgroup owns 16*TM rows x 32 columns of C over the whole of K (or over its K slice when the host splits K
// on top).  Its eight waves take the 128-byte K steps round robin, two steps per wave and round: in round r wave w
// computes steps 16 r + w and 16 r + 8 + w of the whole tile.  Nothing is shared on the way, so the K loop has no
// barrier and no wait on another wave.
//   * Both operands travel global -> LDS with buffer_load ... lds, eight lanes per 128-byte row, rows rotated as
//     in gemm_nt_kernel (lds_slot), into a ring of twenty 1 KiB slots that belongs to the wave alone, and from
//     there into registers with conflict-free ds_read_b128 in the MFMA's lane layout.  (Loading the fragments
//     from global memory straight into that layout was built first and is far slower: neighbouring lanes are
//     neighbouring rows there, the texture addresser merges nothing, and every 16 bytes become a request of
//     their own: 64 cycles per instruction and CU.)
//   * The wave waits for its own copies with s_waitcnt vmcnt(n): copies land in issue order, and the program of a
//     round is fixed, so every n is a compile-time constant.  All of B of the round (the stream from HBM) is
//     requested when the round starts; A (shared by every workgroup, an L2 hit) fills what is left of the ring,
//     is drained into registers as it lands and makes room for the rest of A: two steps of a 128-row tile are
//     40 KiB, twice the ring.  Steps past the end of K are copied like all others (the buffer range check turns
//     them into zeros).
// The eight partial sums meet once, in LDS, and are added in wave order (a fixed order: the same bits every
// run; exact for int32), then scaled, converted and stored like the epilogue of gemm_nt_kernel.
#pragma once
#include "gemm_mfma.cuh"

namespace qgemm {

template <int ARITH_, int TM_, bool BLOCK_SCALE_ = false, int TN_ = 2>
struct SkinnyCfg {
    static constexpr int ARITH = ARITH_;
    // 128-block scales (fp8): every MFMA starts from zero and its product of one K block is folded into the running
    // sum with a_scale[row, kb] * b_scale[strip, kb], as in gemm_nt_kernel.  The strip of 32 (or 64) columns lies inside
    // one 128-column block of b_scale.  a_scale is read with the caller's strides (lane l: row l of the tile, the rows of
    // an MFMA tile picked out of that with ds_bpermute); the scales of a round are requested in front of the round's
    // copies, so they have arrived wherever the copies they precede have.
    static constexpr bool BLOCK_SCALE = BLOCK_SCALE_;
    static_assert(!BLOCK_SCALE_ || ARITH_ == AR_F8 || ARITH_ == AR_I8, "block scales: fp8 and int8 operands");
    // TN = 4 (with TM = 4: a 64 x 64 tile): half the strips, so A is fetched half as often; for shapes with several
    // row tiles, where a CU's load path, not the stream of B from HBM, is what bounds a 32-column strip.
    static constexpr int TM = TM_, TN = TN_;                // 16 x 16 MFMA tiles of the workgroup's tile
    static constexpr int BM = 16 * TM_, BN = 16 * TN_;
    static constexpr int NW = 8, THREADS = NW * kWave;
    static constexpr int SLOTS = 20;                        // ring slots (1 KiB = one copy instruction) per wave
    static constexpr int SA = 2 * TM, SB = 2 * TN;          // slots of one step of A / of B
    static constexpr int RING_BYTES = SLOTS * 1024;
    static constexpr int LDS_BYTES = NW * RING_BYTES;       // the rings; afterwards one partial sum (1 KiB per tile) per wave
    static_assert(TM == 1 || TM == 2 || TM == 4 || TM == 8, "the programs below are written for these tile heights");
    static_assert(TN == 2 || (TN == 4 && TM == 4) || (TN == 1 && TM <= 2), "64-column strips: the 64 x 64 tile; 16-column strips: up to 32 rows");
    // TN = 1 (16-column strips, up to 32 rows; with 64 rows they were level with 32-column strips and a K split or behind): twice the strips of the 32-column rows, for few columns against a long K,
    // where 32-column strips leave half of the CUs idle and a K split across workgroups costs a second launch.
    static constexpr bool ALL_AT_ONCE = 2 * (SA + SB) <= SLOTS;      // both steps of a round fit the ring together
    static_assert(TM * TN * 1024 <= RING_BYTES, "a wave's partial sums fit its ring");
};

// all copies of this wave but the last IN_FLIGHT have landed
template <int IN_FLIGHT>
__device__ inline void wait_landed() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(IN_FLIGHT));
    __builtin_amdgcn_sched_barrier(0);
}

template <class C>
__global__ void __launch_bounds__(C::THREADS) gemm_skinny_kernel(const GemmArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    typedef typename AccT<C::ARITH>::type part_t;                       // one MFMA step: int32 for int8 operands, else fp32
    typedef std::conditional_t<C::BLOCK_SCALE, v4f, part_t> acc_t;      // the running sums: fp32 with block scales
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    QGEMM_STAMP_DECL(6);
    QGEMM_STAMP(0);

    uint32_t wg = blockIdx.x, z = 0;
    if (p.nsplit > 1) {
        z = __builtin_amdgcn_readfirstlane(wg % p.nsplit);
        wg = __builtin_amdgcn_readfirstlane(wg / p.nsplit);
    }
    // column strips side by side (the few row tiles of one strip are neighbours: they share the strip of B in L2)
    // (the 64 x 64 form has many row tiles: there the tiles an XCD holds at one time form a compact block, as in
    // gemm_nt_kernel, so that its L2 fetches each panel of A and B once)
    uint32_t tm, tn;
    if constexpr (C::TN == 4) {
        tile_map(wg, p.tiles_m, p.tiles_n, p.group_m, tm, tn);
        tm = __builtin_amdgcn_readfirstlane(tm);
        tn = __builtin_amdgcn_readfirstlane(tn);
    } else {
        tm = __builtin_amdgcn_readfirstlane(wg % p.tiles_m);
        tn = __builtin_amdgcn_readfirstlane(wg / p.tiles_m);
    }
    const uint32_t row0 = tm * C::BM, col0 = tn * C::BN;
    const uint32_t kbeg = z * p.ksteps_per_split;
    const uint32_t kend = kbeg + p.ksteps_per_split < p.ksteps ? kbeg + p.ksteps_per_split : p.ksteps;
    const int nk = (int)(kend - kbeg);

    // Buffer resources end with the last valid row of the tile and the last byte of the K slice: rows past M / N and
    // steps past the end of K read as zeros.
    const uint32_t a_rows = p.M - row0 < (uint32_t)C::BM ? p.M - row0 : C::BM;
    const uint32_t b_rows = p.N - col0 < (uint32_t)C::BN ? p.N - col0 : C::BN;
    // (a partial last K step: the ranges end with the last byte of K, and in that step the lanes whose 16-byte chunk
    // lies past the end of a row present an offset that is out of range, as in gemm_nt_kernel)
    const bool has_tail = p.k_tail != 0 && kend == p.ksteps && nk > 0;
    const uint32_t kbytes = has_tail ? (uint32_t)(nk - 1) * 128 + p.k_tail : (uint32_t)nk * 128;
    const int kt_tail = has_tail ? nk - 1 : -1;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.A + (size_t)row0 * p.lda + (size_t)kbeg * 128, (a_rows - 1) * p.lda + kbytes);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.B + (size_t)col0 * p.ldb + (size_t)kbeg * 128, (b_rows - 1) * p.ldb + kbytes);
    // a copy moves 8 rows x 128 bytes; lane l fetches the chunk of row l >> 3 that belongs in 16-byte slot l of
    // the kilobyte (rotation by the row: see lds_slot)
    const uint32_t rot = (((lane & 7) - (lane >> 3)) & 7) * 16;
    const uint32_t voff_a = (lane >> 3) * p.lda + rot, voff_b = (lane >> 3) * p.ldb + rot;
    const uint32_t tail_or = (has_tail && rot >= p.k_tail) ? 0x80000000u : 0u;
    char *ring = smem + wave * C::RING_BYTES;
    const int fr = lane & 15, fg = lane >> 4;
    const int off0 = lds_slot(fr, fg) * 16, off1 = lds_slot(fr, 4 + fg) * 16;

    // K step the loop's step kt stands for: the workgroups of a column strip start k_first steps in and wrap round
    // (GemmArgs::k_rot);
    // steps past the end stay past the end (they read zeros)
    const int k_first = p.k_rot && nk > 0 ? (int)((tn * p.k_rot) % (uint32_t)nk) : 0;
    auto kpos = [&](int kt) -> int {
        const int k = kt + k_first;
        return kt >= nk ? kt : (k >= nk ? k - nk : k);
    };
    // copies: n kilobytes of step kt (rows 8 * first ..) of A or B into ring slots slot, slot + 1, ...
    auto copy_a = [&](int kt_loop, int first, int n, int slot) {
        const int kt = kpos(kt_loop);
        const uint32_t va = kt == kt_tail ? (voff_a | tail_or) : voff_a;
#pragma unroll
        for (int i = 0; i < n; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void *)(ring + (slot + i) * 1024), 16, va,
                                                     (first + i) * 8 * p.lda + (uint32_t)kt * 128, 0, 0);
    };
    auto copy_b_part = [&](int kt_loop, int first, int n, int slot) {
        const int kt = kpos(kt_loop);
        const uint32_t vb = kt == kt_tail ? (voff_b | tail_or) : voff_b;
        // B streamed out of memory and read once: the copies carry the streaming hint (nt).  Config 5 with B in rotation
        // through 352 MB: M = 16 5.65 -> 5.40 us, M = 64 6.96 -> 6.82, M = 128 8.35 -> 8.22; level with B resident.
        if (p.b_stream) {
#pragma unroll
            for (int i = 0; i < n; ++i)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_void *)(ring + (slot + i) * 1024), 16, vb,
                                                         (first + i) * 8 * p.ldb + (uint32_t)kt * 128, 0, 2);
        } else {
#pragma unroll
            for (int i = 0; i < n; ++i)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_void *)(ring + (slot + i) * 1024), 16, vb,
                                                         (first + i) * 8 * p.ldb + (uint32_t)kt * 128, 0, 0);
        }
    };
    auto copy_b = [&](int kt, int slot) { copy_b_part(kt, 0, C::SB, slot); };
    // fragments of the two steps of a round: [step][block][half]
    v4i fa[2][C::TM][2], fb[2][C::TN][2];
    auto drain_a = [&](int s, int blk0, int nblk, int slot) {       // blocks blk0 .. of step s sit in ring slots slot ..
#pragma unroll
        for (int i = 0; i < nblk; ++i) {
            fa[s][blk0 + i][0] = *(const v4i *)(ring + slot * 1024 + i * 2048 + off0);
            fa[s][blk0 + i][1] = *(const v4i *)(ring + slot * 1024 + i * 2048 + off1);
        }
    };
    auto drain_b_part = [&](int s, int blk0, int nblk, int slot) {
#pragma unroll
        for (int i = 0; i < nblk; ++i) {
            fb[s][blk0 + i][0] = *(const v4i *)(ring + slot * 1024 + i * 2048 + off0);
            fb[s][blk0 + i][1] = *(const v4i *)(ring + slot * 1024 + i * 2048 + off1);
        }
    };
    auto drain_b = [&](int s, int slot) { drain_b_part(s, 0, C::TN, slot); };
    auto drained = [&]() {                                  // the fragment reads are done: their slots may be refilled
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(waitcnt_lgkm0());
        __builtin_amdgcn_sched_barrier(0);
    };

    acc_t acc[C::TM][C::TN];
#pragma unroll
    for (int a = 0; a < C::TM; ++a)
#pragma unroll
        for (int b = 0; b < C::TN; ++b) acc[a][b] = acc_t{0, 0, 0, 0};

    // block scales of the two steps of the round in hand (cur) and of the round whose copies are on their way (nxt)
    constexpr int NLD = C::BLOCK_SCALE ? (C::BM + 63) / 64 : 1;
    int as_cur[2][NLD], as_nxt[2][NLD];
    float bs_cur[2], bs_nxt[2];
    __amdgpu_buffer_rsrc_t ras = make_rsrc(p.as, 0);
    uint32_t as_voff = 0, bs_base = 0;
    if constexpr (C::BLOCK_SCALE) {
        ras = make_rsrc(p.as, ((p.ksteps - 1) * p.as_ks + (p.M - 1) * p.as_ms + 1) * 4);
        as_voff = (row0 + lane) * p.as_ms * 4;
        uint32_t nb = col0 / 128;
        nb = nb < p.nb_max ? nb : p.nb_max;
        bs_base = nb * p.bs_ns;
    }
    auto fetch_scales = [&](int k) {            // for steps k and k + 8 of this wave (called in front of their copies)
        if constexpr (C::BLOCK_SCALE) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const uint32_t kb = kbeg + (uint32_t)kpos(k + s * C::NW);
                // (a step past the end of K multiplies zeros: any finite scale will do, so keep the reads inside)
                const uint32_t kbc = kb < p.ksteps ? kb : p.ksteps - 1;
#pragma unroll
                for (int j = 0; j < NLD; ++j)
                    as_nxt[s][j] = __builtin_amdgcn_raw_buffer_load_b32(ras, as_voff, (64 * j * p.as_ms + kbc * p.as_ks) * 4, 0);
                bs_nxt[s] = p.bs[bs_base + kbc * p.bs_ks];
            }
        }
    };
    auto take_scales = [&]() {
        if constexpr (C::BLOCK_SCALE) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
#pragma unroll
                for (int j = 0; j < NLD; ++j) as_cur[s][j] = as_nxt[s][j];
                bs_cur[s] = bs_nxt[s];
            }
        }
    };
    auto compute = [&](int s) {
        if constexpr (C::BLOCK_SCALE) {
            float f[C::TM];
#pragma unroll
            for (int a = 0; a < C::TM; ++a)
                f[a] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((((16 * a) & 63) + (lane & 15)) * 4,
                                                                                as_cur[s][(16 * a) / 64])) * bs_cur[s];
            // one MFMA behind: the four FMAs of a tile go behind the MFMA of the next tile and run under it (straight
            // after their own MFMA they would wait for it, and the next MFMA for them)
            part_t part[2];
#pragma unroll
            for (int i = 0; i <= C::TM * C::TN; ++i) {
                if (i < C::TM * C::TN) {
                    const int a = i % C::TM, b = i / C::TM;
                    part[i & 1] = mma128<C::ARITH>(fb[s][b][0], fb[s][b][1], fa[s][a][0], fa[s][a][1], part_t{0, 0, 0, 0});
                }
                if (i > 0) {
                    const int pa = (i - 1) % C::TM, pb = (i - 1) / C::TM;
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[pa][pb][r] += (float)part[(i - 1) & 1][r] * f[pa];
                }
            }
        } else {
#pragma unroll
            for (int b = 0; b < C::TN; ++b)
#pragma unroll
                for (int a = 0; a < C::TM; ++a)
                    acc[a][b] = mma128<C::ARITH>(fb[s][b][0], fb[s][b][1], fa[s][a][0], fa[s][a][1], acc[a][b]);
        }
    };

    // ---- one round = steps k and k + 8 of this wave.  Ring programs by tile height (slots per step: A 2 TM, B 4):
    //   TM <= 2, or 16-column strips (at most 20 slots): everything at once.   B0 B1 A0 A1
    //   TM == 4  (24 slots):  A0 B0 B1 A1[0..4)  | A0 drained ->  A1[4..8)
    //   TM == 8  (40 slots):  A0[0..12) B0 B1    | A0[0..12) drained -> A0[12..16) A1[0..8) | B0 B1 A0[12..16) drained
    //                         -> A1[8..16)
    //   TM == 4, TN == 4 (32 slots, B 8 per step):  A0 B0 B1[0..4) | A0 drained -> B1[4..8) A1[0..4) | B0 drained
    //                         -> A1[4..8)
    // A goes in front of B where the ring cannot take the round at once: the wait for it then does not include
    // the trip to HBM, and its slots turn over while B is still on its way.
    constexpr int SA = C::SA, SB = C::SB;
    auto start_round = [&](int k) {
        fetch_scales(k);
        __builtin_amdgcn_sched_barrier(0);          // (the scale loads stay in front of the copies)
        if constexpr (C::TN == 4) {                   // 64 x 64: A0 B0 B1[0..4) fill the ring
            copy_a(k, 0, 8, 0);
            copy_b(k, 8);
            copy_b_part(k + C::NW, 0, 4, 16);
        } else if constexpr (C::ALL_AT_ONCE) {
            copy_b(k, 0);
            copy_b(k + C::NW, SB);
            copy_a(k, 0, SA, 2 * SB);
            copy_a(k + C::NW, 0, SA, 2 * SB + SA);
        } else if constexpr (C::TM == 4) {
            copy_a(k, 0, 8, 0);
            copy_b(k, 8);
            copy_b(k + C::NW, 12);
            copy_a(k + C::NW, 0, 4, 16);
        } else {
            copy_a(k, 0, 12, 0);
            copy_b(k, 12);
            copy_b(k + C::NW, 16);
        }
    };
    // everything of the round into registers, the MFMAs of its first step, and (next: the round after this one
    // exists) the first copies of the next round as soon as the ring is empty; the MFMAs of the second step last
    auto finish_round = [&](int k, bool next, bool two) {
        take_scales();
        if constexpr (C::TN == 4) {
            // ring: A0 0-7, B0 8-15, B1a 16-19 | A0 drained -> B1b 0-3, A1a 4-7 | B0 drained -> A1b 8-11
            wait_landed<12>();
            drain_a(0, 0, 4, 0);
            drained();
            copy_b_part(k + C::NW, 4, 4, 0);
            copy_a(k + C::NW, 0, 4, 4);
            wait_landed<12>();
            drain_b(0, 8);
            drained();
            copy_a(k + C::NW, 4, 4, 8);
            compute(0);
            wait_landed<12>();
            drain_b_part(1, 0, 2, 16);
            wait_landed<8>();
            drain_b_part(1, 2, 2, 0);
            wait_landed<4>();
            drain_a(1, 0, 2, 4);
            wait_landed<0>();
            drain_a(1, 2, 2, 8);
        } else if constexpr (C::ALL_AT_ONCE) {
            wait_landed<SA>();
            drain_b(0, 0);
            drain_b(1, SB);
            drain_a(0, 0, C::TM, 2 * SB);
            compute(0);
            wait_landed<0>();
            drain_a(1, 0, C::TM, 2 * SB + SA);
        } else if constexpr (C::TM == 4) {
            wait_landed<12>();
            drain_a(0, 0, 4, 0);
            drained();
            copy_a(k + C::NW, 4, 4, 0);
            wait_landed<4>();
            drain_b(0, 8);
            drain_b(1, 12);
            drain_a(1, 0, 2, 16);
            compute(0);
            wait_landed<0>();
            drain_a(1, 2, 2, 0);
        } else {
            wait_landed<8>();
            drain_a(0, 0, 6, 0);
            drained();
            copy_a(k, 12, 4, 0);
            copy_a(k + C::NW, 0, 8, 4);
            wait_landed<8>();
            drain_b(0, 12);
            drain_b(1, 16);
            drain_a(0, 6, 2, 0);
            drained();
            copy_a(k + C::NW, 8, 8, 12);
            compute(0);
            wait_landed<8>();
            drain_a(1, 0, 4, 4);
            wait_landed<0>();
            drain_a(1, 4, 4, 12);
        }
        drained();
        if (next) start_round(k + 2 * C::NW);
        if (two) compute(1);
    };
    int k = wave;
    start_round(k);
    QGEMM_STAMP(1);
    for (; k < nk; k += 2 * C::NW) finish_round(k, k + 2 * C::NW < nk, k + C::NW < nk);
    // (a wave without a step has copies of zeros on their way into its ring, which now takes the partial sums)
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0) & 0xF0FF);
    __builtin_amdgcn_sched_barrier(0);
    QGEMM_STAMP(3);

    // ---- the eight partial sums meet in LDS: partial of wave w, tile t at smem + w * RING_BYTES + t * 1 KiB, lane-linear
    constexpr int T = C::TM * C::TN;
    char *mine = ring + lane * 16;
#pragma unroll
    for (int a = 0; a < C::TM; ++a)
#pragma unroll
        for (int b = 0; b < C::TN; ++b) *(acc_t *)(mine + (a * C::TN + b) * 1024) = acc[a][b];
    __syncthreads();
    QGEMM_STAMP(4);

    float scale = 1.0f;
    if (p.per_matrix_scale) scale = p.as[0] * p.bs[0];
    char *Cz = p.C + (size_t)z * p.split_stride * dtype_bytes(p.out_dtype);
    // wave w finishes tiles w, w + 8, ...
#pragma unroll
    for (int i = 0; i < (T + C::NW - 1) / C::NW; ++i) {
        const int t = wave + i * C::NW;
        if (t >= T) break;
        acc_t s = *(const acc_t *)(smem + (size_t)t * 1024 + lane * 16);
#pragma unroll
        for (int w = 1; w < C::NW; ++w) {
            const acc_t o = *(const acc_t *)(smem + (size_t)w * C::RING_BYTES + (size_t)t * 1024 + lane * 16);
#pragma unroll
            for (int r = 0; r < 4; ++r) s[r] += o[r];
        }
        const int a = t / C::TN, b = t % C::TN;
        const uint32_t m = row0 + a * 16 + (lane & 15);
        const uint32_t n = col0 + b * 16 + (lane >> 4) * 4;
        if (m >= p.M || n >= p.N) continue;
        const size_t idx = (size_t)m * p.ldc + n;
        const bool full = p.vec_store && n + 3 < p.N;
        if constexpr (C::ARITH == AR_I8 && !C::BLOCK_SCALE) {
            if (p.out_dtype == QGEMM_DT_I32) {
                int *dst = (int *)Cz + idx;
                if (full) *(v4i *)dst = s;
                else
                    for (int r = 0; r < 4; ++r)
                        if (n + r < p.N) dst[r] = s[r];
                continue;
            }
        }
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = (float)s[r] * scale;
        if (p.out_dtype == QGEMM_DT_F32) {
            float *dst = (float *)Cz + idx;
            if (full) *(v4f *)dst = v4f{v[0], v[1], v[2], v[3]};
            else
                for (int r = 0; r < 4; ++r)
                    if (n + r < p.N) dst[r] = v[r];
        } else {
            const v2i h = p.out_dtype == QGEMM_DT_BF16 ? pack4_bf16(v[0], v[1], v[2], v[3]) : pack4_f16(v[0], v[1], v[2], v[3]);
            unsigned short *dst = (unsigned short *)Cz + idx;
            if (full) *(v2i *)dst = h;
            else
                for (int r = 0; r < 4; ++r)
                    if (n + r < p.N) dst[r] = pack4_elem(h, r);
        }
    }
    QGEMM_STAMP(5);
    QGEMM_STAMP_WRITE(p.dbg_cycles, blockIdx.x * C::NW + wave, 6, lane == 0);
#endif
}

}  // namespace qgemm

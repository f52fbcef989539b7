// The software-pipelined bf16 prefill kernel with 64 queries per wavefront (included by prefill.hip, inside
// namespace vsp { namespace { ).  Same tiles, fragment layouts, ring and arithmetic as prefill_bf16_pipe_kernel; what
// changes is how much work hangs on every byte that crosses LDS:
//   - a wavefront owns two blocks of 32 queries, so every K and V^T operand it reads from LDS feeds two MFMAs (one per
//     block) instead of one, and every softmax instruction stream is doubled next to them: half the LDS operand reads
//     per FLOP;
//   - a workgroup (4 wavefronts, one per SIMD, up to 512 registers each) owns 256 queries, so every K/V tile crosses
//     from L2 to LDS once per 256 queries instead of once per 128, with one barrier per 32 MFMAs of a wavefront
//     instead of one per 16.
// The price is one workgroup per CU: nothing else on a SIMD covers this wavefront's prologue, drain and output
// stores, which is why the launch code keeps this kernel for contexts long enough that those are a small share.
// Under the causal mask the 256 x 256 block on the diagonal is walked in lockstep (one barrier per step), so the eight
// 32-query blocks of a workgroup are paired (w, 7 - w): every wavefront then has the same number of tile products in
// that block (9), and the number of steps in which some wavefront still has both of its blocks active is the minimum
// (4 of the 8).
//
// Registers.  One wavefront per SIMD may use 512 registers, of which only the 256 architectural ones are visible to
// the vector ALU; left to itself the compiler gives every MFMA result an accumulation register and copies the score
// tiles back and forth (about 400 copies per step).  So the MFMAs are issued from inline asm with the register file of
// every operand spelled out: O^T accumulators and Q^T (loop constants, read by nothing but MFMAs) in accumulation
// registers, score tiles, P and the LDS operands in architectural ones.  The compiler does not see inside the asm, so
// the wait states it would otherwise insert around MFMAs are kept by hand:
//   - an MFMA result must not be read or overwritten by another kind of instruction for ~20 issue slots: the pipeline
//     puts a whole step between the score MFMAs and the softmax that reads them; the mask, the rare rescale and the
//     epilogue wait explicitly (mfma_settle());
//   - an MFMA must not read a register that a vector-ALU instruction wrote in the two issue slots before it: its
//     operands come from LDS (behind a wait), from accumulation registers, or from P computed a step earlier, and no
//     operand is left for the compiler to copy into place in front of the asm (Q^T parked in accumulation registers
//     and copied back before each use is exactly what broke an earlier form of this kernel).
// tests/test_wide_kernel_isa.py checks both rules on the compiled code.  The reference maximum enters the exponent through the
// fused multiply-add in front of the exp2, P = exp2(c * s - m): no tile of -m / c as an MFMA C operand (which would
// have to sit in architectural registers next to the scores).
#pragma once

constexpr int kBMW = 256;   // queries per workgroup of the wide kernel
#ifdef ABL_LEAD6
constexpr int kLeadW = 6;
#else
constexpr int kLeadW = 4;
#endif
//   // LDS operand reads run this many operand slots (two MFMAs each) ahead


template <bool VBLK, int LEAD>
constexpr int reads_behind_n(int s) {
    int n = 0;
    for (int k = 1; k < LEAD; ++k) n += slot_reads<VBLK>(s + k);
    return n;
}

// The MFMAs, each one asm statement together with the wait for its LDS operand (WAIT >= 0: at most that many of this
// wavefront's LDS reads may still be outstanding; they return in order) and, for the step variants outside the steady
// state (PAD), two idle issue slots in front, where the compiler may have had to move a block's accumulators or P
// between registers on the way in.
#define VSP_MFMA_ASM(OPERANDS, OUT, ...)                                                                                        \
    do {                                                                                                                        \
        if constexpr (WAIT >= 0 && PAD) asm volatile("s_waitcnt lgkmcnt(%[w])\n\ts_nop 1\n\tv_mfma_f32_32x32x16_bf16 " OPERANDS : OUT : __VA_ARGS__, [w] "n"(WAIT < 0 ? 0 : WAIT)); \
        else if constexpr (WAIT >= 0) asm volatile("s_waitcnt lgkmcnt(%[w])\n\tv_mfma_f32_32x32x16_bf16 " OPERANDS : OUT : __VA_ARGS__, [w] "n"(WAIT < 0 ? 0 : WAIT)); \
        else if constexpr (PAD) asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 " OPERANDS : OUT : __VA_ARGS__);               \
        else asm volatile("v_mfma_f32_32x32x16_bf16 " OPERANDS : OUT : __VA_ARGS__);                                             \
    } while (0)
// S^T tile (architectural registers) = K rows (architectural, from LDS) * Q^T (accumulation registers), and += the same
template <bool PAD, int WAIT>
__device__ inline void mfma_set_v(f32x16_t& d, const bf16x8_t& a, const bf16x8_t& b) {
    VSP_MFMA_ASM("%[d], %[a], %[b], 0", [d] "=&v"(d), [a] "v"(a), [b] "a"(b));
}
template <bool PAD, int WAIT>
__device__ inline void mfma_acc_v(f32x16_t& d, const bf16x8_t& a, const bf16x8_t& b) {
    VSP_MFMA_ASM("%[d], %[a], %[b], %[d]", [d] "+v"(d), [a] "v"(a), [b] "a"(b));
}
// 16 bytes from global memory into accumulation registers; the caller waits (vmcnt) before the first use
template <int OFFSET_BYTES>
__device__ inline void load_to_agpr(bf16x8_t& d, const void* p) {
    asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "=a"(d) : "v"(p), "n"(OFFSET_BYTES));
}
// O^T tile (accumulation registers) += V^T (architectural, from LDS) * P^T (architectural)
template <bool PAD, int WAIT>
__device__ inline void mfma_acc_a(f32x16_t& d, const bf16x8_t& a, const bf16x8_t& b) {
    VSP_MFMA_ASM("%[d], %[a], %[b], %[d]", [d] "+a"(d), [a] "v"(a), [b] "v"(b));
}
// The steady-state softmax instructions, one per asm statement: asm volatile statements keep their order, so these sit
// exactly where they are written between the MFMAs (left to the compiler they gather behind the second MFMA of a
// slot, and the first MFMA's shadow stays empty while the wavefront waits to issue the second).
__device__ inline void v_fma_exp(float& d, float a, float b, float c) {  // d = exp2(a * b + c)
#ifdef ABL_EXPMUL
    asm volatile("v_fma_f32 %0, %1, %2, %3\n\tv_mul_f32 %0, %0, %0" : "=v"(d) : "v"(a), "v"(b), "v"(c));
#else
    asm volatile("v_fma_f32 %0, %1, %2, %3\n\tv_exp_f32 %0, %0" : "=v"(d) : "v"(a), "v"(b), "v"(c));
#endif
}
__device__ inline void v_fma1(float& d, float a, float b, float c) { asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c)); }
__device__ inline void v_exp1(float& d) { asm volatile("v_exp_f32 %0, %0" : "+v"(d)); }
__device__ inline void v_add(float& d, float a, float b) { asm volatile("v_add_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b)); }
__device__ inline void v_acc(float& d, float a) { asm volatile("v_add_f32 %0, %0, %1" : "+v"(d) : "v"(a)); }
__device__ inline void v_cvt_pk(uint32_t& d, float a, float b) { asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b)); }
__device__ inline void pin(float& x) { asm volatile("" : "+v"(x)); }
__device__ inline void pin(uint32_t& x) { asm volatile("" : "+v"(x)); }
// More wait states than any MFMA of this kernel needs between its issue and a vector-ALU read of its result.
__device__ inline void mfma_settle() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }

template <bool VBLK>
__global__ void __launch_bounds__(256, 1) prefill_bf16_wide_kernel(PrefillArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses device-only builtins
    constexpr int D = 128;
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int CPR = D / 8;
    constexpr int RP = 256 / (2 * D);
    constexpr int NR = 1024 / (2 * D);
    constexpr int NGRP = kUnit / NR;
    constexpr int NLD = NGRP / 4;
    constexpr int SLOT = kUnit * D;
    constexpr int SLOTB = 2 * SLOT;
    constexpr int NRING = 4;
    constexpr int NC = 2;  // 32-query blocks per wavefront
    static_assert(KS == 8 && DB == 4 && NLD == 2, "written for D = 128");

    // K ring (4 slots) | V ring (4 slots)
    __shared__ __attribute__((aligned(1024))) uint16_t smem[2 * NRING * SLOT];
    const uint32_t lds0 = lds_addr(smem);

    const int nbh = a.B * a.Hq;
    int bid = blockIdx.x;
    int tile0 = 0;  // first key tile of this workgroup's share of the context (a split context: cache-plane mode only)
    int split = 0;
    if constexpr (VBLK) {
        if (a.n_splits > 1) {
            const int inner = a.n_qtiles * nbh;
            split = bid / inner;
            bid -= split * inner;
            tile0 = split * a.split_tiles;
        }
    }
    const int qt = a.n_qtiles - 1 - bid / nbh;
    const int bh = xcd_grouped_head(bid % nbh, a.B * a.Hkv, a.n_rep);
    const int b = bh / a.Hq, hq = bh % a.Hq, kvh = hq / a.n_rep;
    int L = a.L;
    int n_chunk = a.T;
    if constexpr (VBLK) {
        if (a.chunk_lens) n_chunk = min(max(a.chunk_lens[b], 0), a.T);
        if (a.seq_lens) L = min(max(a.seq_lens[b], n_chunk), a.L);
    }
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 31, h = lane >> 5;
    const int off = L - n_chunk;
    // the two 32-query blocks of this wavefront: block w and block 7 - w of the workgroup's eight
    int q0c[NC];
    q0c[0] = qt * kBMW + 32 * wave;
    q0c[1] = qt * kBMW + 32 * (7 - wave);

    const uint16_t* Qp = (const uint16_t*)a.q + (int64_t)b * a.sq[0] + (int64_t)hq * a.sq[1];
    const uint16_t* Kp = (const uint16_t*)a.k + (int64_t)b * a.sk[0] + (int64_t)kvh * a.sk[1];
    const uint16_t* Vp = (const uint16_t*)a.v + (int64_t)b * a.sv[0] + (int64_t)kvh * a.sv[1];

    // Q^T goes from global memory straight into accumulation registers (the loads are asm, so the wait for them is
    // by hand too: they are older than the first tile requests, whose wait below therefore covers them).  Q is used
    // exactly as stored; a negative scale is carried by the sign of c = scale * log2(e) in front of the exp2.
    bf16x8_t qf[NC][KS];
    const uint16_t* qp[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) qp[c] = Qp + (int64_t)min(q0c[c] + ql, a.T - 1) * a.sq[2] + 8 * h;
    static_for<NC * KS>([&](auto i_c) {
        constexpr int c = decltype(i_c)::value / KS, ks = decltype(i_c)::value % KS;
        load_to_agpr<32 * ks>(qf[c][ks], qp[c]);
    });
    const float cexp = a.negate_q ? -a.scale_log2 : a.scale_log2;
    const float masked = cexp < 0.f ? INFINITY : -INFINITY;  // the score of a masked key: c * masked = -inf

    const int wg_qmax = min(qt * kBMW + kBMW - 1, a.T - 1);
    const int kv_end_wg = a.causal ? min(L, wg_qmax + off + 1) : L;
    int n_tiles = (kv_end_wg + kUnit - 1) / kUnit;  // tiles the workgroup loads
    int nt_c[NC], fm_c[NC];  // per block: tiles it uses; its first tile that needs the mask
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int q0 = q0c[c];
        const int qmax = min(q0 + 31, a.T - 1);
        const int kv_end = (q0 < a.T) ? (a.causal ? min(L, qmax + off + 1) : L) : 0;
        nt_c[c] = (kv_end + kUnit - 1) / kUnit;
        fm_c[c] = min(nt_c[c], L / kUnit);
        if (a.causal) fm_c[c] = min(fm_c[c], q0 + off - 31 < 0 ? 0 : (q0 + off - 31) / kUnit + 1);
    }
    if constexpr (VBLK) {
        if (a.n_splits > 1) {  // this workgroup's share: tiles [tile0, tile0 + split_tiles), counted from tile0 below
            n_tiles = max(0, min(n_tiles, tile0 + a.split_tiles) - tile0);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                nt_c[c] = min(max(0, nt_c[c] - tile0), n_tiles);
                fm_c[c] = min(max(0, fm_c[c] - tile0), nt_c[c]);
            }
        }
    }
    const int n_fast = max(0, min(fm_c[0], fm_c[1]) - 2);  // steps [0, n_fast): every stage of both blocks active, no mask

    f32x16_t acc[NC][DB];
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int i = 0; i < DB; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[c][i][j] = 0.f;
    float m_ref[NC] = {0.f, 0.f};  // "no reference yet": the first tile sets it
    float l[NC] = {0.f, 0.f};

    // global -> LDS, as in prefill_bf16_pipe_kernel
    const int ld_row = lane / CPR, ld_pos = lane % CPR;
    uint32_t voffK[NLD], voffV[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int r = NR * (wave + 4 * i) + ld_row;
        voffK[i] = (uint32_t)r * (uint32_t)a.sk[2] * 2u + 16u * (uint32_t)(ld_pos ^ ((r / RP) % CPR));
        if constexpr (VBLK) voffV[i] = (uint32_t)(wave + 4 * i) * 1024u + 16u * (uint32_t)lane;  // the tile is contiguous
        else voffV[i] = (uint32_t)r * (uint32_t)a.sv[2] * 2u + 16u * (uint32_t)(ld_pos ^ (((r / RP) % (CPR / 4)) << 2));
    }
    const int64_t rowK = a.sk[2] * 2, rowV = a.sv[2] * 2;
    auto locate_tile = [&](int key0, const char*& kb, const char*& vb, int& local, int& cap, int& rows) {
        kb = (const char*)Kp;
        vb = (const char*)Vp;
        local = key0;
        cap = a.s_pad;
        rows = L - key0;
        if constexpr (VBLK) {
            if (a.page_table) {
                const int pg = key0 / a.page_tokens;
                local = key0 - pg * a.page_tokens;
                cap = a.page_tokens;
                const int64_t slab = (int64_t)a.page_table[(int64_t)b * a.pages_per_seq + pg] * a.Hkv + kvh;
                kb = (const char*)a.k + slab * cap * D * 2;
                vb = (const char*)a.v + slab * cap * D * 2;
                rows = min(rows, cap - local);
            }
        }
    };
    auto load_k_tile = [&](int t, int slot) {
        const char *kb, *vb;
        int local, cap, rows;
        locate_tile((tile0 + t) * kUnit, kb, vb, local, cap, rows);
        __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void*)(kb + (int64_t)local * rowK), 0, (int)((int64_t)rows * rowK), 0x00020000);
        uint16_t* dst = smem + slot * SLOT;
#pragma unroll
        for (int i = 0; i < NLD; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (__attribute__((address_space(3))) void*)(dst + (wave + 4 * i) * 512), 16, voffK[i], 0, 0, 0);
    };
    auto load_v_tile = [&](int t, int slot) {
        const char *kb, *vb;
        int local, cap, rows;
        locate_tile((tile0 + t) * kUnit, kb, vb, local, cap, rows);
        const int64_t v_base = VBLK ? (int64_t)local * D * 2 : (int64_t)local * rowV;
        const int64_t v_bytes = VBLK ? ((int64_t)cap - local) * D * 2 : (int64_t)rows * rowV;
        __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void*)(vb + v_base), 0, (int)v_bytes, 0x00020000);
        uint16_t* dst = smem + (NRING + slot) * SLOT;
#pragma unroll
        for (int i = 0; i < NLD; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (__attribute__((address_space(3))) void*)(dst + (wave + 4 * i) * 512), 16, voffV[i], 0, 0, 0);
    };

    // loop-constant LDS read addresses (ring slot 0 of each operand; the slot is an immediate offset)
    const int krow = VBLK ? ((ql & ~12) | ((ql & 4) << 1) | ((ql & 8) >> 1)) : ql;  // tile row this lane's S^T row holds
    const int kswz = (krow / RP) % CPR;
    uint32_t kaddr[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kaddr[ks] = lds0 + 2u * (uint32_t)(krow * D + 8 * ((2 * ks + h) ^ kswz));
    const int i16 = lane & 15;
    const int vswz = ((i16 >> 2) / RP) % (CPR / 4);
    const int v_lane_off = (4 * h + (i16 >> 2)) * D + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    uint32_t va[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
        va[db] = VBLK ? lds0 + 16u * (uint32_t)(h * D + ql) : lds0 + 2u * (uint32_t)v_lane_off + 64u * (uint32_t)(db ^ vswz);

    Frag fr[16];             // operand of slot s of the current step (slots < kLeadW: already requested)
    f32x16_t sb[2][NC];      // step tau finishes S'(tau+2) in sb[tau & 1] and consumes S'(tau+1) from sb[(tau+1) & 1]
    uint32_t pb[2][NC][8];   // packed bf16 P: step tau consumes P(tau) from pb[tau & 1] and writes P(tau+1) to pb[(tau+1) & 1]
    float negm[NC] = {0.f, 0.f};  // -m_ref of this lane's query (log2 domain)

    // Request the operand of slot S of the step whose ring slot is RS.
    auto request = [&](auto s_c, auto rs_c) {
        constexpr int S = decltype(s_c)::value;
        constexpr int RS = decltype(rs_c)::value;

        if constexpr (kSlotIsQ[S]) {
            constexpr int ks = kSlotIdx[S];
            fr[S].k = lds_read_b128_asm<RS * SLOTB>(kaddr[ks]);
        } else {
            constexpr int p = kSlotIdx[S], j = p / 4, db = p % 4;
            if constexpr (VBLK) {  // token block 2j + h of the tile, rows d = 32 db + ql: one 16-byte read
                fr[S].k = lds_read_b128_asm<(NRING + RS) * SLOTB + (2 * j * D + 32 * db) * 16>(va[db]);
            } else {
                constexpr int VOFF = (NRING + RS) * SLOTB + 16 * j * D * 2;
                fr[S].t0 = lds_read_tr16_b64_asm<VOFF>(va[db]);
                fr[S].t1 = lds_read_tr16_b64_asm<VOFF + 8 * D * 2>(va[db]);
            }
        }
    };

    // One step.  PH = tau & 3 (ring slot of the step's tiles: K(tau+2), V(tau)).  Every variant is one straight line of
    // code (no per-slot guards), chosen per step by wavefront-uniform tests:
    //   MODE 0: all three stages of both blocks, no mask needed;
    //   MODE 1: the same, and the new scores are masked where their tile straddles (or lies beyond) the diagonal or the
    //           end of the context.  Tiles a block does not need are computed too and masked as a whole: P = 0 there,
    //           the running sums do not move, the work is wasted but harmless (tile requests past the end re-read
    //           real rows or zeros, never uninitialised LDS);
    //   MODE 2: as 1 for block 1 only: block 0 (the earlier one) has used its last tile and does nothing;
    //   MODE 3 / 4: the two prologue steps: no PV (there is no P yet, and the V ring is not filled), softmax only in
    //           the second, where it sets the reference from tile 0.
    auto step = [&](int tau, auto ph_c, auto mode_c) {
        constexpr int PH = decltype(ph_c)::value;
        constexpr int MODE = decltype(mode_c)::value;
        constexpr bool FAST = MODE == 0;
        constexpr bool FIRST = MODE == 4;   // step -1: the softmax stage sees tile 0 and sets the reference
        constexpr int C0 = MODE == 2 ? 1 : 0;        // first active block
        constexpr bool PV = MODE < 3, SM = MODE != 3;

        if constexpr (MODE == 3) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");  // first step: K(1) has landed
        else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");  // the tiles of step tau+1 have landed; those of tau+2 may be in flight
#ifdef ABL_NOBAR
        if constexpr (MODE != 0)
#endif
        __builtin_amdgcn_s_barrier();  // waits are explicit: no fence, which would drain every load in flight
        // always four loads per wavefront and step, so that the vmcnt arithmetic holds: past the end the tile index is
        // clamped (the rows fall outside the buffer bound and arrive as zeros, or re-read the last tile; never consumed)
#ifdef ABL_NOLOAD
        if constexpr (MODE != 3 && MODE != 0) {
#else
        if constexpr (MODE != 3) {
#endif
            load_k_tile(min(tau + 5, n_tiles - 1), (PH + 3) & 3);
            load_v_tile(min(tau + 3, n_tiles - 1), (PH + 3) & 3);
        }

        float es[NC][16];
        float lsum[NC] = {0.f, 0.f}, lsum2[NC] = {0.f, 0.f};
        // instruction i of the 32 that turn a block's finished scores into its next P: per pair of scores 2 multiplies,
        // 2 exp2, 1 pack and the row sum (plain adds in steady state; the packed dot product on the rounded values in
        // the boundary steps, so that short contexts are normalised by exactly what was accumulated)
        auto softmax_op = [&](auto c_c, auto i_c) {
            constexpr int c = decltype(c_c)::value;
            constexpr int i = decltype(i_c)::value, p = i / 4, k = i % 4;
            f32x16_t& s_cur = sb[(PH + 1) & 1][c];
            uint32_t(&p_nxt)[8] = pb[(PH + 1) & 1][c];
            // pin(): an empty asm that takes the value just computed as an operand.  Without it the compiler is free to
            // sink these instructions out of the slot (their results are only used a step later, or behind the branch
            // that follows the slots), which would take them out from under the MFMAs.
            if constexpr (k == 0) {
                es[c][2 * p] = __builtin_fmaf(s_cur[2 * p], cexp, negm[c]);
                es[c][2 * p + 1] = __builtin_fmaf(s_cur[2 * p + 1], cexp, negm[c]);
                es[c][2 * p] = __builtin_amdgcn_exp2f(es[c][2 * p]);
                pin(es[c][2 * p]);
                pin(es[c][2 * p + 1]);
            } else if constexpr (k == 1) {
                es[c][2 * p + 1] = __builtin_amdgcn_exp2f(es[c][2 * p + 1]);
                pin(es[c][2 * p + 1]);
            } else if constexpr (k == 2) {
                p_nxt[p] = cvt_pk_bf16(es[c][2 * p], es[c][2 * p + 1]);
                pin(p_nxt[p]);
            } else if constexpr (FAST) {
                if constexpr (p == 0) { lsum[c] = es[c][0]; lsum2[c] = es[c][1]; }
                else { lsum[c] += es[c][2 * p]; lsum2[c] += es[c][2 * p + 1]; }
                pin(lsum[c]);
                pin(lsum2[c]);
            } else {
                lsum[c] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, p_nxt[p]), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), lsum[c], false);
                pin(lsum[c]);
            }
        };

        // Steady state (MODE 0): slot S handles score S of each block, in the shadow of that block's MFMA: the multiply-add
        // and the exp2 of score S, the add of score S-1 into the row sum (a transcendental result must not be
        // consumed by the very next instruction), the pack of the pair finished a slot earlier.  What is left after
        // slot 15 (one add, one pack per block) sits behind the slots.
        auto fast_softmax = [&](auto c_c, auto s_c) {
            constexpr int c = decltype(c_c)::value, S = decltype(s_c)::value;
            f32x16_t& s_cur = sb[(PH + 1) & 1][c];
            uint32_t(&p_nxt)[8] = pb[(PH + 1) & 1][c];
            // (the multiply-add of score S + 1 goes in front of the exp2 of score S, so that no instruction waits on
            // the one right before it; the multiply-add of score 0 sits at the top of the step)
            if constexpr (S < 15) v_fma1(es[c][S + 1], s_cur[S + 1], cexp, negm[c]);
            v_exp1(es[c][S]);
            if constexpr (S == 2) v_add(lsum[c], es[c][0], es[c][1]);
            else if constexpr (S > 2) v_acc(lsum[c], es[c][S - 1]);
            if constexpr (S >= 2 && S % 2 == 0) v_cvt_pk(p_nxt[(S - 2) / 2], es[c][S - 2], es[c][S - 1]);
        };

        if constexpr (FAST) {
            static_for<NC>([&](auto c_c) {
                constexpr int c = decltype(c_c)::value;
                v_fma1(es[c][0], sb[(PH + 1) & 1][c][0], cexp, negm[c]);
            });
        }
        static_for<16>([&](auto s_c) {
            constexpr int S = decltype(s_c)::value;
            // ---- the two MFMAs of this slot share one operand from LDS
            if constexpr (kSlotIsQ[S]) {
                constexpr int ks = kSlotIdx[S];
                constexpr int W = reads_behind_n<VBLK, kLeadW>(S);
                static_for<NC>([&](auto c_c) {
                    constexpr int c = decltype(c_c)::value;
                    if constexpr (c >= C0) {
                        f32x16_t& s_nxt = sb[PH & 1][c];
                        constexpr int WAIT = c == C0 ? W : -1;  // the first MFMA of the slot waits for the operand
                        if constexpr (ks == 0) mfma_set_v<!FAST, WAIT>(s_nxt, __builtin_bit_cast(bf16x8_t, fr[S].k), qf[c][ks]);
                        else mfma_acc_v<!FAST, WAIT>(s_nxt, __builtin_bit_cast(bf16x8_t, fr[S].k), qf[c][ks]);
                        if constexpr (FAST) fast_softmax(c_c, s_c);
                        else if constexpr (SM && !FIRST) softmax_op(c_c, std::integral_constant<int, 2 * S>{});
                    }
                });
            } else {
                constexpr int p = kSlotIdx[S], j = p / 4, db = p % 4;
                constexpr int W = reads_behind_n<VBLK, kLeadW>(S);
                if constexpr (VBLK && !FAST && PV) {
                    frag_wait_k<W>(fr[S].k);  // the operand is patched below: wait for it here
                    // the planes hold stale tokens past L: P is 0 there, V must not be NaN
                    const int nvalid = L - ((tile0 + tau) * kUnit + 16 * j + 8 * h);  // slots e >= nvalid are past the context
                    if (nvalid < 8) {
#pragma unroll
                        for (int w = 0; w < 4; ++w) {
                            uint32_t x = fr[S].k[w];
                            if (2 * w + 1 >= nvalid) x &= 0x0000ffffu;
                            if (2 * w >= nvalid) x = 0;
                            fr[S].k[w] = x;
                        }
                    }
                }
                if constexpr (!PV) {  // the operand was requested all the same: it lands before its registers are reused
                    if constexpr (VBLK) frag_wait_k<W>(fr[S].k);
                    else frag_wait_v<W>(fr[S].t0, fr[S].t1);
                }
                const bf16x8_t vf = VBLK ? __builtin_bit_cast(bf16x8_t, fr[S].k)
                                         : __builtin_bit_cast(bf16x8_t, uint4{fr[S].t0.x, fr[S].t0.y, fr[S].t1.x, fr[S].t1.y});
                static_for<NC>([&](auto c_c) {
                    constexpr int c = decltype(c_c)::value;
                    if constexpr (c >= C0) {
                        if constexpr (PV) {
                            uint32_t(&p_cur)[8] = pb[PH & 1][c];
                            const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, uint4{p_cur[4 * j], p_cur[4 * j + 1], p_cur[4 * j + 2], p_cur[4 * j + 3]});
                            mfma_acc_a<!FAST, (c == C0 ? W : -1)>(acc[c][db], vf, pf);
                        }
                        if constexpr (FAST) fast_softmax(c_c, s_c);
                        else if constexpr (SM && !FIRST) softmax_op(c_c, std::integral_constant<int, 2 * S>{});
                    }
                });
            }
            // ---- the operand of the slot kLeadW ahead (next step's tiles once the index wraps)
#ifdef ABL_NOLDS
            if constexpr (!FAST)
#endif
            {
            if constexpr (S + kLeadW < 16) request(std::integral_constant<int, S + kLeadW>{}, std::integral_constant<int, PH>{});
            else request(std::integral_constant<int, S + kLeadW - 16>{}, std::integral_constant<int, (PH + 1) & 3>{});
            }
            // ---- the rest of this slot's share of the vector-ALU work
            if constexpr (SM && !FIRST && !FAST) {
                static_for<NC>([&](auto c_c) {
                    if constexpr (decltype(c_c)::value >= C0) softmax_op(c_c, std::integral_constant<int, 2 * S + 1>{});
                });
            }
            if constexpr (!FAST && S == 12) {
                static_for<NC>([&](auto c_c) {
                    constexpr int c = decltype(c_c)::value;
                    if constexpr (c >= C0) {
                        f32x16_t& s_nxt = sb[PH & 1][c];
                        const int k0 = (tile0 + tau + 2) * kUnit;
                        if ((a.causal && k0 + kUnit - 1 > q0c[c] + off) || (k0 + kUnit > L) || q0c[c] >= a.T) {
                            mfma_settle();  // the last QK^T MFMA was issued two slots ago, and a prologue step has no other work there
                            const int q_abs = q0c[c] + ql + off;
                            // a block past the end of the chunk has no keys at all
                            const int lim = q0c[c] >= a.T ? -1 : (a.causal ? min(q_abs, L - 1) : L - 1);
#pragma unroll
                            for (int v = 0; v < 16; ++v)
                                if ((VBLK ? k0 + 16 * (v >> 3) + 8 * h + (v & 7) : k0 + 8 * (v >> 2) + 4 * h + (v & 3)) > lim) s_nxt[v] = masked;
                        }
                    }
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (FAST) {
            static_for<NC>([&](auto c_c) {
                constexpr int c = decltype(c_c)::value;
                uint32_t(&p_nxt)[8] = pb[(PH + 1) & 1][c];
                v_acc(lsum[c], es[c][15]);
                v_cvt_pk(p_nxt[7], es[c][14], es[c][15]);
            });
        }
        // outside the steady state the compiler may move accumulators between registers where step variants meet:
        // the MFMAs of this step have drained before that
        if constexpr (!FAST) mfma_settle();
        static_for<NC>([&](auto c_c) {
            constexpr int c = decltype(c_c)::value;
            if constexpr (SM && c >= C0) {
                // A reference that has fallen behind shows in the row sum: below 2^10 no P of the tile exceeds 2^10, far
                // from overflow; otherwise (rare; and always for the first tile, which has no reference yet) take the
                // true maximum of these scores, raise the reference to an integer at or above it (alpha is then a power
                // of two, so everything computed against the old reference rescales exactly) and redo this tile's P.
                f32x16_t& s_cur = sb[(PH + 1) & 1][c];
                constexpr bool first = FIRST;
                if (first || __any(!(lsum[c] + lsum2[c] < 1024.f))) {
                    mfma_settle();  // the accumulators are read below, right behind the last PV MFMAs
                    float mx = s_cur[0] * cexp;
#pragma unroll
                    for (int v = 1; v < 16; ++v) mx = fmaxf(mx, s_cur[v] * cexp);
                    mx = half_swap_max(mx);
                    // raise (first tile: set) the reference to an integer at or above the largest score of the tile
                    float delta = (mx == -INFINITY) ? 0.f : ceilf(mx) + negm[c];
                    if (!first) delta = fmaxf(delta, 0.f);
                    if constexpr (!first) {  // nothing has been accumulated before the first tile
                        const float alpha = __builtin_amdgcn_exp2f(-delta);
                        l[c] *= alpha;
#pragma unroll
                        for (int i = 0; i < DB; ++i)
#pragma unroll
                            for (int j = 0; j < 16; ++j) acc[c][i][j] *= alpha;
                    }
                    lsum[c] = lsum2[c] = 0.f;
                    m_ref[c] += delta;
                    negm[c] = -m_ref[c];
                    static_for<32>([&](auto i_c) { softmax_op(c_c, i_c); });
                }
                l[c] += lsum[c] + lsum2[c];
            }
        });
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    using Fast = std::integral_constant<int, 0>;
    using Masked = std::integral_constant<int, 1>;
    using OneBlock = std::integral_constant<int, 2>;
    using First = std::integral_constant<int, 3>;   // step -2
    using Second = std::integral_constant<int, 4>;  // step -1
    // past the unmasked stretch: both blocks while block 0 still has a tile to multiply into its output, then block 1 alone
    auto late_step = [&](int tau, auto ph_c) {
        if (tau < nt_c[0]) step(tau, ph_c, Masked{});
        else step(tau, ph_c, OneBlock{});
    };

    if (n_tiles > 0) {  // an empty context (cache mode, length 0) has nothing to attend to: zeros below
        // prologue: the tiles of steps -2 and -1 (K(0), K(1)) are requested here, published by the barrier below
        load_k_tile(0, 2);
        load_k_tile(min(1, n_tiles - 1), 3);
        // tiles of steps 0 and 1 (K(2), V(0), K(3), V(1)); from step -1 on every step requests the tiles three steps ahead
        load_k_tile(min(2, n_tiles - 1), 0);
        load_v_tile(0, 0);
        load_k_tile(min(3, n_tiles - 1), 1);
        load_v_tile(min(1, n_tiles - 1), 1);
        asm volatile("s_waitcnt vmcnt(10)" ::: "memory");  // K(0) has landed
        __builtin_amdgcn_s_barrier();  // waits are explicit: no fence, which would drain every load in flight
        static_for<kLeadW>([&](auto s_c) { request(s_c, I2{}); });

        step(-2, I2{}, First{});
        step(-1, I3{}, Second{});
        int tau = 0;
        for (; tau + 4 <= n_fast; tau += 4) {
            step(tau, I0{}, Fast{});
            step(tau + 1, I1{}, Fast{});
            step(tau + 2, I2{}, Fast{});
            step(tau + 3, I3{}, Fast{});
        }
        for (; tau < n_tiles; tau += 4) {
            late_step(tau, I0{});
            if (tau + 1 < n_tiles) late_step(tau + 1, I1{});
            if (tau + 2 < n_tiles) late_step(tau + 2, I2{});
            if (tau + 3 < n_tiles) late_step(tau + 3, I3{});
        }
        // operands requested for a step that does not exist are still in flight: let them land before the registers die
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }

    mfma_settle();
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const float lc = half_swap_sum(l[c]);
        const int qi = q0c[c] + ql;
        if constexpr (VBLK) {
            if (a.n_splits > 1) {  // the unnormalised partial of this share of the context; the combine kernel finishes the row
                if (qi < a.T) {
                    const int64_t row = (((int64_t)b * a.Hq + hq) * a.T + qi) * a.n_splits + split;
                    float* po = a.ws_o + row * D;
#pragma unroll
                    for (int db = 0; db < DB; ++db)
#pragma unroll
                        for (int vq = 0; vq < 4; ++vq)
                            *(float4*)(po + 32 * db + 8 * vq + 4 * h) = float4{acc[c][db][4 * vq], acc[c][db][4 * vq + 1], acc[c][db][4 * vq + 2], acc[c][db][4 * vq + 3]};
                    if (h == 0) {  // a row that met no key in this share (masked, or the share lies past its diagonal) says so
                        a.ws_ml[row * 2] = lc > 0.f ? m_ref[c] : -INFINITY;
                        a.ws_ml[row * 2 + 1] = lc;
                    }
                }
                continue;
            }
        }
        if (qi < a.T) {
            const float inv_l = lc > 0.f ? 1.0f / lc : 0.f;
            uint16_t* op = (uint16_t*)a.out + (int64_t)b * a.so[0] + (int64_t)hq * a.so[1] + (int64_t)qi * a.so[2];
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int vq = 0; vq < 4; ++vq) {
                    const int d = 32 * db + 8 * vq + 4 * h;
                    uint2 w;
                    w.x = cvt_pk_bf16(acc[c][db][4 * vq] * inv_l, acc[c][db][4 * vq + 1] * inv_l);
                    w.y = cvt_pk_bf16(acc[c][db][4 * vq + 2] * inv_l, acc[c][db][4 * vq + 3] * inv_l);
                    *(uint2*)(op + d) = w;
                }
            if (a.lse && h == 0)
                a.lse[(int64_t)b * a.sl[0] + (int64_t)hq * a.sl[1] + (int64_t)qi * a.sl[2]] = (m_ref[c] + __builtin_amdgcn_logf(lc)) * 0.6931471805599453f;
        }
    }
    // the clamped tile requests of the last steps write LDS: they have landed before the workgroup gives its LDS back
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
}

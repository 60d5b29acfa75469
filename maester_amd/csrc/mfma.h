// gfx950 (CDNA4) building blocks shared by the bf16 attention kernels: MFMA fragment types, the
// LDS tile layout, and the row-wise / transposed LDS fragment reads.
//
// MFMA v_mfma_f32_32x32x16_bf16, wave64, lane l, r = l % 32, hh = l / 32:
//   A (32 x 16): lane holds A[r][8*hh .. 8*hh+7]          (8 bf16)
//   B (16 x 32): lane holds B[8*hh .. 8*hh+7][r]          (8 bf16)
//   C (32 x 32): lane holds C[8*(v/4) + 4*hh + v%4][r]    (v = 0..15, fp32)
// Because the C layout of one product has the shape of a B operand (a lane owns one column and
// 16 of its rows), the kernels compute transposed products (S^T = K Q^T, then O^T = V^T P^T) so
// that P never leaves registers; the only thing to arrange is that the other operand enumerates
// the contraction index in the order 16t + 8*(e/4) + 4*hh + e%4 (e = 0..7), see tr_frag().
//
// LDS tile layout ("permuted rows, padded"): a tile of R rows x D bf16 keeps logical row
// 16a + 4m + e at physical row 16a + 4e + m, with a row pitch of D*2 + 16 bytes.  The pitch is
// 4 banks (mod 64) so 16 consecutive physical rows start in 16 distinct 4-bank groups -- a
// row-wise b128 read by 16 lanes with consecutive rows is conflict free -- and the row
// permutation puts the 4 consecutive logical rows a transposed read touches 16 banks apart, so
// that one is conflict free too.  Every access is lane_base + compile-time offset: no address
// arithmetic in the loops.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace ma {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int64_t i64x2 __attribute__((ext_vector_type(2)));

#ifndef MA_LDS
#define MA_LDS __attribute__((address_space(3)))
#endif
typedef MA_LDS char* lds_ptr;

// compile-time loop: f(std::integral_constant<int, I>{}) for I in [B, E)
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

template <int D>
struct Tile {
    static constexpr int kPitch = D * 2 + 16;  // bytes per physical row
    static constexpr int kChunks = D / 8;      // 16-byte chunks per row
    static constexpr int bytes(int rows) { return rows * kPitch; }

    // physical row of a logical row (swap the two 2-bit fields inside each group of 16)
    __device__ __forceinline__ static int prow(int row) {
        return (row & ~15) | ((row & 3) << 2) | ((row >> 2) & 3);
    }
    __device__ __forceinline__ static int off(int row, int col) { return prow(row) * kPitch + col * 2; }

    // ---- row-wise fragments (contraction index contiguous in memory) -------------------------
    // lane (r, hh) reads row row0 + r, elements 16*kk + 8*hh .. +7.  row0 must be a multiple of 32.
    __device__ __forceinline__ static int row_base(int lane) {
        return prow(lane & 31) * kPitch + (lane >> 5) * 16;
    }
    __device__ __forceinline__ static bf16x8 row_frag(lds_ptr tile, int base, int row0, int kk) {
        return *(MA_LDS bf16x8*)(tile + base + row0 * kPitch + kk * 32);
    }

    // ---- transposed fragments through ds_read_b64_tr_b16 -----------------------------------------
    // Within each group of 16 lanes, lane i supplies the address of 4 consecutive elements and
    // receives element i%4 of the rows supplied by lanes i/4, 4+i/4, 8+i/4, 12+i/4.  Lane i of a
    // group points at (row = g + i/4, col = c + 4*(i%4)) and ends up with column c + i of rows
    // g..g+3.  For an A operand (M = tile column, K = tile row) over columns c0..c0+31 and rows
    // r0..r0+15 paired with a C-layout fragment, lane (r, hh) needs column c0 + r and rows
    // r0 + 4*hh + {0..3} and r0 + 8 + 4*hh + {0..3}: two reads, 8 rows apart.
    // r0 must be a multiple of 16, c0 a multiple of 32.
    __device__ __forceinline__ static int tr_base(int lane) {
        const int i = lane & 15, hh = lane >> 5;
        const int row = 4 * hh + (i >> 2);                       // logical row within the group of 16
        const int col = (((lane >> 4) & 1) << 4) + ((i & 3) << 2);
        return prow(row) * kPitch + col * 2;
    }
    __device__ __forceinline__ static bf16x8 tr_frag(lds_ptr tile, int base, int r0, int c0) {
        // logical rows +8 inside a group of 16 are physical rows +2
        const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((MA_LDS bf16x4*)(tile + base + r0 * kPitch + c0 * 2));
        const bf16x4 hi =
            __builtin_amdgcn_ds_read_tr16_b64_v4bf16((MA_LDS bf16x4*)(tile + base + (r0 + 2) * kPitch + c0 * 2));
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
};

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// MFMAs with the register classes of their operands pinned.  Left to itself the register
// allocator keeps long-lived accumulators in AGPRs and shuttles all of them to VGPRs and back
// around every loop iteration as soon as anything (a rare rescale, say) touches them with the
// vector ALU.  Here the accumulators are pinned to VGPRs ("+v": MFMA reads/writes them in place
// and so does the VALU) and the loop-invariant operand fragments can be parked in AGPRs ("a").
// The compiler does not know these asm statements are MFMAs and pads no hazards: callers keep
// VALU readers of c at least 16 wait states behind the last MFMA (mfma_fence()) and VALU writers
// of a/b a few instructions ahead of the first.
__device__ __forceinline__ void mfma32_vv(f32x16& c, bf16x8 a, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma32_va(f32x16& c, bf16x8 a, bf16x8 b_agpr) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b_agpr));
}
__device__ __forceinline__ void mfma32_av(f32x16& c, bf16x8 a_agpr, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "a"(a_agpr), "v"(b));
}
// same with a zero addend: starts an accumulation without a VALU-written zero tile
__device__ __forceinline__ void mfma32_va_zero(f32x16& c, bf16x8 a, bf16x8 b_agpr) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "a"(b_agpr));
}
__device__ __forceinline__ void mfma32_av_zero(f32x16& c, bf16x8 a_agpr, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "a"(a_agpr), "v"(b));
}
__device__ __forceinline__ void mfma32_vv_zero(f32x16& c, bf16x8 a, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
}
// accumulator pinned to AGPRs (for tiles no vector-ALU instruction touches inside the loop)
__device__ __forceinline__ void mfma32_acc_a(f32x16& c, bf16x8 a, bf16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
// pins two operand fragments to AGPRs at this point of the program
__device__ __forceinline__ void park_in_agprs(bf16x8& x, bf16x8& y) { asm volatile("" : "+a"(x), "+a"(y)); }
// 16 wait states: enough for the result of an 8-pass MFMA to be readable by the vector ALU.  The
// tiles are read-write operands so that nothing that uses them can be scheduled above the fence
// (volatile asm statements keep their order among themselves).
__device__ __forceinline__ void mfma_fence() { asm volatile("s_nop 15"); }
template <int I, int N, bool ACC_A>
__device__ __forceinline__ void pin_tiles(f32x16* acc) {
    if constexpr (I < N) {
        if constexpr (ACC_A) asm volatile("" : "+a"(acc[I]));
        else asm volatile("" : "+v"(acc[I]));
        pin_tiles<I + 1, N, ACC_A>(acc);
    }
}
// Pins N freshly computed operand fragments: everything that produces them is scheduled above this
// point, a few wait states ahead of the MFMAs that read them (a vector-ALU result must not be
// consumed by an MFMA in the very next cycles).
template <int I, int N>
__device__ __forceinline__ void pin_frags(bf16x8* f) {
    if constexpr (I < N) {
        if constexpr (I == 0) asm volatile("s_nop 4" : "+v"(f[0]));
        else asm volatile("" : "+v"(f[I]));
        pin_frags<I + 1, N>(f);
    }
}
template <int N, bool ACC_A = false>
__device__ __forceinline__ void mfma_fence_tiles(f32x16* acc) {
    mfma_fence();
    pin_tiles<0, N, ACC_A>(acc);
}

// ---- explicitly pipelined LDS fragment reads ---------------------------------------------------
// The compiler serialises "LDS read -> wait -> MFMA" in these kernels, so the hot loops issue
// their LDS reads through asm statements (kept in program order) and tie the matching
// s_waitcnt to the fragment it guards: lds_wait<N>(x) returns once at most N younger LDS
// operations are still outstanding, and because it takes x as a read-write operand no consumer
// of x can be moved above it.  Extra outstanding operations the compiler adds only make the
// waits more conservative.  The MFMAs stay builtins, so the compiler keeps handling their hazards.
template <int OFF>
__device__ __forceinline__ bf16x8 lds_read_b128(uint32_t addr) {
    bf16x8 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
template <int OFF>
__device__ __forceinline__ bf16x4 lds_read_tr16_b64(uint32_t addr) {
    bf16x4 v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
template <int N>
__device__ __forceinline__ void lds_wait(bf16x8& x) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x) : "n"(N));
}
template <int N>
__device__ __forceinline__ void lds_wait2(bf16x4& x, bf16x4& y) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(x), "+v"(y) : "n"(N));
}
__device__ __forceinline__ uint32_t lds_addr(lds_ptr p) { return (uint32_t)(uintptr_t)p; }

// acc[nb] = sum_kk L(rows 32nb + r, cols 16kk..) x reg[kk] for NB row blocks of 32 at once: a
// software pipeline of depth P over the NB*KK row-wise fragments of an LDS tile (row_addr = lds
// address of the tile + Tile::row_base(lane)).  The register-resident fragments reg[] live in
// AGPRs (REG_A) or VGPRs.  SWAP puts the LDS fragment in the B slot instead (computes the
// transposed product).  acc is overwritten (no zero tile needed) and lives in VGPRs; ends with
// mfma_fence().
struct NoHook {
    template <typename I>
    __device__ __forceinline__ void operator()(I) const {}
};

// hook(integral_constant<int, i>) runs right after MFMA i has been issued: the kernels use it to
// spread the global -> LDS loads of the next step over the chain instead of issuing them in one
// burst (a burst fills the memory pipeline and stalls the wave with the matrix cores idle).
template <int D, int NB, int P, bool SWAP = false, bool REG_A = true, typename Hook = NoHook>
__device__ __forceinline__ void rowfrag_gemm(uint32_t row_addr, const bf16x8* reg, f32x16* acc, Hook&& hook = Hook{}) {
    using TL = Tile<D>;
    constexpr int KK = D / 16;
    constexpr int N = NB * KK;
    bf16x8 t[N];
    auto rd = [&](auto idx) {
        constexpr int i = decltype(idx)::value;
        constexpr int kk = i / NB, nb = i % NB;
        t[i] = lds_read_b128<nb * 32 * TL::kPitch + kk * 32>(row_addr);
    };
    auto step = [&](auto idx) {
        constexpr int i = decltype(idx)::value;
        constexpr int kk = i / NB, nb = i % NB;
        constexpr int younger = (N - 1 - i) < (P - 1) ? (N - 1 - i) : (P - 1);
        lds_wait<younger>(t[i]);
        if constexpr (kk == 0) {
            if constexpr (!REG_A) { if constexpr (SWAP) mfma32_vv_zero(acc[nb], reg[kk], t[i]); else mfma32_vv_zero(acc[nb], t[i], reg[kk]); }
            else if constexpr (SWAP) mfma32_av_zero(acc[nb], reg[kk], t[i]);
            else mfma32_va_zero(acc[nb], t[i], reg[kk]);
        } else {
            if constexpr (!REG_A) { if constexpr (SWAP) mfma32_vv(acc[nb], reg[kk], t[i]); else mfma32_vv(acc[nb], t[i], reg[kk]); }
            else if constexpr (SWAP) mfma32_av(acc[nb], reg[kk], t[i]);
            else mfma32_va(acc[nb], t[i], reg[kk]);
        }
    };
    static_for<0, (P < N ? P : N)>(rd);
    static_for<0, N>([&](auto idx) {
        constexpr int i = decltype(idx)::value;
        step(idx);
        if constexpr (i + P < N) rd(std::integral_constant<int, i + P>{});
        hook(idx);
    });
    mfma_fence_tiles<NB>(acc);
}

// Two independent products of that kind, from two LDS tiles, in one read pipeline:
//   acc0 = sum_kk L0(rows r, cols 16kk..) x reg0[kk],  acc1 = sum_kk L1(...) x reg1[kk].
// SEQ = false interleaves them MFMA by MFMA; SEQ = true finishes acc0 (MFMAs 0..KK-1) before acc1
// (MFMAs KK..2KK-1), so that hooks of the second half can already work on acc0 with the vector ALU
// (from MFMA KK+1 on: the result of an MFMA is readable two MFMAs later).
// PRESET: the accumulators come in holding the addends of the two products instead of being overwritten.
template <int D, int P, bool SWAP = false, bool REG_A = true, typename Hook = NoHook, bool SEQ = false, bool PRESET = false>
__device__ __forceinline__ void rowfrag_gemm2(uint32_t row_addr0, const bf16x8* reg0, f32x16& acc0, uint32_t row_addr1,
                                              const bf16x8* reg1, f32x16& acc1, Hook&& hook = Hook{}) {
    constexpr int KK = D / 16;
    constexpr int N = 2 * KK;
    bf16x8 t[N];
    auto rd = [&](auto idx) {
        constexpr int i = decltype(idx)::value;
        constexpr int kk = SEQ ? i % KK : i / 2, which = SEQ ? i / KK : i % 2;
        t[i] = lds_read_b128<kk * 32>(which ? row_addr1 : row_addr0);
    };
    auto step = [&](auto idx) {
        constexpr int i = decltype(idx)::value;
        constexpr int kk = SEQ ? i % KK : i / 2, which = SEQ ? i / KK : i % 2;
        constexpr int younger = (N - 1 - i) < (P - 1) ? (N - 1 - i) : (P - 1);
        lds_wait<younger>(t[i]);
        // the register fragment is handed to the asm statement as it is (no copy: a copy of an
        // AGPR-resident fragment would need AGPRs of its own)
        auto one = [&](f32x16& acc, const bf16x8& rg) {
            if constexpr (kk == 0 && !PRESET) {
                if constexpr (!REG_A) { if constexpr (SWAP) mfma32_vv_zero(acc, rg, t[i]); else mfma32_vv_zero(acc, t[i], rg); }
                else if constexpr (SWAP) mfma32_av_zero(acc, rg, t[i]);
                else mfma32_va_zero(acc, t[i], rg);
            } else {
                if constexpr (!REG_A) { if constexpr (SWAP) mfma32_vv(acc, rg, t[i]); else mfma32_vv(acc, t[i], rg); }
                else if constexpr (SWAP) mfma32_av(acc, rg, t[i]);
                else mfma32_va(acc, t[i], rg);
            }
        };
        if constexpr (which) one(acc1, reg1[kk]);
        else one(acc0, reg0[kk]);
    };
    static_for<0, (P < N ? P : N)>(rd);
    static_for<0, N>([&](auto idx) {
        constexpr int i = decltype(idx)::value;
        step(idx);
        if constexpr (i + P < N) rd(std::integral_constant<int, i + P>{});
        // SEQ: acc0 is final after MFMA KK-1 and may be read by the vector ALU once two more MFMAs have
        // been issued.  Pinning it here keeps whatever the hooks do with it below this point (their
        // arithmetic is ordinary code, which the compiler would otherwise move up to MFMA KK-1).
        if constexpr (SEQ && i == KK + 1) asm volatile("" : "+v"(acc0));
        hook(idx);
    });
    mfma_fence();
    asm volatile("" : "+v"(acc0));
    asm volatile("" : "+v"(acc1));
}

// acc[db] += L^T(rows 16j.., cols 32db..) x reg[j] over NJ 16-row slabs of an LDS tile through
// transposed fragments (tr_addr = lds address of the tile + Tile::tr_base(lane)).  Pipeline of
// depth P over the NJ * DB fragments (two LDS reads each).  reg lives in VGPRs, acc in VGPRs or
// (ACC_A) AGPRs; ends with mfma_fence().
// READY: how many of the reg fragments are complete when the chain starts; the others are
// produced by the hooks of earlier MFMAs (fragment j is first used by MFMA j*DB) and are picked up
// from reg_in just before their first use.
template <int D, int NJ, int P, bool ACC_A = false, typename Hook = NoHook, int READY = NJ>
__device__ __forceinline__ void trfrag_gemm(uint32_t tr_addr, const bf16x8* reg_in, f32x16* acc, Hook&& hook = Hook{}) {
    using TL = Tile<D>;
    constexpr int DB = D / 32;
    constexpr int N = NJ * DB;
    bf16x8 reg[NJ];
#pragma unroll
    for (int j = 0; j < READY; ++j) reg[j] = reg_in[j];
    pin_frags<0, READY>(reg);
    bf16x4 lo[N], hi[N];
    auto rd = [&](auto idx) {
        constexpr int i = decltype(idx)::value;
        constexpr int j = i / DB, db = i % DB;
        lo[i] = lds_read_tr16_b64<(16 * j) * TL::kPitch + db * 64>(tr_addr);
        hi[i] = lds_read_tr16_b64<(16 * j + 2) * TL::kPitch + db * 64>(tr_addr);
    };
    auto step = [&](auto idx) {
        constexpr int i = decltype(idx)::value;
        constexpr int j = i / DB, db = i % DB;
        constexpr int younger = (N - 1 - i) < (P - 1) ? (N - 1 - i) : (P - 1);
        if constexpr (j >= READY && db == 0) {  // a fragment the hooks have just finished
            reg[j] = reg_in[j];
            asm volatile("s_nop 4" : "+v"(reg[j]));
        }
        // wait on the two halves themselves: a copy made while assembling the 8-element fragment
        // must not read them before the data has landed
        lds_wait2<2 * younger>(lo[i], hi[i]);
        const bf16x8 f = __builtin_shufflevector(lo[i], hi[i], 0, 1, 2, 3, 4, 5, 6, 7);
        if constexpr (ACC_A) mfma32_acc_a(acc[db], f, reg[j]);
        else mfma32_vv(acc[db], f, reg[j]);
    };
    static_for<0, (P < N ? P : N)>(rd);
    static_for<0, N>([&](auto idx) {
        constexpr int i = decltype(idx)::value;
        step(idx);
        if constexpr (i + P < N) rd(std::integral_constant<int, i + P>{});
        hook(idx);
    });
    mfma_fence_tiles<DB, ACC_A>(acc);  // whatever comes next may read acc with the vector ALU
}

// Two products of that kind, from two LDS tiles into two sets of AGPR accumulators, as ONE read
// pipeline: acc0[db] += L0^T x reg0[j] (MFMAs 0 .. NJ*DB-1), then acc1[db] += L1^T x reg1[j].  The
// first fragments of the second product are requested while the last MFMAs of the first are issued,
// so the pipeline is filled once instead of twice (a chain that starts cold waits a full LDS latency
// for its first fragment) and one fence serves both.
template <int D, int NJ, int P, typename Hook = NoHook>
__device__ __forceinline__ void trfrag_gemm_two(uint32_t tr_addr0, const bf16x8* reg0_in, f32x16* acc0, uint32_t tr_addr1,
                                                const bf16x8* reg1_in, f32x16* acc1, Hook&& hook = Hook{}) {
    using TL = Tile<D>;
    constexpr int DB = D / 32;
    constexpr int H = NJ * DB;
    constexpr int N = 2 * H;
    bf16x8 reg0[NJ], reg1[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) { reg0[j] = reg0_in[j]; reg1[j] = reg1_in[j]; }
    pin_frags<0, NJ>(reg0);
    pin_frags<0, NJ>(reg1);
    bf16x4 lo[N], hi[N];
    auto rd = [&](auto idx) {
        constexpr int i = decltype(idx)::value;
        constexpr int j = (i % H) / DB, db = i % DB;
        lo[i] = lds_read_tr16_b64<(16 * j) * TL::kPitch + db * 64>(i < H ? tr_addr0 : tr_addr1);
        hi[i] = lds_read_tr16_b64<(16 * j + 2) * TL::kPitch + db * 64>(i < H ? tr_addr0 : tr_addr1);
    };
    static_for<0, (P < N ? P : N)>(rd);
    static_for<0, N>([&](auto idx) {
        constexpr int i = decltype(idx)::value;
        constexpr int j = (i % H) / DB, db = i % DB;
        constexpr int younger = (N - 1 - i) < (P - 1) ? (N - 1 - i) : (P - 1);
        lds_wait2<2 * younger>(lo[i], hi[i]);
        const bf16x8 f = __builtin_shufflevector(lo[i], hi[i], 0, 1, 2, 3, 4, 5, 6, 7);
        if constexpr (i < H) mfma32_acc_a(acc0[db], f, reg0[j]);
        else mfma32_acc_a(acc1[db], f, reg1[j]);
        if constexpr (i + P < N) rd(std::integral_constant<int, i + P>{});
        hook(idx);
    });
    mfma_fence_tiles<DB, true>(acc0);
    pin_tiles<0, DB, true>(acc1);
}

// ---- register-blocked variants: every LDS fragment feeds two MFMAs ---------------------------------
// For two query heads that share a kv head, the K (or V) fragment read from LDS is the same for both:
// reading it once halves the LDS traffic per MFMA (the transposed reads of the second product are
// what bounds a single-head chain).  Hooks are numbered by MFMA (two per fragment).
//
// accA = sum_kk L(rows r, cols 16kk..) x regA[kk], accB = the same with regB; 32 rows of the tile at
// row_addr; register fragments in VGPRs; accumulators (overwritten) in VGPRs.
template <int D, int P, typename Hook = NoHook>
__device__ __forceinline__ void rowfrag_gemm_dual(uint32_t row_addr, const bf16x8* regA, const bf16x8* regB, f32x16& accA,
                                                  f32x16& accB, Hook&& hook = Hook{}) {
    constexpr int N = D / 16;
    bf16x8 t[N];
    auto rd = [&](auto idx) {
        constexpr int i = decltype(idx)::value;
        t[i] = lds_read_b128<i * 32>(row_addr);
    };
    static_for<0, (P < N ? P : N)>(rd);
    static_for<0, N>([&](auto idx) {
        constexpr int i = decltype(idx)::value;
        constexpr int younger = (N - 1 - i) < (P - 1) ? (N - 1 - i) : (P - 1);
        lds_wait<younger>(t[i]);
        if constexpr (i == 0) mfma32_vv_zero(accA, t[i], regA[i]);
        else mfma32_vv(accA, t[i], regA[i]);
        hook(std::integral_constant<int, 2 * i>{});
        if constexpr (i == 0) mfma32_vv_zero(accB, t[i], regB[i]);
        else mfma32_vv(accB, t[i], regB[i]);
        if constexpr (i + P < N) rd(std::integral_constant<int, i + P>{});
        hook(std::integral_constant<int, 2 * i + 1>{});
    });
    mfma_fence();
    asm volatile("" : "+v"(accA));
    asm volatile("" : "+v"(accB));
}

// accA[db] += L^T(rows 16j.., cols 32db..) x regA[j], accB[db] += the same x regB[j], over NJ
// 16-row slabs of the tile at tr_addr; accumulators in AGPRs.
template <int D, int NJ, int P, typename Hook = NoHook>
__device__ __forceinline__ void trfrag_gemm_dual(uint32_t tr_addr, const bf16x8* regA_in, const bf16x8* regB_in, f32x16* accA,
                                                 f32x16* accB, Hook&& hook = Hook{}) {
    using TL = Tile<D>;
    constexpr int DB = D / 32;
    constexpr int N = NJ * DB;
    bf16x8 regA[NJ], regB[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) { regA[j] = regA_in[j]; regB[j] = regB_in[j]; }
    pin_frags<0, NJ>(regA);
    pin_frags<0, NJ>(regB);
    bf16x4 lo[N], hi[N];
    auto rd = [&](auto idx) {
        constexpr int i = decltype(idx)::value;
        constexpr int j = i / DB, db = i % DB;
        lo[i] = lds_read_tr16_b64<(16 * j) * TL::kPitch + db * 64>(tr_addr);
        hi[i] = lds_read_tr16_b64<(16 * j + 2) * TL::kPitch + db * 64>(tr_addr);
    };
    static_for<0, (P < N ? P : N)>(rd);
    static_for<0, N>([&](auto idx) {
        constexpr int i = decltype(idx)::value;
        constexpr int j = i / DB, db = i % DB;
        constexpr int younger = (N - 1 - i) < (P - 1) ? (N - 1 - i) : (P - 1);
        lds_wait2<2 * younger>(lo[i], hi[i]);
        const bf16x8 f = __builtin_shufflevector(lo[i], hi[i], 0, 1, 2, 3, 4, 5, 6, 7);
        mfma32_acc_a(accA[db], f, regA[j]);
        hook(std::integral_constant<int, 2 * i>{});
        mfma32_acc_a(accB[db], f, regB[j]);
        if constexpr (i + P < N) rd(std::integral_constant<int, i + P>{});
        hook(std::integral_constant<int, 2 * i + 1>{});
    });
    mfma_fence_tiles<DB, true>(accA);
    pin_tiles<0, DB, true>(accB);
}

// Global -> registers -> LDS staging of a ROWS x D bf16 tile by NT threads.  load() issues all the
// global loads of the thread back to back (rows past the end are clamped to the last valid row so
// that the loads need no branches; their data is zeroed in store()), store() writes them to LDS.
// Splitting the two lets the loads of the next tile fly while the current one is being consumed.
template <int D, int ROWS, int NT>
struct Stager {
    static constexpr int CH = D / 8;
    static constexpr int N = ROWS * CH / NT;  // chunks per thread
    static constexpr int RPP = NT / CH;       // rows covered per pass
    static_assert((ROWS * CH) % NT == 0 && NT % CH == 0, "staging shape");
    u32x4 v[N];

    __device__ __forceinline__ void load(const __bf16* g, int64_t stride, int rows_valid, int tid) {
        const int c = tid % CH, r0 = tid / CH;
#pragma unroll
        for (int n = 0; n < N; ++n) {
            const int row = min(r0 + n * RPP, rows_valid - 1);
            v[n] = *(const u32x4*)(g + (int64_t)row * stride + c * 8);
        }
    }
    __device__ __forceinline__ void store(lds_ptr tile, int rows_valid, int tid) {
        const int c = tid % CH, r0 = tid / CH;
        if (rows_valid < ROWS) {
#pragma unroll
            for (int n = 0; n < N; ++n)
                if (r0 + n * RPP >= rows_valid) v[n] = u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int n = 0; n < N; ++n) *(MA_LDS u32x4*)(tile + Tile<D>::off(r0 + n * RPP, c * 8)) = v[n];
    }
};

// Global -> LDS staging without registers (gfx950 global_load_lds_dwordx4): every lane of a wave
// moves 16 bytes from an address of its own to LDS at wave_base + 16*lane, asynchronously (counted
// by vmcnt).  The tile is cut into runs of 64 consecutive 16-byte slots (the pad slot of each row
// included; it receives a copy of chunk 0); run t is moved by wave t % NWAVES.  Which global
// (row, chunk) lands in a slot is decided on the global side, so the permuted/padded layout costs
// nothing.  Rows at or beyond rows_valid re-read the last valid row (callers mask them).
#define MA_GLB __attribute__((address_space(1)))
// One run: 64 lanes x 16 bytes from (wave-uniform base + per-lane byte offset) to LDS at the
// wave-uniform address lds .. lds + 1023.  An asm statement so that it keeps its place among the
// MFMAs and LDS reads of a chain (which are asm statements too).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"  // m0 is clobbered on purpose: it carries the LDS address
__device__ __forceinline__ void global_to_lds_run(const void* base, uint32_t voff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff), "s"(base) : "m0");
}
// the same with the non-temporal hint: for data that is read exactly once (it does not displace what other workgroups share)
__device__ __forceinline__ void global_to_lds_run_nt(const void* base, uint32_t voff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds), "v"(voff), "s"(base) : "m0");
}
// The same through a buffer descriptor: the lane's byte offset into the tile is a ready-made register
// (row * row stride + offset inside the row, the same for every tile of one tensor), and rows past the
// end of the tile are out of the descriptor's range: such lanes touch no memory and zeros land in LDS.
// Three instructions per run instead of seven; the descriptor takes the place of the clamp.
//   rsrc = {address bits 31..0, address bits 47..32 (stride field 0: raw buffer), bytes in range, format word}
__device__ __forceinline__ u32x4 tile_rsrc(uint64_t base, uint32_t bytes_in_range) {
    // (the arguments are wave-uniform values that sit in SGPRs already: the descriptor is put together on
    // the scalar side, and the empty asm statement says so to the compiler)
    u32x4 r;
    r[0] = (uint32_t)base;
    r[1] = (uint32_t)(base >> 32) & 0xffffu;
    r[2] = bytes_in_range;
    r[3] = 0x00020000u;  // 32-bit data format, no swizzle (gfx9 raw buffer)
    asm volatile("" : "+s"(r));
    return r;
}
// (the same two with the LDS address given as a wave-uniform base plus a compile-time constant: the sum goes
// straight into m0, one instruction less than adding first and moving then)
template <int IMM>
__device__ __forceinline__ void global_to_lds_run_at(const void* base, uint32_t voff, uint32_t lds_base) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(base), "n"(IMM) : "m0", "scc");
}
template <int IMM>
__device__ __forceinline__ void buffer_to_lds_run_at(const u32x4 rsrc, uint32_t voff, uint32_t lds_base) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_base), "v"(voff), "s"(rsrc), "n"(IMM) : "m0", "scc");
}
__device__ __forceinline__ void buffer_to_lds_run(const u32x4 rsrc, uint32_t voff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds), "v"(voff), "s"(rsrc) : "m0");
}
#pragma clang diagnostic pop
template <int D, int ROWS, int NWAVES>
struct DirectStager {
    using TL = Tile<D>;
    static constexpr int SPR = TL::kChunks + 1;  // slots per row
    static constexpr int SLOTS = ROWS * SPR;
    static_assert(SLOTS % 64 == 0, "tile must be a whole number of wave runs");
    static constexpr int NL = SLOTS / 64;
    static constexpr int PER = (NL + NWAVES - 1) / NWAVES;
    // (source row << 16 | byte offset inside the row) of this lane for each of its runs: the same for
    // every tile of this shape, whatever its row stride
    uint32_t rc[PER];

    __device__ __forceinline__ static void slot(int t, int lane, int& row, int& chunk) {
        const int s = t * 64 + lane;
        const int rho = s / SPR;
        chunk = s - rho * SPR;
        if (chunk == TL::kChunks) chunk = 0;
        row = TL::prow(rho);  // prow is its own inverse
    }
    __device__ __forceinline__ void init(int w, int lane) {
#pragma unroll
        for (int p = 0; p < PER; ++p) {
            int row, chunk;
            slot(w + p * NWAVES, lane, row, chunk);
            rc[p] = (uint32_t)(row << 16 | chunk * 16);
        }
    }
    // number of runs wave w moves per tile
    __device__ __forceinline__ static int runs_of(int w) { return (NL - w + NWAVES - 1) / NWAVES; }
    __device__ __forceinline__ uint32_t offset(int p, uint32_t stride_bytes, int last_row) const {
        return (uint32_t)min((int)(rc[p] >> 16), last_row) * stride_bytes + (rc[p] & 0xffffu);
    }
    // run P of this wave for a whole tile (all ROWS rows valid), if P < limit (wave-uniform)
    template <int P, bool NT = false>
    __device__ __forceinline__ void issue_one(const __bf16* g, uint32_t tile_addr, int w, int limit, uint32_t stride_bytes) const {
        if constexpr (P < PER) {
            if (P < limit) {
                if constexpr (NT) global_to_lds_run_nt(g, (rc[P] >> 16) * stride_bytes + (rc[P] & 0xffffu), tile_addr + (w + P * NWAVES) * 1024);
                else global_to_lds_run(g, (rc[P] >> 16) * stride_bytes + (rc[P] & 0xffffu), tile_addr + (w + P * NWAVES) * 1024);
            }
        }
    }
    // the whole tile at once; rows at or beyond rows_valid re-read the last valid row
    template <bool NT = false>
    __device__ __forceinline__ void issue(const __bf16* g, lds_ptr tile, int w, int lane, int rows_valid,
                                          int64_t stride) const {
        const uint32_t sb = (uint32_t)(stride * 2);
        const int runs = runs_of(w);
#pragma unroll
        for (int p = 0; p < PER; ++p)
            if (p < runs) {
                if constexpr (NT) global_to_lds_run_nt(g, offset(p, sb, rows_valid - 1), lds_addr(tile) + (w + p * NWAVES) * 1024);
                else global_to_lds_run(g, offset(p, sb, rows_valid - 1), lds_addr(tile) + (w + p * NWAVES) * 1024);
            }
    }
};

// waits until this wave's outstanding global (and global->LDS) loads have landed
__device__ __forceinline__ void wait_vmem() { __builtin_amdgcn_s_waitcnt(0x0f70); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32, 64); }

}  // namespace ma

// Building blocks of the kernels that run 16-step blocks on the matrix cores (gfx950, wave64).
//
// Every 16x16 matrix lives in the accumulator layout of v_mfma_f32_16x16x4_f32 (4 VGPRs: lane l,
// register r holds element [4*(l/16) + r][l % 16]).  In that layout register r of a matrix is
// directly the B operand of the r-th MFMA of a product, and the A operand of the transposed
// matrix, so the primitive is  tn(X, Y, acc) = acc + X^T Y  with no data movement between products.
#pragma once
#include <hip/hip_runtime.h>

namespace fwp {

typedef float v4f __attribute__((ext_vector_type(4)));

// acc + X^T Y for 16x16 matrices in the accumulator layout
__device__ __forceinline__ v4f tn(v4f X, v4f Y, v4f acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(X[0], Y[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(X[1], Y[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(X[2], Y[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(X[3], Y[3], acc, 0, 0, 0);
    return acc;
}

constexpr int kBlk = 16;   // steps per block = MFMA tile edge
constexpr int kAuxHeader = 16;   // floats before the per-block matrices in the auxiliary buffer

// Position of this lane's four registers in the accumulator layout.
struct Geo16 {
    int g, c;
    bool up[4], lo[4], di[4];   // row < column, row > column, row == column for register r
    __device__ explicit Geo16(int lane) : g(lane / 16), c(lane % 16) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            up[r] = 4 * g + r < c;
            lo[r] = c < 4 * g + r;
            di[r] = 4 * g + r == c;
        }
    }
};

// The buffer-load intrinsics, declared by their LLVM names (the clang builtin for the 128-bit load
// comes out as a 32-bit load with this compiler).
typedef int v4i __attribute__((ext_vector_type(4)));
__device__ float llvm_raw_buffer_load_f32(v4i rsrc, int voffset, int soffset, int aux) __asm("llvm.amdgcn.raw.buffer.load.f32");
__device__ v4f llvm_raw_buffer_load_v4f32(v4i rsrc, int voffset, int soffset, int aux) __asm("llvm.amdgcn.raw.buffer.load.v4f32");
__device__ void llvm_raw_buffer_store_f32(float x, v4i rsrc, int voffset, int soffset, int aux) __asm("llvm.amdgcn.raw.buffer.store.f32");
__device__ void llvm_raw_buffer_store_v4f32(v4f x, v4i rsrc, int voffset, int soffset, int aux) __asm("llvm.amdgcn.raw.buffer.store.v4f32");

// Access to one sequence's rows of a tensor through a buffer resource: the address of a load or store
// is (descriptor base) + (32-bit byte offset per lane, VGPR) + (byte offset per block, SGPR) +
// (immediate), so moving on to the next block costs one scalar multiply and no vector address
// arithmetic.  All offsets stay below 2^31 (checked on the host).  The hardware checks the sum of
// the three offsets against the size: loads beyond it return 0 and stores beyond it are dropped,
// which is how the rows of a last, partial block of 16 steps are dealt with.
struct RowBuf {
    v4i rsrc;       // base address (48 bits, stride 0), size in bytes, 32-bit data format
    __device__ __forceinline__ RowBuf(const float *base, uint32_t bytes) {
        const uint64_t a = reinterpret_cast<uint64_t>(base);
        rsrc = v4i{(int)(uint32_t)a, (int)(uint32_t)((a >> 32) & 0xffff), (int)bytes, 0x00020000};
    }
    __device__ __forceinline__ float f(unsigned lane_bytes, unsigned block_bytes) const {
        return llvm_raw_buffer_load_f32(rsrc, (int)lane_bytes, (int)block_bytes, 0);
    }
    __device__ __forceinline__ v4f f4(unsigned lane_bytes, unsigned block_bytes) const {
        return llvm_raw_buffer_load_v4f32(rsrc, (int)lane_bytes, (int)block_bytes, 0);
    }
    __device__ __forceinline__ void st(float x, unsigned lane_bytes, unsigned block_bytes) const {
        llvm_raw_buffer_store_f32(x, rsrc, (int)lane_bytes, (int)block_bytes, 0);
    }
    // A 16-byte store takes the whole offset in the VGPR.  With the block offset in an SGPR the
    // compiler sees no hazard between the store and a vector instruction that overwrites the data
    // registers right behind it, and the hardware has one: the store then writes the new value for
    // some lanes (seen as zeros in the first dword of the last four lanes of each row, and only
    // with several waves per SIMD).  Without the SGPR the compiler leaves the wait state.
    __device__ __forceinline__ void st4(const v4f &x, unsigned lane_bytes, unsigned block_bytes) const {
        llvm_raw_buffer_store_v4f32(x, rsrc, (int)(lane_bytes + block_bytes), 0, 0);
    }
};

// Workgroup barrier that orders the LDS hand-over only.  __syncthreads() also waits for every
// global load and store of the wave, the prefetches of the coming blocks included.
// FWP_TIMING_WITHOUT_BARRIERS (measurement only, never the product's build): the waves keep every instruction
// and every LDS wait but do not wait for each other, which bounds what any hand-over protocol without a
// workgroup barrier could gain.  Results are wrong; no address depends on data, so such a build is safe to time.
__device__ __forceinline__ void lds_barrier() {
#ifdef FWP_TIMING_WITHOUT_BARRIERS
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#else
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#endif
}

__device__ __forceinline__ float4 as_float4(const v4f &x) { return make_float4(x[0], x[1], x[2], x[3]); }
__device__ __forceinline__ v4f from_float4(const float4 &x) { return v4f{x.x, x.y, x.z, x.w}; }

// A 16x16 matrix in LDS as the 64 lanes' register quadruples.  put() followed by get() hands a
// matrix over as it is; put_t() followed by get() hands over its transpose: lane (g, c) holds
// X[4g + r][c], which the reader of the transpose wants in lane (c / 4, 4g + r) as register c % 4.
// A transpose costs four scattered LDS writes instead of the four MFMAs of a product with the
// identity; each group of 16 lanes is followed by 16 bytes of padding, which spreads those
// writes over all banks.  Within one wave LDS operations execute in order, so a wave may read
// back what it has just written without a barrier.
struct LdsMat {
    float4 q[68];
    // where lane `l` keeps its quadruple
    __device__ __forceinline__ float4 &at(int l) { return q[l + l / 16]; }
    __device__ __forceinline__ const float4 &at(int l) const { return q[l + l / 16]; }
    __device__ __forceinline__ void put(int lane, const v4f &x) { at(lane) = as_float4(x); }
    __device__ __forceinline__ void put_t(const Geo16 &p, const v4f &x) {
        float *f = reinterpret_cast<float *>(q) + 68 * (p.c / 4) + 16 * p.g + p.c % 4;
#pragma unroll
        for (int r = 0; r < 4; r++) f[4 * r] = x[r];
    }
    __device__ __forceinline__ v4f get(int lane) const { return from_float4(at(lane)); }
};

// (I + At)^-1 for a strictly triangular 16x16 matrix given both as A and as its transpose At:
// (I - At)(I + At^2)(I + At^4)(I + At^8) with the transposes of the squares taken through LDS
// (`scratch`: two matrices owned by the calling wave), 6 products.
__device__ __forceinline__ v4f inv_unit_triangular_lds(v4f A, v4f At, v4f identity, LdsMat *scratch,
                                                       const Geo16 &p, int lane) {
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    v4f T = identity - At;
    const v4f A2 = tn(At, A, zero);
    scratch[0].put_t(p, A2);
    T = tn(A2, T, T);
    __builtin_amdgcn_wave_barrier();
    const v4f At2 = scratch[0].get(lane);
    const v4f A4 = tn(At2, A2, zero);
    scratch[1].put_t(p, A4);
    T = tn(A4, T, T);
    __builtin_amdgcn_wave_barrier();
    const v4f At4 = scratch[1].get(lane);
    const v4f A8 = tn(At4, A4, zero);
    return tn(A8, T, T);
}

// T = (I + A)^-1 for A = strict_lower(diag(b) G), G = K K^T, without multiplying it out on the matrix
// cores (six products per block): T (I + A) = I is solved by substitution, column by column from the
// right, T[c][j] = [c == j] - sum_{i > j} T[c][i] b_i G[i][j], 120 multiply-adds per row.  A wave
// does a group of four blocks at once: lane 16 jb + c computes row c of block jb, reading G and b
// from LDS (the 16 lanes of a block read the same address).
constexpr int kGrp = 4;     // blocks per group

// G per block of the group in the accumulator layout, 64 lanes + 4 of padding so that the four
// blocks' reads fall on different banks; b likewise
struct SolveLds {
    float4 gm[kGrp][68];
    float bl[kGrp][20];
    // by the whole wave, for block j of the group: G in the accumulator layout, bcol = b[t0 + c]
    __device__ __forceinline__ void put(int j, int lane, const Geo16 &p, const v4f &G, float bcol) {
        gm[j][lane] = as_float4(G);
        if (p.g == 0) bl[j][p.c] = bcol;
    }
};

// A lane's row of T and what it carries between the steps of the substitution.
struct SolveRow {
    float be[16], T[16], Wn[16];
    __device__ __forceinline__ void begin(const SolveLds &s, const Geo16 &p) {
#pragma unroll
        for (int a = 0; a < 4; a++) {
            const float4 b4 = *reinterpret_cast<const float4 *>(&s.bl[p.g][4 * a]);
            be[4 * a] = b4.x, be[4 * a + 1] = b4.y, be[4 * a + 2] = b4.z, be[4 * a + 3] = b4.w;
        }
    }
    // columns HI down to LO of the row (the columns above HI done before).  Column j needs the row's
    // entries i > j; only the newest of them, i = j + 1, has just been computed, so the terms i >= j + 2
    // are summed first, in two chains that do not wait for it, and the newest term is added last: the
    // dependent path through the row is two operations per column instead of a chain of up to fifteen.
    template <int HI, int LO>
    __device__ __forceinline__ void columns(const SolveLds &s, const Geo16 &p) {
        const float4 *gq = s.gm[p.g];
#pragma unroll
        for (int jj = HI; jj >= LO; jj--) {
            float far0 = p.c == jj ? 1.f : 0.f, far1 = 0.f, near = 0.f;
#pragma unroll
            for (int a = (jj + 1) / 4; a < 4; a++) {
                const float4 g4 = gq[16 * a + jj];          // G[4a .. 4a + 3][jj]
                const float gg[4] = {g4.x, g4.y, g4.z, g4.w};
#pragma unroll
                for (int x = 0; x < 4; x++) {
                    const int i = 4 * a + x;
                    if (i == jj + 1) near = gg[x];
                    else if (i > jj + 1 && (i & 1)) far1 = fmaf(Wn[i], gg[x], far1);
                    else if (i > jj + 1) far0 = fmaf(Wn[i], gg[x], far0);
                }
            }
            const float acc = jj < 15 ? fmaf(Wn[jj < 15 ? jj + 1 : 15], near, far0 + far1) : far0;
            T[jj] = acc;
            Wn[jj] = -(acc * be[jj]);
        }
    }
    // (I + A)^-T of the lane's block as the accumulator layout wants it: lane (g', c) then reads
    // register r = T[c][4g' + r]
    __device__ __forceinline__ void store(LdsMat &m, const Geo16 &p) const {
#pragma unroll
        for (int a = 0; a < 4; a++) m.at(16 * a + p.c) = make_float4(T[4 * a], T[4 * a + 1], T[4 * a + 2], T[4 * a + 3]);
    }
};

// v - v_old can be had from U = diag(beta)(v - v_old) by a division only where every beta of the
// block is large enough for its reciprocal to be finite and exact enough (rows past the end of the
// sequence read beta = 0; zeros and denormals may also come from the caller).
__device__ __forceinline__ bool betas_divide(const v4f &brow) {
    constexpr float kMin = 1e-30f;
    return __builtin_amdgcn_ballot_w64(!(fabsf(brow[0]) >= kMin) || !(fabsf(brow[1]) >= kMin) ||
                                       !(fabsf(brow[2]) >= kMin) || !(fabsf(brow[3]) >= kMin)) == 0;
}

// Index of the checkpoint chunk a block lies in: block / blocks_per_chunk as a multiplication
// (exact while block * blocks_per_chunk < 2^32), the remainder alongside.
struct ChunkOf {
    unsigned bpc, magic;
    __device__ explicit ChunkOf(int chunk) : bpc(chunk / kBlk), magic(0xFFFFFFFFu / bpc + 1) {}
    __device__ __forceinline__ unsigned operator()(unsigned block) const { return __umulhi(block, magic); }
    // is `block` the last one of its chunk?
    __device__ __forceinline__ bool closes(unsigned block) const {
        return (block + 1) - (*this)(block + 1) * bpc == 0;
    }
};

// The per-block loop of one wave: `step(e, raw)` for e = 0 .. n-1 with the data of the coming PF
// blocks in flight in a ring of registers, one workgroup barrier per block (none for kernels of one wave).  `load(raw, e)` is asked for
// e <= n - 1 only (past the end the last block is loaded again and not used).  Memory latency is
// several block times here, so one block ahead is not enough.
template <int PF, class Raw, bool BARRIER = true, class Load, class Step>
__device__ __forceinline__ void ring_loop(int n, Load load, Step step) {
    Raw ring[PF];
#pragma unroll
    for (int j = 0; j < PF; j++) load(ring[j], min(j, n - 1));
    int e = 0;
    for (; e + PF <= n; e += PF) {
#pragma unroll
        for (int j = 0; j < PF; j++) {
            step(e + j, ring[j]);
            load(ring[j], min(e + j + PF, n - 1));
            __builtin_amdgcn_sched_barrier(0);     // the loads are issued here, not next to their use
            if constexpr (BARRIER) lds_barrier();
        }
    }
#pragma unroll
    for (int j = 0; j < PF; j++) {
        if (e + j < n) {
            step(e + j, ring[j]);
            if constexpr (BARRIER) lds_barrier();
        }
    }
}

}  // namespace fwp

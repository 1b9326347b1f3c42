// Prompt-sized product of bfloat16 activations with Q4_0 weights on the matrix
// cores of gfx950: Y[M, N] = X[M, K] . W[N, K]^T, X and Y bfloat16, W in ggml
// Q4_0 blocks, float32 accumulation (Tensor.MatMulT with a half x and a
// block-quantized w, tensor/quant.go:45-48: x is cast to float32, multiplied,
// and the result rounded once to x's dtype).
//
// The arithmetic is exact up to the order of the float32 sums, not a product
// with weights rounded to 16 bits. A weight is (n - 8) * d with a 4-bit n and a
// binary16 d: up to 15 significant bits, more than bfloat16's 8. So each weight
// goes to the matrix cores as two bfloat16 numbers, hi = the upper 16 bits of
// w and lo = w - hi, which together are w exactly (lo has at most 7
// significant bits), and Y = X . hi^T + X . lo^T with every product exact in float32
// (8 x 8 bits). That doubles the MFMA count and leaves nothing per output to do
// on the vector unit inside the loop; the split itself is done once per weight
// while the tile is staged (convert, one FMA by the scale, round, subtract,
// round: about five vector instructions a weight, shared by all rows of X).
//
// A workgroup of four wavefronts computes a 64 or 128 x 128 tile of Y over
// steps of two Q4_0 blocks (64 of K): X rows and the two halves of the weights
// are staged through LDS (rows padded to 144 bytes, which makes the 128-bit
// fragment reads conflict-free). The loads that feed a step are what bounds
// this kernel if they are not coalesced (a wavefront load that touches 64
// cache lines costs 64 cycles of the L1's time), so eight lanes share the 128
// bytes a row of X contributes to a step. Loading, splitting and multiplying
// must overlap, and wavefronts that all do the same thing between the same
// barriers do not overlap anything (two workgroups on a compute unit fall into
// step with each other too). So the workgroup's eight wavefronts have two
// roles: four multiply (fragment reads and MFMAs only), four feed them (loads
// two steps ahead, the split on the vector unit, LDS stores into the other of
// two buffers). Each SIMD holds one of each, and the hardware interleaves
// them; one barrier a step hands a buffer over.
// v_mfma_f32_32x32x16_bf16 takes, per lane, eight consecutive k of row
// (lane % 32), the lane's half (lane / 32) choosing which eight of the sixteen;
// its result holds column (lane % 32) and rows 8 (i / 4) + 4 (lane / 32) + i % 4
// in register i.
//
// A second, approximate form (template argument HALF, chosen by the caller; never
// by default) rounds each weight once to binary16 and multiplies with
// v_mfma_f32_32x32x16_f16: one plane instead of two, and a nibble becomes a weight
// in three packed instructions per pair. A weight is then off by at most 2^-11 of
// itself (the results by about 2e-4 of their root mean square at K = 4096 and by
// 1e-3 of it at worst: at the edge of the 1e-3 asked of this product, which is why
// it is not the default); |d| above 8188 overflows. X is brought to binary16
// beforehand by a pass of its own that scales each row by a power of two, so that
// its largest element lands in [2^14, 2^15): bfloat16's 8 significant bits fit
// binary16's 11, so the conversion is exact for every element within 2^28 of the
// row's largest, whatever the row's range, and the results are scaled back
// (exactly) when they are written.
#include "device_util.h"
#include "half_rows.h"
#include "kernels.h"

namespace mimir {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kBN = 128;        // columns of Y (rows of W) per workgroup
constexpr int kKS = 64;         // K per step: two Q4_0 blocks
constexpr int kLd = kKS + 8;    // bfloat16 elements per LDS row

constexpr size_t stage_bytes(int BM, bool half = false) { return (size_t)(BM + (half ? 1 : 2) * kBN) * kLd * 2; }  // X, hi, lo (binary16: X, w)

// The barrier of the main loop. __syncthreads() also waits for every global load
// in flight (its fence covers all memory), which would stall each step for a
// full trip to memory and undo the prefetching; the loop only hands LDS
// buffers over, so it waits for LDS traffic alone.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Two floats to a packed pair of bfloat16, rounded to nearest even.
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    f32x2 f = {a, b};
    bf16x2 h = __builtin_convertvector(f, bf16x2);
    uint32_t u;
    __builtin_memcpy(&u, &h, 4);
    return u;
}

// MT 32-row tiles per multiplying wavefront: the workgroup's tile is (64 MT) x 128. HALF: X is binary16 (rows
// scaled, row m's results to be multiplied by row_scale[m]) and the weights are rounded to binary16.
template <int MT, bool OUT_F32, bool HALF>
__global__ __launch_bounds__(512) void qgemm_q4_0_kernel(const uint16_t* __restrict__ X, const uint8_t* __restrict__ W,
                                                            void* __restrict__ Yv, int M, int N, int K, int64_t x_row_stride,
                                                            int tiles_m, int ntiles, const float* __restrict__ row_scale) {
    constexpr int BM = 64 * MT;
    constexpr size_t kStage = stage_bytes(BM, HALF);
    constexpr int AV = BM * 8 / 256;      // 16-byte pieces of the X tile per thread (4 or 2): piece p is row p / 8, bytes 16 (p % 8)..
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const bool feeder = wave >= 4;          // wavefronts 4..7 stage, 0..3 multiply
    const int tid = threadIdx.x & 255;      // index within the role
    const int wm = (wave & 3) >> 1, wn = wave & 1, l32 = lane & 31, lh = lane >> 5;

    // Consecutive workgroup ids go round the chip's eight dies; give each die a
    // run of consecutive tiles, ordered so that the tiles a die works on at one
    // time share their rows of X: a row tile of X (BM x K bfloat16, 1 or 2 MB)
    // stays in the die's 4 MB L2 while the strips of W (0.3 MB each) stream
    // through, instead of all of X streaming in again for every strip.
    const int per = (ntiles + 7) >> 3;
    const int tile = ((int)blockIdx.x & 7) * per + ((int)blockIdx.x >> 3);
    if (tile >= ntiles) return;
    const int tiles_n = ntiles / tiles_m;
    const int m0 = (tile / tiles_n) * BM, n0 = (tile % tiles_n) * kBN;
    const int nb = K >> 5;
    const int64_t w_row_bytes = (int64_t)nb * 18;

    // what this thread stages: pieces tid, tid + 256, .. of the X tile, and one
    // block of one row of W (sixteen consecutive lanes take sixteen consecutive
    // rows, so that their 16-byte LDS stores spread over all banks)
    const uint16_t* a_src[AV];
    int a_dst[AV];
#pragma unroll
    for (int i = 0; i < AV; i++) {
        const int p = tid + 256 * i, row = p >> 3, chunk = p & 7;
        const int m = m0 + row < M ? m0 + row : M - 1;
        a_src[i] = X + (int64_t)m * x_row_stride + chunk * 8;
        a_dst[i] = row * kLd + chunk * 8;
    }
    const int w_col = tid & (kBN - 1), w_blk = tid >> 7;
    const int w_n = n0 + w_col < N ? n0 + w_col : N - 1;
    const uint8_t* w_src = W + (int64_t)w_n * w_row_bytes + w_blk * 18;

    const int nk = K / kKS;
    // W reaches the feeders in one of two ways. With 64- and 128-row tiles there
    // is room in LDS for a raw panel of four steps of W (144 bytes a row, two
    // buffers): nine lanes share a row's 144 bytes, so a wavefront load touches
    // about ten cache lines instead of 64, and each feeder then picks its block
    // out of LDS. With 256-row tiles every feeder loads its own 18 bytes.
    constexpr bool PANEL = MT <= 2 || HALF;  // one plane of weights leaves room for the panel beside 256-row tiles too
    constexpr int kPanelBytes = kBN * 144, kPanelPieces = kBN * 9;
    uint8_t* raw = smem + 2 * kStage;
    struct Fetched {  // what one step needs from memory
        u32x4 ra[AV], rq;
        uint16_t rd;
    };
    auto fetch = [&](int kb, Fetched& f) {
        kb = kb < nk ? kb : nk - 1;  // past the end: a valid step again, unused (no branch in the loop body)
#pragma unroll
        for (int i = 0; i < AV; i++) __builtin_memcpy(&f.ra[i], __builtin_assume_aligned(a_src[i] + (int64_t)kb * kKS, 16), 16);
        if (!PANEL) {
            const uint8_t* wp = w_src + (int64_t)kb * 36;
            f.rd = *(const uint16_t*)wp;
            f.rq = load_u32x4_unaligned(wp + 2);
        }
    };
    u32x4 pw[5];
    auto panel_fetch = [&](int q) {
        const int np = nk >> 2;
        q = q < np ? q : np - 1;
#pragma unroll
        for (int i = 0; i < 5; i++) {
            const int pid = tid + 256 * i;
            if (pid < kPanelPieces) {
                const int row = pid / 9, pc = pid % 9;
                const int n = n0 + row < N ? n0 + row : N - 1;
                __builtin_memcpy(&pw[i], __builtin_assume_aligned(W + (int64_t)n * w_row_bytes + (int64_t)q * 144 + pc * 16, 16), 16);
            }
        }
    };
    auto panel_store = [&](int q) {
#pragma unroll
        for (int i = 0; i < 5; i++) {
            const int pid = tid + 256 * i;
            if (pid < kPanelPieces) *(u32x4*)(raw + (q & 1) * kPanelBytes + (pid / 9) * 144 + (pid % 9) * 16) = pw[i];
        }
    };
    auto stage = [&](int buf, const Fetched& f, int step) {
        uint16_t* As = (uint16_t*)(smem + (size_t)buf * kStage);
        uint16_t* Bh = As + BM * kLd;
        uint16_t* Bl = Bh + kBN * kLd;
        const u32x4* ra = f.ra;
        u32x4 rq = f.rq;
        uint16_t rd = f.rd;
        if (PANEL) {  // this thread's block of the step, out of the raw panel
            const uint8_t* pb = raw + ((step >> 2) & 1) * kPanelBytes + w_col * 144 + ((step & 3) * 2 + w_blk) * 18;
            rd = *(const uint16_t*)pb;
            __builtin_memcpy(&rq, __builtin_assume_aligned(pb + 2, 2), 16);
        }
#pragma unroll
        for (int i = 0; i < AV; i++) *(u32x4*)(As + a_dst[i]) = ra[i];
        // byte j of the block's 16 holds element j (low nibble) and 16 + j (high
        // nibble). All of it in full-rate integer and float instructions: the
        // nibble goes into the mantissa of 2^23 (v_perm), minus 2^23 + 8 is n - 8,
        // times d is the weight, exactly; its upper 16 bits are a bfloat16 (hi,
        // truncated, not rounded: w - hi then has at most 7 significant bits and
        // its upper 16 bits are lo, exactly).
        if (HALF) {
            // the nibble into the mantissa of binary16's 1024 (v_perm, two at a time), minus 1032 is n - 8, times d
            // rounds once: the weight to the nearest binary16
            const _Float16 dh = __builtin_bit_cast(_Float16, rd);
            const f16x2 d2 = {dh, dh}, off = {(_Float16)1032.f, (_Float16)1032.f};
            u32x4 wq[4];
#pragma unroll
            for (int half = 0; half < 2; half++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t nib = (rq[i] >> (4 * half)) & 0x0f0f0f0fu;
                    const uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, nib, 0x04010400u);
                    const uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, nib, 0x04030402u);
                    const f16x2 w0 = (__builtin_bit_cast(f16x2, p0) - off) * d2;
                    const f16x2 w1 = (__builtin_bit_cast(f16x2, p1) - off) * d2;
                    wq[2 * half + (i >> 1)][2 * (i & 1)] = __builtin_bit_cast(uint32_t, w0);
                    wq[2 * half + (i >> 1)][2 * (i & 1) + 1] = __builtin_bit_cast(uint32_t, w1);
                }
            uint16_t* hrow = Bh + w_col * kLd + w_blk * 32;
#pragma unroll
            for (int v = 0; v < 4; v++) *(u32x4*)(hrow + 8 * v) = wq[v];
            return;
        }
        const float d = f16_bits_to_f32(rd);
        u32x4 hi[4], lo[4];  // elements 0..7, 8..15 (low nibbles), 16..23, 24..31 (high nibbles)
#pragma unroll
        for (int half = 0; half < 2; half++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t nib = (rq[i] >> (4 * half)) & 0x0f0f0f0fu;
                uint32_t wb[4], rb[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float t = __uint_as_float(__builtin_amdgcn_perm(0x4b000000u, nib, 0x070c0c00u | (uint32_t)j)) - 8388616.0f;
                    const float w = t * d;
                    wb[j] = __float_as_uint(w);
                    rb[j] = __float_as_uint(w - __uint_as_float(wb[j] & 0xffff0000u));
                }
                hi[2 * half + (i >> 1)][2 * (i & 1)] = __builtin_amdgcn_perm(wb[1], wb[0], 0x07060302u);
                hi[2 * half + (i >> 1)][2 * (i & 1) + 1] = __builtin_amdgcn_perm(wb[3], wb[2], 0x07060302u);
                lo[2 * half + (i >> 1)][2 * (i & 1)] = __builtin_amdgcn_perm(rb[1], rb[0], 0x07060302u);
                lo[2 * half + (i >> 1)][2 * (i & 1) + 1] = __builtin_amdgcn_perm(rb[3], rb[2], 0x07060302u);
            }
        uint16_t* hrow = Bh + w_col * kLd + w_blk * 32;
        uint16_t* lrow = Bl + w_col * kLd + w_blk * 32;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            *(u32x4*)(hrow + 8 * v) = hi[v];
            *(u32x4*)(lrow + 8 * v) = lo[v];
        }
    };

    f32x16 total[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int i = 0; i < 16; i++) total[mt][nt][i] = 0.f;

    // A step is four slices of 16 of K. The fragments of slice i + 1 are read from
    // LDS while the MFMAs of slice i run (two sets of fragment registers), so
    // that only the first slice's reads are waited for.
    auto compute = [&](int buf) {
        const uint16_t* As = (const uint16_t*)(smem + (size_t)buf * kStage);
        const uint16_t* Bh = As + BM * kLd;
        const uint16_t* Bl = Bh + kBN * kLd;
        bf16x8 a[2][MT], bh[2][2], bl[2][2];
        auto read_slice = [&](int set, int sl) {  // slice sl: block sl / 2, half sl % 2
            const int koff = (sl >> 1) * 32 + (sl & 1) * 16 + lh * 8;
            if (!HALF) {
#pragma unroll
                for (int nt = 0; nt < 2; nt++) bl[set][nt] = *(const bf16x8*)(Bl + (wn * 64 + nt * 32 + l32) * kLd + koff);
            }
#pragma unroll
            for (int mt = 0; mt < MT; mt++) a[set][mt] = *(const bf16x8*)(As + (wm * (32 * MT) + mt * 32 + l32) * kLd + koff);
#pragma unroll
            for (int nt = 0; nt < 2; nt++) bh[set][nt] = *(const bf16x8*)(Bh + (wn * 64 + nt * 32 + l32) * kLd + koff);
        };
        read_slice(0, 0);
#pragma unroll
        for (int sl = 0; sl < 4; sl++) {
            if (sl < 3) read_slice((sl + 1) & 1, sl + 1);
            if (HALF) {
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int nt = 0; nt < 2; nt++) {
                        const bf16x8 av = a[sl & 1][mt], bv = bh[sl & 1][nt];
                        total[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, av), __builtin_bit_cast(f16x8, bv),
                                                                               total[mt][nt], 0, 0, 0);
                    }
                continue;
            }
            // the tiles in turn for each operand pair, so that consecutive MFMAs are independent
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++)
                    total[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[sl & 1][mt], bl[sl & 1][nt], total[mt][nt], 0, 0, 0);
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++)
                    total[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[sl & 1][mt], bh[sl & 1][nt], total[mt][nt], 0, 0, 0);
        }
        // the order asked of the scheduler: slice 0's reads, then slice by slice the
        // next slice's reads ahead of this slice's MFMAs
        constexpr int kReads = MT + (HALF ? 2 : 4), kMfmas = (HALF ? 2 : 4) * MT;
        __builtin_amdgcn_sched_group_barrier(0x100, kReads, 0);
#pragma unroll
        for (int sl = 0; sl < 3; sl++) {
            __builtin_amdgcn_sched_group_barrier(0x100, kReads, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, kMfmas, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, kMfmas, 0);
    };

    // Buffer kb & 1 holds step kb. Within step kb the feeders fill the other
    // buffer with step kb + 1 while the multipliers read this one; the barrier
    // that ends the step says both are done.
    if (feeder) {
        // Loads run four steps ahead of their use (four sets of registers, and the
        // raw panel a panel ahead): under load a request takes longer than a step.
        Fetched f0, f1, f2, f3;
        if (PANEL) {
            panel_fetch(0);
            panel_store(0);
            panel_fetch(1);
        }
        fetch(0, f0);
        fetch(1, f1);
        fetch(2, f2);
        fetch(3, f3);
        lds_barrier();  // raw panel 0 is in place
        stage(0, f0, 0);
        lds_barrier();
        // each turn first requests the loads of three steps ahead (into the set of
        // registers the turn before consumed), so that the load unit works through
        // them while this wavefront does the arithmetic of the step it stages
        for (int kb = 0; kb < nk; kb += 4) {
            fetch(kb + 4, f0);
            stage(1, f1, kb + 1);  // step kb + 1 while step kb is multiplied
            lds_barrier();
            if (kb + 1 >= nk) break;
            fetch(kb + 5, f1);
            stage(0, f2, kb + 2);
            lds_barrier();
            if (kb + 2 >= nk) break;
            fetch(kb + 6, f2);
            if (PANEL) panel_store((kb >> 2) + 1);  // the next panel into the other raw buffer, a step before its first use
            if (PANEL) panel_fetch((kb >> 2) + 2);
            stage(1, f3, kb + 3);
            lds_barrier();
            if (kb + 3 >= nk) break;
            fetch(kb + 7, f3);
            stage(0, f0, kb + 4);
            lds_barrier();
        }
        return;
    }
    lds_barrier();
    lds_barrier();
    for (int kb = 0; kb < nk; kb++) {  // one body: the accumulators stay where they are from step to step
        compute(kb & 1);
        lds_barrier();
    }

    // One rounding to the output's dtype (f32ToBF16, backend/cpu/half.go:42-51). An MFMA leaves a lane one column of Y and
    // four consecutive rows per group of four registers: transposed within each quad of lanes (quad_transpose) a group is
    // one row and four consecutive columns a lane, stored with one 8-byte (bfloat16) or 16-byte (float32) store.
    const bool wide_ok = (N & 3) == 0 && ((uintptr_t)Yv & 15) == 0;
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int m = m0 + wm * (32 * MT) + mt * 32 + q * 8 + lh * 4 + (l32 & 3);
            float back = 1.f;
            if (HALF) back = m < M ? row_scale[m] : 0.f;
#pragma unroll
            for (int nt = 0; nt < 2; nt++) {
                float v[4] = {total[mt][nt][4 * q], total[mt][nt][4 * q + 1], total[mt][nt][4 * q + 2], total[mt][nt][4 * q + 3]};
                quad_transpose(v, l32);
                const int n = n0 + wn * 64 + nt * 32 + (l32 & ~3);
                if (m >= M || n >= N) continue;
                if (HALF) {
#pragma unroll
                    for (int k = 0; k < 4; k++) v[k] *= back;
                }
                if (wide_ok && n + 3 < N) {
                    if (OUT_F32) {
                        const f32x4 o = {v[0], v[1], v[2], v[3]};
                        *(f32x4*)((float*)Yv + (int64_t)m * N + n) = o;
                    } else {
                        const u32x2 o = {(uint32_t)f32_to_bf16_bits(v[0]) | (uint32_t)f32_to_bf16_bits(v[1]) << 16,
                                         (uint32_t)f32_to_bf16_bits(v[2]) | (uint32_t)f32_to_bf16_bits(v[3]) << 16};
                        *(u32x2*)((uint16_t*)Yv + (int64_t)m * N + n) = o;
                    }
                } else {
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        if (n + k >= N) continue;
                        if (OUT_F32) ((float*)Yv)[(int64_t)m * N + n + k] = v[k];
                        else ((uint16_t*)Yv)[(int64_t)m * N + n + k] = f32_to_bf16_bits(v[k]);
                    }
                }
            }
        }
}

__global__ __launch_bounds__(256) void bf16_rows_to_f32_kernel(const uint16_t* __restrict__ x, float* __restrict__ y, int64_t M, int64_t K,
                                                               int64_t x_row_stride) {
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < M * K; t += (int64_t)gridDim.x * 256)
        y[t] = bf16_bits_to_f32(x[(t / K) * x_row_stride + t % K]);
}

__global__ __launch_bounds__(256) void bf16_rows_to_f16_scaled_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                                      float* __restrict__ scale_back, int64_t K, int64_t x_row_stride) {
    bf16_row_to_f16_scaled(x, y, scale_back, K, x_row_stride, blockIdx.x);
}

__global__ __launch_bounds__(256) void f32_to_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ y, int64_t n) {
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < n; t += (int64_t)gridDim.x * 256) y[t] = f32_to_bf16_bits(x[t]);
}

}  // namespace

hipError_t bf16_rows_to_f32(const void* x, float* y, int64_t M, int64_t K, int64_t x_row_stride, hipStream_t st) {
    int64_t g = (M * K + 255) / 256;
    hipLaunchKernelGGL(bf16_rows_to_f32_kernel, dim3((unsigned)(g > 65536 ? 65536 : g)), dim3(256), 0, st, (const uint16_t*)x, y, M, K,
                       x_row_stride);
    return hipGetLastError();
}

hipError_t f32_to_bf16(const float* x, void* y, int64_t n, hipStream_t st) {
    int64_t g = (n + 255) / 256;
    hipLaunchKernelGGL(f32_to_bf16_kernel, dim3((unsigned)(g > 65536 ? 65536 : g)), dim3(256), 0, st, x, (uint16_t*)y, n);
    return hipGetLastError();
}

// Whether the matrix-core kernel takes this product: K in panels of 256, rows
// of X and of W aligned for 16-byte loads.
bool qgemm_q4_0_ok(const void* W, const void* X, int64_t M, int64_t N, int64_t K, int64_t x_row_stride) {
    return M > 0 && N > 0 && K > 0 && K % 256 == 0 && ((uintptr_t)X & 15) == 0 && x_row_stride % 8 == 0 && ((uintptr_t)W & 15) == 0 &&
           M <= (1 << 24) && N <= (1 << 24) && K <= (1 << 24);
}

// X [M, K] bfloat16 (rows x_row_stride elements apart), W [N, K] Q4_0 with
// finite scales, Y [M, N] bfloat16, or float32 if out_f32.
// With half_ws (qgemm_q4_0_half_ws_bytes(M, K) bytes, 16-byte aligned) the product takes its approximate form:
// X converted into half_ws first, weights rounded to binary16.
// With `panel` the workspace also holds W as a binary16 panel, and products for which qgemm_f16_panel_pays take the
// two launches of qgemm_f16_panel.hip (the same weights, bit for bit; the sums in another order).
static size_t half_x_bytes(int64_t M, int64_t K) { return ((size_t)M * K * 2 + 255) & ~(size_t)255; }
static size_t half_scale_bytes(int64_t M) { return ((size_t)M * 4 + 255) & ~(size_t)255; }
size_t qgemm_q4_0_half_ws_bytes(int64_t M, int64_t N, int64_t K, bool panel) {
    return half_x_bytes(M, K) + half_scale_bytes(M) + (panel && qgemm_f16_panel_pays(M, N, K) ? qgemm_f16_panel_bytes(N, K) : 0);
}

hipError_t qgemm_q4_0_bf16(const void* W, const void* X, void* Y, int64_t M, int64_t N, int64_t K, int64_t x_row_stride, bool out_f32,
                           void* half_ws, bool panel, hipStream_t st) {
    const bool half = half_ws != nullptr;
    const float* row_scale = nullptr;
    if (half) {
        float* sb = (float*)((uint8_t*)half_ws + half_x_bytes(M, K));
        if (panel && qgemm_f16_panel_pays(M, N, K))
            return qgemm_f16_panel(W, X, x_row_stride, half_ws, sb, Y, M, N, K, out_f32, (uint8_t*)half_ws + half_x_bytes(M, K) + half_scale_bytes(M), st);
        hipLaunchKernelGGL(bf16_rows_to_f16_scaled_kernel, dim3((unsigned)M), dim3(256), 0, st, (const uint16_t*)X, (uint16_t*)half_ws, sb, K,
                           x_row_stride);
        X = half_ws;
        x_row_stride = K;
        row_scale = sb;
    }
    // the tallest tiles that still give three quarters of the compute units work: a taller tile reads less from
    // LDS per MFMA (a wavefront multiplies 32 MT x 64 of it), which is worth more than the idle quarter (measured at
    // 512 x 14336 and 2048 x 4096: 224 and 256 tiles of 256 rows beat 448 and 512 tiles of 128 rows by a fifth)
    const int64_t tiles_n = (N + kBN - 1) / kBN;
    const int MT = ((M + 255) / 256) * tiles_n >= 192 ? 4 : ((M + 127) / 128) * tiles_n >= 192 ? 2 : 1;
    const int BM = 64 * MT;
    const int tiles_m = (int)((M + BM - 1) / BM);
    const int ntiles = (int)(tiles_m * tiles_n);
    dim3 grid((unsigned)(((ntiles + 7) / 8) * 8));
    const size_t lds = 2 * stage_bytes(BM, half) + (MT <= 2 || half ? 2 * kBN * 144 : 0);
    {  // more dynamic LDS than a kernel gets by default
        static std::atomic<bool> raised{false};  // threads may race here: both then set the same attribute
        if (!raised) {
            const int most = 160 * 1024;
            hipError_t e = hipSuccess;
#define QGEMM_RAISE(MT_, F32_)                                                                                                                  \
    if (e == hipSuccess) e = hipFuncSetAttribute((const void*)qgemm_q4_0_kernel<MT_, F32_, false>, hipFuncAttributeMaxDynamicSharedMemorySize, most); \
    if (e == hipSuccess) e = hipFuncSetAttribute((const void*)qgemm_q4_0_kernel<MT_, F32_, true>, hipFuncAttributeMaxDynamicSharedMemorySize, most)
            QGEMM_RAISE(1, true); QGEMM_RAISE(1, false); QGEMM_RAISE(2, true); QGEMM_RAISE(2, false); QGEMM_RAISE(4, true); QGEMM_RAISE(4, false);
#undef QGEMM_RAISE
            if (e != hipSuccess) return e;
            raised = true;
        }
    }
#define QGEMM_LAUNCH(MT_, F32_)                                                                                                              \
    do {                                                                                                                                     \
        if (half)                                                                                                                            \
            hipLaunchKernelGGL((qgemm_q4_0_kernel<MT_, F32_, true>), grid, dim3(512), lds, st, (const uint16_t*)X, (const uint8_t*)W, Y,     \
                               (int)M, (int)N, (int)K, x_row_stride, tiles_m, ntiles, row_scale);                                            \
        else                                                                                                                                 \
            hipLaunchKernelGGL((qgemm_q4_0_kernel<MT_, F32_, false>), grid, dim3(512), lds, st, (const uint16_t*)X, (const uint8_t*)W, Y,    \
                               (int)M, (int)N, (int)K, x_row_stride, tiles_m, ntiles, row_scale);                                            \
    } while (0)
    note_kernel("qgemm_q4_0_kernel<%d, %s, %s>", MT, out_f32 ? "true" : "false", half ? "true" : "false");
    if (MT == 4) {
        if (out_f32) QGEMM_LAUNCH(4, true); else QGEMM_LAUNCH(4, false);
    } else if (MT == 2) {
        if (out_f32) QGEMM_LAUNCH(2, true); else QGEMM_LAUNCH(2, false);
    } else {
        if (out_f32) QGEMM_LAUNCH(1, true); else QGEMM_LAUNCH(1, false);
    }
#undef QGEMM_LAUNCH
    return hipGetLastError();
}

}  // namespace mimir

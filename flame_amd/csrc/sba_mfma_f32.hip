// fp32 matrix-core kernels (head_dim 64 and 128): the same sweeps, carry tables and per-step arithmetic
// as the bf16 kernels, with every product on v_mfma_f32_32x32x2_f32.  The reference runs fp32
// inputs through its one tiled kernel as well (stickbreaking_attention/utils.py:8 ALLOW_TF32,
// sb_attn/sb_fwd.py:139-253); here fp32 stays fp32 end to end (the 1e-4 tolerance class), the
// backward has no atomics and is bit-reproducible.  These are correctness-first kernels: one
// variant for every grid size, tiles staged through registers, one workgroup barrier pair per
// step; the matrix pipe runs fp32 at 1/16 of its bf16 rate anyway.
//
// Geometry as in sba_mfma.h: a workgroup is 4 waves, wave w owns 32 query rows, a step covers
// 64 keys, score tiles are computed transposed (S^T = K Q^T), and MFMA row M of tile t holds key
//     key_local = 32*((M>>2)&1) + 16*t + 4*(M>>3) + (M&3)
// so that lane (n, h) has the 32 consecutive keys 32*h + idx of query n in registers
// (idx = 16*t + r): the product chains and prefix sums of sba_mfma.h apply unchanged.
// The 32x32x2 MFMA takes one float per lane for A (row = lane%32, k = lane/32) and for B
// (column = lane%32, k = lane/32).  The contraction index is spread so that a lane fetches four
// consecutive floats at a time: head-dim products use d = 8*j + 4*(lane/32) + i in MFMA 4*j + i;
// key products (P*V, dQ) use key 32*(lane/32) + idx in MFMA idx, which is exactly the register
// the weight of that key sits in.
#include "sba_mfma.h"

namespace sba {
namespace f32 {

constexpr int SK = 64 + 4;                 // row stride of a transposed [D][64 keys] tile and of the weight tiles
template <int D> constexpr int row_stride() { return D + 4; }     // row stride (floats) of a [rows][D] tile: conflict-free b128 reads down a column
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ inline f32x16 mfma32(float a, float b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
__device__ inline int key_of_row(int t, int M) { return 32 * ((M >> 2) & 1) + 16 * t + 4 * (M >> 3) + (M & 3); }

// rows row0 .. row0+R-1 of a [rows, D] fp32 tensor -> registers (zeros past `len`); 256 threads
template <int R, int D> struct TileRegs {
    static constexpr int SD = row_stride<D>();
    static constexpr int kPer = R * D / 4 / kThreads;         // float4 chunks per thread: 4 (R = 64) or 8 (R = 128)
    f32x4 v[kPer];
    __device__ inline void load(const TensorArg& t, int64_t base, int row0, int len) {
        const int tid = threadIdx.x;
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int c = tid + i * kThreads, row = c / (D / 4), col = 4 * (c % (D / 4));
            f32x4 x = {0.f, 0.f, 0.f, 0.f};
            if (row0 + row < len) x = *(const f32x4*)(t.ptr + 4 * (base + (int64_t)(row0 + row) * t.st + col));
            v[i] = x;
        }
    }
    __device__ inline void store_natural(float* tile) const {                 // tile[row][SD]
        const int tid = threadIdx.x;
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int c = tid + i * kThreads, row = c / (D / 4), col = 4 * (c % (D / 4));
            *(f32x4*)(tile + row * SD + col) = v[i];
        }
    }
    __device__ inline void store_transposed(float* tile) const {              // tile[d][SK], R = 64 rows
        const int tid = threadIdx.x;
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int c = tid + i * kThreads, row = c / (D / 4), col = 4 * (c % (D / 4));
#pragma unroll
            for (int e = 0; e < 4; ++e) tile[(col + e) * SK + row] = v[i][e];
        }
    }
};

// this lane's share of row `row` for the head-dim products: f[4*j + i] = x[row][8*j + 4*h + i] * s
template <int D>
__device__ inline void load_row_share(float (&f)[D / 2], const TensorArg& t, int64_t base, int row, int len, int h, float s) {
    const char* ptr = t.ptr + 4 * (base + (int64_t)row * t.st + 4 * h);
#pragma unroll
    for (int j = 0; j < D / 8; ++j) {
        f32x4 x = {0.f, 0.f, 0.f, 0.f};
        if (row < len) x = *(const f32x4*)(ptr + 32 * j);
#pragma unroll
        for (int i = 0; i < 4; ++i) f[4 * j + i] = x[i] * s;
    }
}

// x[16*t + r] = sum_d tile[key(t, row)][d] * f[d-share]: S^T (tile = K, f = scaled Q) or dP^T (tile = V, f = dO)
template <int D>
__device__ inline void head_dim_product(float (&x)[32], const float* tile, const float (&f)[D / 2], int lane) {
    constexpr int SD = row_stride<D>();
    const int m = lane & 31, h = lane >> 5;
#pragma unroll
    for (int t = 1; t >= 0; --t) {
        const float* row = tile + key_of_row(t, m) * SD + 4 * h;
        f32x16 acc = {0};
#pragma unroll
        for (int j = 0; j < D / 8; ++j) {
            const f32x4 a = *(const f32x4*)(row + 8 * j);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc = mfma32(a[i], f[4 * j + i], acc);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) x[16 * t + r] = acc[r];
    }
}

// acc[db] (rows d = 32*db + .., column = query) += sum_keys tileT[d][key] * w[key]: O^T += V^T P^T, dQ^T += K^T dZ^T
template <int D>
__device__ inline void key_product(f32x16 (&acc)[D / 32], const float* tileT, const float (&w)[32], int lane) {
    const int m = lane & 31, h = lane >> 5;
#pragma unroll
    for (int db = 0; db < D / 32; ++db) {
        const float* row = tileT + (32 * db + m) * SK + 32 * h;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const f32x4 a = *(const f32x4*)(row + 4 * j);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[db] = mfma32(a[i], w[4 * j + i], acc[db]);
        }
    }
}

// rows d = 32*db + 8*g + 4*h + 0..3 of an accumulator pair, column = this lane's query -> one [tokens, D] row
template <int D>
__device__ inline void store_query_row(const TensorArg& t, int64_t base, int row, int lane, const f32x16 (&acc)[D / 32], float s) {
    const int h = lane >> 5;
    char* ptr = t.ptr + 4 * (base + (int64_t)row * t.st + 4 * h);
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f32x4 x = {acc[db][4 * g] * s, acc[db][4 * g + 1] * s, acc[db][4 * g + 2] * s, acc[db][4 * g + 3] * s};
            *(f32x4*)(ptr + 4 * (32 * db + 8 * g)) = x;
        }
}

// ---------------------------------------------------------------- forward
template <int D, bool kCarryOnly>
__global__ __launch_bounds__(kThreads) void fwd_kernel(KParams p) {
    constexpr int SD = row_stride<D>();
    __shared__ __attribute__((aligned(16))) float ktile[64 * SD];
    __shared__ __attribute__((aligned(16))) float vT[D * SK];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 31, h = lane >> 5;
    const int head = blockIdx.x % p.n_heads;
    const Job job = decode_job(p, order_job(blockIdx.x / p.n_heads, p.n_jobs, false));
    const int strict = p.attend_current ? 0 : 1;
    const int m0 = job.rb * kRowBlock, q0w = m0 + 32 * wave, qi = q0w + n;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;

    float qf[D / 2];
    load_row_share<D>(qf, p.q, qbase, qi, job.len, h, p.scale2);
    f32x16 oacc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; ++db) oacc[db] = f32x16{0};
    float R = 1.0f;
    const int imax = min(m0 + kRowBlock - 1, job.len - 1);
    const int kmax = imax - strict;
    const int n_steps = kmax >= 0 ? kmax / kKeyBlock + 1 : 0;
    const int64_t tabq = tab_index(p, head, job, job.rb, 0) + 32 * wave + n;

    for (int step = n_steps - 1; step >= 0; --step) {
        const int key0 = step * kKeyBlock;
        TileRegs<64, D> kr, vr;
        kr.load(p.k, kbase, key0, job.len);
        if (!kCarryOnly) vr.load(p.v, vbase, key0, job.len);
        __syncthreads();                       // the previous step's tiles have been read
        kr.store_natural(ktile);
        if (!kCarryOnly) vr.store_transposed(vT);
        __syncthreads();
        if (key0 + strict > q0w + 31) continue;           // whole step right of this wave's last query (uniform per wave)
        if (p.save && h == 0 && qi < job.len) p.rtab[tabq + step * kRowBlock] = R;
        float x[32];
        head_dim_product<D>(x, ktile, qf, lane);
        if (key0 + 63 + strict > q0w) mask_step(x, key0 + 32 * h, qi, strict);
        float dummy[1];
        stick_weights<false>(x, dummy, R, lane);
        if (!kCarryOnly) key_product<D>(oacc, vT, x, lane);
    }
    if (qi < job.len && !kCarryOnly) {
        store_query_row<D>(p.o, (int64_t)job.seq * p.o.sb + (int64_t)head * p.o.sh + (int64_t)job.tok0 * p.o.st, qi, lane, oacc, 1.0f);
        if (h == 0) ((float*)p.rem.ptr)[(int64_t)job.seq * p.rem.sb + (int64_t)head * p.rem.sh + job.tok0 + qi] = R;
    }
}

// ---------------------------------------------------------------- backward pass 1: dQ + prefix table
template <int D>
__global__ __launch_bounds__(kThreads) void bwd_dq_kernel(KParams p) {
    constexpr int SD = row_stride<D>();
    __shared__ __attribute__((aligned(16))) float ktile[64 * SD];
    __shared__ __attribute__((aligned(16))) float vtile[64 * SD];
    __shared__ __attribute__((aligned(16))) float kT[D * SK];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 31, h = lane >> 5;
    const int head = blockIdx.x % p.n_heads;
    const Job job = decode_job(p, order_job(blockIdx.x / p.n_heads, p.n_jobs, false));
    const int strict = p.attend_current ? 0 : 1;
    const int m0 = job.rb * kRowBlock, q0w = m0 + 32 * wave, qi = q0w + n;
    const bool row_ok = qi < job.len;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;
    const int64_t dobase = (int64_t)job.seq * p.d_o.sb + (int64_t)head * p.d_o.sh + (int64_t)job.tok0 * p.d_o.st;

    float qf[D / 2], dof[D / 2];
    load_row_share<D>(qf, p.q, qbase, qi, job.len, h, p.scale2);
    load_row_share<D>(dof, p.d_o, dobase, qi, job.len, h, 1.0f);
    float dr = 0.f;
    if (row_ok && p.d_rem.ptr)
        dr = ((const float*)p.d_rem.ptr)[(int64_t)job.seq * p.d_rem.sb + (int64_t)head * p.d_rem.sh + job.tok0 + qi];
    f32x16 dqacc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; ++db) dqacc[db] = f32x16{0};
    float Gc = 0.f;
    const int imax = min(m0 + kRowBlock - 1, job.len - 1);
    const int kmax = imax - strict;
    const int n_steps = kmax >= 0 ? kmax / kKeyBlock + 1 : 0;
    const int64_t tix0 = tab_index(p, head, job, job.rb, 0) + 32 * wave + n;

    for (int step = 0; step < n_steps; ++step) {
        const int key0 = step * kKeyBlock;
        TileRegs<64, D> kr, vr;
        kr.load(p.k, kbase, key0, job.len);
        vr.load(p.v, vbase, key0, job.len);
        __syncthreads();
        kr.store_natural(ktile);
        kr.store_transposed(kT);
        vr.store_natural(vtile);
        __syncthreads();
        if (key0 + strict > q0w + 31) continue;
        float R = row_ok ? p.rtab[tix0 + step * kRowBlock] : 1.0f;
        float x[32], beta[32], dp[32];
        head_dim_product<D>(x, ktile, qf, lane);
        head_dim_product<D>(dp, vtile, dof, lane);
        if (key0 + 63 + strict > q0w) mask_step(x, key0 + 32 * h, qi, strict);
        stick_weights<true>(x, beta, R, lane);
        // the gradient of rem rides in the prefix as the constant d_rem * rem (see the bf16 dQ kernel)
        if (step == 0) Gc = dr * R;
        if (row_ok && h == 0) p.gtab[tix0 + step * kRowBlock] = Gc;
        logit_grads<true>(x, beta, dp, Gc, lane);
        key_product<D>(dqacc, kT, dp, lane);
    }
    // the scaled Q share carries scale * log2(e): dq = scale * dZ K
    if (row_ok)
        store_query_row<D>(p.dq, (int64_t)job.seq * p.dq.sb + (int64_t)head * p.dq.sh + (int64_t)job.tok0 * p.dq.st, qi, lane, dqacc, p.scale);
}

// ---------------------------------------------------------------- backward pass 2: dK, dV
// One workgroup per (64-key block, head); a step covers 128 queries.  Each wave turns its 32
// queries into weights and logit gradients (carries from the two tables); the workgroup shares
// them through an LDS tile [query][key] together with the step's Q and dO rows, and every wave
// reduces its [32 keys x 32 d] tiles of dV, then of dK (tile (wave&1, wave>>1), at head_dim 128
// also (wave&1, (wave>>1) + 2)).  At head_dim 128 the step's queries reach the reductions in two
// parts of 64 (waves 0-1, then waves 2-3 deposit their rows), which is what fits the LDS.
template <int D>
__global__ __launch_bounds__(kThreads) void bwd_dkv_kernel(KParams p) {
    constexpr int SD = row_stride<D>();
    constexpr int kParts = D / 64;             // 1 or 2
    constexpr int kPart = kRowBlock / kParts;  // queries per part
    constexpr int kMine = D / 64;              // output tiles per wave and tensor
    __shared__ __attribute__((aligned(16))) float ktile[64 * SD];
    __shared__ __attribute__((aligned(16))) float vtile[64 * SD];
    __shared__ __attribute__((aligned(16))) float qtile[kPart * SD];         // scaled Q rows of the part
    __shared__ __attribute__((aligned(16))) float dotile[kPart * SD];
    __shared__ __attribute__((aligned(16))) float ztile[kPart * SK];         // a, then dz: [query][key]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 31, h = lane >> 5;
    const int head = blockIdx.x % p.n_heads;
    const int slot = blockIdx.x / p.n_heads;   // two 64-key blocks per scheduled 128-row job
    const Job job = decode_key_job(p, slot >> 1);
    const int kb = 2 * job.rb + (slot & 1);
    const int key0 = kb * kKeyBlock;
    if (key0 >= job.len) return;               // uniform over the workgroup
    const int strict = p.attend_current ? 0 : 1;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;
    const int64_t dobase = (int64_t)job.seq * p.d_o.sb + (int64_t)head * p.d_o.sh + (int64_t)job.tok0 * p.d_o.st;
    {
        TileRegs<64, D> kr, vr;
        kr.load(p.k, kbase, key0, job.len);
        vr.load(p.v, vbase, key0, job.len);
        kr.store_natural(ktile);
        vr.store_natural(vtile);
    }
    __syncthreads();                           // K, V tiles visible
    const int kh = wave & 1, dbw = wave >> 1;  // this wave's output tiles: key half kh, d-blocks dbw + 2*j
    const int part_of_wave = 32 * wave / kPart, lrow = 32 * wave - part_of_wave * kPart + n;
    f32x16 dkacc[kMine], dvacc[kMine];
#pragma unroll
    for (int j = 0; j < kMine; ++j) { dkacc[j] = f32x16{0}; dvacc[j] = f32x16{0}; }
    const int n_qb = (job.len + kRowBlock - 1) / kRowBlock;
    for (int qb = job.rb; qb < n_qb; ++qb) {
        const int q0w = qb * kRowBlock + 32 * wave, qi = q0w + n;
        float qf[D / 2], dof[D / 2];
        load_row_share<D>(qf, p.q, qbase, qi, job.len, h, p.scale2);
        load_row_share<D>(dof, p.d_o, dobase, qi, job.len, h, 1.0f);
        float x[32], dp[32];
        const bool skip = key0 + strict > q0w + 31 || q0w >= job.len;
        if (!skip) {
            float R = 0.f, Gc = 0.f;           // rows past the end: zero carries make weights and gradients exactly zero
            if (qi < job.len) {
                const int64_t t = tab_index(p, head, job, qb, kb) + 32 * wave + n;
                R = p.rtab[t]; Gc = p.gtab[t];
            }
            float beta[32];
            head_dim_product<D>(x, ktile, qf, lane);
            head_dim_product<D>(dp, vtile, dof, lane);
            if (key0 + 63 + strict > q0w) mask_step(x, key0 + 32 * h, qi, strict);
            stick_weights<true>(x, beta, R, lane);
            logit_grads<true>(x, beta, dp, Gc, lane);
        } else {
#pragma unroll
            for (int idx = 0; idx < 32; ++idx) { x[idx] = 0.f; dp[idx] = 0.f; }
        }
#pragma unroll
        for (int part = 0; part < kParts; ++part) {
            const bool mine = part_of_wave == part;
            __syncthreads();                   // the previous reduction is done: the tiles are free
            if (mine) {
#pragma unroll
                for (int j = 0; j < D / 8; ++j) {
                    *(f32x4*)(qtile + lrow * SD + 8 * j + 4 * h) = f32x4{qf[4 * j], qf[4 * j + 1], qf[4 * j + 2], qf[4 * j + 3]};
                    *(f32x4*)(dotile + lrow * SD + 8 * j + 4 * h) = f32x4{dof[4 * j], dof[4 * j + 1], dof[4 * j + 2], dof[4 * j + 3]};
                }
#pragma unroll
                for (int c = 0; c < 8; ++c) *(f32x4*)(ztile + lrow * SK + 32 * h + 4 * c) = f32x4{x[4 * c], x[4 * c + 1], x[4 * c + 2], x[4 * c + 3]};
            }
            __syncthreads();
            // dV[key][d] += sum_q a[q][key] dO[q][d]
#pragma unroll
            for (int j = 0; j < kMine; ++j)
#pragma unroll 8
                for (int i = 0; i < kPart / 2; ++i)
                    dvacc[j] = mfma32(ztile[(2 * i + h) * SK + 32 * kh + n], dotile[(2 * i + h) * SD + 32 * (dbw + 2 * j) + n], dvacc[j]);
            __syncthreads();
            if (mine) {
#pragma unroll
                for (int c = 0; c < 8; ++c) *(f32x4*)(ztile + lrow * SK + 32 * h + 4 * c) = f32x4{dp[4 * c], dp[4 * c + 1], dp[4 * c + 2], dp[4 * c + 3]};
            }
            __syncthreads();
            // dK[key][d] += sum_q dz[q][key] Q[q][d]
#pragma unroll
            for (int j = 0; j < kMine; ++j)
#pragma unroll 8
                for (int i = 0; i < kPart / 2; ++i)
                    dkacc[j] = mfma32(ztile[(2 * i + h) * SK + 32 * kh + n], qtile[(2 * i + h) * SD + 32 * (dbw + 2 * j) + n], dkacc[j]);
        }
    }
    // accumulator rows are keys 32*kh + 8*(r/4) + 4*h + r%4, column d = 32*(dbw + 2j) + n.  The Q rows carried
    // scale * log2(e): dk = scale * dZ^T Q = (scale / scale2) * the sum.
    const float ks = p.scale / p.scale2;
    const int64_t dkbase = (int64_t)job.seq * p.dk.sb + (int64_t)head * p.dk.sh + (int64_t)job.tok0 * p.dk.st;
    const int64_t dvbase = (int64_t)job.seq * p.dv.sb + (int64_t)head * p.dv.sh + (int64_t)job.tok0 * p.dv.st;
#pragma unroll
    for (int j = 0; j < kMine; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = key0 + 32 * kh + 8 * (r >> 2) + 4 * h + (r & 3);
            if (key < job.len) {
                ((float*)p.dk.ptr)[dkbase + (int64_t)key * p.dk.st + 32 * (dbw + 2 * j) + n] = dkacc[j][r] * ks;
                ((float*)p.dv.ptr)[dvbase + (int64_t)key * p.dv.st + 32 * (dbw + 2 * j) + n] = dvacc[j][r];
            }
        }
}

}  // namespace f32
}  // namespace sba

int sba_launch_mfma_f32_fwd(const sba::KParams& kp, hipStream_t s) {
    using namespace sba;
    dim3 grid((unsigned)kp.n_jobs * kp.n_heads);
    if (kp.head_dim == 64) {
        if (kp.carry_only) hipLaunchKernelGGL((f32::fwd_kernel<64, true>), grid, dim3(kThreads), 0, s, kp);
        else hipLaunchKernelGGL((f32::fwd_kernel<64, false>), grid, dim3(kThreads), 0, s, kp);
    } else {
        if (kp.carry_only) hipLaunchKernelGGL((f32::fwd_kernel<128, true>), grid, dim3(kThreads), 0, s, kp);
        else hipLaunchKernelGGL((f32::fwd_kernel<128, false>), grid, dim3(kThreads), 0, s, kp);
    }
    return hipGetLastError() == hipSuccess ? SBA_OK : SBA_ERR_LAUNCH;
}

int sba_launch_mfma_f32_bwd(const sba::KParams& kp, int phases, hipStream_t s) {
    using namespace sba;
    if (!kp.rtab || !kp.gtab) return SBA_ERR_WORKSPACE;
    dim3 grid((unsigned)kp.n_jobs * kp.n_heads);
    if (kp.head_dim == 64) {
        if (phases != 2) hipLaunchKernelGGL((f32::bwd_dq_kernel<64>), grid, dim3(kThreads), 0, s, kp);
        if (phases != 1) hipLaunchKernelGGL((f32::bwd_dkv_kernel<64>), dim3(2 * grid.x), dim3(kThreads), 0, s, kp);
    } else {
        if (phases != 2) hipLaunchKernelGGL((f32::bwd_dq_kernel<128>), grid, dim3(kThreads), 0, s, kp);
        if (phases != 1) hipLaunchKernelGGL((f32::bwd_dkv_kernel<128>), dim3(2 * grid.x), dim3(kThreads), 0, s, kp);
    }
    return hipGetLastError() == hipSuccess ? SBA_OK : SBA_ERR_LAUNCH;
}

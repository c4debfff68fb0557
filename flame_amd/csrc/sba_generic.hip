// Generic stick-breaking attention kernels: any head_dim <= 256, fp32, bf16 or float16 storage,
// fp32 arithmetic on the vector ALUs (no matrix cores).  This is the fp32 path of the
// operator (the 1e-4 tolerance class) and the path for head dims the MFMA kernels do
// not cover.  One thread owns one query row; a workgroup owns a row-block of 128 queries
// and sweeps the keys right-to-left from the diagonal, 32 keys at a time through LDS.
//
// Mathematics (reference: sb_varlen/sb_varlen_fwd.py:26-78 forward tile,
// sb_varlen/sb_varlen_bwd.py:412-430 gradient algebra), in linear space:
//   e = exp(z), u = 1/(1+e) = 1-beta,  R_j = prod_{k>j} u_k,  A_ij = e*u*R_j,  rem = R_{-1}.
//   g_ij = A_ij (dO_i.v_j - drem_i),  dz_ik = g_ik - beta_ik * sum_{j<=k} g_ij.
// The backward makes two right-to-left sweeps per row: the first one sums g over the row,
// the second turns the running suffix sum into the prefix sum it needs.
#include "sba_common.h"

namespace sba {

constexpr int kGenThreads = kRowBlock;   // 128
constexpr int kGenChunk = 32;            // keys per LDS chunk
constexpr float kMaxLogitNat = 20.794415f;  // kMaxLogit2 * ln 2

template <typename T, int DP>
__device__ inline void load_rows_to_lds(float* dst, const TensorArg& t, int64_t base, int row0,
                                        int len, int D) {
    // dst[kGenChunk][DP]; rows row0..row0+31 of the sequence, zero beyond len / D.
    for (int idx = threadIdx.x; idx < kGenChunk * DP; idx += kGenThreads) {
        int r = idx / DP, d = idx % DP;
        int row = row0 + r;
        float v = 0.f;
        if (row < len && d < D) v = Elem<T>::load(t.ptr, base + (int64_t)row * t.st + d);
        dst[idx] = v;
    }
}

template <typename T, int DP>
__global__ __launch_bounds__(kGenThreads) void generic_fwd_kernel(KParams p) {
    __shared__ float Ks[kGenChunk * DP];
    __shared__ float Vs[kGenChunk * DP];
    const int head = blockIdx.x % p.n_heads;
    const Job job = decode_job(p, blockIdx.x / p.n_heads);
    const int D = p.head_dim;
    const int i = job.rb * kRowBlock + threadIdx.x;
    const bool active = i < job.len;
    const int strict = p.attend_current ? 0 : 1;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;

    float q[DP], acc[DP];
#pragma unroll
    for (int d = 0; d < DP; ++d) {
        q[d] = (active && d < D) ? Elem<T>::load(p.q.ptr, qbase + (int64_t)i * p.q.st + d) * p.scale : 0.f;
        acc[d] = 0.f;
    }
    float R = 1.f;
    const int imax = min(job.rb * kRowBlock + kRowBlock - 1, job.len - 1);
    const int kmax = imax - strict;
    for (int c = (kmax >= 0 ? kmax / kGenChunk : -1); c >= 0; --c) {
        __syncthreads();
        load_rows_to_lds<T, DP>(Ks, p.k, kbase, c * kGenChunk, job.len, D);
        load_rows_to_lds<T, DP>(Vs, p.v, vbase, c * kGenChunk, job.len, D);
        __syncthreads();
        for (int jj = kGenChunk - 1; jj >= 0; --jj) {
            const int j = c * kGenChunk + jj;
            float z = 0.f;
#pragma unroll
            for (int d = 0; d < DP; ++d) z = __builtin_fmaf(q[d], Ks[jj * DP + d], z);
            const bool valid = active && (j + strict <= i);
            if (valid) {
                float e = expf(fminf(z, kMaxLogitNat));
                float u = 1.0f / (1.0f + e);
                float pw = e * u * R;
                R *= u;
#pragma unroll
                for (int d = 0; d < DP; ++d) acc[d] = __builtin_fmaf(pw, Vs[jj * DP + d], acc[d]);
            }
        }
    }
    if (active) {
        const int64_t obase = (int64_t)job.seq * p.o.sb + (int64_t)head * p.o.sh + (int64_t)(job.tok0 + i) * p.o.st;
#pragma unroll
        for (int d = 0; d < DP; ++d)
            if (d < D) Elem<T>::store(p.o.ptr, obase + d, acc[d]);
        Elem<T>::store(p.rem.ptr, (int64_t)job.seq * p.rem.sb + (int64_t)head * p.rem.sh + job.tok0 + i, R);
    }
}

// The attention weights A_ij themselves, the reference's `return_attention` debug output (sb_attn/sb_fwd.py:141-172,
// sb_varlen/sb_varlen_fwd.py:195-201 and :409-446): fp32, dense [B, H, T, T], packed [H, sum T, sum T] (a document's
// block on the diagonal); entries of pairs that are not allowed are left as they are (the caller zero-fills, as the
// reference does).  The forward sweep of generic_fwd_kernel without V.
template <typename T, int DP>
__global__ __launch_bounds__(kGenThreads) void generic_weights_kernel(KParams p) {
    __shared__ float Ks[kGenChunk * DP];
    const int head = blockIdx.x % p.n_heads;
    const Job job = decode_job(p, blockIdx.x / p.n_heads);
    const int D = p.head_dim;
    const int i = job.rb * kRowBlock + threadIdx.x;
    const bool active = i < job.len;
    const int strict = p.attend_current ? 0 : 1;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    // row (token i) of this head's [tokens x tokens] matrix, first column of the sequence
    const int64_t side = p.cu_seqlens ? (int64_t)p.total_tokens : (int64_t)p.seq_len;
    const int64_t plane = p.cu_seqlens ? (int64_t)head : (int64_t)job.seq * p.n_heads + head;
    float* const wrow = p.weights + (plane * side + job.tok0 + i) * side + job.tok0;

    float q[DP];
#pragma unroll
    for (int d = 0; d < DP; ++d)
        q[d] = (active && d < D) ? Elem<T>::load(p.q.ptr, qbase + (int64_t)i * p.q.st + d) * p.scale : 0.f;
    float R = 1.f;
    const int imax = min(job.rb * kRowBlock + kRowBlock - 1, job.len - 1);
    const int kmax = imax - strict;
    for (int c = (kmax >= 0 ? kmax / kGenChunk : -1); c >= 0; --c) {
        __syncthreads();
        load_rows_to_lds<T, DP>(Ks, p.k, kbase, c * kGenChunk, job.len, D);
        __syncthreads();
        for (int jj = kGenChunk - 1; jj >= 0; --jj) {
            const int j = c * kGenChunk + jj;
            float z = 0.f;
#pragma unroll
            for (int d = 0; d < DP; ++d) z = __builtin_fmaf(q[d], Ks[jj * DP + d], z);
            if (active && (j + strict <= i)) {
                const float e = expf(fminf(z, kMaxLogitNat));
                const float u = 1.0f / (1.0f + e);
                wrow[j] = e * u * R;
                R *= u;
            }
        }
    }
}

// fp32 accumulators for dk and dv: [2][tab_tokens][H][DP] -> index helper
__device__ inline int64_t acc_index(const KParams& p, int which, int64_t tok, int head, int DP) {
    return (((int64_t)which * p.tab_tokens + tok) * p.n_heads + head) * DP;
}

__global__ void generic_zero_kernel(float* buf, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) buf[i] = 0.f;
}

template <typename T, int DP>
__global__ __launch_bounds__(kGenThreads) void generic_bwd_kernel(KParams p) {
    __shared__ float Ks[kGenChunk * DP];
    __shared__ float Vs[kGenChunk * DP];
    const int head = blockIdx.x % p.n_heads;
    const Job job = decode_job(p, blockIdx.x / p.n_heads);
    const int D = p.head_dim;
    const int i = job.rb * kRowBlock + threadIdx.x;
    const bool active = i < job.len;
    const int strict = p.attend_current ? 0 : 1;
    const int64_t qbase = (int64_t)job.seq * p.q.sb + (int64_t)head * p.q.sh + (int64_t)job.tok0 * p.q.st;
    const int64_t kbase = (int64_t)job.seq * p.k.sb + (int64_t)head * p.k.sh + (int64_t)job.tok0 * p.k.st;
    const int64_t vbase = (int64_t)job.seq * p.v.sb + (int64_t)head * p.v.sh + (int64_t)job.tok0 * p.v.st;
    const int64_t dobase = (int64_t)job.seq * p.d_o.sb + (int64_t)head * p.d_o.sh + (int64_t)job.tok0 * p.d_o.st;

    float q[DP], dO[DP], dq[DP];
#pragma unroll
    for (int d = 0; d < DP; ++d) {
        bool ok = active && d < D;
        q[d] = ok ? Elem<T>::load(p.q.ptr, qbase + (int64_t)i * p.q.st + d) : 0.f;
        dO[d] = ok ? Elem<T>::load(p.d_o.ptr, dobase + (int64_t)i * p.d_o.st + d) : 0.f;
        dq[d] = 0.f;
    }
    float dr = 0.f;
    if (active && p.d_rem.ptr)
        dr = Elem<T>::load(p.d_rem.ptr, (int64_t)job.seq * p.d_rem.sb + (int64_t)head * p.d_rem.sh + job.tok0 + i);

    const int imax = min(job.rb * kRowBlock + kRowBlock - 1, job.len - 1);
    const int kmax = imax - strict;
    const int cmax = (kmax >= 0 ? kmax / kGenChunk : -1);
    float delta = 0.f;    // sum_j g_ij
    for (int sweep = 0; sweep < 2; ++sweep) {
        float R = 1.f;
        float suffix = 0.f;   // sum_{j > k} g_ij while sweeping right-to-left
        for (int c = cmax; c >= 0; --c) {
            __syncthreads();
            load_rows_to_lds<T, DP>(Ks, p.k, kbase, c * kGenChunk, job.len, D);
            load_rows_to_lds<T, DP>(Vs, p.v, vbase, c * kGenChunk, job.len, D);
            __syncthreads();
            for (int jj = kGenChunk - 1; jj >= 0; --jj) {
                const int j = c * kGenChunk + jj;
                float z = 0.f, dp = 0.f;
#pragma unroll
                for (int d = 0; d < DP; ++d) {
                    z = __builtin_fmaf(q[d], Ks[jj * DP + d], z);
                    dp = __builtin_fmaf(dO[d], Vs[jj * DP + d], dp);
                }
                const bool valid = active && (j + strict <= i);
                float pw = 0.f, dz = 0.f;
                if (valid) {
                    float e = expf(fminf(z * p.scale, kMaxLogitNat));
                    float u = 1.0f / (1.0f + e);
                    float beta = e * u;
                    pw = beta * R;
                    R *= u;
                    float g = pw * (dp - dr);
                    if (sweep == 0) {
                        delta += g;
                    } else {
                        float G = delta - suffix;   // sum_{j' <= j} g
                        suffix += g;
                        dz = g - beta * G;
                    }
                }
                if (sweep == 1 && j < job.len) {
                    // the branch is uniform per wave (j, job.len are); invalid lanes add 0
                    const int64_t tok = tab_token(p, job, j);
                    float* dk32 = p.dkv32 + acc_index(p, 0, tok, head, DP);
                    float* dv32 = p.dkv32 + acc_index(p, 1, tok, head, DP);
#pragma unroll
                    for (int d = 0; d < DP; ++d) {
                        dq[d] = __builtin_fmaf(dz, Ks[jj * DP + d], dq[d]);
                        float a = dz * q[d], b = pw * dO[d];
                        // wave reduction, then one atomic per wave
                        for (int off = 32; off >= 1; off >>= 1) {
                            a += __shfl_xor(a, off);
                            b += __shfl_xor(b, off);
                        }
                        if ((threadIdx.x & 63) == 0) {
                            atomicAdd(dk32 + d, a);
                            atomicAdd(dv32 + d, b);
                        }
                    }
                }
            }
        }
    }
    if (active) {
        const int64_t dqb = (int64_t)job.seq * p.dq.sb + (int64_t)head * p.dq.sh + (int64_t)(job.tok0 + i) * p.dq.st;
#pragma unroll
        for (int d = 0; d < DP; ++d)
            if (d < D) Elem<T>::store(p.dq.ptr, dqb + d, dq[d] * p.scale);
    }
}

// dk = scale * dk32, dv = dv32, written with the caller's strides and dtype.
template <typename T, int DP>
__global__ void generic_finish_kernel(KParams p) {
    const int64_t n = p.tab_tokens * p.n_heads * (int64_t)p.head_dim;
    const int D = p.head_dim;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n;
         idx += (int64_t)gridDim.x * blockDim.x) {
        int d = idx % D;
        int head = (idx / D) % p.n_heads;
        int64_t tok = idx / ((int64_t)D * p.n_heads);
        int64_t seq = (p.cu_seqlens == nullptr) ? tok / p.seq_len : 0;
        int64_t t = (p.cu_seqlens == nullptr) ? tok % p.seq_len : tok;
        float a = p.dkv32[acc_index(p, 0, tok, head, DP) + d] * p.scale;
        float b = p.dkv32[acc_index(p, 1, tok, head, DP) + d];
        Elem<T>::store(p.dk.ptr, seq * p.dk.sb + (int64_t)head * p.dk.sh + t * p.dk.st + d, a);
        Elem<T>::store(p.dv.ptr, seq * p.dv.sb + (int64_t)head * p.dv.sh + t * p.dv.st + d, b);
    }
}

template <typename T, int DP>
static int launch_fwd(const KParams& kp, hipStream_t s) {
    dim3 grid((unsigned)kp.n_jobs * kp.n_heads);
    hipLaunchKernelGGL((generic_fwd_kernel<T, DP>), grid, dim3(kGenThreads), 0, s, kp);
    return hipGetLastError() == hipSuccess ? SBA_OK : SBA_ERR_LAUNCH;
}

template <typename T, int DP>
static int launch_bwd(const KParams& kp, hipStream_t s) {
    const int64_t n = 2 * kp.tab_tokens * kp.n_heads * (int64_t)DP;
    hipLaunchKernelGGL(generic_zero_kernel, dim3(1024), dim3(256), 0, s, kp.dkv32, n);
    dim3 grid((unsigned)kp.n_jobs * kp.n_heads);
    hipLaunchKernelGGL((generic_bwd_kernel<T, DP>), grid, dim3(kGenThreads), 0, s, kp);
    hipLaunchKernelGGL((generic_finish_kernel<T, DP>), dim3(1024), dim3(256), 0, s, kp);
    return hipGetLastError() == hipSuccess ? SBA_OK : SBA_ERR_LAUNCH;
}

}  // namespace sba

int sba_generic_padded_dim(int D) { return D <= 32 ? 32 : (D <= 64 ? 64 : (D <= 128 ? 128 : 256)); }

int sba_launch_generic_fwd(const sba::KParams& kp, int dtype, hipStream_t s) {
    using namespace sba;
    const int DP = sba_generic_padded_dim(kp.head_dim);
    if (dtype == SBA_DTYPE_F32) {
        if (DP == 32) return launch_fwd<float, 32>(kp, s);
        if (DP == 64) return launch_fwd<float, 64>(kp, s);
        if (DP == 128) return launch_fwd<float, 128>(kp, s);
        return launch_fwd<float, 256>(kp, s);
    }
    if (dtype == SBA_DTYPE_F16) {
        if (DP == 32) return launch_fwd<_Float16, 32>(kp, s);
        if (DP == 64) return launch_fwd<_Float16, 64>(kp, s);
        if (DP == 128) return launch_fwd<_Float16, 128>(kp, s);
        return launch_fwd<_Float16, 256>(kp, s);
    }
    if (DP == 32) return launch_fwd<uint16_t, 32>(kp, s);
    if (DP == 64) return launch_fwd<uint16_t, 64>(kp, s);
    if (DP == 128) return launch_fwd<uint16_t, 128>(kp, s);
    return launch_fwd<uint16_t, 256>(kp, s);
}

template <typename T> static int launch_weights(const sba::KParams& kp, int DP, hipStream_t s) {
    using namespace sba;
    dim3 grid((unsigned)kp.n_jobs * kp.n_heads);
    if (DP == 32) hipLaunchKernelGGL((generic_weights_kernel<T, 32>), grid, dim3(kGenThreads), 0, s, kp);
    else if (DP == 64) hipLaunchKernelGGL((generic_weights_kernel<T, 64>), grid, dim3(kGenThreads), 0, s, kp);
    else if (DP == 128) hipLaunchKernelGGL((generic_weights_kernel<T, 128>), grid, dim3(kGenThreads), 0, s, kp);
    else hipLaunchKernelGGL((generic_weights_kernel<T, 256>), grid, dim3(kGenThreads), 0, s, kp);
    return hipGetLastError() == hipSuccess ? SBA_OK : SBA_ERR_LAUNCH;
}

int sba_launch_generic_weights(const sba::KParams& kp, int dtype, hipStream_t s) {
    const int DP = sba_generic_padded_dim(kp.head_dim);
    if (dtype == SBA_DTYPE_F16) return launch_weights<_Float16>(kp, DP, s);
    return dtype == SBA_DTYPE_F32 ? launch_weights<float>(kp, DP, s) : launch_weights<uint16_t>(kp, DP, s);
}

int sba_launch_generic_bwd(const sba::KParams& kp, int dtype, hipStream_t s) {
    using namespace sba;
    const int DP = sba_generic_padded_dim(kp.head_dim);
    if (dtype == SBA_DTYPE_F32) {
        if (DP == 32) return launch_bwd<float, 32>(kp, s);
        if (DP == 64) return launch_bwd<float, 64>(kp, s);
        if (DP == 128) return launch_bwd<float, 128>(kp, s);
        return launch_bwd<float, 256>(kp, s);
    }
    if (dtype == SBA_DTYPE_F16) {
        if (DP == 32) return launch_bwd<_Float16, 32>(kp, s);
        if (DP == 64) return launch_bwd<_Float16, 64>(kp, s);
        if (DP == 128) return launch_bwd<_Float16, 128>(kp, s);
        return launch_bwd<_Float16, 256>(kp, s);
    }
    if (DP == 32) return launch_bwd<uint16_t, 32>(kp, s);
    if (DP == 64) return launch_bwd<uint16_t, 64>(kp, s);
    if (DP == 128) return launch_bwd<uint16_t, 128>(kp, s);
    return launch_bwd<uint16_t, 256>(kp, s);
}

// Matrix-memory recurrence (mLSTM) over a flat batch of portions and single tokens.
//
// Per head, with a query q and key k of dk channels and a value v of dv channels, a log input
// gate i and a log forget gate f (both softly capped), and a running maximum m that starts at 0:
//
//   m_t = max(f_t + m_{t-1}, i_t)
//   S_t = exp(f_t + m_{t-1} - m_t) S_{t-1} + exp(i_t - m_t) k_t v_t^T        [dk x dv]
//   n_t = exp(f_t + m_{t-1} - m_t) n_{t-1} + exp(i_t - m_t) k_t              [dk]
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
//
// n is one more column of S (the column of a value that is always 1), and n_t . q_t is that
// column's output: the kernels below carry dv + 1 columns and divide afterwards.  Everything
// here is float32: gates, maxima, decays, state and outputs; the element type only decides how
// the packed projections are read and the finished rows are stored.
//
// Three kernels a step:
//   gates   one wave per (request, head): i, f, the maxima m_t, and per token the logarithms
//           of the two decay factors (log keep = f_t + m_{t-1} - m_t, log take = i_t - m_t,
//           both <= 0).  Activations of 64 tokens are computed side by side, the max-plus
//           recurrence walks them in order.
//   scan    per (request, head, block of columns): the state update and S^T q token by token,
//           the tokens' rows staged through LDS sixteen at a time.
//   finish  per (token, head): the division, the head's unit root mean square, the weight over
//           all heads' channels and the sigmoid gate.
// State per request slot: S [slot, head, dk, dv], n [slot, head, dk], m [slot, head], float32,
// zero at the start of a request.
#include "common.h"

#define ML_TOKENS 16   // tokens staged per round of the scan
#define ML_DREG 32     // state rows a lane holds of its column

__device__ inline float soft_cap(float x, float cap) { return cap * tanhf(x / cap); }

__device__ inline float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// gate_pre [tokens, 2 * heads]: the input gates' pre-activations, then the forget gates'.
__global__ __launch_bounds__(RL_WAVE) void mlstm_gates_kernel(
    const float* __restrict__ gate_pre, const float* __restrict__ gate_bias,
    const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots, float* __restrict__ m_state,
    float* __restrict__ log_keep, float* __restrict__ log_take, float* __restrict__ m_tok, int heads,
    float cap) {
    const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
    const int slot = seq_slots[s];
    float m = m_state[(size_t)slot * heads + h];
    const float bi = gate_bias ? gate_bias[h] : 0.f;
    const float bf = gate_bias ? gate_bias[heads + h] : 0.f;
    for (int base = t0; base < t1; base += RL_WAVE) {
        const int t = base + lane;
        const bool valid = t < t1;
        float gi = 0.f, gf = 0.f;
        if (valid) {
            gi = soft_cap(gate_pre[(size_t)t * 2 * heads + h] + bi, cap);
            gf = log_sigmoid(soft_cap(gate_pre[(size_t)t * 2 * heads + heads + h] + bf, cap));
        }
        const int count = min(RL_WAVE, t1 - base);
        float before = 0.f, mine = 0.f;
        for (int u = 0; u < count; ++u) {
            const float fu = __shfl(gf, u, RL_WAVE);
            const float iu = __shfl(gi, u, RL_WAVE);
            const float m_new = fmaxf(fu + m, iu);
            if (lane == u) {
                before = m;
                mine = m_new;
            }
            m = m_new;
        }
        if (valid) {
            const size_t at = (size_t)t * heads + h;
            log_keep[at] = gf + before - mine;
            log_take[at] = gi - mine;
            m_tok[at] = mine;
        }
    }
    if (lane == 0) m_state[(size_t)slot * heads + h] = m;
}

// One wave per (request, head, block of columns).  A wave's 64 lanes are `slices` groups of
// `cols` = 64 / slices lanes: lane l holds, of column blockIdx.z * cols + l % cols, the state
// rows d = l / cols + r * slices (r < ML_DREG).  Column dv is the normaliser n.
// raw [tokens, heads, dv + 1]: S_t^T q_t (q scaled), the last entry n_t . q_t.
template <typename T>
__global__ __launch_bounds__(RL_WAVE) void mlstm_scan_kernel(
    const T* __restrict__ packed, int row_width, int q_col, int k_col, int v_col,
    const float* __restrict__ log_keep, const float* __restrict__ log_take,
    const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots, float* __restrict__ S_state,
    float* __restrict__ n_state, float* __restrict__ raw, int heads, int dk, int dv, int slices,
    float q_scale) {
    __shared__ float sq[ML_TOKENS][256];
    __shared__ float sk[ML_TOKENS][256];
    __shared__ float sv[ML_TOKENS][RL_WAVE];
    __shared__ float skeep[ML_TOKENS];
    __shared__ float stake[ML_TOKENS];
    const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int cols = RL_WAVE / slices;
    const int slice = lane / cols;
    const int j0 = blockIdx.z * cols;
    const int j = j0 + lane % cols;
    const bool live = j <= dv;
    const bool is_n = j == dv;
    const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
    const int slot = seq_slots[s];
    float* column = is_n ? n_state + ((size_t)slot * heads + h) * dk
                         : S_state + ((size_t)slot * heads + h) * dk * dv + j;
    const size_t stride = is_n ? 1 : dv;
    float S[ML_DREG];
#pragma unroll
    for (int r = 0; r < ML_DREG; ++r) {
        const int d = slice + r * slices;
        S[r] = (live && d < dk) ? column[(size_t)d * stride] : 0.f;
    }
    for (int base = t0; base < t1; base += ML_TOKENS) {
        const int count = min(ML_TOKENS, t1 - base);
        __syncthreads();
        for (int idx = lane; idx < count * dk; idx += RL_WAVE) {
            const int u = idx / dk, d = idx - u * dk;
            const T* row = packed + (size_t)(base + u) * row_width + (size_t)h * dk + d;
            sq[u][d] = to_float(row[q_col]);
            sk[u][d] = to_float(row[k_col]);
        }
        for (int idx = lane; idx < count * cols; idx += RL_WAVE) {
            const int u = idx / cols, c = idx - u * cols;
            const int jj = j0 + c;
            sv[u][c] = jj < dv ? to_float(packed[(size_t)(base + u) * row_width + v_col + (size_t)h * dv + jj])
                               : (jj == dv ? 1.f : 0.f);
        }
        if (lane < count) {
            skeep[lane] = expf(log_keep[(size_t)(base + lane) * heads + h]);
            stake[lane] = expf(log_take[(size_t)(base + lane) * heads + h]);
        }
        __syncthreads();
        for (int u = 0; u < count; ++u) {
            const float keep = skeep[u];
            const float tv = stake[u] * sv[u][lane % cols];
            float acc = 0.f;
#pragma unroll
            for (int r = 0; r < ML_DREG; ++r) {
                const int d = slice + r * slices;
                if (d < dk) {
                    S[r] = keep * S[r] + tv * sk[u][d];
                    acc += S[r] * sq[u][d];
                }
            }
            for (int off = cols; off < RL_WAVE; off <<= 1) acc += __shfl_xor(acc, off, RL_WAVE);
            if (slice == 0 && live) raw[((size_t)(base + u) * heads + h) * (dv + 1) + j] = acc * q_scale;
        }
    }
    if (live) {
#pragma unroll
        for (int r = 0; r < ML_DREG; ++r) {
            const int d = slice + r * slices;
            if (d < dk) column[(size_t)d * stride] = S[r];
        }
    }
}

// out[t, h * dv + j] = o_j / rms(o) * weight[h * dv + j] * sigmoid(gate[t, h * dv + j]) with
// o = raw[.., :dv] / (max(|raw[.., dv]|, exp(-m_t)) + 1e-6).  One wave per (token, head).
template <typename T>
__global__ __launch_bounds__(256) void mlstm_finish_kernel(
    const float* __restrict__ raw, const float* __restrict__ m_tok, const T* __restrict__ packed,
    int row_width, int g_col, const float* __restrict__ weight, T* __restrict__ out, int heads, int dv,
    float eps) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & (RL_WAVE - 1);
    const int h = blockIdx.y * (blockDim.x / RL_WAVE) + threadIdx.x / RL_WAVE;
    if (h >= heads) return;
    const float* r = raw + ((size_t)t * heads + h) * (dv + 1);
    const float den = fmaxf(fabsf(r[dv]), expf(-m_tok[(size_t)t * heads + h])) + 1e-6f;
    float ss = 0.f;
    for (int j = lane; j < dv; j += RL_WAVE) {
        const float o = r[j] / den;
        ss += o * o;
    }
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)dv + eps);
    const T* gate = packed + (size_t)t * row_width + g_col + (size_t)h * dv;
    T* dst = out + ((size_t)t * heads + h) * dv;
    for (int j = lane; j < dv; j += RL_WAVE) {
        const float g = to_float(gate[j]);
        dst[j] = from_float<T>(r[j] / den * inv * weight[(size_t)h * dv + j] / (1.f + expf(-g)));
    }
}

extern "C" int rl_mlstm_max_key_dim() { return 256; }

// slices of a column's state rows over lanes: the fewest that leave a lane ML_DREG rows
static int mlstm_slices(int dk) {
    int slices = 1;
    while (slices * ML_DREG < dk) slices *= 2;
    return slices;
}

extern "C" int rl_mlstm_gates(const float* gate_pre, const float* gate_bias, const int* cu_seqlens,
                              const int* seq_slots, float* m_state, float* log_keep, float* log_take,
                              float* m_tok, int num_seqs, int heads, float cap, hipStream_t stream) {
    if (num_seqs <= 0) return RL_OK;
    if (heads < 1 || heads > 65535 || !(cap > 0.f)) return RL_ERR_ARG;
    hipLaunchKernelGGL(mlstm_gates_kernel, dim3(num_seqs, heads), dim3(RL_WAVE), 0, stream, gate_pre,
                       gate_bias, cu_seqlens, seq_slots, m_state, log_keep, log_take, m_tok, heads, cap);
    return rl_launch_status();
}

extern "C" int rl_mlstm_scan(const void* packed, int row_width, int q_col, int k_col, int v_col,
                             const float* log_keep, const float* log_take, const int* cu_seqlens,
                             const int* seq_slots, float* S_state, float* n_state, float* raw,
                             int num_seqs, int heads, int dk, int dv, float q_scale, int act_type,
                             hipStream_t stream) {
    if (num_seqs <= 0) return RL_OK;
    if (heads < 1 || heads > 65535 || dk < 1 || dk > 256 || dv < 1) return RL_ERR_ARG;
    if (q_col < 0 || k_col < 0 || v_col < 0 || q_col + heads * dk > row_width ||
        k_col + heads * dk > row_width || v_col + heads * dv > row_width)
        return RL_ERR_ARG;
    const int slices = mlstm_slices(dk);
    const int cols = RL_WAVE / slices;
    const int blocks = (dv + 1 + cols - 1) / cols;
    if (blocks > 65535) return RL_ERR_ARG;
    dim3 grid(num_seqs, heads, blocks), block(RL_WAVE);
    if (act_type == RL_F32)
        hipLaunchKernelGGL(mlstm_scan_kernel<float>, grid, block, 0, stream, (const float*)packed, row_width,
                           q_col, k_col, v_col, log_keep, log_take, cu_seqlens, seq_slots, S_state, n_state,
                           raw, heads, dk, dv, slices, q_scale);
    else if (act_type == RL_BF16)
        hipLaunchKernelGGL(mlstm_scan_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)packed, row_width,
                           q_col, k_col, v_col, log_keep, log_take, cu_seqlens, seq_slots, S_state, n_state,
                           raw, heads, dk, dv, slices, q_scale);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}

extern "C" int rl_mlstm_finish(const float* raw, const float* m_tok, const void* packed, int row_width,
                               int g_col, const float* weight, void* out, int tokens, int heads, int dv,
                               float eps, int act_type, hipStream_t stream) {
    if (tokens <= 0) return RL_OK;
    if (heads < 1 || dv < 1 || g_col < 0 || g_col + heads * dv > row_width) return RL_ERR_ARG;
    const int head_groups = (heads + 3) / 4;
    if (head_groups > 65535) return RL_ERR_ARG;
    dim3 grid(tokens, head_groups), block(256);
    if (act_type == RL_F32)
        hipLaunchKernelGGL(mlstm_finish_kernel<float>, grid, block, 0, stream, raw, m_tok, (const float*)packed,
                           row_width, g_col, weight, (float*)out, heads, dv, eps);
    else if (act_type == RL_BF16)
        hipLaunchKernelGGL(mlstm_finish_kernel<bf16_t>, grid, block, 0, stream, raw, m_tok,
                           (const bf16_t*)packed, row_width, g_col, weight, (bf16_t*)out, heads, dv, eps);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}

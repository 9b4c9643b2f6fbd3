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

// --------------------------------------------------------------------------- //
// The same recurrence in chunks of 64 tokens, on the matrix cores' float32 instruction
// (v_mfma_f32_16x16x4_f32), for steps that bring portions of prompts.  With a_t = log keep and
// b_t = log take of the gates kernel, and A_t the sum of a over the chunk's tokens up to t:
//
//   entering state S_in; for a token t of the chunk
//   S_t^T q_t = exp(A_t) S_in^T q_t + sum_{s <= t} exp(A_t - A_s + b_s) (q_t . k_s) v_s
//   S_out     = exp(A_last) S_in + sum_s exp(A_last - A_s + b_s) k_s v_s^T
//
// Every exponent is <= 0.  Three kernels: `state` computes every chunk's own sum U_c in
// parallel; `carry` walks a request's chunks, S_c = exp(A_last,c) S_{c-1} + U_c, leaves in U_c's
// place the state that enters chunk c and in the slot the state after the last; `output`
// computes every chunk's rows in parallel.  n is carried beside S as the column of the value 1.
//
// chunks[c] = {request (index into seq_slots), first token (flat), tokens, -}.
// seq_chunks[i] = {first chunk, chunks} of request i.
// --------------------------------------------------------------------------- //
typedef float f32x4 __attribute__((ext_vector_type(4)));
#define MC_L 64      // tokens a chunk
#define MC_JB 128    // value channels a workgroup
#define MC_CT 8      // = MC_JB / 16
#define MC_SLAB 32   // query / key channels staged at a time by the output kernel

__device__ inline float wave_inclusive_sum(float v) {
    const int lane = threadIdx.x & (RL_WAVE - 1);
#pragma unroll
    for (int off = 1; off < RL_WAVE; off <<= 1) {
        const float up = __shfl_up(v, off, RL_WAVE);
        if (lane >= off) v += up;
    }
    return v;
}

// sA[s] = A_s (inclusive sums of log keep over the chunk's tokens), sB[s] = log take; entries
// beyond the chunk's tokens repeat the last sum and take nothing.  Called by every thread.
__device__ inline void chunk_gates(const float* __restrict__ log_keep, const float* __restrict__ log_take,
                                   int begin, int count, int heads, int h, float* sA, float* sB) {
    if (threadIdx.x < RL_WAVE) {
        const int u = threadIdx.x;
        const float a = u < count ? log_keep[(size_t)(begin + u) * heads + h] : 0.f;
        sA[u] = wave_inclusive_sum(a);
        sB[u] = u < count ? log_take[(size_t)(begin + u) * heads + h] : -INFINITY;
    }
    __syncthreads();
}

// U[c][h][d][j] = sum_s w_s k_s[d] v_s[j], Un[c][h][d] = sum_s w_s k_s[d], decay[c][h] = A_last.
// Wave w owns the rows d of the tiles w, w + 4, ... (RT of them), and all MC_CT column tiles.
template <typename T, int RT>
__global__ __launch_bounds__(256) void mlstm_chunk_state_kernel(
    const T* __restrict__ packed, int row_width, int k_col, int v_col, const float* __restrict__ log_keep,
    const float* __restrict__ log_take, const int* __restrict__ chunks, float* __restrict__ U,
    float* __restrict__ Un, float* __restrict__ decay, int heads, int dk, int dv) {
    __shared__ float sK[16][256 + 16];
    __shared__ float sA[MC_L], sB[MC_L], sW[MC_L];
    const int c = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * MC_JB;
    const int begin = chunks[4 * c + 1], count = chunks[4 * c + 2];
    const int lane = threadIdx.x & (RL_WAVE - 1), wave = threadIdx.x / RL_WAVE;
    const int l16 = lane & 15, g = lane >> 4;
    const int dk16 = (dk + 15) & ~15;
    chunk_gates(log_keep, log_take, begin, count, heads, h, sA, sB);
    const float a_last = sA[count - 1];
    if (threadIdx.x < MC_L) sW[threadIdx.x] = threadIdx.x < count ? expf(a_last - sA[threadIdx.x] + sB[threadIdx.x]) : 0.f;
    if (threadIdx.x == 0 && blockIdx.z == 0) decay[(size_t)c * heads + h] = a_last;
    f32x4 acc[RT][MC_CT];
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int ct = 0; ct < MC_CT; ++ct) acc[i][ct] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float un = 0.f;
    for (int base = 0; base < count; base += 16) {
        __syncthreads();  // sW is written; the last slab is read
        for (int idx = threadIdx.x; idx < 16 * dk16; idx += 256) {
            const int u = idx / dk16, d = idx - u * dk16;
            float v = 0.f;
            if (base + u < count && d < dk)
                v = sW[base + u] * to_float(packed[(size_t)(begin + base + u) * row_width + k_col + (size_t)h * dk + d]);
            sK[u][d] = v;
        }
        __syncthreads();
        if (blockIdx.z == 0 && (int)threadIdx.x < dk) {
#pragma unroll
            for (int u = 0; u < 16; ++u) un += sK[u][threadIdx.x];
        }
#pragma unroll
        for (int kk = 0; kk < 16; kk += 4) {
            const int u = kk + g;
            float a[RT];
#pragma unroll
            for (int i = 0; i < RT; ++i) {
                const int d0 = 16 * (wave + 4 * i);
                a[i] = d0 < dk16 ? sK[u][d0 + l16] : 0.f;
            }
            const bool live = base + u < count;
            const T* vrow = packed + (size_t)(begin + base + u) * row_width + v_col + (size_t)h * dv;
#pragma unroll
            for (int ct = 0; ct < MC_CT; ++ct) {
                const int j = j0 + 16 * ct + l16;
                const float b = (live && j < dv) ? to_float(vrow[j]) : 0.f;
#pragma unroll
                for (int i = 0; i < RT; ++i)
                    acc[i][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b, acc[i][ct], 0, 0, 0);
            }
        }
    }
    float* out = U + ((size_t)c * heads + h) * dk * dv;
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int ct = 0; ct < MC_CT; ++ct)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int d = 16 * (wave + 4 * i) + 4 * g + r, j = j0 + 16 * ct + l16;
                if (d < dk && j < dv) out[(size_t)d * dv + j] = acc[i][ct][r];
            }
    if (blockIdx.z == 0 && (int)threadIdx.x < dk) Un[((size_t)c * heads + h) * dk + threadIdx.x] = un;
}

// One thread per element of a head's state (dk * dv of S, then dk of n), walking the request's
// chunks: what enters chunk c takes U_c's place.
__global__ __launch_bounds__(256) void mlstm_chunk_carry_kernel(
    float* __restrict__ U, float* __restrict__ Un, const float* __restrict__ decay,
    const int* __restrict__ seq_chunks, const int* __restrict__ seq_slots, float* __restrict__ S_state,
    float* __restrict__ n_state, int heads, int dk, int dv) {
    const int i = blockIdx.z, h = blockIdx.y;
    const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t per = (size_t)dk * dv;
    if (e >= per + dk) return;
    const int c0 = seq_chunks[2 * i], nc = seq_chunks[2 * i + 1];
    const int slot = seq_slots[i];
    const bool is_n = e >= per;
    float* state = is_n ? n_state + ((size_t)slot * heads + h) * dk + (e - per)
                        : S_state + ((size_t)slot * heads + h) * per + e;
    float* buf = is_n ? Un + (size_t)h * dk + (e - per) : U + (size_t)h * per + e;
    const size_t stride = is_n ? (size_t)heads * dk : (size_t)heads * per;
    float s = *state;
    int c = 0;
    for (; c + 4 <= nc; c += 4) {
        float u[4], f[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            u[k] = buf[(size_t)(c0 + c + k) * stride];
            f[k] = expf(decay[(size_t)(c0 + c + k) * heads + h]);
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            buf[(size_t)(c0 + c + k) * stride] = s;
            s = f[k] * s + u[k];
        }
    }
    for (; c < nc; ++c) {
        const float u = buf[(size_t)(c0 + c) * stride];
        buf[(size_t)(c0 + c) * stride] = s;
        s = expf(decay[(size_t)(c0 + c) * heads + h]) * s + u;
    }
    *state = s;
}

// raw[t][h][j] = q_scale * (exp(A_t) S_in^T q_t + sum_{s<=t} w_ts (q_t . k_s) v_s)[j]; the entry
// dv of a row is the same with n_in and the value 1.  Wave w owns the rows 16 w .. 16 w + 15.
template <typename T>
__global__ __launch_bounds__(256) void mlstm_chunk_output_kernel(
    const T* __restrict__ packed, int row_width, int q_col, int k_col, int v_col,
    const float* __restrict__ log_keep, const float* __restrict__ log_take, const int* __restrict__ chunks,
    const float* __restrict__ U, const float* __restrict__ Un, float* __restrict__ raw, int heads, int dk,
    int dv, float q_scale) {
    __shared__ float sQ[MC_L][MC_SLAB + 2];
    __shared__ float sK[MC_L][MC_SLAB + 2];
    __shared__ float sP[MC_L][MC_L + 2];
    __shared__ float sA[MC_L], sB[MC_L], sE[MC_L], sRow[MC_L], sDot[MC_L];
    __shared__ float sN[256];
    const int c = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * MC_JB;
    const int begin = chunks[4 * c + 1], count = chunks[4 * c + 2];
    const int lane = threadIdx.x & (RL_WAVE - 1), wave = threadIdx.x / RL_WAVE;
    const int l16 = lane & 15, g = lane >> 4;
    const int dk4 = (dk + 3) & ~3;
    const bool first = blockIdx.z == 0;
    chunk_gates(log_keep, log_take, begin, count, heads, h, sA, sB);
    if (threadIdx.x < MC_L) sE[threadIdx.x] = expf(sA[threadIdx.x]);
    if (first && (int)threadIdx.x < dk) sN[threadIdx.x] = Un[((size_t)c * heads + h) * dk + threadIdx.x];

    auto stage = [&](int d0, bool keys) {
        for (int idx = threadIdx.x; idx < MC_L * MC_SLAB; idx += 256) {
            const int t = idx / MC_SLAB, dd = idx - t * MC_SLAB;
            float q = 0.f, k = 0.f;
            if (t < count && d0 + dd < dk) {
                const T* row = packed + (size_t)(begin + t) * row_width + (size_t)h * dk + d0 + dd;
                q = to_float(row[q_col]);
                if (keys) k = to_float(row[k_col]);
            }
            sQ[t][dd] = q;
            if (keys) sK[t][dd] = k;
        }
    };

    // ---- scores of the chunk's own tokens
    f32x4 p[4];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) p[ct] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float dot = 0.f;  // q_t . n_in, by the thread of row t
    for (int d0 = 0; d0 < dk4; d0 += MC_SLAB) {
        __syncthreads();
        stage(d0, true);
        __syncthreads();
        if (first && threadIdx.x < MC_L) {
            for (int dd = 0; dd < MC_SLAB && d0 + dd < dk; ++dd) dot += sQ[threadIdx.x][dd] * sN[d0 + dd];
        }
#pragma unroll
        for (int kk = 0; kk < MC_SLAB; kk += 4) {
            const float a = sQ[16 * wave + l16][kk + g];
#pragma unroll
            for (int ct = 0; ct < 4; ++ct)
                p[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, sK[16 * ct + l16][kk + g], p[ct], 0, 0, 0);
        }
    }
    // ---- decay weights, the causal mask, row sums (the normaliser's column)
    float rs[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int t = 16 * wave + 4 * g + r, s = 16 * ct + l16;
            const float w = (s <= t && t < count) ? expf(sA[t] - sA[s] + sB[s]) * p[ct][r] : 0.f;
            sP[t][s] = w;
            rs[r] += w;
        }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) rs[r] += __shfl_xor(rs[r], off, RL_WAVE);
        if (l16 == 0) sRow[16 * wave + 4 * g + r] = rs[r];
    }
    if (first && threadIdx.x < MC_L) sDot[threadIdx.x] = dot;
    __syncthreads();
    // ---- weights times values
    f32x4 acc[MC_CT];
#pragma unroll
    for (int ct = 0; ct < MC_CT; ++ct) acc[ct] = (f32x4){0.f, 0.f, 0.f, 0.f};
    for (int kk = 0; kk < count; kk += 4) {
        const float a = sP[16 * wave + l16][kk + g];
        const bool live = kk + g < count;
        const T* vrow = packed + (size_t)(begin + kk + g) * row_width + v_col + (size_t)h * dv;
#pragma unroll
        for (int ct = 0; ct < MC_CT; ++ct) {
            const int j = j0 + 16 * ct + l16;
            const float b = (live && j < dv) ? to_float(vrow[j]) : 0.f;
            acc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[ct], 0, 0, 0);
        }
    }
    // ---- the entering state: rows of q times exp(A_t)
    const float* Sin = U + ((size_t)c * heads + h) * dk * dv;
    const float e_row = sE[16 * wave + l16];
    for (int d0 = 0; d0 < dk4; d0 += MC_SLAB) {
        __syncthreads();
        stage(d0, false);
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < MC_SLAB; kk += 4) {
            const int d = d0 + kk + g;
            const float a = sQ[16 * wave + l16][kk + g] * e_row;
#pragma unroll
            for (int ct = 0; ct < MC_CT; ++ct) {
                const int j = j0 + 16 * ct + l16;
                const float b = (d < dk && j < dv) ? Sin[(size_t)d * dv + j] : 0.f;
                acc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[ct], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int ct = 0; ct < MC_CT; ++ct)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int t = 16 * wave + 4 * g + r, j = j0 + 16 * ct + l16;
            if (t < count && j < dv) raw[((size_t)(begin + t) * heads + h) * (dv + 1) + j] = acc[ct][r] * q_scale;
        }
    if (first && (int)threadIdx.x < count) {
        const int t = threadIdx.x;
        raw[((size_t)(begin + t) * heads + h) * (dv + 1) + dv] = (sRow[t] + sE[t] * sDot[t]) * q_scale;
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

// The chunked form of rl_mlstm_scan.  U [nchunks, heads, dk, dv], Un [nchunks, heads, dk] and
// decay [nchunks, heads] are scratch of the call.
extern "C" int rl_mlstm_chunked(const void* packed, int row_width, int q_col, int k_col, int v_col,
                                const float* log_keep, const float* log_take, const int* chunks, int nchunks,
                                const int* seq_chunks, const int* seq_slots, int num_seqs, float* U, float* Un,
                                float* decay, float* S_state, float* n_state, float* raw, int heads, int dk,
                                int dv, float q_scale, int act_type, hipStream_t stream) {
    if (nchunks <= 0 || num_seqs <= 0) return RL_OK;
    if (heads < 1 || heads > 65535 || num_seqs > 65535 || dk < 1 || dk > 256 || dv < 1) return RL_ERR_ARG;
    if (q_col < 0 || k_col < 0 || v_col < 0 || q_col + heads * dk > row_width ||
        k_col + heads * dk > row_width || v_col + heads * dv > row_width)
        return RL_ERR_ARG;
    const int jblocks = (dv + MC_JB - 1) / MC_JB;
    if (jblocks > 65535) return RL_ERR_ARG;
    const int row_tiles = ((dk + 15) / 16 + 3) / 4;  // tiles of 16 state rows a wave
    dim3 grid(nchunks, heads, jblocks), block(256);
#define ML_STATE(TT, RTV)                                                                                      \
    hipLaunchKernelGGL((mlstm_chunk_state_kernel<TT, RTV>), grid, block, 0, stream, (const TT*)packed, row_width, \
                       k_col, v_col, log_keep, log_take, chunks, U, Un, decay, heads, dk, dv)
#define ML_STATE_T(TT)          \
    if (row_tiles <= 1)         \
        ML_STATE(TT, 1);        \
    else if (row_tiles == 2)    \
        ML_STATE(TT, 2);        \
    else                        \
        ML_STATE(TT, 4)
    if (act_type == RL_F32) {
        ML_STATE_T(float);
    } else if (act_type == RL_BF16) {
        ML_STATE_T(bf16_t);
    } else {
        return RL_ERR_ARG;
    }
#undef ML_STATE_T
#undef ML_STATE
    const size_t elements = (size_t)dk * dv + dk;
    hipLaunchKernelGGL(mlstm_chunk_carry_kernel, dim3((unsigned)((elements + 255) / 256), heads, num_seqs), block, 0,
                       stream, U, Un, decay, seq_chunks, seq_slots, S_state, n_state, heads, dk, dv);
    if (act_type == RL_F32)
        hipLaunchKernelGGL(mlstm_chunk_output_kernel<float>, grid, block, 0, stream, (const float*)packed, row_width,
                           q_col, k_col, v_col, log_keep, log_take, chunks, U, Un, raw, heads, dk, dv, q_scale);
    else
        hipLaunchKernelGGL(mlstm_chunk_output_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)packed,
                           row_width, q_col, k_col, v_col, log_keep, log_take, chunks, U, Un, raw, heads, dk, dv,
                           q_scale);
    return rl_launch_status();
}

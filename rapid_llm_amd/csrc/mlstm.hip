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
// A step runs the gates kernel, one of three forms of the recurrence, and the finishing kernel:
//   gates   one workgroup per (request, head): i, f, the maxima m_t, and per token the
//           logarithms of the two decay factors (log keep = f_t + m_{t-1} - m_t, log take =
//           i_t - m_t, both <= 0 up to rounding).  Activations side by side, the max-plus
//           recurrence as a scan over the workgroup.
//   step    every request brings one token: per (token, head, 64 columns) the state is read,
//           updated and written back once, as a stream.
//   scan    short portions: per (request, head, block of columns) the state stays in registers
//           and the tokens' rows are staged through LDS sixteen at a time.
//   chunked portions of prompts: chunks of 64 tokens on the float32 matrix instruction, three
//           kernels (every chunk's own sum, the carry over a request's chunks, every chunk's
//           outputs); described where they stand.
//   finish  per (token, head): the division, the head's unit root mean square, the weight over
//           all heads' channels and the sigmoid gate.
// The gates' pre-activations come from gate_product (or from the few-row product of the core
// library) as float32.
// State per request slot: S [slot, head, dk, dv], n [slot, head, dk], m [slot, head], float32,
// zero at the start of a request.
#include "common.h"

// A (token, head) row of the unfinished outputs: dv numerators, then n . q, padded so that
// every row starts at a multiple of 16 bytes.
__host__ __device__ inline int raw_width(int dv) { return (dv + 4) & ~3; }

#define ML_TOKENS 16   // tokens staged at a time by the scan
#define ML_DREG 32     // state rows a lane holds of its column

template <typename T>
struct alignas(sizeof(T) * 4) Vec4 {
    T v[4];
};

__device__ inline float soft_cap(float x, float cap) { return cap * tanhf(x / cap); }

__device__ inline float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// gate_pre [tokens, 2 * heads]: the input gates' pre-activations, then the forget gates'.
// A token maps the maximum m to max(m + f, i).  Two tokens in a row map it to
// max(m + f1 + f2, max(i1 + f2, i2)): such pairs (F, G) are folded over a wave by an inclusive
// scan, the waves' totals over the workgroup through LDS, and every lane applies its pair to
// the maximum that entered.  A workgroup of W waves takes 64 W tokens at a time.
__global__ __launch_bounds__(1024) void mlstm_gates_kernel(
    const float* __restrict__ gate_pre, const float* __restrict__ gate_bias,
    const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots, float* __restrict__ m_state,
    float* __restrict__ log_keep, float* __restrict__ log_take, float* __restrict__ m_tok, int heads,
    float cap) {
    __shared__ float wF[16], wG[16];
    const int s = blockIdx.x, h = blockIdx.y;
    const int lane = threadIdx.x & (RL_WAVE - 1), wave = threadIdx.x / RL_WAVE;
    const int waves = blockDim.x / RL_WAVE;
    const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
    const int slot = seq_slots[s];
    float m = m_state[(size_t)slot * heads + h];  // the maximum that enters these tokens
    const float bi = gate_bias ? gate_bias[h] : 0.f;
    const float bf = gate_bias ? gate_bias[heads + h] : 0.f;
    for (int base = t0; base < t1; base += blockDim.x) {
        const int t = base + threadIdx.x;
        const bool valid = t < t1;
        float gi = 0.f, gf = 0.f;
        if (valid) {
            gi = soft_cap(gate_pre[(size_t)t * 2 * heads + h] + bi, cap);
            gf = log_sigmoid(soft_cap(gate_pre[(size_t)t * 2 * heads + heads + h] + bf, cap));
        }
        float F = valid ? gf : 0.f, G = valid ? gi : -INFINITY;
#pragma unroll
        for (int off = 1; off < RL_WAVE; off <<= 1) {
            const float Fu = __shfl_up(F, off, RL_WAVE);
            const float Gu = __shfl_up(G, off, RL_WAVE);
            if (lane >= off) {
                G = fmaxf(Gu + F, G);
                F = Fu + F;
            }
        }
        __syncthreads();  // the totals of the tokens before are still read
        if (lane == RL_WAVE - 1) {
            wF[wave] = F;
            wG[wave] = G;
        }
        __syncthreads();
        float m_in = m;  // what enters this wave's 64 tokens
        for (int w = 0; w < wave; ++w) m_in = fmaxf(m_in + wF[w], wG[w]);
        const float mine = fmaxf(m_in + F, G);
        const float up = __shfl_up(mine, 1, RL_WAVE);
        const float before = lane == 0 ? m_in : up;
        for (int w = 0; w < waves; ++w) m = fmaxf(m + wF[w], wG[w]);
        if (valid) {
            const size_t at = (size_t)t * heads + h;
            log_keep[at] = gf + before - mine;
            log_take[at] = gi - mine;
            m_tok[at] = mine;
        }
    }
    if (threadIdx.x == 0) m_state[(size_t)slot * heads + h] = m;
}

// One wave per (request, head, block of columns).  A wave's 64 lanes are `slices` groups of
// `cols` = 64 / slices lanes: lane l holds, of column blockIdx.z * cols + l % cols, the state
// rows d = l / cols + r * slices (r < ML_DREG).  Column dv is the normaliser n.
// raw [tokens, heads, raw_width(dv)]: S_t^T q_t (q scaled), entry dv of a row is n_t . q_t.
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
            if (slice == 0 && live) raw[((size_t)(base + u) * heads + h) * raw_width(dv) + j] = acc * q_scale;
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

// A step of single tokens: the state is read, updated and written back once, as a stream.
// One workgroup per (token, head, 64 columns): lane = column (64 consecutive floats of a state
// row are one 256-byte access), the four waves split the rows and their sums meet in LDS.
template <typename T>
__global__ __launch_bounds__(256) void mlstm_step_kernel(
    const T* __restrict__ packed, int row_width, int q_col, int k_col, int v_col,
    const float* __restrict__ log_keep, const float* __restrict__ log_take,
    const int* __restrict__ seq_slots, float* __restrict__ S_state, float* __restrict__ n_state,
    float* __restrict__ raw, int heads, int dk, int dv, float q_scale) {
    __shared__ float sq[256], sk[256];
    __shared__ float part[4][RL_WAVE];
    const int t = blockIdx.x, h = blockIdx.y;
    const int lane = threadIdx.x & (RL_WAVE - 1), wave = threadIdx.x / RL_WAVE;
    const int j = blockIdx.z * RL_WAVE + lane;
    const int slot = seq_slots[t];
    const T* row = packed + (size_t)t * row_width;
    if ((int)threadIdx.x < dk) {
        sq[threadIdx.x] = to_float(row[q_col + (size_t)h * dk + threadIdx.x]);
        sk[threadIdx.x] = to_float(row[k_col + (size_t)h * dk + threadIdx.x]);
    }
    const float keep = expf(log_keep[(size_t)t * heads + h]);
    const float take = expf(log_take[(size_t)t * heads + h]);
    __syncthreads();
    const bool live = j <= dv, is_n = j == dv;
    const float tv = take * (is_n ? 1.f : (j < dv ? to_float(row[v_col + (size_t)h * dv + j]) : 0.f));
    float* column = is_n ? n_state + ((size_t)slot * heads + h) * dk
                         : S_state + ((size_t)slot * heads + h) * dk * dv + j;
    const size_t stride = is_n ? 1 : dv;
    const int per = (dk + 3) / 4;
    const int d_lo = wave * per, d_hi = min(dk, d_lo + per);
    float acc = 0.f;
    if (live) {
        int d = d_lo;
        for (; d + 8 <= d_hi; d += 8) {
            float s[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) s[u] = column[(size_t)(d + u) * stride];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                s[u] = keep * s[u] + tv * sk[d + u];
                acc += s[u] * sq[d + u];
                column[(size_t)(d + u) * stride] = s[u];
            }
        }
        for (; d < d_hi; ++d) {
            const float v = keep * column[(size_t)d * stride] + tv * sk[d];
            acc += v * sq[d];
            column[(size_t)d * stride] = v;
        }
    }
    part[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && live)
        raw[((size_t)t * heads + h) * raw_width(dv) + j] =
            (part[0][lane] + part[1][lane] + part[2][lane] + part[3][lane]) * q_scale;
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
    const float* r = raw + ((size_t)t * heads + h) * raw_width(dv);
    const float den = fmaxf(fabsf(r[dv]), expf(-m_tok[(size_t)t * heads + h])) + 1e-6f;
    const T* gate = packed + (size_t)t * row_width + g_col + (size_t)h * dv;
    const float* w = weight + (size_t)h * dv;
    T* dst = out + ((size_t)t * heads + h) * dv;
    // four channels a lane where every row involved starts on a multiple of four elements
    if (dv % 4 == 0 && row_width % 4 == 0 && g_col % 4 == 0) {
        float ss = 0.f;
        for (int j = 4 * lane; j < dv; j += 4 * RL_WAVE) {
            const float4 o = *reinterpret_cast<const float4*>(r + j);
            const float a = o.x / den, b = o.y / den, c = o.z / den, d = o.w / den;
            ss += a * a + b * b + c * c + d * d;
        }
        ss = wave_sum(ss);
        const float inv = 1.f / sqrtf(ss / (float)dv + eps);
        for (int j = 4 * lane; j < dv; j += 4 * RL_WAVE) {
            const float4 o = *reinterpret_cast<const float4*>(r + j);
            const float4 wv = *reinterpret_cast<const float4*>(w + j);
            const Vec4<T> gv = *reinterpret_cast<const Vec4<T>*>(gate + j);
            const float ov[4] = {o.x, o.y, o.z, o.w}, ww[4] = {wv.x, wv.y, wv.z, wv.w};
            Vec4<T> y;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                y.v[k] = from_float<T>(ov[k] / den * inv * ww[k] / (1.f + expf(-to_float(gv.v[k]))));
            *reinterpret_cast<Vec4<T>*>(dst + j) = y;
        }
        return;
    }
    float ss = 0.f;
    for (int j = lane; j < dv; j += RL_WAVE) {
        const float o = r[j] / den;
        ss += o * o;
    }
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)dv + eps);
    for (int j = lane; j < dv; j += RL_WAVE) {
        const float g = to_float(gate[j]);
        dst[j] = from_float<T>(r[j] / den * inv * w[j] / (1.f + expf(-g)));
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
// Wave w owns the column tiles 2 w and 2 w + 1 and all RT row tiles of 16 state rows: a value
// is loaded by one wave only and meets every key row of the slab.
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
    f32x4 acc[RT][2];
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) acc[i][ct] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float un = 0.f;
    // thread d holds channel d of the keys of a slab's 16 tokens: sixteen loads asked for at
    // once, the next slab's while this one is multiplied
    // (no load stands behind a condition: addresses are clamped into the chunk and what lies
    // beyond it is dropped afterwards, so that the loads of a batch travel together)
    const int kd = threadIdx.x;
    const T* kcol = packed + (size_t)begin * row_width + k_col + (size_t)h * dk + min(kd, dk - 1);
    float kv[16];
    auto load_keys = [&](int base) {
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const float x = to_float(kcol[(size_t)min(base + u, count - 1) * row_width]);
            kv[u] = (kd < dk && base + u < count) ? x : 0.f;
        }
    };
    load_keys(0);
    for (int base = 0; base < count; base += 16) {
        __syncthreads();  // sW is written; the last slab is read
        if (kd < dk16) {
#pragma unroll
            for (int u = 0; u < 16; ++u) sK[u][kd] = sW[base + u] * kv[u];
        }
        __syncthreads();
        if (base + 16 < count) load_keys(base + 16);
        if (blockIdx.z == 0 && (int)threadIdx.x < dk) {
#pragma unroll
            for (int u = 0; u < 16; ++u) un += sK[u][threadIdx.x];
        }
#pragma unroll
        for (int kk = 0; kk < 16; kk += 4) {
            const int u = kk + g;
            const bool live = base + u < count;
            const T* vrow = packed + (size_t)(begin + min(base + u, count - 1)) * row_width + v_col + (size_t)h * dv;
            float b[2];
#pragma unroll
            for (int ct = 0; ct < 2; ++ct) {
                const int j = j0 + 16 * (2 * wave + ct) + l16;
                const float x = to_float(vrow[min(j, dv - 1)]);
                b[ct] = (live && j < dv) ? x : 0.f;
            }
#pragma unroll
            for (int i = 0; i < RT; ++i) {
                const float a = 16 * i < dk16 ? sK[u][16 * i + l16] : 0.f;
#pragma unroll
                for (int ct = 0; ct < 2; ++ct)
                    acc[i][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b[ct], acc[i][ct], 0, 0, 0);
            }
        }
    }
    float* out = U + ((size_t)c * heads + h) * dk * dv;
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int d = 16 * i + 4 * g + r, j = j0 + 16 * (2 * wave + ct) + l16;
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
    for (; c + 8 <= nc; c += 8) {
        float u[8], f[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            u[k] = buf[(size_t)(c0 + c + k) * stride];
            f[k] = expf(decay[(size_t)(c0 + c + k) * heads + h]);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
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
// dv of a row is the same with n_in and the value 1.  For the scores wave w owns the rows
// 16 w .. 16 w + 15; for the products with values and state it owns the column tiles 2 w and
// 2 w + 1 of all 64 rows, so that a value or a state element is loaded by one wave only.
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

    // thread (t0, dd) holds channel d0 + dd of the tokens t0, t0 + 8, ...: eight (or sixteen)
    // loads asked for at once
    const int sdd = threadIdx.x % MC_SLAB, st0 = threadIdx.x / MC_SLAB;
    float gq[8], gk[8];
    auto stage_load = [&](int d0, bool keys) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int t = st0 + 8 * i;
            const bool live = t < count && d0 + sdd < dk;
            const T* row = packed + (size_t)(begin + min(t, count - 1)) * row_width + (size_t)h * dk +
                           min(d0 + sdd, dk - 1);
            const float xq = to_float(row[q_col]);
            gq[i] = live ? xq : 0.f;
            if (keys) {
                const float xk = to_float(row[k_col]);
                gk[i] = live ? xk : 0.f;
            }
        }
    };
    auto stage_store = [&](bool keys) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            sQ[st0 + 8 * i][sdd] = gq[i];
            if (keys) sK[st0 + 8 * i][sdd] = gk[i];
        }
    };

    const int jw = j0 + 32 * wave + l16;  // this lane's column of the wave's first tile
    // ---- scores of the chunk's own tokens
    f32x4 p[4];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) p[ct] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float dot = 0.f;  // q_t . n_in, by the thread of row t
    stage_load(0, true);
    for (int d0 = 0; d0 < dk4; d0 += MC_SLAB) {
        __syncthreads();
        stage_store(true);
        __syncthreads();
        if (d0 + MC_SLAB < dk4) stage_load(d0 + MC_SLAB, true);  // the next slab travels meanwhile
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
    // the chunk's values of this wave's two column tiles and the first slab of the queries
    // again, asked for while the weights are made
    float bv[MC_L / 4][2];
#pragma unroll
    for (int kq = 0; kq < MC_L / 4; ++kq) {
        const int u = 4 * kq + g;
        const T* vrow = packed + (size_t)(begin + min(u, count - 1)) * row_width + v_col + (size_t)h * dv;
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) {
            const float x = to_float(vrow[min(jw + 16 * ct, dv - 1)]);
            bv[kq][ct] = (u < count && jw + 16 * ct < dv) ? x : 0.f;
        }
    }
    stage_load(0, false);
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
    f32x4 acc[4][2];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) acc[rt][ct] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kq = 0; kq < MC_L / 4; ++kq) {
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const float a = sP[16 * rt + l16][4 * kq + g];
#pragma unroll
            for (int ct = 0; ct < 2; ++ct)
                acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bv[kq][ct], acc[rt][ct], 0, 0, 0);
        }
    }
    // ---- the entering state: rows of q times exp(A_t)
    const float* Sin = U + ((size_t)c * heads + h) * dk * dv;
    float e_row[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) e_row[rt] = sE[16 * rt + l16];
    float bs[MC_SLAB / 4][2];  // a slab's rows of the entering state, asked for a slab ahead
    auto load_state = [&](int d0) {
#pragma unroll
        for (int kq = 0; kq < MC_SLAB / 4; ++kq) {
            const int d = d0 + 4 * kq + g;
#pragma unroll
            for (int ct = 0; ct < 2; ++ct) {
                const float x = Sin[(size_t)min(d, dk - 1) * dv + min(jw + 16 * ct, dv - 1)];
                bs[kq][ct] = (d < dk && jw + 16 * ct < dv) ? x : 0.f;
            }
        }
    };
    load_state(0);
    for (int d0 = 0; d0 < dk4; d0 += MC_SLAB) {
        __syncthreads();
        stage_store(false);
        __syncthreads();
        if (d0 + MC_SLAB < dk4) stage_load(d0 + MC_SLAB, false);
        float b[MC_SLAB / 4][2];
#pragma unroll
        for (int kq = 0; kq < MC_SLAB / 4; ++kq) {
            b[kq][0] = bs[kq][0];
            b[kq][1] = bs[kq][1];
        }
        if (d0 + MC_SLAB < dk4) load_state(d0 + MC_SLAB);
#pragma unroll
        for (int kq = 0; kq < MC_SLAB / 4; ++kq) {
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const float a = sQ[16 * rt + l16][4 * kq + g] * e_row[rt];
#pragma unroll
                for (int ct = 0; ct < 2; ++ct)
                    acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b[kq][ct], acc[rt][ct], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = 16 * rt + 4 * g + r, j = jw + 16 * ct;
                if (t < count && j < dv)
                    raw[((size_t)(begin + t) * heads + h) * raw_width(dv) + j] = acc[rt][ct][r] * q_scale;
            }
    if (first && (int)threadIdx.x < count) {
        const int t = threadIdx.x;
        raw[((size_t)(begin + t) * heads + h) * raw_width(dv) + dv] = (sRow[t] + sE[t] * sDot[t]) * q_scale;
    }
}

// The gates' projection: out[t][n] = sum_k x[t][k] w[n][k] in float32, for the few rows of w
// that a recurrence's gates have (two a head).  One workgroup per token: its 256 threads walk K
// four channels a thread at a time; sixteen outputs are accumulated side by side and folded over
// the workgroup at the end.  The weights (a few hundred KB) stay in the caches for every token.
template <typename T>
__global__ __launch_bounds__(256) void gate_product_kernel(const T* __restrict__ x, const float* __restrict__ w,
                                                           float* __restrict__ out, int tokens, int K, int N) {
    __shared__ float part[4][16];
    const int lane = threadIdx.x & (RL_WAVE - 1), wave = threadIdx.x / RL_WAVE;
    const int t = blockIdx.x;
    const T* row = x + (size_t)t * K;
    for (int n0 = 0; n0 < N; n0 += 16) {
        float acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
        if (K % 4 == 0) {  // whole groups of four channels: sixteen 16-byte loads at once
            for (int k = 4 * threadIdx.x; k < K; k += 4 * 256) {
                float xv[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) xv[j] = to_float(row[k + j]);
                float4 wv[16];
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    wv[i] = *reinterpret_cast<const float4*>(w + (size_t)min(n0 + i, N - 1) * K + k);
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    acc[i] += xv[0] * wv[i].x + xv[1] * wv[i].y + xv[2] * wv[i].z + xv[3] * wv[i].w;
            }
        } else {
            for (int k = threadIdx.x; k < K; k += 256) {
                const float xv = to_float(row[k]);
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[i] += xv * w[(size_t)min(n0 + i, N - 1) * K + k];
            }
        }
        __syncthreads();  // the sums of the columns before are still read
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float total = wave_sum(acc[i]);
            if (lane == 0) part[wave][i] = total;
        }
        __syncthreads();
        if (threadIdx.x < 16 && n0 + (int)threadIdx.x < N)
            out[(size_t)t * N + n0 + threadIdx.x] =
                part[0][threadIdx.x] + part[1][threadIdx.x] + part[2][threadIdx.x] + part[3][threadIdx.x];
    }
}

extern "C" int rl_gate_product(const void* x, const float* w, float* out, int tokens, int K, int N, int act_type,
                               hipStream_t stream) {
    if (tokens <= 0 || N <= 0) return RL_OK;
    if (K < 1) return RL_ERR_ARG;
    dim3 grid(tokens), block(256);
    if (act_type == RL_F32)
        hipLaunchKernelGGL(gate_product_kernel<float>, grid, block, 0, stream, (const float*)x, w, out, tokens, K, N);
    else if (act_type == RL_BF16)
        hipLaunchKernelGGL(gate_product_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)x, w, out, tokens, K, N);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}

// the largest key size the kernels take (the step and scan kernels stage a head's query and
// key in LDS, the chunk kernels hold up to sixteen tiles of state rows a wave)
extern "C" int rl_mlstm_max_key_dim() { return 256; }

// slices of a column's state rows over lanes: the fewest that leave a lane ML_DREG rows
static int mlstm_slices(int dk) {
    int slices = 1;
    while (slices * ML_DREG < dk) slices *= 2;
    return slices;
}

extern "C" int rl_mlstm_gates(const float* gate_pre, const float* gate_bias, const int* cu_seqlens,
                              const int* seq_slots, float* m_state, float* log_keep, float* log_take,
                              float* m_tok, int num_seqs, int heads, float cap, int longest,
                              hipStream_t stream) {
    if (num_seqs <= 0) return RL_OK;
    if (heads < 1 || heads > 65535 || !(cap > 0.f)) return RL_ERR_ARG;
    // as many waves as the longest request of the step has blocks of 64 tokens, up to 16
    int waves = (longest + RL_WAVE - 1) / RL_WAVE;
    waves = waves < 1 ? 1 : (waves > 16 ? 16 : waves);
    hipLaunchKernelGGL(mlstm_gates_kernel, dim3(num_seqs, heads), dim3(waves * RL_WAVE), 0, stream, gate_pre,
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
    const int row_tiles = (dk + 15) / 16;  // tiles of 16 state rows
    dim3 grid(nchunks, heads, jblocks), block(256);
#define ML_STATE(TT, RTV)                                                                                      \
    hipLaunchKernelGGL((mlstm_chunk_state_kernel<TT, RTV>), grid, block, 0, stream, (const TT*)packed, row_width, \
                       k_col, v_col, log_keep, log_take, chunks, U, Un, decay, heads, dk, dv)
#define ML_STATE_T(TT)          \
    if (row_tiles <= 2)         \
        ML_STATE(TT, 2);        \
    else if (row_tiles <= 4)    \
        ML_STATE(TT, 4);        \
    else if (row_tiles <= 8)    \
        ML_STATE(TT, 8);        \
    else                        \
        ML_STATE(TT, 16)
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

// rl_mlstm_scan for a step in which every request brings one token (request i = token i).
extern "C" int rl_mlstm_step(const void* packed, int row_width, int q_col, int k_col, int v_col,
                             const float* log_keep, const float* log_take, const int* seq_slots,
                             float* S_state, float* n_state, float* raw, int tokens, int heads, int dk,
                             int dv, float q_scale, int act_type, hipStream_t stream) {
    if (tokens <= 0) return RL_OK;
    if (heads < 1 || heads > 65535 || dk < 1 || dk > 256 || dv < 1) return RL_ERR_ARG;
    if (q_col < 0 || k_col < 0 || v_col < 0 || q_col + heads * dk > row_width ||
        k_col + heads * dk > row_width || v_col + heads * dv > row_width)
        return RL_ERR_ARG;
    const int blocks = (dv + 1 + RL_WAVE - 1) / RL_WAVE;
    if (blocks > 65535) return RL_ERR_ARG;
    dim3 grid(tokens, heads, blocks), block(256);
    if (act_type == RL_F32)
        hipLaunchKernelGGL(mlstm_step_kernel<float>, grid, block, 0, stream, (const float*)packed, row_width,
                           q_col, k_col, v_col, log_keep, log_take, seq_slots, S_state, n_state, raw, heads, dk,
                           dv, q_scale);
    else if (act_type == RL_BF16)
        hipLaunchKernelGGL(mlstm_step_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)packed, row_width,
                           q_col, k_col, v_col, log_keep, log_take, seq_slots, S_state, n_state, raw, heads, dk,
                           dv, q_scale);
    else
        return RL_ERR_ARG;
    return rl_launch_status();
}

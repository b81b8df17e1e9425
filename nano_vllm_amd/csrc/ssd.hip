// A selective state-space layer with a scalar decay per head and token, after its input projection.
//
// The projection's row is [z | x B C | dt]: z and x of H * P channels (H heads of P), B and C of G * N
// (G groups, N state rows; head h reads group h / (H / G)), dt of H.  Per request the layer keeps, in
// the request's slot, S [H, N, P] and the last K - 1 inputs of the convolution [C, K - 1] (C = H * P +
// 2 G N channels), both float, taken as zero where the request starts (seq_starts == 0).
//
//   conv      u_t[c] = silu(b[c] + sum_j w[c][j] * in_(t - (K - 1) + j)[c])          over x, B and C; in before the
//                                                                                    request's start is zero
//   step      dt_t[h] = softplus(dt_raw + dt_bias[h]);  a_t[h] = exp(-exp(A_log[h]) * dt_t[h])
//   state     S_t = a_t S_(t-1) + dt_t B_t x_t^T;  y_t = S_t^T C_t + D[h] x_t
//   finish    y <- y * silu(z), then y / sqrt(mean(y^2) + eps) * w in norm_groups equal parts of the H * P channels
//
// The convolution's sums and silu are float and rounded once to the element type; everything after
// (step sizes, decays, the state, the read-out, gate and norm) is float with the accurate exponential
// and logarithm in both builds, rounded once at the output.
//
// Kernels: conv (a thread per token and channel, or eight tokens in a row; it also leaves B and C as floats
// and every head's step size and decay; a request that brings one token shifts its kept inputs there),
// conv_state (the kept inputs of requests that bring a portion), single (requests that bring one token),
// scan (portions), chain and inter (blocks), finish.  The scan gives every thread one column of S (up to 64 of
// its rows, in registers: a state of more rows is shared out over 2 or 4 lanes, whose sums meet by shuffles);
// B, C and x of 16 tokens at a time are staged in LDS for the wave.  A long portion is cut into blocks that
// run side by side, each from a zero state (the first from the request's); a pass over the blocks makes
// every block's true state at its end, E_b = exp(sum of the block's log-decays) E_(b-1) + U_b, and a
// second pass, a float product on the matrix cores, adds what the state before a block contributes,
// exp(log-decay up to t) E_(b-1)^T C_t.
#include "common.h"

#define SSD_MAX_TAPS 16
#define SSD_CONV_TOKENS 8 // tokens in a row that a thread of the convolution takes, in steps of many tokens
#define SSD_TB 16          // tokens whose inputs the recurrence stages at a time

__device__ __forceinline__ float ssd_silu(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float ssd_softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

// ---------------------------------------------------------------------------- convolution
template <typename T>
__global__ void __launch_bounds__(256)
ssd_conv_kernel(const T* __restrict__ proj, int64_t stride, int col0, int channels, int taps,
                const T* __restrict__ conv_w, const T* __restrict__ conv_b, float* __restrict__ conv_state,
                const int32_t* __restrict__ token_seq, const int32_t* __restrict__ cu_seqlens,
                const int32_t* __restrict__ seq_starts, const int32_t* __restrict__ state_slots,
                T* __restrict__ out, float* __restrict__ bc, int np, int n_state, int groups, float* __restrict__ dtd,
                int heads, int dt_col, const float* __restrict__ dt_bias, const float* __restrict__ a_log, int64_t tokens,
                int per_thread) {
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    // a thread takes per_thread tokens in a row with its channel's weights in registers
    float wt[SSD_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < SSD_MAX_TAPS; ++j)
        if (j < taps) wt[j] = to_float(conv_w[(int64_t)c * taps + j]);
    const float bias_c = to_float(conv_b[c]);
    const int hist = taps - 1;
    const int inner = channels - 2 * groups * n_state;
    for (int64_t t = (int64_t)blockIdx.x * per_thread; t < min(tokens, ((int64_t)blockIdx.x + 1) * per_thread); ++t) {
        const int s = token_seq[t];
        const int begin = cu_seqlens[s], n = cu_seqlens[s + 1] - begin;
        const int i = (int)(t - begin);                      // the token's place in its request's portion
        const bool carried = seq_starts[s] > 0;
        float* kept = conv_state + ((int64_t)state_slots[s] * channels + c) * hist;
        float in[SSD_MAX_TAPS];
#pragma unroll
        for (int j = 0; j < SSD_MAX_TAPS; ++j) {
            if (j >= taps) break;
            const int src = i - (hist - j);                  // place in the portion of tap j's input
            if (src >= 0) in[j] = to_float(proj[(t - (hist - j)) * stride + col0 + c]);
            else in[j] = carried ? kept[i + j] : 0.f;        // hist + src = i + j
        }
        float sum = bias_c;
#pragma unroll
        for (int j = 0; j < SSD_MAX_TAPS; ++j) {
            if (j >= taps) break;
            sum += wt[j] * in[j];
        }
        const T rounded = from_float<T>(ssd_silu(sum));
        out[t * channels + c] = rounded;
        // B and C once more as floats, [token][group][B | C][np] (np rows, those beyond the state's zero): the
        // recurrence reads them from there.  And, by the first threads, the step size and the decay of
        // every head: dtd[token][head] = (dt, exp(-exp(A_log) dt)).
        if (c >= inner) {
            const int idx = c - inner, gn = groups * n_state;
            bc[((t * groups + (idx % gn) / n_state) * 2 + idx / gn) * np + idx % n_state] = to_float(rounded);
        }
        if (c < heads) {
            const float dt = ssd_softplus(to_float(proj[t * stride + dt_col + c]) + dt_bias[c]);
            dtd[(t * heads + c) * 2] = dt;
            dtd[(t * heads + c) * 2 + 1] = expf(-expf(a_log[c]) * dt);
        }
        if (n == 1) {                                        // a single token: the kept inputs move on by one
#pragma unroll
            for (int j = 0; j < SSD_MAX_TAPS - 1; ++j) {
                if (j >= hist) break;
                kept[j] = in[j + 1];
            }
        }
    }
}

// The kept inputs of the requests that bring more than one token: the last K - 1 inputs of the portion,
// or, where the portion is shorter, the old ones moved on.  A thread per (request, channel) reads all it
// needs before it writes.
template <typename T>
__global__ void __launch_bounds__(256)
ssd_conv_state_kernel(const T* __restrict__ proj, int64_t stride, int col0, int channels, int taps,
                      float* __restrict__ conv_state, const int32_t* __restrict__ cu_seqlens,
                      const int32_t* __restrict__ seq_starts, const int32_t* __restrict__ state_slots, int first_seq) {
    const int s = first_seq + blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int begin = cu_seqlens[s], n = cu_seqlens[s + 1] - begin;
    if (n <= 1) return;
    const bool carried = seq_starts[s] > 0;
    const int hist = taps - 1;
    float* kept = conv_state + ((int64_t)state_slots[s] * channels + c) * hist;
    float next[SSD_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < SSD_MAX_TAPS - 1; ++j) {
        if (j >= hist) break;
        const int src = n - hist + j;
        if (src >= 0) next[j] = to_float(proj[(int64_t)(begin + src) * stride + col0 + c]);
        else next[j] = carried ? kept[j + n] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < SSD_MAX_TAPS - 1; ++j) {
        if (j >= hist) break;
        kept[j] = next[j];
    }
}

// ---------------------------------------------------------------------------- the recurrence
// One wave per (unit, head, 64 columns of S).  A unit is a run of tokens of one request: a whole
// request's tokens of this step (units == null: unit u is request first_seq + u), or a block of a
// portion (units[u] = request, first token within the portion, tokens, blocks of the portion).
// mode 0: from the request's state (zero at its start) to its new state, which is written back.
// mode 1 (blocks): a portion's first block starts from the request's state, the others from zero; every
//         block leaves its end state in block_states[u] and its tokens' log-decays, summed from the block's
//         start, in cum[t, h]; the request's state is not written.
// mode 2 (blocks, second pass): the blocks after a portion's first add exp(cum_t) E^T C_t to y, E the true
//         state before the block (block_states[u - 1] after the pass over the blocks).
// B, C, the step size and the decay of a token are the same for all lanes of a wave.  Where a thread holds a whole
// column of S (NSPLIT 1: up to 64 rows, or 128 where asked for) they are read from global memory by addresses that are the same in
// every lane, which the compiler turns into scalar loads: they cost no vector register and no LDS, and are
// operands of the multiply-adds as they are.  Where a column is shared out over lanes, B and C of 16 tokens at a
// time go through LDS.
template <typename T, int NPER, int NSPLIT>
__global__ void __launch_bounds__(NVA_WAVE)
ssd_scan_kernel(const T* __restrict__ conv, int channels, const float* __restrict__ bc, int np,
                const float* __restrict__ dtd, int heads, int vdim, int n_state, int groups,
                const float* __restrict__ a_log, const float* __restrict__ d_skip, float* __restrict__ state,
                const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_starts,
                const int32_t* __restrict__ state_slots, int first_seq, const int32_t* __restrict__ units, int mode,
                int carried_only, float* __restrict__ block_states, float* __restrict__ cum, float* __restrict__ y) {
    // B, C, x, the step size and the decay of SSD_TB tokens at a time: their loads are on their way
    // together, and the tokens of a batch run from LDS
    constexpr bool SC = NSPLIT == 1;
    __shared__ __attribute__((aligned(16))) float b_s[SC ? 1 : SSD_TB][NPER * NSPLIT], c_s[SC ? 1 : SSD_TB][NPER * NSPLIT];
    __shared__ float x_s[SSD_TB][NVA_WAVE];
    // a wave's lanes: NSPLIT parts of the state's rows (NPER rows each) times 64 / NSPLIT columns
    constexpr int NMAX = NPER * NSPLIT, PL = NVA_WAVE / NSPLIT;
    const int u = blockIdx.z, h = blockIdx.y;
    const int part = threadIdx.x / PL, row0 = part * NPER;
    const int p = blockIdx.x * PL + threadIdx.x % PL;
    const bool mine = p < vdim;
    int s, t0, n, first_block = 1;
    if (units) {
        s = first_seq + units[4 * u];
        t0 = cu_seqlens[s] + units[4 * u + 1];
        n = units[4 * u + 2];
        first_block = units[4 * u + 1] == 0;
    } else {
        s = first_seq + u;
        t0 = cu_seqlens[s];
        n = cu_seqlens[s + 1] - t0;
    }
    if (mode == 2 && first_block) return;
    // (carried_only: the blocks from a zero state have a kernel of their own; this one takes those that go on from
    // the request's state)
    if (mode == 1 && carried_only && !(first_block && seq_starts[s] > 0)) return;
    const int inner = heads * vdim;
    const int g = h / (heads / groups);
    const float* bc_g = bc + (int64_t)g * 2 * np;             // token t: + t * groups * 2 * np; C: + np
    const int64_t bc_stride = (int64_t)groups * 2 * np;
    float* own = state + (((int64_t)state_slots[s] * heads + h) * n_state) * vdim + p;
    float* block = block_states ? block_states + (((int64_t)u * heads + h) * n_state) * vdim + p : nullptr;

    float S[NPER];                                  // rows row0 .. row0 + NPER - 1 of column p
    if (mode == 2) {
        const float* before = block - (int64_t)heads * n_state * vdim;       // the unit before: the block before
#pragma unroll
        for (int i = 0; i < NPER; ++i) S[i] = mine && row0 + i < n_state ? before[(int64_t)(row0 + i) * vdim] : 0.f;
    } else {
        const bool carried = first_block && seq_starts[s] > 0;
#pragma unroll
        for (int i = 0; i < NPER; ++i) S[i] = carried && mine && row0 + i < n_state ? own[(int64_t)(row0 + i) * vdim] : 0.f;
    }
    // the read-out of a column: the sum over the lanes that hold its parts, in all of them
    auto whole = [&](float v) -> float {
#pragma unroll
        for (int off = PL; off < NVA_WAVE; off <<= 1) v += __shfl_xor(v, off, NVA_WAVE);
        return v;
    };
    const float rate = -expf(a_log[h]), skip = d_skip[h];
    float log_decay = 0.f;
    const int lane = threadIdx.x;
    for (int i0 = 0; i0 < n; i0 += SSD_TB) {
        const int nb = min(SSD_TB, n - i0);
        const int64_t tb = t0 + i0;
        __syncthreads();
        // (every load of a batch is asked for before any is used: a loop of load and store would wait for each in turn)
        if (!SC) {
            // a token's B and C lie side by side in bc, 2 np floats: the wave copies them 16 bytes a lane (np == NMAX here)
            constexpr int PER = 2 * NMAX / 4 / NVA_WAVE > 0 ? 2 * NMAX / 4 / NVA_WAVE : 1;     // float4 a lane and token
            float4 v[SSD_TB][PER];
#pragma unroll
            for (int j = 0; j < SSD_TB; ++j)
#pragma unroll
                for (int q = 0; q < PER; ++q) {
                    const int at = (q * NVA_WAVE + lane) * 4;
                    v[j][q] = j < nb && at < 2 * NMAX ? *reinterpret_cast<const float4*>(bc_g + (tb + j) * bc_stride + at)
                                                      : make_float4(0.f, 0.f, 0.f, 0.f);
                }
            // (rows of a short batch beyond its tokens are written too, as zeros: a store behind a branch would hold up
            // the others)
#pragma unroll
            for (int j = 0; j < SSD_TB; ++j)
#pragma unroll
                for (int q = 0; q < PER; ++q) {
                    const int at = (q * NVA_WAVE + lane) * 4;
                    if (at < NMAX) *reinterpret_cast<float4*>(&b_s[j][at]) = v[j][q];
                    else if (at < 2 * NMAX) *reinterpret_cast<float4*>(&c_s[j][at - NMAX]) = v[j][q];
                }
        }
        if (mode != 2) {
            float xv[SSD_TB];
#pragma unroll
            for (int j = 0; j < SSD_TB; ++j) xv[j] = j < nb && mine ? to_float(conv[(tb + j) * channels + h * vdim + p]) : 0.f;
#pragma unroll
            for (int j = 0; j < SSD_TB; ++j) x_s[j][lane] = xv[j];          // (a column's lanes hold the same)
        }
        __syncthreads();
        auto step = [&](int j) __attribute__((always_inline)) {
            const int64_t t = tb + j;
            // (the constant address space: a load from it at an address that is the same in every lane is a scalar load)
            typedef const __attribute__((address_space(4))) float* scalar_ptr;
            scalar_ptr bt_c = (scalar_ptr)(uintptr_t)(bc_g + t * bc_stride), ct_c = bt_c + np;
            const float* bt_l = &b_s[SC ? 0 : j][row0];
            const float* ct_l = &c_s[SC ? 0 : j][row0];
#define SSD_B(k) (SC ? bt_c[k] : bt_l[k])
#define SSD_C(k) (SC ? ct_c[k] : ct_l[k])
            if (mode == 2) {
                float acc = 0.f;
#pragma unroll
                for (int k = 0; k < NPER; ++k) acc += S[k] * SSD_C(k);
                acc = whole(acc);
                if (mine && part == 0) y[t * inner + h * vdim + p] += expf(cum[t * heads + h]) * acc;
                return;
            }
            scalar_ptr dd = (scalar_ptr)(uintptr_t)(dtd + (t * heads + h) * 2);
            const float dt = dd[0], decay = dd[1];
            const float x = x_s[j][lane];
            const float dx = dt * x;
            float acc = 0.f;
#pragma unroll
            for (int k = 0; k < NPER; ++k) {
                S[k] = decay * S[k] + SSD_B(k) * dx;
                acc += S[k] * SSD_C(k);
            }
            acc = whole(acc);
            if (mine && part == 0) y[t * inner + h * vdim + p] = acc + skip * x;
            if (mode == 1) {
                log_decay += rate * dt;
                if (lane == 0 && blockIdx.x == 0) cum[t * heads + h] = log_decay;
            }
        };
        // a full batch with the tokens' numbers known at compile time: the next token's operands can be asked for
        // during this token's sums
        if (nb == SSD_TB) {
#pragma unroll
            for (int j = 0; j < SSD_TB; ++j) step(j);
        } else {
            for (int j = 0; j < nb; ++j) step(j);
        }
    }
#undef SSD_B
#undef SSD_C
    if (mode == 2 || !mine) return;
    // (a portion of one block has no pass over its blocks: its end state is the request's new state)
    float* dst = mode == 1 && units[4 * u + 3] > 1 ? block : own;
#pragma unroll
    for (int i = 0; i < NPER; ++i)
        if (row0 + i < n_state) dst[(int64_t)(row0 + i) * vdim] = S[i];
}

// The pass over a portion's blocks: block_states[b] <- exp(total log-decay of block b) * block_states[b - 1]
// + block_states[b] for b = 1 ..., and the request's state <- the last.  chains[c] = (first unit, blocks,
// request, tokens of the last block).  A thread per entry of S.
__global__ void __launch_bounds__(256)
ssd_chain_kernel(float* __restrict__ block_states, const float* __restrict__ cum, float* __restrict__ state,
                 const int32_t* __restrict__ chains, const int32_t* __restrict__ units,
                 const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ state_slots, int first_seq, int heads,
                 int n_state, int vdim) {
    const int c = blockIdx.z, h = blockIdx.y;
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    const int per_head = n_state * vdim;
    if (e >= per_head) return;
    const int u0 = chains[4 * c], blocks = chains[4 * c + 1], s = first_seq + chains[4 * c + 2];
    const int64_t unit_stride = (int64_t)heads * per_head;
    float* at = block_states + (int64_t)u0 * unit_stride + (int64_t)h * per_head + e;
    float carry = at[0];
    for (int b = 1; b < blocks; ++b) {
        const int u = u0 + b;
        const int64_t last = cu_seqlens[first_seq + units[4 * u]] + units[4 * u + 1] + units[4 * u + 2] - 1;
        carry = expf(cum[last * heads + h]) * carry + at[b * unit_stride];
        at[b * unit_stride] = carry;
    }
    state[((int64_t)state_slots[s] * heads + h) * per_head + e] = carry;
}

// ---------------------------------------------------------------------------- single tokens
// A request that brings one token: the step is the state's bytes, read once and written once.  A workgroup of four
// waves takes (request, head, 64 columns of S); a thread one column and every fourth row, all of its rows asked
// for before B, C and the step size arrive; the four partial read-outs of a column meet in LDS.
__global__ void __launch_bounds__(256)
ssd_single_kernel(const void* __restrict__ conv, int conv_is_f32, int channels, const float* __restrict__ bc, int np,
                  const float* __restrict__ dtd, int heads, int vdim, int n_state, int groups,
                  const float* __restrict__ d_skip, float* __restrict__ state, const int32_t* __restrict__ cu_seqlens,
                  const int32_t* __restrict__ seq_starts, const int32_t* __restrict__ state_slots,
                  float* __restrict__ y) {
    __shared__ float b_s[256], c_s[256], part_s[4][64];
    const int s = blockIdx.z, h = blockIdx.y;
    const int pl = threadIdx.x % 64, rg = threadIdx.x / 64;
    const int p = blockIdx.x * 64 + pl;
    const bool mine = p < vdim;
    const int64_t t = cu_seqlens[s];
    const bool carried = seq_starts[s] > 0;
    float* own = state + (((int64_t)state_slots[s] * heads + h) * n_state) * vdim + p;
    constexpr int ROWS = 64;                          // rows of a thread: every fourth of up to 256
    float S[ROWS];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        const int r = rg + 4 * i;
        S[i] = carried && mine && r < n_state ? own[(int64_t)r * vdim] : 0.f;
    }
    const int g = h / (heads / groups);
    const float* bt = bc + (t * groups + g) * 2 * (int64_t)np;
    for (int k = threadIdx.x; k < n_state; k += 256) {
        b_s[k] = bt[k];
        c_s[k] = bt[np + k];
    }
    const float dt = dtd[(t * heads + h) * 2], decay = dtd[(t * heads + h) * 2 + 1];
    const int64_t xi = t * channels + h * vdim + p;
    const float x = !mine ? 0.f : conv_is_f32 ? static_cast<const float*>(conv)[xi] : to_float(static_cast<const __bf16*>(conv)[xi]);
    __syncthreads();
    const float dx = dt * x;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        const int r = rg + 4 * i;
        if (r < n_state) {
            S[i] = decay * S[i] + b_s[r] * dx;
            acc += S[i] * c_s[r];
            if (mine) own[(int64_t)r * vdim] = S[i];
        }
    }
    part_s[rg][pl] = acc;
    __syncthreads();
    if (rg == 0 && mine)
        y[t * heads * vdim + h * vdim + p] = part_s[0][pl] + part_s[1][pl] + part_s[2][pl] + part_s[3][pl] + d_skip[h] * x;
}

typedef __attribute__((ext_vector_type(16))) float ssd_f32x16;

// ---------------------------------------------------------------------------- a block from a zero state, as products
// With cum_t the sum of the log-decays of the block's tokens up to t, a block that starts from a zero state gives
//     y_t = sum over s <= t of exp(cum_t - cum_s) dt_s (C_t . B_s) x_s + D x_t         and leaves
//     U   = sum over s of exp(cum_last - cum_s) dt_s B_s x_s^T                          as its end state:
// no recurrence, three float products (C B^T, the masked and weighted result times X, B^T times the weighted X) on
// the matrix cores (v_mfma_f32_32x32x2_f32).  Every exponent is a difference of sums of logarithms that is <= 0.
// A workgroup of four waves takes a block of up to 64 tokens, a head and 64 columns; C, B and X are staged in LDS,
// the masked product goes through LDS to become an operand.  States of up to 128 rows.
__global__ void __launch_bounds__(256)
ssd_block_kernel(const void* __restrict__ conv, int conv_is_f32, int channels, const float* __restrict__ bc, int np,
                 const float* __restrict__ dtd, int heads, int vdim, int n_state, int groups,
                 const float* __restrict__ a_log, const float* __restrict__ d_skip, float* __restrict__ state,
                 const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_starts,
                 const int32_t* __restrict__ state_slots, int first_seq, const int32_t* __restrict__ units,
                 float* __restrict__ block_states, float* __restrict__ cum, float* __restrict__ y) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int u = blockIdx.z, h = blockIdx.y, pw = blockIdx.x * 64;
    const int s = first_seq + units[4 * u];
    const bool first_block = units[4 * u + 1] == 0;
    if (first_block && seq_starts[s] > 0) return;          // goes on from the request's state: the recurrence's kernel
    const int n = units[4 * u + 2], blocks = units[4 * u + 3];
    const int64_t t0 = cu_seqlens[s] + units[4 * u + 1];
    const int nt = (n_state + 31) / 32;                    // tiles of 32 rows of the state
    const int ld = 32 * nt + 1;                            // C and B rows in LDS, zero beyond the state's rows
    float* c_s = lds;                                      // [64][ld]
    float* b_s = c_s + 64 * ld;                            // [64][ld]
    float* x_s = b_s + 64 * ld;                            // [64][65]
    float* m_s = x_s + 64 * 65;                            // [64][65]
    float* cum_s = m_s + 64 * 65;                          // [64]
    float* dt_s = cum_s + 64;                              // [64]
    const int tid = threadIdx.x, wave = tid / NVA_WAVE, lane = tid % NVA_WAVE;
    const int g = h / (heads / groups);
    const int64_t bc_stride = (int64_t)groups * 2 * np;
    const float* bc_g = bc + (int64_t)g * 2 * np;
    const int width = 32 * nt;
    // B and C of the block's tokens, 16 bytes a load, every load asked for before any is used (the rows are padded
    // with zeros up to np in memory; beyond np and beyond the block's tokens zeros are written)
    {
        const int w4 = width / 4;                          // float4 a row
        constexpr int MAXQ = 64 * 32 / 256;                // a row has at most 128 floats
        float4 vb[MAXQ], vc[MAXQ];
#pragma unroll
        for (int q = 0; q < MAXQ; ++q) {
            const int idx = q * 256 + tid, r = idx / w4, k = (idx % w4) * 4;
            const bool ok = idx < 64 * w4 && r < n && k < np;
            vb[q] = ok ? *reinterpret_cast<const float4*>(bc_g + (t0 + r) * bc_stride + k) : make_float4(0.f, 0.f, 0.f, 0.f);
            vc[q] = ok ? *reinterpret_cast<const float4*>(bc_g + (t0 + r) * bc_stride + np + k) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int q = 0; q < MAXQ; ++q) {
            const int idx = q * 256 + tid;
            if (idx < 64 * w4) {
                float* bd = b_s + (idx / w4) * ld + (idx % w4) * 4;
                float* cd = c_s + (idx / w4) * ld + (idx % w4) * 4;
                bd[0] = vb[q].x, bd[1] = vb[q].y, bd[2] = vb[q].z, bd[3] = vb[q].w;
                cd[0] = vc[q].x, cd[1] = vc[q].y, cd[2] = vc[q].z, cd[3] = vc[q].w;
            }
        }
    }
    {
        float vx[16];
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const int idx = q * 256 + tid, r = idx / 64, j = idx % 64;
            const int64_t at = (t0 + r) * channels + h * vdim + pw + j;
            vx[q] = r < n && pw + j < vdim ? (conv_is_f32 ? static_cast<const float*>(conv)[at]
                                                         : to_float(static_cast<const __bf16*>(conv)[at])) : 0.f;
        }
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const int idx = q * 256 + tid;
            x_s[(idx / 64) * 65 + idx % 64] = vx[q];
        }
    }
    if (wave == 0) {
        // the tokens' log-decays summed along the block, by one wave
        const float dt = lane < n ? dtd[((t0 + lane) * heads + h) * 2] : 0.f;
        float c = -expf(a_log[h]) * dt;
#pragma unroll
        for (int off = 1; off < NVA_WAVE; off <<= 1) {
            const float up = __shfl_up(c, off, NVA_WAVE);
            if (lane >= off) c += up;
        }
        cum_s[lane] = c;
        dt_s[lane] = dt;
        if (lane < n && blockIdx.x == 0) cum[(t0 + lane) * heads + h] = c;
    }
    __syncthreads();
    const int i = lane % 32, half = lane / 32;
    typedef ssd_f32x16 acc_t;
    // ---- G = C B^T, tile (ti, si) of 32 tokens t by 32 tokens s; then masked and weighted into m_s
    {
        const int ti = wave / 2, si = wave % 2;
        acc_t acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
        if (si <= ti) {                                      // (the tile above the diagonal is all zero)
            const float* crow = c_s + (32 * ti + i) * ld + half;
            const float* brow = b_s + (32 * si + i) * ld + half;
#pragma unroll 8
            for (int k = 0; k < width; k += 2) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(crow[k], brow[k], acc, 0, 0, 0);
        }
        const int sc = 32 * si + i;
        const float cum_sc = cum_s[sc], dt_sc = dt_s[sc];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int t = 32 * ti + 8 * (r / 4) + 4 * half + r % 4;
            m_s[t * 65 + sc] = sc <= t ? acc[r] * expf(cum_s[t] - cum_sc) * dt_sc : 0.f;
        }
    }
    __syncthreads();
    const int inner = heads * vdim;
    // ---- Y = M X, tile (ti, pi) of 32 tokens by 32 columns
    {
        const int ti = wave / 2, pi = wave % 2;
        acc_t acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
        const float* mrow = m_s + (32 * ti + i) * 65 + half;
        const float* xcol = x_s + half * 65 + 32 * pi + i;
#pragma unroll 8
        for (int k = 0; k < 32 * (ti + 1); k += 2) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(mrow[k], xcol[k * 65], acc, 0, 0, 0);
        const float skip = d_skip[h];
        const int pc = pw + 32 * pi + i;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int t = 32 * ti + 8 * (r / 4) + 4 * half + r % 4;
            if (t < n && pc < vdim) y[(t0 + t) * inner + h * vdim + pc] = acc[r] + skip * x_s[t * 65 + 32 * pi + i];
        }
    }
    // ---- U = B^T diag(w) X with w_s = exp(cum_last - cum_s) dt_s: tiles of 32 state rows by 32 columns
    const float cum_last = cum_s[63];                        // (tokens beyond the block's add nothing to the sum)
    float* dst = blocks > 1 ? block_states + (((int64_t)u * heads + h) * n_state) * vdim
                            : state + (((int64_t)state_slots[s] * heads + h) * n_state) * vdim;
    for (int tile = wave; tile < 2 * nt; tile += 4) {
        const int ni = tile / 2, pi = tile % 2;
        acc_t acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
        const float* bcol = b_s + half * ld + 32 * ni + i;
        const float* xcol = x_s + half * 65 + 32 * pi + i;
#pragma unroll 8
        for (int k = 0; k < 64; k += 2) {
            const float w = expf(cum_last - cum_s[k + half]) * dt_s[k + half];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bcol[k * ld], w * xcol[k * 65], acc, 0, 0, 0);
        }
        const int pc = pw + 32 * pi + i;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = 32 * ni + 8 * (r / 4) + 4 * half + r % 4;
            if (row < n_state && pc < vdim) dst[(int64_t)row * vdim + pc] = acc[r];
        }
    }
}

// ---------------------------------------------------------------------------- what the state before a block adds
// y[t, p] += exp(cum[t]) * sum_n C[t, n] E[n, p] for the tokens t of a block, E the true state before the block: one float
// product per block and head, on the matrix cores (v_mfma_f32_32x32x2_f32: float operands, float sums).  A workgroup of
// four waves takes 64 tokens of a block and 64 columns; C of those tokens and the 64 columns of E are staged in LDS (rows
// beyond the state's are zero there).

__global__ void __launch_bounds__(256)
ssd_inter_kernel(const float* __restrict__ bc, int np, int heads, int vdim, int n_state, int groups,
                 const int32_t* __restrict__ cu_seqlens, int first_seq, const int32_t* __restrict__ units, int subs,
                 const float* __restrict__ block_states, const float* __restrict__ cum, float* __restrict__ y) {
    extern __shared__ __attribute__((aligned(16))) float c_lds[];          // [64 tokens][kp + 1], then E [kp][64]
    const int u = blockIdx.z / subs, sub = blockIdx.z % subs, h = blockIdx.y;
    if (units[4 * u + 1] == 0) return;                                      // a portion's first block started from the true state
    const int n = units[4 * u + 2];
    const int i0 = sub * 64;
    if (i0 >= n) return;
    const int64_t t0 = cu_seqlens[first_seq + units[4 * u]] + units[4 * u + 1] + i0;
    const int rows = min(64, n - i0);
    const int kp = (n_state + 1) & ~1;                                      // k in pairs
    const int ld = kp + 1;
    const int g = h / (heads / groups);
    const int64_t bc_stride = (int64_t)groups * 2 * np;
    const float* c_g = bc + (int64_t)g * 2 * np + np;
    float* e_lds = c_lds + 64 * ld;
    const float* e = block_states + (((int64_t)(u - 1) * heads + h) * n_state) * vdim;
    const int pw = blockIdx.x * 64;                                        // the workgroup's first column
    // (eight loads asked for before any is used: a loop of load and store would wait for each in turn)
    for (int base = 0; base < 64 * kp; base += 8 * 256) {
        float vc[8], ve[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const int idx = base + q * 256 + threadIdx.x;
            const int r = idx / kp, k = idx % kp;                           // C: token r, row k
            vc[q] = idx < 64 * kp && r < rows && k < n_state ? c_g[(t0 + r) * bc_stride + k] : 0.f;
            const int ke = idx / 64, j = idx % 64;                          // E: row ke, column j
            ve[q] = idx < 64 * kp && ke < n_state && pw + j < vdim ? e[(int64_t)ke * vdim + pw + j] : 0.f;
        }
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const int idx = base + q * 256 + threadIdx.x;
            if (idx < 64 * kp) {
                c_lds[(idx / kp) * ld + idx % kp] = vc[q];
                e_lds[idx] = ve[q];
            }
        }
    }
    __syncthreads();
    const int wave = threadIdx.x / NVA_WAVE, lane = threadIdx.x % NVA_WAVE;
    const int tt = wave / 2, p0 = blockIdx.x * 64 + (wave % 2) * 32;
    if (tt * 32 >= rows || p0 >= vdim) return;
    const int i = lane % 32, half = lane / 32;
    const int inner = heads * vdim;
    const bool col_ok = p0 + i < vdim;
    ssd_f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    const float* crow = c_lds + (tt * 32 + i) * ld + half;
    const float* ecol = e_lds + half * 64 + (wave % 2) * 32 + i;
#pragma unroll 8
    for (int k = 0; k < kp; k += 2) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(crow[k], ecol[k * 64], acc, 0, 0, 0);
    // acc[r] is the sum of row 8 (r / 4) + 4 half + r % 4, column i
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int row = tt * 32 + 8 * (r / 4) + 4 * half + r % 4;
        if (row < rows && col_ok) {
            const int64_t t = t0 + row;
            y[t * inner + h * vdim + p0 + i] += expf(cum[t * heads + h]) * acc[r];
        }
    }
}

// ---------------------------------------------------------------------------- gate and grouped norm
template <typename T>
__global__ void __launch_bounds__(1024)
ssd_finish_kernel(const float* __restrict__ y, const T* __restrict__ proj, int64_t stride, const float* __restrict__ weight,
                  int inner, int group_size, float eps, T* __restrict__ out, int64_t out_stride) {
    __shared__ float scratch[16];
    const int64_t t = blockIdx.x;
    const int g = blockIdx.y;
    const float* yr = y + t * inner + g * group_size;
    const T* zr = proj + t * stride + g * group_size;
    float ss = 0.f;
    for (int i = threadIdx.x; i < group_size; i += blockDim.x) {
        const float v = yr[i] * ssd_silu(to_float(zr[i]));
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float scale = rsqrtf(ss / (float)group_size + eps);
    for (int i = threadIdx.x; i < group_size; i += blockDim.x) {
        const float v = yr[i] * ssd_silu(to_float(zr[i]));
        out[t * out_stride + g * group_size + i] = from_float<T>(v * scale * weight[g * group_size + i]);
    }
}

struct ScanArgs {
    const elem_t* conv; int channels; const float* bc; int np; const float* dtd; int heads, vdim, n_state, groups;
    const float *a_log, *d_skip; float* state; const int32_t *cu, *starts, *slots;
    float *block_states, *cum, *y;
};

// Rows of B and C per token and group in the float copy the recurrence reads: the rows a thread (or the lanes that
// share a column) hold, the state's rounded up.
static int ssd_padded_rows(int n_state) {
    return n_state <= 16 ? 16 : n_state <= 32 ? 32 : n_state <= 64 ? 64 : n_state <= 128 ? 128 : 256;
}
NVA_EXPORT int NVA_NAME(nva_state_space_padded_rows)(int n_state) { return ssd_padded_rows(n_state); }

template <int NPER, int NSPLIT>
static void launch_scan(const ScanArgs& a, unsigned units, int first_seq, const int32_t* us, int mode, int carried_only,
                        hipStream_t stream) {
    constexpr int PL = NVA_WAVE / NSPLIT;
    const dim3 grid((unsigned)((a.vdim + PL - 1) / PL), (unsigned)a.heads, units);
    hipLaunchKernelGGL((ssd_scan_kernel<elem_t, NPER, NSPLIT>), grid, dim3(NVA_WAVE), 0, stream, a.conv, a.channels, a.bc,
                       a.np, a.dtd, a.heads, a.vdim, a.n_state, a.groups, a.a_log, a.d_skip, a.state, a.cu, a.starts, a.slots,
                       first_seq, us, mode, carried_only, a.block_states, a.cum, a.y);
}

// proj: [tokens, 2 H P + 2 G N + H] with rows `stride` apart.  conv_out [tokens, C] (elements), y_raw [tokens, H P]
// and cum [tokens, H] (float) are scratch.  state [slots, H, N, P], conv_state [slots, C, K - 1], float.
// The first num_single requests bring one token each.  units / chains (with block_states [units, H, N, P]): the
// portions of the requests from num_single on cut into blocks (units[u] = request counted from num_single, first token,
// tokens, blocks of the portion; block_tokens: the most tokens of a block; shape: 0, or how a state of 65 to 128 rows is held (1: a thread a column, 2: four
// lanes a column, 3: the second pass on the vector units, 4: single
// tokens through the kernel that serves portions, 6: blocks from a zero state
// as products on the matrix cores; measurements); chains[c] = first unit, blocks, request, tokens of the last block, for every
// portion of more than one block); null: every portion runs as one.
// bc: float [tokens, groups, 2, padded rows] (zero where the padded rows exceed the state's: the caller clears it then),
// dtd: float [tokens, heads, 2]: scratch as well.
NVA_EXPORT int NVA_NAME(nva_state_space)(const void* proj, int64_t stride, void* conv_out, float* bc, float* dtd,
                                         float* y_raw, float* cum, void* out,
                                         int64_t out_stride, float* state, float* conv_state, int64_t slots,
                                         const int32_t* token_seq, const int32_t* cu_seqlens, const int32_t* seq_starts,
                                         const int32_t* state_slots, int64_t seqs, int64_t tokens, int64_t num_single,
                                         int heads, int vdim, int n_state, int groups, int taps, const void* conv_w,
                                         const void* conv_b, const float* dt_bias, const float* a_log, const float* d_skip,
                                         const float* norm_w, int norm_groups, float eps, const int32_t* units,
                                         int64_t n_units, const int32_t* chains, int64_t n_chains, int block_tokens,
                                         float* block_states, int shape, hipStream_t stream) {
    if (tokens == 0) return 0;
    if (tokens < 0 || seqs <= 0 || seqs > 65535 || num_single < 0 || num_single > seqs || slots <= 0)
        return nva_fail("state_space: bad counts tokens=%lld requests=%lld", (long long)tokens, (long long)seqs);
    if (heads <= 0 || vdim <= 0 || n_state <= 0 || groups <= 0 || heads % groups || norm_groups <= 0 ||
        (heads * vdim) % norm_groups || heads > 65535)
        return nva_fail("state_space: bad sizes heads=%d vdim=%d state=%d groups=%d norm_groups=%d", heads, vdim, n_state,
                        groups, norm_groups);
    if (taps < 1 || taps > SSD_MAX_TAPS) return nva_fail("state_space: %d taps (1..%d are built)", taps, SSD_MAX_TAPS);
    if (n_state > 256) return nva_fail("state_space: a state of %d rows (up to 256 are built)", n_state);
    const int inner = heads * vdim, channels = inner + 2 * groups * n_state;
    if (stride < 2 * inner + 2 * groups * n_state + heads) return nva_fail("state_space: rows too short");
    if (!proj || !conv_out || !bc || !dtd || !y_raw || !out || !state || (!conv_state && taps > 1) || !token_seq || !cu_seqlens || !seq_starts ||
        !state_slots || !conv_w || !conv_b || !dt_bias || !a_log || !d_skip || !norm_w)
        return nva_fail("state_space: a tensor is missing");
    if (n_chains && (!units || !chains || !block_states || !cum || block_tokens <= 0 || n_units * ((block_tokens + 63) / 64) > 65535))
        return nva_fail("state_space: blocks need their scratch and their size");
    const elem_t* pj = (const elem_t*)proj;
    if (tokens > 0x7fffffff || (channels + 255) / 256 > 65535) return nva_fail("state_space: too many tokens or channels");
    const int per_thread = tokens >= 1024 ? SSD_CONV_TOKENS : 1;
    hipLaunchKernelGGL((ssd_conv_kernel<elem_t>),
                       dim3((unsigned)((tokens + per_thread - 1) / per_thread), (channels + 255) / 256), dim3(256), 0, stream, pj,
                       stride, inner, channels, taps, (const elem_t*)conv_w, (const elem_t*)conv_b, conv_state, token_seq,
                       cu_seqlens, seq_starts, state_slots, (elem_t*)conv_out, bc, ssd_padded_rows(n_state), n_state, groups, dtd,
                       heads, inner + channels, dt_bias, a_log, tokens, per_thread);
    if (seqs > num_single && taps > 1)
        hipLaunchKernelGGL((ssd_conv_state_kernel<elem_t>), dim3((channels + 255) / 256, (unsigned)(seqs - num_single)),
                           dim3(256), 0, stream, pj, stride, inner, channels, taps, conv_state, cu_seqlens, seq_starts,
                           state_slots, (int)num_single);
    const ScanArgs args{(const elem_t*)conv_out, channels, bc, ssd_padded_rows(n_state), dtd, heads, vdim, n_state, groups,
                        a_log, d_skip, state, cu_seqlens, seq_starts, state_slots, block_states, cum, y_raw};
    // a thread holds up to 64 rows of a column of S; a state of more rows is shared out over 2 or 4 lanes
    auto scan = [&](unsigned units, int first_seq, const int32_t* us, int mode, int carried_only = 0) {
        if (n_state <= 16) launch_scan<16, 1>(args, units, first_seq, us, mode, carried_only, stream);
        else if (n_state <= 32) launch_scan<32, 1>(args, units, first_seq, us, mode, carried_only, stream);
        else if (n_state <= 64) launch_scan<64, 1>(args, units, first_seq, us, mode, carried_only, stream);
        else if (n_state <= 128 && shape == 1) launch_scan<128, 1>(args, units, first_seq, us, mode, carried_only, stream);
        else if (n_state <= 128 && shape == 2) launch_scan<32, 4>(args, units, first_seq, us, mode, carried_only, stream);
        else if (n_state <= 128) launch_scan<64, 2>(args, units, first_seq, us, mode, carried_only, stream);
        else launch_scan<64, 4>(args, units, first_seq, us, mode, carried_only, stream);
    };
    // the requests that bring one token (they come first) have a kernel of their own
    auto single = [&]() {
        if (num_single && shape != 4)
            hipLaunchKernelGGL(ssd_single_kernel, dim3((unsigned)((vdim + 63) / 64), (unsigned)heads, (unsigned)num_single), dim3(256),
                               0, stream, conv_out, (int)(sizeof(elem_t) == 4), channels, bc, ssd_padded_rows(n_state), dtd, heads,
                               vdim, n_state, groups, d_skip, state, cu_seqlens, seq_starts, state_slots, y_raw);
        else if (num_single)
            scan((unsigned)num_single, 0, nullptr, 0);
    };
    if (n_chains) {
        if (n_units <= 0 || n_units > 65535) return nva_fail("state_space: bad block count %lld", (long long)n_units);
        single();
        // blocks of up to 64 tokens from a zero state can run as three products on the matrix cores (shape 6; a portion's
        // first block that goes on from the request's state, taller states and longer blocks run the recurrence): as
        // fast as the recurrence where measured, and not the kernel that serves
        const bool products = shape == 6 && block_tokens <= 64 && n_state <= 128;
        if (products) {
            const int nt = (n_state + 31) / 32;
            const size_t lds = (size_t)(2 * 64 * (32 * nt + 1) + 2 * 64 * 65 + 128) * sizeof(float);
            static bool raised_block = false;
            if (!raised_block) {
                if (hipFuncSetAttribute((const void*)ssd_block_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)((2 * 64 * 129 + 2 * 64 * 65 + 128) * sizeof(float))) != hipSuccess)
                    return nva_fail("state_space: cannot have the LDS of the blocks' products");
                raised_block = true;
            }
            hipLaunchKernelGGL(ssd_block_kernel, dim3((unsigned)((vdim + 63) / 64), (unsigned)heads, (unsigned)n_units), dim3(256),
                               lds, stream, conv_out, (int)(sizeof(elem_t) == 4), channels, bc, ssd_padded_rows(n_state), dtd,
                               heads, vdim, n_state, groups, a_log, d_skip, state, cu_seqlens, seq_starts, state_slots,
                               (int)num_single, units, block_states, cum, y_raw);
        }
        scan((unsigned)n_units, (int)num_single, units, 1, products ? 1 : 0);
        hipLaunchKernelGGL(ssd_chain_kernel, dim3((n_state * vdim + 255) / 256, heads, (unsigned)n_chains), dim3(256), 0, stream,
                           block_states, cum, state, chains, units, cu_seqlens, state_slots, (int)num_single, heads, n_state,
                           vdim);
        if (shape == 3) {
            scan((unsigned)n_units, (int)num_single, units, 2);              // (on the vector units: measurements)
        } else {
            // the blocks' tokens: `block_tokens` at most, 64 a workgroup
            const int subs = (block_tokens + 63) / 64;
            const int kp = (n_state + 1) & ~1;
            static bool raised = false;              // the kernel's LDS limit, lifted once to what the tallest state needs
            if (!raised) {
                if (hipFuncSetAttribute((const void*)ssd_inter_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)((64 * 257 + 256 * 64) * sizeof(float))) != hipSuccess)
                    return nva_fail("state_space: cannot have the LDS of the blocks' second pass");
                raised = true;
            }
            hipLaunchKernelGGL(ssd_inter_kernel, dim3((unsigned)((vdim + 63) / 64), (unsigned)heads, (unsigned)(n_units * subs)),
                               dim3(256), (size_t)(64 * (kp + 1) + kp * 64) * sizeof(float), stream, bc, ssd_padded_rows(n_state), heads, vdim,
                               n_state, groups, cu_seqlens, (int)num_single, units, subs, block_states, cum, y_raw);
        }
    } else {
        single();
        if (seqs > num_single) {
            // (units == null: unit u is request first_seq + u)
            scan((unsigned)(seqs - num_single), (int)num_single, nullptr, 0);
        }
    }
    const int group_size = inner / norm_groups;
    // (few tokens: more threads a row, so that a row's loads are on their way at once)
    hipLaunchKernelGGL((ssd_finish_kernel<elem_t>), dim3((unsigned)tokens, norm_groups),
                       dim3(tokens <= 64 && group_size >= 2048 ? 1024 : 256), 0, stream, y_raw, pj,
                       stride, norm_w, inner, group_size, eps, (elem_t*)out, out_stride);
    return nva_check_launch("state_space");
}

NVA_DEFINE_LAST_ERROR(nva_ssd)

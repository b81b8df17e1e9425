// Retention: linear attention with a fixed decay per head, no softmax and no denominator.
//
// Per head, with a state S [D, DV] that starts at zero and is carried from token to token:
//     q, k <- rotation of the first R channels in pairs (i, i + R/2) by the angle p * f_i
//     k    <- k * k_scale
//     S_t  = decay * S_(t-1) + k_t v_t^T          o_t = S_t^T q_t
// and afterwards (the finishing kernel), per token and head,
//     y = o / sqrt(mean(o^2) + eps) * silu(g)
//
// A step brings, for every request, one token or a portion of a prompt.  The portion is taken in
// chunks of RET_C tokens.  With S the state before a chunk of n tokens and i, j its tokens:
//     o_i  = decay^(i+1) S^T q_i + sum_{j <= i} decay^(i-j) (q_i . k_j) v_j
//     S'   = decay^n S + sum_j decay^(n-1-j) k_j v_j^T
// No quotient of powers is ever taken, so small decays do not overflow.  The columns of S (the value
// channels) do not depend on each other: a workgroup takes one request, one head and a slice of
// value channels, keeps its part of S in LDS over all the chunks, and writes it back at the end.
//
// Everything here is float: the rotation (angles from the float position and float frequencies,
// accurate sine and cosine), the scores, the decay powers (a table [heads, RET_C + 1] made on the
// host in double), the state and the sums.  Only the projections are read as elements, and the
// finished y is rounded once.
//
// The step's metadata is read on the device only (cu_seqlens_q, seq_starts, state_slots), so a
// captured step replays for other requests.  seq_starts[s] == 0 starts from a zero state.
#include "common.h"

#define RET_C 32                  // tokens of a chunk
#define RET_THREADS 256
#define RET_MAX_VSLICE 32         // value channels of a workgroup

__host__ __device__ inline size_t ret_lds_floats(int dim, int vslice) {
    // q and k [RET_C][dim + 1], v [RET_C][vslice], scores [RET_C][RET_C + 1], state [dim][vslice]
    return (size_t)2 * RET_C * (dim + 1) + (size_t)RET_C * vslice + (size_t)RET_C * (RET_C + 1) + (size_t)dim * vslice;
}

template <typename T>
__global__ void __launch_bounds__(RET_THREADS)
retention_chunk_kernel(const T* __restrict__ proj, int64_t stride, float* __restrict__ o_raw, int64_t o_stride,
                       float* __restrict__ state, const int32_t* __restrict__ cu_seqlens_q,
                       const int32_t* __restrict__ seq_starts, const int32_t* __restrict__ state_slots,
                       const float* __restrict__ decay_pow, const float* __restrict__ inv_freq, int rot,
                       int heads, int dim, int vdim, int vslice, int nslices, float k_scale) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int DS = dim + 1;
    float* const q_s = lds;                              // [RET_C][DS]
    float* const k_s = q_s + RET_C * DS;                 // [RET_C][DS]
    float* const v_s = k_s + RET_C * DS;                 // [RET_C][vslice]
    float* const a_s = v_s + RET_C * vslice;             // [RET_C][RET_C + 1]
    float* const s_s = a_s + RET_C * (RET_C + 1);        // [dim][vslice]

    const int h = blockIdx.x / nslices, slice = blockIdx.x % nslices;
    const int seq = blockIdx.y;
    const int c0 = slice * vslice;
    const int nc = min(vslice, vdim - c0);               // this slice's channels
    const int tid = threadIdx.x;
    const int q_begin = cu_seqlens_q[seq];
    const int q_len = cu_seqlens_q[seq + 1] - q_begin;
    const int start = seq_starts[seq];
    const int slot = state_slots[seq];
    const float* pw = decay_pow + (int64_t)h * (RET_C + 1);
    float* const s_g = state + (((int64_t)slot * heads + h) * dim) * vdim + c0;      // [dim][vdim] of (slot, head), at this slice
    const int half = rot / 2;
    const int64_t q_off = (int64_t)h * dim, k_off = (int64_t)(heads + h) * dim;
    const int64_t v_off = (int64_t)2 * heads * dim + (int64_t)h * vdim + c0;

    for (int e = tid; e < dim * nc; e += RET_THREADS) {
        const int d = e / nc, c = e % nc;
        s_s[d * vslice + c] = start > 0 ? s_g[(int64_t)d * vdim + c] : 0.f;
    }

    for (int t0 = 0; t0 < q_len; t0 += RET_C) {
        const int n = min(RET_C, q_len - t0);
        __syncthreads();                                 // the chunk before is done with q, k, v and the scores
        // ---- q and k of the chunk, rotated, k scaled; v
        for (int e = tid; e < n * dim; e += RET_THREADS) {
            const int r = e / dim, d = e % dim;
            const T* row = proj + (int64_t)(q_begin + t0 + r) * stride;
            float qv = to_float(row[q_off + d]), kv = to_float(row[k_off + d]);
            if (d < rot) {
                const bool lower = d < half;
                const int partner = lower ? d + half : d - half;
                const float angle = (float)(start + t0 + r) * inv_freq[lower ? d : d - half];
                float sn, cs;
                sincosf(angle, &sn, &cs);
                const float qp = to_float(row[q_off + partner]), kp = to_float(row[k_off + partner]);
                qv = lower ? qv * cs - qp * sn : qv * cs + qp * sn;
                kv = lower ? kv * cs - kp * sn : kv * cs + kp * sn;
            }
            q_s[r * DS + d] = qv;
            k_s[r * DS + d] = kv * k_scale;
        }
        for (int e = tid; e < n * nc; e += RET_THREADS) {
            const int r = e / nc, c = e % nc;
            v_s[r * vslice + c] = to_float(proj[(int64_t)(q_begin + t0 + r) * stride + v_off + c]);
        }
        __syncthreads();
        // ---- scores of the chunk with their decay: a[i][j] = decay^(i-j) q_i . k_j for j <= i
        for (int e = tid; e < n * n; e += RET_THREADS) {
            const int i = e / n, j = e % n;
            float dot = 0.f;
            if (j <= i) {
                const float* qi = q_s + i * DS;
                const float* kj = k_s + j * DS;
                for (int d = 0; d < dim; ++d) dot += qi[d] * kj[d];
                dot *= pw[i - j];
            }
            a_s[i * (RET_C + 1) + j] = dot;
        }
        __syncthreads();
        // ---- outputs: what the state before the chunk gives, and the chunk's own tokens
        for (int e = tid; e < n * nc; e += RET_THREADS) {
            const int i = e / nc, c = e % nc;
            const float* qi = q_s + i * DS;
            float from_state = 0.f;
            for (int d = 0; d < dim; ++d) from_state += qi[d] * s_s[d * vslice + c];
            float own = 0.f;
            const float* ai = a_s + i * (RET_C + 1);
            for (int j = 0; j <= i; ++j) own += ai[j] * v_s[j * vslice + c];
            o_raw[(int64_t)(q_begin + t0 + i) * o_stride + (int64_t)h * vdim + c0 + c] = pw[i + 1] * from_state + own;
        }
        __syncthreads();
        // ---- the state after the chunk
        const float all = pw[n];
        for (int e = tid; e < dim * nc; e += RET_THREADS) {
            const int d = e / nc, c = e % nc;
            float add = 0.f;
            for (int j = 0; j < n; ++j) add += pw[n - 1 - j] * k_s[j * DS + d] * v_s[j * vslice + c];
            s_s[d * vslice + c] = all * s_s[d * vslice + c] + add;
        }
    }
    __syncthreads();
    for (int e = tid; e < dim * nc; e += RET_THREADS) {
        const int d = e / nc, c = e % nc;
        s_g[(int64_t)d * vdim + c] = s_s[d * vslice + c];
    }
}

// ---------------------------------------------------------------------------- single tokens
// A request that brings one token: S <- decay S + k v^T, o = S^T q, nothing else.  The step is the
// state's bytes, read once and written once: a workgroup takes (request, head, 32 value channels),
// a thread one channel and every eighth row of S, which it asks for before anything else; q and k
// are rotated into LDS meanwhile, and the eight partial sums of a channel meet in LDS.
#define RET_DEC_ROWS 32           // rows of S a thread keeps: heads of up to 8 * 32 channels
template <typename T>
__global__ void __launch_bounds__(256)
retention_decode_kernel(const T* __restrict__ proj, int64_t stride, float* __restrict__ o_raw, int64_t o_stride,
                        float* __restrict__ state, const int32_t* __restrict__ cu_seqlens_q,
                        const int32_t* __restrict__ seq_starts, const int32_t* __restrict__ state_slots,
                        const float* __restrict__ decay_pow, const float* __restrict__ inv_freq, int rot,
                        int heads, int dim, int vdim, int nslices, float k_scale) {
    __shared__ float q_s[8 * RET_DEC_ROWS], k_s[8 * RET_DEC_ROWS], part_s[8][33];
    const int h = blockIdx.x / nslices, c0 = 32 * (blockIdx.x % nslices);
    const int seq = blockIdx.y;
    const int tid = threadIdx.x, c = tid & 31, dg = tid >> 5;
    const bool has = c0 + c < vdim;
    const int64_t tok = cu_seqlens_q[seq];
    const int start = seq_starts[seq];
    const int slot = state_slots[seq];
    float* const s_g = state + (((int64_t)slot * heads + h) * dim) * vdim + c0 + c;
    float S[RET_DEC_ROWS];
#pragma unroll
    for (int i = 0; i < RET_DEC_ROWS; ++i) {
        const int d = dg + 8 * i;
        S[i] = has && d < dim && start > 0 ? s_g[(int64_t)d * vdim] : 0.f;
    }
    const T* row = proj + tok * stride;
    const int half = rot / 2;
    for (int d = tid; d < dim; d += blockDim.x) {
        float qv = to_float(row[(int64_t)h * dim + d]), kv = to_float(row[(int64_t)(heads + h) * dim + d]);
        if (d < rot) {
            const bool lower = d < half;
            const int partner = lower ? d + half : d - half;
            float sn, cs;
            sincosf((float)start * inv_freq[lower ? d : d - half], &sn, &cs);
            const float qp = to_float(row[(int64_t)h * dim + partner]), kp = to_float(row[(int64_t)(heads + h) * dim + partner]);
            qv = lower ? qv * cs - qp * sn : qv * cs + qp * sn;
            kv = lower ? kv * cs - kp * sn : kv * cs + kp * sn;
        }
        q_s[d] = qv;
        k_s[d] = kv * k_scale;
    }
    const float v = has ? to_float(row[(int64_t)2 * heads * dim + (int64_t)h * vdim + c0 + c]) : 0.f;
    const float decay = decay_pow[(int64_t)h * (RET_C + 1) + 1];
    __syncthreads();
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < RET_DEC_ROWS; ++i) {
        const int d = dg + 8 * i;
        if (d < dim) {
            S[i] = decay * S[i] + k_s[d] * v;
            o += S[i] * q_s[d];
            if (has) s_g[(int64_t)d * vdim] = S[i];
        }
    }
    part_s[dg][c] = o;
    __syncthreads();
    if (dg == 0 && has) {
        float sum = 0.f;
#pragma unroll
        for (int g = 0; g < 8; ++g) sum += part_s[g][c];
        o_raw[tok * o_stride + (int64_t)h * vdim + c0 + c] = sum;
    }
}

// ---------------------------------------------------------------------------- on the matrix cores, in float
// The same chunks with their four products as 32 x 32 x 2 float MFMAs (float operands, float sums:
// nothing is rounded to a shorter type).  One wave per (request, head, 32 value channels), up to four
// waves of one head in a workgroup, which share the chunk's q and k in LDS; heads of 32 DT channels.
// The wave keeps its part of the state, S[:, 32 channels], in DT accumulator tiles
// for the whole portion: it is the B operand of the product with q as it lies (register r of a tile
// holds, in the lanes' lower and upper halves, rows 8 (r/4) + r%4 and that + 4, so step r of the sum
// over a tile's 32 rows takes these two rows, and q is read from LDS to match), and the accumulator
// of the product k^T v.  Per chunk: scores q k^T (DT * 16 MFMAs), masked and weighted by the decay
// powers and passed through LDS to become an A operand; o = scores v + decay^(i+1) q S (16 + DT * 16);
// S <- decay^n S + k^T (decay^(n-1-j) v) (DT * 16).  Rows of a short chunk beyond its n tokens are zero.
// cos_sin: float [tokens, rot], cosines then sines of each token's angles (made once per step by
// retention_angles_kernel, with the accurate routines), or null where nothing is rotated.
typedef __attribute__((ext_vector_type(16))) float f32x16;

__global__ void __launch_bounds__(256)
retention_angles_kernel(const int32_t* __restrict__ positions, const float* __restrict__ inv_freq, int half,
                        float* __restrict__ cos_sin, int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const int64_t t = e / half;
    const int i = (int)(e % half);
    float sn, cs;
    sincosf((float)positions[t] * inv_freq[i], &sn, &cs);
    cos_sin[t * 2 * half + i] = cs;
    cos_sin[t * 2 * half + half + i] = sn;
}

#define RET_MFMA_WAVES 4

// Eight consecutive elements as they were loaded (16 bytes of bfloat16, 32 of float), widened when used.
template <typename T> struct Raw8;
template <> struct Raw8<__bf16> {
    typedef __attribute__((ext_vector_type(8))) __bf16 v8;
    v8 v;
    __device__ __forceinline__ void load(const __bf16* p) { v = *reinterpret_cast<const v8*>(p); }
    __device__ __forceinline__ float get(int i) const { return static_cast<float>(v[i]); }
};
template <> struct Raw8<float> {
    float4 a, b;
    __device__ __forceinline__ void load(const float* p) {
        a = reinterpret_cast<const float4*>(p)[0];
        b = reinterpret_cast<const float4*>(p)[1];
    }
    __device__ __forceinline__ float get(int i) const {
        return i == 0 ? a.x : i == 1 ? a.y : i == 2 ? a.z : i == 3 ? a.w : i == 4 ? b.x : i == 5 ? b.y : i == 6 ? b.z : b.w;
    }
};

__host__ __device__ inline size_t ret_mfma_lds_floats(int dim, int waves) {
    return (size_t)2 * RET_C * (dim + 1) + (size_t)waves * 2 * RET_C * (RET_C + 1) + 64;
}

// A long portion is cut into blocks of `bt` tokens (units: int32 [n][4] = request, first token of the
// block within the portion, its tokens, blocks of the portion) that run side by side, each from a
// zero state but the first: mode 0 leaves a block's outputs without what the state at its start
// would give, and the block's own end state in scratch[unit] (a portion of one block writes the
// request's slot itself); retention_scan_kernel then makes every block's true end state,
// E_b = decay^len_b E_(b-1) + (end state from zero), and the request's new state; mode 1 adds
// decay^(i+1) q_i E_(b-1) to the outputs of every block but the first.  units null: one block a request.
// NW: waves of the workgroup.  vec: rows, offsets and the rotation allow loads of eight elements; the
// chunk after the one at hand is then asked for before the products start and waits in registers.
template <typename T, int DT, int NW>
__global__ void __launch_bounds__(NW * NVA_WAVE)
retention_mfma_kernel(const T* __restrict__ proj, int64_t stride, float* __restrict__ o_raw, int64_t o_stride,
                      float* __restrict__ state, const int32_t* __restrict__ cu_seqlens_q,
                      const int32_t* __restrict__ seq_starts, const int32_t* __restrict__ state_slots,
                      const float* __restrict__ decay_pow, const float* __restrict__ cos_sin, int rot,
                      int heads, int vdim, float k_scale, int vec, const int32_t* __restrict__ units,
                      float* __restrict__ scratch, int mode) {
    static_assert(RET_C == 32, "a chunk is one MFMA tile of rows");
    constexpr int D = 32 * DT, DS = D + 1, VS = RET_C + 1;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int waves = NW;
    const int wave = threadIdx.x / NVA_WAVE;
    float* const q_s = lds;                                   // [32][DS], all waves'
    float* const k_s = q_s + RET_C * DS;                      // [32][DS]
    float* const pw_s = k_s + RET_C * DS;                     // [33] (+ padding to 64)
    float* const v_s = pw_s + 64 + wave * 2 * RET_C * VS;     // [32][33], this wave's
    float* const a_s = v_s + RET_C * VS;                      // [32][33]

    const int lane = threadIdx.x % NVA_WAVE, col = lane & 31, up = lane >> 5;
    const int nslices = vdim / 32, groups = (nslices + waves - 1) / waves;
    const int h = blockIdx.x / groups;
    const int slice = (blockIdx.x % groups) * waves + wave;
    const bool active = slice < nslices;                      // a wave without a slice only helps to load q and k
    const int c0 = 32 * (active ? slice : 0);
    int seq = blockIdx.y, first_token = 0, unit_len = -1, blocks = 1;
    if (units) {
        const int32_t* u = units + 4 * (int64_t)blockIdx.y;
        seq = u[0], first_token = u[1], unit_len = u[2], blocks = u[3];
    }
    if (mode == 1 && first_token == 0) return;                  // a first block has its state from the start
    const int q_begin = cu_seqlens_q[seq] + first_token;
    const int q_len = units ? unit_len : cu_seqlens_q[seq + 1] - q_begin;
    // a block after the first starts from zero (mode 0) or reads the block before's end state (mode 1)
    const int start = first_token == 0 ? seq_starts[seq] : 0;
    const int slot = state_slots[seq];
    float* const s_slot = state + (((int64_t)slot * heads + h) * D) * vdim + c0 + col;
    float* const s_unit = scratch ? scratch + (((int64_t)blockIdx.y * heads + h) * D) * vdim + c0 + col : s_slot;
    const float* const s_from = mode == 1 ? s_unit - (int64_t)heads * D * vdim : s_slot;
    float* const s_to = blocks == 1 ? s_slot : s_unit;
    const int half = rot / 2;
    const int64_t q_off = (int64_t)h * D, k_off = (int64_t)(heads + h) * D;
    const int64_t v_off = (int64_t)2 * heads * D + (int64_t)h * vdim + c0;
    // register r of an accumulator tile holds row rowmap(r) of the tile in this lane's half of the wave
    auto rowmap = [&](int r) { return 8 * (r >> 2) + 4 * up + (r & 3); };

    if (threadIdx.x <= RET_C) pw_s[threadIdx.x] = decay_pow[(int64_t)h * (RET_C + 1) + threadIdx.x];
    f32x16 S[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            S[dt][r] = (start > 0 || mode == 1) && active ? s_from[(int64_t)(32 * dt + rowmap(r)) * vdim] : 0.f;
    float chunks_decay = 1.f;                     // decay^(32 c) at the block's chunk c (mode 1)

    // blocks of eight elements: of q and k [32][D / 8] over all threads, of v [32][4] over a wave's lanes
    constexpr int QK_BLOCKS = RET_C * D / 8, PQ = (QK_BLOCKS + NW * NVA_WAVE - 1) / (NW * NVA_WAVE);
    constexpr bool PREFETCH = PQ <= 4;
    constexpr int PQR = PREFETCH ? PQ : 1;
    Raw8<T> rq[PQR], rqp[PQR], rk[PQR], rkp[PQR], rv[2];
    float4 rcs[PQR][2], rsn[PQR][2];
    const bool fast = PREFETCH && vec;
    auto ask = [&](int t0) __attribute__((always_inline)) {
        const int n = min(RET_C, q_len - t0);
#pragma unroll
        for (int p = 0; p < PQR; ++p) {
            const int b = threadIdx.x + p * NW * NVA_WAVE;
            const int r = b / (D / 8), d = (b % (D / 8)) * 8;
            if (b < QK_BLOCKS && r < n) {
                const int64_t tok = q_begin + t0 + r;
                const T* row = proj + tok * stride;
                rq[p].load(row + q_off + d);
                rk[p].load(row + k_off + d);
                if (d < rot) {
                    const int partner = d < half ? d + half : d - half, i0 = d < half ? d : d - half;
                    rqp[p].load(row + q_off + partner);
                    rkp[p].load(row + k_off + partner);
                    const float* cs_row = cos_sin + tok * rot + i0;
                    rcs[p][0] = reinterpret_cast<const float4*>(cs_row)[0];
                    rcs[p][1] = reinterpret_cast<const float4*>(cs_row)[1];
                    rsn[p][0] = reinterpret_cast<const float4*>(cs_row + half)[0];
                    rsn[p][1] = reinterpret_cast<const float4*>(cs_row + half)[1];
                }
            }
        }
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int b = lane + p * NVA_WAVE, r = b >> 2, c = (b & 3) * 8;
            if (r < n) rv[p].load(proj + (int64_t)(q_begin + t0 + r) * stride + v_off + c);
        }
    };
    auto put = [&](int n) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < PQR; ++p) {
            const int b = threadIdx.x + p * NW * NVA_WAVE;
            const int r = b / (D / 8), d = (b % (D / 8)) * 8;
            if (b < QK_BLOCKS) {
                const bool lower = d < half;
                const float cs[8] = {rcs[p][0].x, rcs[p][0].y, rcs[p][0].z, rcs[p][0].w, rcs[p][1].x, rcs[p][1].y, rcs[p][1].z, rcs[p][1].w};
                const float sn[8] = {rsn[p][0].x, rsn[p][0].y, rsn[p][0].z, rsn[p][0].w, rsn[p][1].x, rsn[p][1].y, rsn[p][1].z, rsn[p][1].w};
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float qv = 0.f, kv = 0.f;
                    if (r < n) {
                        qv = rq[p].get(e), kv = rk[p].get(e);
                        if (d < rot) {
                            const float qp = rqp[p].get(e), kp = rkp[p].get(e);
                            qv = lower ? qv * cs[e] - qp * sn[e] : qv * cs[e] + qp * sn[e];
                            kv = lower ? kv * cs[e] - kp * sn[e] : kv * cs[e] + kp * sn[e];
                        }
                    }
                    q_s[r * DS + d + e] = qv;
                    k_s[r * DS + d + e] = kv * k_scale;
                }
            }
        }
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int b = lane + p * NVA_WAVE, r = b >> 2, c = (b & 3) * 8;
#pragma unroll
            for (int e = 0; e < 8; ++e) v_s[r * VS + c + e] = r < n ? rv[p].get(e) : 0.f;
        }
    };
    if (fast) ask(0);

    for (int t0 = 0; t0 < q_len; t0 += RET_C) {
        const int n = min(RET_C, q_len - t0);
        __syncthreads();                          // the chunk before is done with LDS
        if (fast) {
            put(n);
            if (t0 + RET_C < q_len) ask(t0 + RET_C);      // on its way during this chunk's products
        } else {
        for (int e = threadIdx.x; e < RET_C * D; e += blockDim.x) {
            const int r = e / D, d = e % D;
            float qv = 0.f, kv = 0.f;
            if (r < n) {
                const int64_t tok = q_begin + t0 + r;
                const T* row = proj + tok * stride;
                qv = to_float(row[q_off + d]);
                kv = to_float(row[k_off + d]);
                if (d < rot) {
                    const bool lower = d < half;
                    const int partner = lower ? d + half : d - half;
                    const float* cs_row = cos_sin + tok * rot;
                    const float cs = cs_row[lower ? d : d - half], sn = cs_row[half + (lower ? d : d - half)];
                    const float qp = to_float(row[q_off + partner]), kp = to_float(row[k_off + partner]);
                    qv = lower ? qv * cs - qp * sn : qv * cs + qp * sn;
                    kv = lower ? kv * cs - kp * sn : kv * cs + kp * sn;
                }
            }
            q_s[r * DS + d] = qv;
            k_s[r * DS + d] = kv * k_scale;
        }
        for (int e = lane; e < RET_C * 32; e += NVA_WAVE) {
            const int r = e >> 5, c = e & 31;
            v_s[r * VS + c] = r < n ? to_float(proj[(int64_t)(q_begin + t0 + r) * stride + v_off + c]) : 0.f;
        }
        }
        __syncthreads();
        f32x16 acc;
        if (mode == 1) {
            // ---- what the state at the block's start gives, added to the outputs that are there
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = rowmap(r);
                acc[r] = i < n && active ? o_raw[(int64_t)(q_begin + t0 + i) * o_stride + (int64_t)h * vdim + c0 + col] : 0.f;
            }
            const float row_decay = pw_s[col + 1] * chunks_decay;
            const float* qa = q_s + col * DS + 4 * up;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[32 * dt + 8 * (r >> 2) + (r & 3)] * row_decay, S[dt][r],
                                                               acc, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = rowmap(r);
                if (i < n && active) o_raw[(int64_t)(q_begin + t0 + i) * o_stride + (int64_t)h * vdim + c0 + col] = acc[r];
            }
            chunks_decay *= pw_s[RET_C];
            continue;
        }
        // ---- scores: A[i][j] = q_i . k_j
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
        {
            const float* qa = q_s + col * DS + up;
            const float* kb = k_s + col * DS + up;
#pragma unroll 8
            for (int kk = 0; kk < D / 2; ++kk)
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[2 * kk], kb[2 * kk], acc, 0, 0, 0);
        }
        // masked and weighted by the decay's powers, then through LDS to become an A operand
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int i = rowmap(r);
            a_s[i * VS + col] = col <= i ? acc[r] * pw_s[i - col] : 0.f;
        }
        __syncthreads();
        // ---- outputs: o = A v + decay^(i+1) q S
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
        {
            const float* aa = a_s + col * VS + up;
            const float* vb = v_s + up * VS + col;
#pragma unroll
            for (int kk = 0; kk < RET_C / 2; ++kk)
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(aa[2 * kk], vb[2 * kk * VS], acc, 0, 0, 0);
            const float row_decay = pw_s[col + 1];
            const float* qa = q_s + col * DS + 4 * up;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[32 * dt + 8 * (r >> 2) + (r & 3)] * row_decay, S[dt][r],
                                                               acc, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int i = rowmap(r);
            if (i < n && active) o_raw[(int64_t)(q_begin + t0 + i) * o_stride + (int64_t)h * vdim + c0 + col] = acc[r];
        }
        // ---- the state after the chunk: S <- decay^n S + k^T (decay^(n-1-j) v)
        {
            const float all = pw_s[n];
            float vb[RET_C / 2];
#pragma unroll
            for (int kk = 0; kk < RET_C / 2; ++kk) {
                const int j = 2 * kk + up;
                vb[kk] = j < n ? v_s[j * VS + col] * pw_s[n - 1 - j] : 0.f;
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                for (int r = 0; r < 16; ++r) S[dt][r] *= all;
                const float* ka = k_s + up * DS + 32 * dt + col;
#pragma unroll
                for (int kk = 0; kk < RET_C / 2; ++kk)
                    S[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[2 * kk * DS], vb[kk], S[dt], 0, 0, 0);
            }
        }
    }
    if (!active || mode == 1) return;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) s_to[(int64_t)(32 * dt + rowmap(r)) * vdim] = S[dt][r];
}

// The blocks' end states from zero, one after the other, into their true end states, and the last
// into the request's slot.  chains: int32 [n][4] = first unit, blocks, request, tokens of the last block.
__global__ void __launch_bounds__(256)
retention_scan_kernel(float* __restrict__ scratch, float* __restrict__ state, const int32_t* __restrict__ chains,
                      const int32_t* __restrict__ state_slots, const float* __restrict__ decay_pow, int heads,
                      int64_t per_head, int bt) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= heads * per_head) return;
    const int32_t* c = chains + 4 * (int64_t)blockIdx.y;
    const int first_unit = c[0], blocks = c[1], seq = c[2], last_len = c[3];
    const float* pw = decay_pow + (e / per_head) * (RET_C + 1);
    float whole = 1.f, last = pw[last_len % RET_C];
    for (int i = 0; i < bt / RET_C; ++i) whole *= pw[RET_C];
    for (int i = 0; i < last_len / RET_C; ++i) last *= pw[RET_C];
    const int64_t unit = heads * per_head;
    float* at = scratch + (int64_t)first_unit * unit + e;
    float E = at[0];
    for (int b = 1; b < blocks; ++b) {
        E = (b == blocks - 1 ? last : whole) * E + at[b * unit];
        at[b * unit] = E;
    }
    state[(int64_t)state_slots[seq] * unit + e] = E;
}

// y[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * silu(g[t, h, :]); one wave per (token, head).
template <typename T>
__global__ void __launch_bounds__(NVA_WAVE)
retention_finish_kernel(const float* __restrict__ o_raw, int64_t o_stride, const T* __restrict__ gate, int64_t g_stride,
                        T* __restrict__ y, int64_t y_stride, int vdim, float eps) {
    const int64_t t = blockIdx.x;
    const int h = blockIdx.y, lane = threadIdx.x;
    const float* o = o_raw + t * o_stride + (int64_t)h * vdim;
    const T* g = gate + t * g_stride + (int64_t)h * vdim;
    T* out = y + t * y_stride + (int64_t)h * vdim;
    float ss = 0.f;
    for (int c = lane; c < vdim; c += NVA_WAVE) ss += o[c] * o[c];
    ss = wave_sum(ss);
    const float scale = rsqrtf(ss / (float)vdim + eps);
    for (int c = lane; c < vdim; c += NVA_WAVE) {
        const float gv = to_float(g[c]);
        out[c] = from_float<T>(o[c] * scale * (gv / (1.f + expf(-gv))));
    }
}

// proj: [tokens, 2 * heads * dim + 2 * heads * vdim] = [q | k | v | g], rows `stride` elements apart.
// o_raw: float [tokens, heads * vdim] scratch.  y: [tokens, heads * vdim] elements.
// state: float [slots, heads, dim, vdim].  decay_pow: float [heads, RET_C + 1], decay_h^m.
// inv_freq: float [rot / 2] (rot 0: no rotation).  vslice: value channels per workgroup (1..32).
// matrix_cores != 0: heads of a multiple of 32 channels (up to 256) and values of a multiple of 32 run
// the MFMA kernel, which wants the tokens' positions and float [tokens, rot] of scratch for the angles.
NVA_EXPORT int NVA_NAME(nva_retention)(const void* proj, int64_t stride, float* o_raw, void* y, int64_t y_stride,
                                       float* state, int64_t num_slots, const int32_t* cu_seqlens_q,
                                       const int32_t* seq_starts, const int32_t* state_slots, int64_t num_seqs,
                                       int64_t tokens, const float* decay_pow, const float* inv_freq, int rot,
                                       int heads, int dim, int vdim, int vslice, float k_scale, float eps,
                                       const int32_t* positions, float* cos_sin, int matrix_cores, int64_t num_decode,
                                       const int32_t* units, int64_t num_units, const int32_t* chains,
                                       int64_t num_chains, int block_tokens, float* block_states, hipStream_t stream) {
    if (num_seqs == 0 || tokens == 0) return 0;
    if (num_seqs < 0 || num_seqs > 65535 || tokens < 0 || tokens > 0x7fffffff)
        return nva_fail("retention: bad counts requests=%lld tokens=%lld", (long long)num_seqs, (long long)tokens);
    if (heads <= 0 || heads > 65535 || dim <= 0 || vdim <= 0 || vslice <= 0 || vslice > RET_MAX_VSLICE)
        return nva_fail("retention: bad sizes heads=%d dim=%d vdim=%d vslice=%d", heads, dim, vdim, vslice);
    if (rot < 0 || rot % 2 || rot > dim || (rot && !inv_freq))
        return nva_fail("retention: %d rotated channels of a head of %d", rot, dim);
    const int64_t width = (int64_t)2 * heads * dim + (int64_t)2 * heads * vdim;
    if (stride < width || y_stride < (int64_t)heads * vdim) return nva_fail("retention: rows are too short");
    if (!proj || !o_raw || !y || !state || !cu_seqlens_q || !seq_starts || !state_slots || !decay_pow || num_slots <= 0)
        return nva_fail("retention: a needed tensor is missing");
    const elem_t* p = (const elem_t*)proj;
    const elem_t* gate = p + (int64_t)2 * heads * dim + (int64_t)heads * vdim;
    // The first num_decode requests bring one token each (the caller puts them first): their kernel
    // streams the state; the portions after them run in chunks.
    if (num_decode < 0 || num_decode > num_seqs) return nva_fail("retention: %lld single tokens of %lld requests", (long long)num_decode, (long long)num_seqs);
    if (num_decode > 0 && dim <= 8 * RET_DEC_ROWS) {
        const int nsl = (vdim + 31) / 32;
        hipLaunchKernelGGL((retention_decode_kernel<elem_t>), dim3((unsigned)(heads * nsl), (unsigned)num_decode), dim3(256), 0,
                           stream, p, stride, o_raw, (int64_t)heads * vdim, state, cu_seqlens_q, seq_starts, state_slots,
                           decay_pow, inv_freq, rot, heads, dim, vdim, nsl, k_scale);
        int rc = nva_check_launch("retention (single tokens)");
        if (rc) return rc;
        cu_seqlens_q += num_decode, seq_starts += num_decode, state_slots += num_decode;
        num_seqs -= num_decode;
        if (num_seqs == 0) {
            hipLaunchKernelGGL((retention_finish_kernel<elem_t>), dim3((unsigned)tokens, (unsigned)heads), dim3(NVA_WAVE), 0,
                               stream, o_raw, (int64_t)heads * vdim, gate, stride, (elem_t*)y, y_stride, vdim, eps);
            return nva_check_launch("retention_finish");
        }
    }
    if (matrix_cores && dim % 32 == 0 && dim <= 256 && vdim % 32 == 0) {
        // positions: int32 [tokens]; cos_sin: float [tokens, rot] scratch (both needed with a rotation)
        if (rot && (!positions || !cos_sin)) return nva_fail("retention: the rotation needs positions and room for the angles");
        if (rot) {
            const int64_t total = tokens * (rot / 2);
            hipLaunchKernelGGL(retention_angles_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, positions,
                               inv_freq, rot / 2, cos_sin, total);
        }
        const int nsl = vdim / 32;
        const int waves = nsl <= 2 ? nsl : RET_MFMA_WAVES;
        // loads of eight elements: rows and parts of rows that start at multiples of eight elements, 16 bytes
        // aligned, and a rotation whose halves are multiples of eight channels
        const int vec = stride % 8 == 0 && nva_aligned(proj, 8 * sizeof(elem_t) > 16 ? 16 : 8 * sizeof(elem_t)) &&
                        rot % 16 == 0 && (!rot || nva_aligned(cos_sin, 16));
        const int groups = (nsl + waves - 1) / waves;
        const size_t bytes = ret_mfma_lds_floats(dim, waves) * sizeof(float);
        // units: the portions cut into blocks that run side by side (see retention_mfma_kernel); the requests
        // they name are counted from the first that brings a portion
        if (units && (num_units <= 0 || num_units > 65535 || !block_states || block_tokens < RET_C || block_tokens % RET_C ||
                      num_chains < 0 || num_chains > 65535 || (num_chains && !chains)))
            return nva_fail("retention: bad blocks (%lld units, %lld chains, %d tokens a block)", (long long)num_units,
                            (long long)num_chains, block_tokens);
        dim3 grid((unsigned)(heads * groups), (unsigned)(units ? num_units : num_seqs));
        for (int mode = 0; mode < (units && num_chains ? 2 : 1); ++mode) {
        if (mode == 1) {
            const int64_t per_head = (int64_t)dim * vdim;
            hipLaunchKernelGGL(retention_scan_kernel, dim3((unsigned)((heads * per_head + 255) / 256), (unsigned)num_chains),
                               dim3(256), 0, stream, block_states, state, chains, state_slots, decay_pow, heads, per_head,
                               block_tokens);
        }
#define RET_LAUNCH_W(DTT, NWW)                                                                                      \
        {                                                                                                           \
            auto kernel = retention_mfma_kernel<elem_t, DTT, NWW>;                                                   \
            static bool raised = false;                                                                              \
            if (!raised && bytes > 48 * 1024) {                                                                       \
                if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) \
                    return nva_fail("retention: cannot have %zu bytes of LDS", bytes);                               \
                raised = true;                                                                                       \
            }                                                                                                        \
            hipLaunchKernelGGL(kernel, grid, dim3(NWW * NVA_WAVE), bytes, stream, p, stride, o_raw,                 \
                               (int64_t)heads * vdim, state, cu_seqlens_q, seq_starts, state_slots, decay_pow, cos_sin, \
                               rot, heads, vdim, k_scale, vec, units, units ? block_states : nullptr, mode);         \
        }
#define RET_LAUNCH(DTT)                                                                                             \
        if (waves == 1) RET_LAUNCH_W(DTT, 1) else if (waves == 2) RET_LAUNCH_W(DTT, 2) else RET_LAUNCH_W(DTT, 4)
        switch (dim / 32) {
            case 1: RET_LAUNCH(1); break;
            case 2: RET_LAUNCH(2); break;
            case 3: RET_LAUNCH(3); break;
            case 4: RET_LAUNCH(4); break;
            case 5: RET_LAUNCH(5); break;
            case 6: RET_LAUNCH(6); break;
            case 7: RET_LAUNCH(7); break;
            default: RET_LAUNCH(8); break;
        }
#undef RET_LAUNCH_W
#undef RET_LAUNCH
        }
        int rc = nva_check_launch("retention (matrix cores)");
        if (rc) return rc;
        hipLaunchKernelGGL((retention_finish_kernel<elem_t>), dim3((unsigned)tokens, (unsigned)heads), dim3(NVA_WAVE), 0,
                           stream, o_raw, (int64_t)heads * vdim, gate, stride, (elem_t*)y, y_stride, vdim, eps);
        return nva_check_launch("retention_finish");
    }
    const int nslices = (vdim + vslice - 1) / vslice;
    if ((int64_t)heads * nslices > 0x7fffffff) return nva_fail("retention: too many workgroups");
    const size_t lds = ret_lds_floats(dim, vslice) * sizeof(float);
    if (lds > 160 * 1024) return nva_fail("retention: a head of %d channels does not fit the LDS", dim);
    auto kernel = retention_chunk_kernel<elem_t>;
    static size_t raised = 48 * 1024;
    if (lds > raised) {
        if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
            return nva_fail("retention: cannot have %zu bytes of LDS", lds);
        raised = 160 * 1024;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)(heads * nslices), (unsigned)num_seqs), dim3(RET_THREADS), lds, stream, p,
                       stride, o_raw, (int64_t)heads * vdim, state, cu_seqlens_q, seq_starts, state_slots, decay_pow,
                       inv_freq, rot, heads, dim, vdim, vslice, nslices, k_scale);
    int rc = nva_check_launch("retention");
    if (rc) return rc;
    hipLaunchKernelGGL((retention_finish_kernel<elem_t>), dim3((unsigned)tokens, (unsigned)heads), dim3(NVA_WAVE), 0, stream,
                       o_raw, (int64_t)heads * vdim, gate, stride, (elem_t*)y, y_stride, vdim, eps);
    return nva_check_launch("retention_finish");
}

NVA_EXPORT int NVA_NAME(nva_retention_chunk)() { return RET_C; }

NVA_DEFINE_LAST_ERROR(nva_retention)

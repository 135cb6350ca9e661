// The gated delta rule: a recurrent mixer with a matrix of state a head.
//
// Per row t of a sequence (G key heads of size dk, H value heads of size dv, value head h reads key
// head h / (H / G)), from the raw projections q, k, v [T, channels]:
//
//   prepare:     c  = silu(causal convolution over time, per channel, `taps` taps, zeros before position 0)
//                q' = unit(c_q) / sqrt(dk),  k' = unit(c_k),  unit(x) = x / sqrt(sum(x^2) + 1e-6),  v' = c_v
//                beta = sigmoid(b),  decay = exp(-exp(A_log) * softplus(a + dt_bias))
//   recurrence:  S <- decay S;  u = beta (v' - S^T k');  S <- S + k' u^T;  o = S^T q'
//   gated norm:  y = o / sqrt(mean(o^2) + eps) * w * silu(gate)         per head, over dv
//
// S is float32 [dk, dv] a head and lives in a slot of per-request state (in the order the recurrence
// kernel's lanes hold it, see there), as do the last taps - 1 raw rows that the convolution reads.  A sequence that starts at position 0 has no history: its slot is
// not read.  Everything after the projections is float32.
//
// The recurrence walks a sequence's rows one after the other.  Columns of S are independent, so a
// column belongs to 16 neighbouring lanes, each holding every 16th of its dk elements in registers; the
// two dot products of a row (k'.S and q'.S, both with the old S, since
// o = decay (q'.S_old) + (q'.k') u) are reduced over those lanes together.
#include "common.h"

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

// ---------------------------------------------------------------------------------------------
// prepare: a workgroup takes one row and one piece of it: a key head (its q and k vectors: convolution,
// silu, unit vectors, their dot product; piece 0 also the row's beta and decay), or 256 channels of v
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) delta_prepare_kernel(
    const T* __restrict__ proj, int ld, const float* __restrict__ conv_w, const T* __restrict__ kept,
    const float* __restrict__ ba, long long ba_row, long long ba_col, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, const int* __restrict__ positions, const int* __restrict__ seq_of_row,
    const int* __restrict__ row_start, const int* __restrict__ slots, float* __restrict__ qn, float* __restrict__ kn,
    float* __restrict__ vc, float* __restrict__ beta, float* __restrict__ decay, float* __restrict__ qk, int H, int G,
    int dk, int dv, int taps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x, piece = blockIdx.y;
    const int seq = seq_of_row[r], pos = positions[r];
    const int in_step = r - row_start[seq];        // rows of this sequence that stand before r in the step
    const int qd = G * dk, C = 2 * qd + H * dv;
    const T* mine = kept ? kept + (size_t)slots[seq] * (taps - 1) * C : nullptr;
    auto conv_silu = [&](int c) {
        float acc = 0.f;
        for (int j = 0; j < taps; ++j) {
            const int back = taps - 1 - j;          // the tap's row lies this many positions before r
            if (back > pos) continue;               // before the sequence's first position: zero
            float x;
            if (back <= in_step) x = to_f32(proj[(size_t)(r - back) * ld + c]);
            else x = to_f32(mine[(size_t)(taps - 1 + in_step - back) * C + c]);
            acc = fmaf(conv_w[(size_t)j * C + c], x, acc);
        }
        return silu_f(acc);
    };
    if (piece >= G) {
        const int c = (piece - G) * 256 + threadIdx.x;
        if (c < H * dv) vc[(size_t)r * H * dv + c] = conv_silu(2 * qd + c);
        return;
    }
    const int i = threadIdx.x;                      // dk <= 256: an element of q and of k a thread
    const bool has = i < dk;
    const float q = has ? conv_silu(piece * dk + i) : 0.f;
    const float k = has ? conv_silu(qd + piece * dk + i) : 0.f;
    const float sq = block_sum(q * q, scratch), sk = block_sum(k * k, scratch);
    const float qu = q * (1.0f / sqrtf(sq + 1e-6f)) * (1.0f / sqrtf((float)dk));
    const float ku = k * (1.0f / sqrtf(sk + 1e-6f));
    const float dot = block_sum(qu * ku, scratch);
    if (has) {
        qn[(size_t)r * qd + (size_t)piece * dk + i] = qu;
        kn[(size_t)r * qd + (size_t)piece * dk + i] = ku;
    }
    if (i == 0) qk[(size_t)r * G + piece] = dot;
    if (piece == 0 && i < H) {
        const float b = ba[(size_t)r * ba_row + (size_t)i * ba_col];
        const float a = ba[(size_t)r * ba_row + (size_t)(H + i) * ba_col] + dt_bias[i];
        beta[(size_t)r * H + i] = 1.0f / (1.0f + expf(-b));
        const float sp = fmaxf(a, 0.f) + log1pf(expf(-fabsf(a)));
        decay[(size_t)r * H + i] = expf(-expf(a_log[i]) * sp);
    }
}

// The last taps - 1 raw rows of every sequence become its kept rows (oldest first).  Row j of the
// new kept rows is row n - (taps - 1) + j of the step's n rows, or, where that is negative, kept row
// n + j of before (zero for a sequence with no history): always a row further on than the one
// written, so the rows are moved in ascending order in place.
template <typename T>
__global__ void delta_conv_keep_kernel(const T* __restrict__ proj, int ld, T* __restrict__ kept,
                                       const int* __restrict__ row_start, const int* __restrict__ seq_start,
                                       const int* __restrict__ slots, int C, int taps) {
    const int seq = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int r0 = row_start[seq], n = row_start[seq + 1] - r0;
    const bool fresh = seq_start[seq] == 0;
    T* mine = kept + (size_t)slots[seq] * (taps - 1) * C;
    for (int j = 0; j < taps - 1; ++j) {
        const int row = n - (taps - 1) + j;
        T x;
        if (row >= 0) x = proj[(size_t)(r0 + row) * ld + c];
        else if (fresh) from_f32(&x, 0.f);
        else x = mine[(size_t)(n + j) * C + c];
        mine[(size_t)j * C + c] = x;
    }
}

// ---------------------------------------------------------------------------------------------
// recurrence
// ---------------------------------------------------------------------------------------------
#define DELTA_LANES 16         // lanes that share a column of S: one row of 16 lanes, summed over with DPP moves
#define DELTA_COLS 16          // columns a workgroup of 256 threads walks

// Sum over the 16 lanes of a row, every lane gets it: neighbours, pairs (quad permutations), then the mirror
// image inside each half row and inside the row (by then the lanes of a quad, of a half row, hold the same).
__device__ __forceinline__ float row16_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));   // row_half_mirror
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));   // row_mirror
    return v;
}

template <int RPT>             // elements of a column a lane holds: dk <= 16 * RPT
__global__ __launch_bounds__(256) void delta_recurrence_kernel(
    const float* __restrict__ qn, const float* __restrict__ kn, const float* __restrict__ vc,
    const float* __restrict__ beta, const float* __restrict__ decay, const float* __restrict__ qk,
    float* __restrict__ state, float* __restrict__ out, const int* __restrict__ row_start,
    const int* __restrict__ seq_start, const int* __restrict__ slots, int H, int G, int dk, int dv) {
    // A sequence's rows pass through LDS in chunks of CT: the whole workgroup fetches a chunk with loads that
    // do not wait for each other (into registers, while the chunk before is worked on), so the walk along the
    // rows waits for LDS only.  In LDS an element i = part + 16 r of k or q lies at part * RPT + r: a lane's
    // share of a row is one run.
    constexpr int CT = RPT == 16 ? 16 : 32;      // rows a chunk (k and q of a chunk: 2 * CT * 16 RPT floats)
    constexpr int DKP = DELTA_LANES * RPT;
    constexpr int NK = CT * DKP / 256;           // elements of k (and of q) a thread fetches a chunk
    constexpr int NV = CT * DELTA_COLS / 256;    // of v
    __shared__ float ks[CT * DKP], qs[CT * DKP], vs[CT * DELTA_COLS], sc[3 * CT];
    const int seq = blockIdx.z, head = blockIdx.y;
    const int part = threadIdx.x % DELTA_LANES;
    const int local = threadIdx.x / DELTA_LANES;
    const int col_raw = blockIdx.x * DELTA_COLS + local;
    const bool live = col_raw < dv;
    const int col = live ? col_raw : dv - 1;
    const int kvh = head / (H / G);
    const int r0 = row_start[seq], r1 = row_start[seq + 1];
    const bool fresh = seq_start[seq] == 0;
    // The state of a slot: [head][block of 16 columns][r][column][part], element i = part + 16 r of a column: a
    // wave's 64 lanes read and write 64 floats in a row.  Elements past dk and columns past dv exist there too
    // (they stay 0: their k is 0, and the v of a column past dv is read as 0).
    float* mine = state + ((((size_t)slots[seq] * H + head) * gridDim.x + blockIdx.x) * RPT * DELTA_COLS + local) * DELTA_LANES + part;
    float S[RPT];
#pragma unroll
    for (int r = 0; r < RPT; ++r) S[r] = fresh ? 0.f : mine[(size_t)r * DELTA_COLS * DELTA_LANES];
    const size_t qd = (size_t)G * dk, vd = (size_t)H * dv;
    float pk[NK], pq[NK], pv[NV], ps = 0.f;
    auto fetch = [&](int c0) {                   // the chunk that starts at row c0, into registers
#pragma unroll
        for (int n = 0; n < NK; ++n) {
            const int e = threadIdx.x + n * 256, t = e / DKP, i = e % DKP;
            const bool ok = c0 + t < r1 && i < dk;
            pk[n] = ok ? kn[(size_t)(c0 + t) * qd + (size_t)kvh * dk + i] : 0.f;
            pq[n] = ok ? qn[(size_t)(c0 + t) * qd + (size_t)kvh * dk + i] : 0.f;
        }
#pragma unroll
        for (int n = 0; n < NV; ++n) {
            const int e = threadIdx.x + n * 256, t = e / DELTA_COLS, j = blockIdx.x * DELTA_COLS + e % DELTA_COLS;
            pv[n] = (c0 + t < r1 && j < dv) ? vc[(size_t)(c0 + t) * vd + (size_t)head * dv + j] : 0.f;
        }
        if (threadIdx.x < 3 * CT) {
            const int which = threadIdx.x / CT, t = threadIdx.x % CT;
            if (c0 + t < r1)
                ps = which == 0 ? beta[(size_t)(c0 + t) * H + head]
                                : which == 1 ? decay[(size_t)(c0 + t) * H + head] : qk[(size_t)(c0 + t) * G + kvh];
        }
    };
    if (r0 < r1) fetch(r0);
    for (int c0 = r0; c0 < r1; c0 += CT) {
        __syncthreads();                         // the chunk before has been walked
#pragma unroll
        for (int n = 0; n < NK; ++n) {
            const int e = threadIdx.x + n * 256, t = e / DKP, i = e % DKP;
            const int at = t * DKP + (i % DELTA_LANES) * RPT + i / DELTA_LANES;
            ks[at] = pk[n];
            qs[at] = pq[n];
        }
#pragma unroll
        for (int n = 0; n < NV; ++n) vs[threadIdx.x + n * 256] = pv[n];
        if (threadIdx.x < 3 * CT) sc[threadIdx.x] = ps;
        __syncthreads();
        if (c0 + CT < r1) fetch(c0 + CT);
        const int rows = min(CT, r1 - c0);
        // the row after the current one is read from LDS while the current one is worked on: two sets of
        // registers take turns, two rows a round of the loop
        auto read_row = [&](int t, float (&kx)[RPT], float (&qx)[RPT], float (&sx)[4]) {
            const float* kp = ks + t * DKP + part * RPT;
            const float* qp = qs + t * DKP + part * RPT;
#pragma unroll
            for (int r = 0; r < RPT; ++r) { kx[r] = kp[r]; qx[r] = qp[r]; }
            sx[0] = vs[t * DELTA_COLS + local];
            sx[1] = sc[t]; sx[2] = sc[CT + t]; sx[3] = sc[2 * CT + t];
        };
        auto walk_row = [&](int t, const float (&k)[RPT], const float (&q)[RPT], const float (&sx)[4]) {
            float d1[2] = {0.f, 0.f}, d2[2] = {0.f, 0.f};          // two sums each: shorter chains of dependent additions
#pragma unroll
            for (int r = 0; r < RPT; ++r) {
                d1[r & 1] = fmaf(k[r], S[r], d1[r & 1]);
                d2[r & 1] = fmaf(q[r], S[r], d2[r & 1]);
            }
            const float s1 = row16_sum(d1[0] + d1[1]), s2 = row16_sum(d2[0] + d2[1]);
            const float g0 = sx[2];
            const float u = sx[1] * (sx[0] - g0 * s1);
#pragma unroll
            for (int r = 0; r < RPT; ++r) S[r] = fmaf(k[r], u, g0 * S[r]);
            if (part == 0 && live) out[(size_t)(c0 + t) * vd + (size_t)head * dv + col] = fmaf(sx[3], u, g0 * s2);
        };
        float ka[RPT], qa[RPT], sa[4], kb[RPT], qb[RPT], sb[4];
        read_row(0, ka, qa, sa);
        int t = 0;
        for (; t + 1 < rows; t += 2) {
            read_row(t + 1, kb, qb, sb);
            walk_row(t, ka, qa, sa);
            read_row(min(t + 2, CT - 1), ka, qa, sa);
            walk_row(t + 1, kb, qb, sb);
        }
        if (t < rows) walk_row(t, ka, qa, sa);
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r) mine[(size_t)r * DELTA_COLS * DELTA_LANES] = S[r];
}

// ---------------------------------------------------------------------------------------------
// gated norm of the heads' outputs: one wave a (row, head)
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ o, const T* __restrict__ gate, int gate_ld,
                                     const float* __restrict__ weight, T* __restrict__ out, int H, int dv, float eps,
                                     long long pairs) {
    const long long p = (long long)blockIdx.x * (blockDim.x / TLI_WAVE) + threadIdx.x / TLI_WAVE;
    if (p >= pairs) return;
    const int lane = threadIdx.x % TLI_WAVE;
    const long long row = p / H;
    const int h = (int)(p - row * H);
    const float* x = o + (size_t)p * dv;
    const T* gt = gate + (size_t)row * gate_ld + (size_t)h * dv;
    float ss = 0.f;
    for (int i = lane; i < dv; i += TLI_WAVE) ss += x[i] * x[i];
    ss = wave_sum(ss);
    const float scale = 1.0f / sqrtf(ss / (float)dv + eps);
    T* y = out + (size_t)p * dv;
    for (int i = lane; i < dv; i += TLI_WAVE) from_f32(y + i, x[i] * scale * weight[i] * silu_f(to_f32(gt[i])));
}

// ---------------------------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------------------------
#define DELTA_MAX_DK 256

// proj: [T, ld] raw projections, channels q (G dk), k (G dk), v (H dv) first; conv_w: float32
// [taps, channels], oldest tap first; kept: [slots, taps - 1, channels] or null for one tap;
// ba: float32, b then a: number n of row t at t * ba_row + n * ba_col.  Outputs are float32: qn, kn [T, G dk], vc [T, H dv], beta, decay
// [T, H], qk [T, G].  `keep`: also move the kept rows on (after every row was read).
extern "C" int tli_delta_prepare(const void* proj, int ld, const float* conv_w, void* kept, const float* ba,
                                 long long ba_row, long long ba_col, const float* a_log, const float* dt_bias, const int* positions,
                                 const int* seq_of_row, const int* row_start, const int* seq_start, const int* slots,
                                 float* qn, float* kn, float* vc, float* beta, float* decay, float* qk, int T,
                                 int seqs, int H, int G, int dk, int dv, int taps, int dtype, void* stream) {
    if (T <= 0) return 0;
    if (H <= 0 || G <= 0 || H % G || dk <= 0 || dv <= 0 || taps <= 0)
        return tli_fail("delta_prepare: bad sizes (heads %d, key heads %d, dk %d, dv %d, taps %d)", H, G, dk, dv, taps);
    const int C = 2 * G * dk + H * dv;
    if (ld < C) return tli_fail("delta_prepare: rows of %d hold fewer than the %d channels", ld, C);
    if (taps > 1 && !kept) return tli_fail("delta_prepare: %d taps need the sequences' kept rows", taps);
    if (H > 256) return tli_fail("delta_prepare: at most 256 heads, got %d", H);
    if (dk > DELTA_MAX_DK) return tli_fail("delta_prepare: key heads of at most %d, got %d", DELTA_MAX_DK, dk);
    if (G + (H * dv + 255) / 256 > 65535) return tli_fail("delta_prepare: too many channels for one launch");
    const dim3 grid(T, G + (H * dv + 255) / 256);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TLI_F32) {
        hipLaunchKernelGGL((delta_prepare_kernel<float>), grid, dim3(256), 0, s, (const float*)proj, ld, conv_w,
                           (const float*)kept, ba, ba_row, ba_col, a_log, dt_bias, positions, seq_of_row, row_start, slots, qn, kn, vc,
                           beta, decay, qk, H, G, dk, dv, taps);
        if (taps > 1)
            hipLaunchKernelGGL((delta_conv_keep_kernel<float>), dim3((C + 255) / 256, seqs), dim3(256), 0, s,
                               (const float*)proj, ld, (float*)kept, row_start, seq_start, slots, C, taps);
    } else if (dtype == TLI_BF16) {
        hipLaunchKernelGGL((delta_prepare_kernel<bf16_t>), grid, dim3(256), 0, s, (const bf16_t*)proj, ld, conv_w,
                           (const bf16_t*)kept, ba, ba_row, ba_col, a_log, dt_bias, positions, seq_of_row, row_start, slots, qn, kn,
                           vc, beta, decay, qk, H, G, dk, dv, taps);
        if (taps > 1)
            hipLaunchKernelGGL((delta_conv_keep_kernel<bf16_t>), dim3((C + 255) / 256, seqs), dim3(256), 0, s,
                               (const bf16_t*)proj, ld, (bf16_t*)kept, row_start, seq_start, slots, C, taps);
    } else {
        return tli_fail("delta_prepare: unknown dtype %d", dtype);
    }
    return tli_check_launch("delta_prepare");
}

// Floats of state a head: columns in blocks of 16, key elements padded to 16 * RPT (RPT = 1, 2, 4, 8 or 16).
extern "C" int tli_delta_state_floats(int dk, int dv) {
    if (dk <= 0 || dv <= 0 || dk > DELTA_MAX_DK) return 0;
    const int rpt = dk <= 16 ? 1 : dk <= 32 ? 2 : dk <= 64 ? 4 : dk <= 128 ? 8 : 16;
    return ((dv + DELTA_COLS - 1) / DELTA_COLS) * rpt * DELTA_COLS * DELTA_LANES;
}

extern "C" int tli_delta_recurrence(const float* qn, const float* kn, const float* vc, const float* beta,
                                    const float* decay, const float* qk, float* state, float* out,
                                    const int* row_start, const int* seq_start, const int* slots, int seqs, int H,
                                    int G, int dk, int dv, void* stream) {
    if (seqs <= 0) return 0;
    if (H <= 0 || G <= 0 || H % G || dk <= 0 || dv <= 0 || dk > DELTA_MAX_DK)
        return tli_fail("delta_recurrence: bad sizes (heads %d, key heads %d, dk %d (at most %d), dv %d)", H, G, dk,
                        DELTA_MAX_DK, dv);
    if (H > 65535 || seqs > 65535) return tli_fail("delta_recurrence: too many heads or sequences for one launch");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((dv + DELTA_COLS - 1) / DELTA_COLS, H, seqs);
#define TLI_DELTA(RPT) hipLaunchKernelGGL((delta_recurrence_kernel<RPT>), grid, dim3(256), 0, s, qn, kn, vc, beta, \
                                          decay, qk, state, out, row_start, seq_start, slots, H, G, dk, dv)
    if (dk <= 16) TLI_DELTA(1);
    else if (dk <= 32) TLI_DELTA(2);
    else if (dk <= 64) TLI_DELTA(4);
    else if (dk <= 128) TLI_DELTA(8);
    else TLI_DELTA(16);
#undef TLI_DELTA
    return tli_check_launch("delta_recurrence");
}

extern "C" int tli_gated_rmsnorm(const float* o, const void* gate, int gate_ld, const float* weight, void* out,
                                 int T, int H, int dv, float eps, int dtype, void* stream) {
    if (T <= 0) return 0;
    if (H <= 0 || dv <= 0 || gate_ld < H * dv) return tli_fail("gated_rmsnorm: bad sizes");
    hipStream_t s = (hipStream_t)stream;
    const long long pairs = (long long)T * H;
    const int blocks = (int)((pairs + 3) / 4);
    if (dtype == TLI_F32)
        hipLaunchKernelGGL((gated_rmsnorm_kernel<float>), dim3(blocks), dim3(256), 0, s, o, (const float*)gate, gate_ld,
                           weight, (float*)out, H, dv, eps, pairs);
    else if (dtype == TLI_BF16)
        hipLaunchKernelGGL((gated_rmsnorm_kernel<bf16_t>), dim3(blocks), dim3(256), 0, s, o, (const bf16_t*)gate,
                           gate_ld, weight, (bf16_t*)out, H, dv, eps, pairs);
    else
        return tli_fail("gated_rmsnorm: unknown dtype %d", dtype);
    return tli_check_launch("gated_rmsnorm");
}

// Mixers that carry a state of fixed size from token to token instead of keys and values: the kernels of their
// recurrences, for prompt and decode steps alike.  Every state lives in float32 in the cache's state area, a row per
// sequence slot; a kernel finds a sequence's row through the step's device-side slot ids and its tokens either through
// a list of tiles (one tile a sequence: sequence, first row, rows, position of the first; a tile of no rows is skipped)
// or, tiles == null, as row b = the one new token of sequence b (seq_lens[b] == 0: a padding row, nothing is touched).
// Everything that enters a recurrence is float32: decays, gates, exponentials, the state; the projections that feed
// them arrive in the activations' type.  The order of every sum is a function of the sizes alone.
//
//   token shift   mix_s[t] = h[t] + (h[t-1] - h[t]) * mu_s; h[-1] of a step is the state's copy of the last h, 0 at position 0
//   wkv           o_t = (S + diag(u) k_t v_t^T)^T r_t;  S <- diag(w_t) S + k_t v_t^T;  w_t = exp(-exp(d_t + w0))   per head
//   head norm     y = o / sqrt(mean_head(o^2) + eps) * weight * silu(gate)
//   min-GRU       z = sigmoid(a + bz); c = b + bx; cand = c >= 0 ? c + 1/2 : sigmoid(c); S <- (1 - z) S + z cand; y = S silu(g)
#include "common.h"
#include <math.h>

struct SeqRange { int seq, row0, n, pos0; };

// A barrier of the workgroup that orders its shared memory only.  __syncthreads() also waits for everything that the wave
// has asked from or sent to global memory; this one leaves loads and stores in flight (whoever needs a load's data waits
// for it there), which is what lets a kernel ask for its next tokens before it walks the current ones.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ __forceinline__ SeqRange seq_range(const int* tiles, const int* seq_lens, int idx) {
    SeqRange r;
    if (tiles) {
        const int* t = tiles + 4 * idx;
        r.seq = t[0]; r.row0 = t[1]; r.n = t[2]; r.pos0 = t[3];
    } else {
        r.seq = idx; r.row0 = idx; r.pos0 = seq_lens[idx] - 1; r.n = r.pos0 >= 0 ? 1 : 0;
    }
    return r;
}

// ---- token shift ----------------------------------------------------------------------------------------------------
// out[s, t, :] for s < n_mix.  The previous row of the flattened batch is the previous token when it belongs to the same
// sequence; else the sequence's state holds it (zero at position 0).  The state is read only: the recurrence's
// kernel stores the step's last h afterwards, when every reader is done.
template <typename T>
__global__ void token_shift_kernel(T* __restrict__ out, const T* __restrict__ h, const float* __restrict__ mu,
                                   const float* __restrict__ state, size_t state_stride, const int* __restrict__ positions,
                                   const int* __restrict__ seq_index, const int* __restrict__ slot_ids, int T_rows, int D,
                                   int n_mix) {
    const int t = blockIdx.x;
    const int pos = positions[t], seq = seq_index[t];
    const int before = t > 0 ? t - 1 : 0;
    const int pos_b = positions[before], seq_b = seq_index[before], slot = slot_ids[seq];     // all asked for together
    const T* cur = h + (size_t)t * D;
    const bool inside = t > 0 && pos > 0 && seq_b == seq && pos_b == pos - 1;
    // both candidates for the previous row are loaded, from places that exist, and one is chosen: a load under a
    // branch would be waited for where it stands, element after element
    const T* prev_row = h + (size_t)(inside ? t - 1 : t) * D;
    const float* prev_state = state + (size_t)slot * state_stride;
#pragma unroll 4
    for (int e = threadIdx.x; e < D; e += blockDim.x) {
        const float c = to_f32(cur[e]);
        const float pr = to_f32(prev_row[e]), ps = prev_state[e];
        const float p = inside ? pr : (pos > 0 ? ps : 0.f);
        const float d = p - c;
        for (int s = 0; s < n_mix; ++s)
            out[((size_t)s * T_rows + t) * D + e] = from_f32<T>(pos >= 0 ? fmaf(d, mu[(size_t)s * D + e], c) : 0.f);
    }
}

extern "C" int bn_token_shift(int dtype, void* out, const void* h, const float* mu, const float* state,
                              long long state_stride, const int* positions, const int* seq_index, const int* slot_ids,
                              int n_tokens, int D, int n_mix, hipStream_t s) {
    if (n_tokens <= 0 || D <= 0 || n_mix <= 0 || !out || !h || !mu || !state || !positions || !seq_index || !slot_ids)
        return BN_ERR_ARG;
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(token_shift_kernel<float>, dim3(n_tokens), dim3(256), 0, s, (float*)out, (const float*)h, mu, state,
                           (size_t)state_stride, positions, seq_index, slot_ids, n_tokens, D, n_mix);
    else if (dtype == BN_DT_BF16)
        hipLaunchKernelGGL(token_shift_kernel<bf16>, dim3(n_tokens), dim3(256), 0, s, (bf16*)out, (const bf16*)h, mu, state,
                           (size_t)state_stride, positions, seq_index, slot_ids, n_tokens, D, n_mix);
    else
        return BN_ERR_DTYPE;
    return bn_launch_status();
}

// ---- the wkv recurrence -----------------------------------------------------------------------------------------------
// A workgroup owns (sequence, head, a block of CB value columns).  Column j of a head's state S[dk, dv] depends on no
// other column, so the columns are spread over threads and workgroups freely (the host picks CB so that a launch fills
// the chip); the dk rows of a column are spread over P threads (P a power of two <= 16, neighbouring lanes), each holding
// WKV_KR consecutive rows in registers, rows p WKV_KR .. p WKV_KR + WKV_KR - 1.  The tokens of a sequence come in chunks
// of TC: r, k, the decay and the block's v are staged in shared memory once a chunk (rows beyond dk zero, which leaves the
// unused registers zero) by waves of the workgroup that do nothing else: while the walking waves run a chunk's tokens
// without a barrier, every thread reading its rows 16 bytes at a time, the staging waves fill the other buffer with the
// next chunk, exponentials of the decay included, so the walk never waits for memory.  A column's sum over the rows is formed in four
// partial sums per thread and a butterfly over the P threads: an order that depends on the head size alone.
#define WKV_KR 16
#define WKV_MAX_DIM 256
#define WKV_MAX_THREADS 256

struct WkvArgs {
    const void* r; const void* k; const void* v; const void* d;     // [T, ld*]: head h at h * dk (v: h * dv)
    int ldr, ldk, ldv, ldd;
    const float* w0;          // [H * dk] added to d before the exponentials
    const float* u;           // [H * dk] the bonus of the current token
    float* o;                 // [T, H * dv] float32
    const void* h;            // [T, D]: the mixer's input, whose last row of every sequence becomes the state's copy
    float* state;             // [slots, state_stride]: S per head in the walkers' order (wkv_state_at), then D values of the last h
    size_t state_stride;
    const int* tiles; const int* seq_lens; const int* slot_ids;
    int H, dk, dv, D, P, CB, TC, walkers;
};

// The sum over the P neighbouring lanes that share a column, every lane getting it: a butterfly whose steps of 1 and
// 2 lanes are exchanges inside a group of four and whose steps of 4 and 8 lanes are mirrors of 8 and 16 lanes (after the
// first two steps a group of four holds one value, so a mirror meets the same partner group as an exchange would).
// Data-parallel moves inside a row of 16 lanes: no trip through shared memory.
__device__ __forceinline__ float wkv_lane_sum(float v, int P) {
    if (P >= 2) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));     // lanes 1 0 3 2
    if (P >= 4) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));     // lanes 2 3 0 1
    if (P >= 8) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));    // mirror of 8
    if (P >= 16) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));   // mirror of 16
    return v;
}

// One token of one column: o = sum_i r_i (S_i + u_i k_i v), then S_i <- w_i S_i + k_i v, over this thread's rows; the
// sum in four partial sums and the lanes' butterfly.
__device__ __forceinline__ float wkv_token(const float4 (&r4)[WKV_KR / 4], const float4 (&k4)[WKV_KR / 4],
                                           const float4 (&w4)[WKV_KR / 4], float vj, const float (&ub)[WKV_KR],
                                           float (&S)[WKV_KR], int P) {
    float part[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int q4 = 0; q4 < WKV_KR / 4; ++q4) {
        const float rv[4] = {r4[q4].x, r4[q4].y, r4[q4].z, r4[q4].w}, kv4[4] = {k4[q4].x, k4[q4].y, k4[q4].z, k4[q4].w},
                    wv[4] = {w4[q4].x, w4[q4].y, w4[q4].z, w4[q4].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int ii = q4 * 4 + e;
            const float kv = kv4[e] * vj;
            part[e] = fmaf(rv[e], fmaf(ub[ii], kv, S[ii]), part[e]);
            S[ii] = fmaf(wv[e], S[ii], kv);
        }
    }
    return wkv_lane_sum((part[0] + part[1]) + (part[2] + part[3]), P);
}

template <typename T>
__global__ __launch_bounds__(WKV_MAX_THREADS + 128) void wkv_scan_kernel(WkvArgs a) {
    extern __shared__ __align__(16) float smem[];
    const SeqRange sr = seq_range(a.tiles, a.seq_lens, blockIdx.x);
    if (sr.n <= 0 || sr.pos0 < 0) return;
    const int head = blockIdx.y, cb = blockIdx.z;
    const int P = a.P, dk = a.dk, dv = a.dv, TC = a.TC, CB = a.CB;
    const int dkp = P * WKV_KR;                           // staged rows, zero beyond dk
    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int n_walk = a.walkers;                         // the first n_walk threads walk the tokens, the rest stage them
    const bool walker = tid < n_walk;
    const int p = tid % P, jl = tid / P;
    const int j = cb * CB + jl;                           // a walker's value column
    const bool owns = walker && jl < CB && j < dv;
    const int buf_floats = TC * (3 * dkp + CB);           // one staged chunk: r, k, w as [TC][dkp], then v as [TC][CB]

    // A head's state lies in the order in which the walkers hold it: element (row p WKV_KR + ii, column j) at
    // (ii dv + j) P + p, so that the lanes of a wave, p fastest and then the columns, read and write runs of memory.
    float* S_g = a.state + (size_t)a.slot_ids[sr.seq] * a.state_stride + (size_t)head * dkp * dv;
    float S[WKV_KR], ub[WKV_KR];
#pragma unroll
    for (int ii = 0; ii < WKV_KR; ++ii) {
        const int i = p * WKV_KR + ii;
        S[ii] = (owns && sr.pos0 > 0) ? S_g[((size_t)ii * dv + j) * P + p] : 0.f;        // rows beyond dk hold zeros
        ub[ii] = (owns && i < dk) ? a.u[(size_t)head * dk + i] : 0.f;
    }

    // the staging threads' work: chunk c0 into buffer b
    auto stage = [&](int c0, int b) {
        float* r_s = smem + (size_t)b * buf_floats;
        float* k_s = r_s + TC * dkp;
        float* w_s = k_s + TC * dkp;
        float* v_s = w_s + TC * dkp;
        const int nc = min(TC, sr.n - c0), lt = tid - n_walk, nl = nthreads - n_walk;
        // eight elements a turn, their loads asked for together (unconditional loads from clamped places: a load
        // under a branch would make the compiler wait for each before the next)
        const int total = nc * dkp;
        for (int base = lt; base < total; base += 8 * nl) {
            float rv[8], kv[8], dv4[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int idx = min(base + q * nl, total - 1);
                const int tt = idx / dkp, i = min(idx - tt * dkp, dk - 1);
                const size_t row = (size_t)(sr.row0 + c0 + tt), c = (size_t)head * dk + i;
                rv[q] = to_f32(reinterpret_cast<const T*>(a.r)[row * a.ldr + c]);
                kv[q] = to_f32(reinterpret_cast<const T*>(a.k)[row * a.ldk + c]);
                dv4[q] = to_f32(reinterpret_cast<const T*>(a.d)[row * a.ldd + c]) + a.w0[c];
            }
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int idx = base + q * nl;
                if (idx < total) {
                    const bool in = idx % dkp < dk;
                    r_s[idx] = in ? rv[q] : 0.f;
                    k_s[idx] = in ? kv[q] : 0.f;
                    w_s[idx] = in ? expf(-expf(dv4[q])) : 0.f;
                }
            }
        }
        const int total_v = nc * CB;
        for (int base = lt; base < total_v; base += 4 * nl) {
            float vv[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int idx = min(base + q * nl, total_v - 1);
                const int tt = idx / CB, col = min(cb * CB + (idx - tt * CB), dv - 1);
                vv[q] = to_f32(reinterpret_cast<const T*>(a.v)[(size_t)(sr.row0 + c0 + tt) * a.ldv + (size_t)head * dv + col]);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int idx = base + q * nl;
                if (idx < total_v) v_s[idx] = cb * CB + idx % CB < dv ? vv[q] : 0.f;
            }
        }
    };

    if (!walker) stage(0, 0);
    lds_barrier();
    int b = 0;
    for (int c0 = 0; c0 < sr.n; c0 += TC, b ^= 1) {
        const int nc = min(TC, sr.n - c0);
        if (!walker) {
            if (c0 + TC < sr.n) stage(c0 + TC, b ^ 1);
        } else if (jl < CB) {
            const float* r_s = smem + (size_t)b * buf_floats;
            const float* k_s = r_s + TC * dkp;
            const float* w_s = k_s + TC * dkp;
            const float* v_s = w_s + TC * dkp;
            // two tokens a turn: both tokens' rows are asked for before the first is used, so the second's way from
            // shared memory is covered by the first's arithmetic
            for (int tt = 0; tt < nc; tt += 2) {
                const bool two = tt + 1 < nc;
                const int t1 = two ? tt + 1 : tt;
                float4 ra[WKV_KR / 4], ka[WKV_KR / 4], wa[WKV_KR / 4], rb[WKV_KR / 4], kb[WKV_KR / 4], wb[WKV_KR / 4];
#pragma unroll
                for (int q4 = 0; q4 < WKV_KR / 4; ++q4) {
                    ra[q4] = reinterpret_cast<const float4*>(r_s + tt * dkp + p * WKV_KR)[q4];
                    ka[q4] = reinterpret_cast<const float4*>(k_s + tt * dkp + p * WKV_KR)[q4];
                    wa[q4] = reinterpret_cast<const float4*>(w_s + tt * dkp + p * WKV_KR)[q4];
                }
                const float va = v_s[tt * CB + jl];
#pragma unroll
                for (int q4 = 0; q4 < WKV_KR / 4; ++q4) {
                    rb[q4] = reinterpret_cast<const float4*>(r_s + t1 * dkp + p * WKV_KR)[q4];
                    kb[q4] = reinterpret_cast<const float4*>(k_s + t1 * dkp + p * WKV_KR)[q4];
                    wb[q4] = reinterpret_cast<const float4*>(w_s + t1 * dkp + p * WKV_KR)[q4];
                }
                const float vb = v_s[t1 * CB + jl];
                const float acc_a = wkv_token(ra, ka, wa, va, ub, S, P);
                if (p == 0 && owns) a.o[(size_t)(sr.row0 + c0 + tt) * (a.H * dv) + (size_t)head * dv + j] = acc_a;
                if (two) {
                    const float acc_b = wkv_token(rb, kb, wb, vb, ub, S, P);
                    if (p == 0 && owns) a.o[(size_t)(sr.row0 + c0 + t1) * (a.H * dv) + (size_t)head * dv + j] = acc_b;
                }
            }
        }
        lds_barrier();                                    // the chunk has been walked and the next one is staged
    }
#pragma unroll
    for (int ii = 0; ii < WKV_KR; ++ii)
        if (owns) S_g[((size_t)ii * dv + j) * P + p] = S[ii];
    if (head == 0 && cb == 0) {                           // the step's last h of this sequence, for the next step's shift
        float* hp = a.state + (size_t)a.slot_ids[sr.seq] * a.state_stride + (size_t)a.H * dkp * dv;
        const T* last = reinterpret_cast<const T*>(a.h) + (size_t)(sr.row0 + sr.n - 1) * a.D;
        for (int e = tid; e < a.D; e += nthreads) hp[e] = to_f32(last[e]);
    }
}

// The split of a head over threads and workgroups (P, CB, TC, threads).  P follows from the head size alone (it fixes the
// order of a column's sum); CB, the columns of a workgroup, is the largest that still gives the launch `want_wgs`
// workgroups, down to one wave of threads, so that a prompt of one sequence spreads over the chip as a batch does.
static bool wkv_shape(int dk, int dv, int groups, int& P, int& CB, int& TC, int& walkers, int& threads) {
    if (dk < 1 || dv < 1 || dk > WKV_MAX_DIM || dv > WKV_MAX_DIM) return false;
    P = 1;
    while (P * WKV_KR < dk) P <<= 1;                      // <= 16
    const int most = WKV_MAX_THREADS / P, least = BN_WAVE / P;          // columns of a full set of walkers, of one wave
    CB = dv < most ? dv : most;
    while (CB > least && (long long)groups * ((dv + CB - 1) / CB) < 256) CB = (CB + 1) / 2 < least ? least : (CB + 1) / 2;
    walkers = ((CB * P + BN_WAVE - 1) / BN_WAVE) * BN_WAVE;
    threads = walkers + 128;                              // and the staging waves
    TC = 32;                                              // the longest chunk whose two buffers fit beside each other
    while (TC > 4 && (size_t)2 * TC * (3 * P * WKV_KR + CB) * sizeof(float) > 60 * 1024) TC >>= 1;
    return true;
}

extern "C" int bn_wkv_supports(int dk, int dv) {
    int P, CB, TC, wk, th;
    return wkv_shape(dk, dv, 1, P, CB, TC, wk, th) ? 1 : 0;
}

// float32 values of one head's state: dk rounded up to the rows that the walkers hold (a power of two times WKV_KR), times dv
extern "C" int bn_wkv_state_floats(int dk, int dv) {
    int P, CB, TC, wk, th;
    return wkv_shape(dk, dv, 1, P, CB, TC, wk, th) ? P * WKV_KR * dv : 0;
}

extern "C" int bn_wkv_scan(int dtype, const void* r, int ldr, const void* k, int ldk, const void* v, int ldv, const void* d,
                           int ldd, const float* w0, const float* u, float* o, const void* h, float* state,
                           long long state_stride, const int* tiles, int n_tiles, const int* seq_lens, const int* slot_ids,
                           int H, int dk, int dv, int D, hipStream_t s) {
    WkvArgs a;
    int threads;
    if (n_tiles <= 0 || H <= 0 || D <= 0 || !wkv_shape(dk, dv, n_tiles * H, a.P, a.CB, a.TC, a.walkers, threads)) return BN_ERR_ARG;
    if (!r || !k || !v || !d || !w0 || !u || !o || !h || !state || !slot_ids || (!tiles && !seq_lens)) return BN_ERR_ARG;
    if (state_stride < (long long)H * a.P * WKV_KR * dv + D) return BN_ERR_ARG;
    a.r = r; a.k = k; a.v = v; a.d = d; a.ldr = ldr; a.ldk = ldk; a.ldv = ldv; a.ldd = ldd;
    a.w0 = w0; a.u = u; a.o = o; a.h = h; a.state = state; a.state_stride = (size_t)state_stride;
    a.tiles = tiles; a.seq_lens = seq_lens; a.slot_ids = slot_ids;
    a.H = H; a.dk = dk; a.dv = dv; a.D = D;
    const size_t smem = (size_t)2 * a.TC * (3 * a.P * WKV_KR + a.CB) * sizeof(float);      // two staged chunks
    const dim3 grid(n_tiles, H, (dv + a.CB - 1) / a.CB);
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(wkv_scan_kernel<float>, grid, dim3(threads), smem, s, a);
    else if (dtype == BN_DT_BF16) hipLaunchKernelGGL(wkv_scan_kernel<bf16>, grid, dim3(threads), smem, s, a);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}

// ---- per-head RMS of the recurrence's output, its weight and the gate -----------------------------------------------
// one wave per (row, head): y = o / sqrt(mean(o^2) + eps) * weight * silu(gate)
template <typename T>
__global__ __launch_bounds__(BN_WAVE) void head_norm_gate_kernel(T* __restrict__ y, const float* __restrict__ o,
                                                                  const T* __restrict__ gate, int ldg,
                                                                  const float* __restrict__ weight, int H, int dv, float eps) {
    const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const float* ov = o + ((size_t)t * H + head) * dv;
    float ss = 0.f;
    for (int e = lane; e < dv; e += BN_WAVE) ss = fmaf(ov[e], ov[e], ss);
    ss = wave_sum(ss);
    const float f = 1.0f / sqrtf(ss / (float)dv + eps);
    for (int e = lane; e < dv; e += BN_WAVE) {
        const float g = to_f32(gate[(size_t)t * ldg + (size_t)head * dv + e]);
        y[((size_t)t * H + head) * dv + e] = from_f32<T>(ov[e] * f * weight[(size_t)head * dv + e] * bn_unary_act(g, BN_UNARY_SILU));
    }
}

extern "C" int bn_head_norm_gate(int dtype, void* y, const float* o, const void* gate, int ldg, const float* weight,
                                 int n_tokens, int H, int dv, float eps, hipStream_t s) {
    if (n_tokens <= 0 || H <= 0 || dv <= 0 || !y || !o || !gate || !weight || ldg < H * dv) return BN_ERR_ARG;
    const dim3 grid(n_tokens, H);
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(head_norm_gate_kernel<float>, grid, dim3(BN_WAVE), 0, s, (float*)y, o, (const float*)gate, ldg, weight, H, dv, eps);
    else if (dtype == BN_DT_BF16)
        hipLaunchKernelGGL(head_norm_gate_kernel<bf16>, grid, dim3(BN_WAVE), 0, s, (bf16*)y, o, (const bf16*)gate, ldg, weight, H, dv, eps);
    else
        return BN_ERR_DTYPE;
    return bn_launch_status();
}

// ---- min-GRU ------------------------------------------------------------------------------------------------------
// zxg [T, ld]: the three projections side by side (update gate at 0, candidate at W, output gate at 2 W), without their
// biases.  A workgroup owns GRU_CH channels of one sequence.  Its tokens come in stages of GRU_TC: all threads load a
// stage (the next one is asked for before the current one is walked), turn it into gate, candidate and silu(g) and
// park those in shared memory; one thread a channel then walks the stage, S <- S + z (cand - S), and leaves S silu(g),
// which all threads store.  The chain of a channel is the same operations in the same order whatever the step holds.
#define GRU_CH 64
#define GRU_TC 64
#define GRU_THREADS 256
#define GRU_PER_THREAD (GRU_CH * GRU_TC / GRU_THREADS)

template <typename T>
__global__ __launch_bounds__(GRU_THREADS) void mingru_scan_kernel(T* __restrict__ y, const T* __restrict__ zxg, int ld,
                                                                   const float* __restrict__ bz, const float* __restrict__ bx,
                                                                   float* __restrict__ state, size_t state_stride,
                                                                   const int* __restrict__ tiles, const int* __restrict__ seq_lens,
                                                                   const int* __restrict__ slot_ids, int W) {
    __shared__ float z_s[GRU_TC][GRU_CH], c_s[GRU_TC][GRU_CH], g_s[GRU_TC][GRU_CH];
    const SeqRange sr = seq_range(tiles, seq_lens, blockIdx.x);
    if (sr.n <= 0 || sr.pos0 < 0) return;
    const int tid = threadIdx.x;
    const int cc = tid % GRU_CH, t_first = tid / GRU_CH;            // this thread's channel and its first token of a stage
    const int c = blockIdx.y * GRU_CH + cc;
    const bool has = c < W;
    float* sp = state + (size_t)slot_ids[sr.seq] * state_stride + c;
    float S = (has && tid < GRU_CH && sr.pos0 > 0) ? *sp : 0.f;
    const float biasz = (has && bz) ? bz[c] : 0.f, biasx = (has && bx) ? bx[c] : 0.f;
    const T* in = zxg + (size_t)sr.row0 * ld + (has ? c : 0);
    T* out = y + (size_t)sr.row0 * W + c;
    float zr[GRU_PER_THREAD], cr[GRU_PER_THREAD], gr[GRU_PER_THREAD];
    auto fetch = [&](int t0) {
#pragma unroll
        for (int i = 0; i < GRU_PER_THREAD; ++i) {
            // unconditional loads from clamped places (a load under a branch is waited for where it stands); what a
            // thread without a channel or a token loads is never stored
            const int t = min(t0 + t_first + i * (GRU_THREADS / GRU_CH), sr.n - 1);
            zr[i] = to_f32(in[(size_t)t * ld]);
            cr[i] = to_f32(in[(size_t)t * ld + W]);
            gr[i] = to_f32(in[(size_t)t * ld + 2 * W]);
        }
    };
    fetch(0);
    for (int t0 = 0; t0 < sr.n; t0 += GRU_TC) {
#pragma unroll
        for (int i = 0; i < GRU_PER_THREAD; ++i) {
            const int tt = t_first + i * (GRU_THREADS / GRU_CH);
            const float cp = cr[i] + biasx;
            z_s[tt][cc] = 1.0f / (1.0f + expf(-(zr[i] + biasz)));
            c_s[tt][cc] = cp >= 0.f ? cp + 0.5f : 1.0f / (1.0f + expf(-cp));
            g_s[tt][cc] = bn_unary_act(gr[i], BN_UNARY_SILU);
        }
        lds_barrier();
        if (t0 + GRU_TC < sr.n) fetch(t0 + GRU_TC);
        const int nt = min(GRU_TC, sr.n - t0);
        if (tid < GRU_CH) {
            for (int tt = 0; tt < nt; tt += 8) {                    // eight tokens' values at once, then their chain
                float z8[8], c8[8], g8[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) { z8[i] = z_s[tt + i][cc]; c8[i] = c_s[tt + i][cc]; g8[i] = g_s[tt + i][cc]; }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (tt + i < nt) {
                        S = fmaf(z8[i], c8[i] - S, S);              // (1 - z) S + z cand
                        g_s[tt + i][cc] = S * g8[i];
                    }
                }
            }
        }
        lds_barrier();
#pragma unroll
        for (int i = 0; i < GRU_PER_THREAD; ++i) {
            const int tt = t_first + i * (GRU_THREADS / GRU_CH);
            if (has && tt < nt) out[(size_t)(t0 + tt) * W] = from_f32<T>(g_s[tt][cc]);
        }
        lds_barrier();
    }
    if (has && tid < GRU_CH) *sp = S;
}

extern "C" int bn_mingru_scan(int dtype, void* y, const void* zxg, int ld, const float* bz, const float* bx, float* state,
                              long long state_stride, const int* tiles, int n_tiles, const int* seq_lens,
                              const int* slot_ids, int W, hipStream_t s) {
    if (n_tiles <= 0 || W <= 0 || ld < 3 * W || !y || !zxg || !state || !slot_ids || (!tiles && !seq_lens)) return BN_ERR_ARG;
    if (state_stride < W) return BN_ERR_ARG;
    const dim3 grid(n_tiles, (W + GRU_CH - 1) / GRU_CH);
    if (dtype == BN_DT_F32)
        hipLaunchKernelGGL(mingru_scan_kernel<float>, grid, dim3(GRU_THREADS), 0, s, (float*)y, (const float*)zxg, ld, bz, bx, state,
                           (size_t)state_stride, tiles, seq_lens, slot_ids, W);
    else if (dtype == BN_DT_BF16)
        hipLaunchKernelGGL(mingru_scan_kernel<bf16>, grid, dim3(GRU_THREADS), 0, s, (bf16*)y, (const bf16*)zxg, ld, bz, bx, state,
                           (size_t)state_stride, tiles, seq_lens, slot_ids, W);
    else
        return BN_ERR_DTYPE;
    return bn_launch_status();
}

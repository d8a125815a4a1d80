// A mixture-of-experts feed-forward whose experts have no gate: expert e is  W_down[e] act(W_up[e] x).
//
//   bn_moe_route     router logits z = W_r h in float32 (one wave a token), scores sigmoid(z) or softmax(z), the top_k
//                    largest (ties: the lower index), optionally divided by their sum -> expert ids and weights [T, top_k]
//   bn_moe_experts   for every (token, choice) pair: y = W_down[e] act(W_up[e] (w h)) when the weight multiplies the
//                    expert's input, w * W_down[e] act(W_up[e] h) when it multiplies the output; one workgroup a pair, which
//                    reads the expert's two matrices once.  The products accumulate in float32; the scaled input and the
//                    hidden vector are rounded to the activations' type as a product of that type would see them.
//   bn_moe_plan      pairs ordered by expert, and tiles of up to MOE_TILE rows of one expert each, for the grouped products
//   bn_moe_grouped   (bf16) the same two products on the matrix cores over those tiles: a tile's rows share an expert
// The outputs of a token's choices land in slab j of y [top_k, T, D] (float32) and are added by whoever consumes y.
#include "common.h"
#include <math.h>

#define MOE_MAX_EXPERTS 1024
#define MOE_PER_LANE (MOE_MAX_EXPERTS / BN_WAVE)
#define MOE_SCORE_SIGMOID 0
#define MOE_SCORE_SOFTMAX 1

struct RouteArgs {
    const void* h;            // [T, ld]
    const float* wr;          // [E, D] float32
    int* ids;                 // [T, K]
    float* wts;               // [T, K]
    int ld, D, E, K, scoring, renorm;
};

template <typename T>
__global__ __launch_bounds__(BN_WAVE) void moe_route_kernel(RouteArgs a) {
    extern __shared__ float hs[];                        // the token's row as float32
    const int t = blockIdx.x, lane = threadIdx.x;
    const T* h = reinterpret_cast<const T*>(a.h) + (size_t)t * a.ld;
    for (int d = lane; d < a.D; d += BN_WAVE) hs[d] = to_f32(h[d]);
    __syncthreads();
    float z[MOE_PER_LANE];                               // expert lane + 64 j
#pragma unroll
    for (int j = 0; j < MOE_PER_LANE; ++j) z[j] = -INFINITY;
    for (int e = 0; e < a.E; ++e) {
        const float* w = a.wr + (size_t)e * a.D;
        float s = 0.f;
        for (int d = lane; d < a.D; d += BN_WAVE) s = fmaf(hs[d], w[d], s);
        s = wave_sum(s);
#pragma unroll
        for (int j = 0; j < MOE_PER_LANE; ++j)
            if (e == lane + BN_WAVE * j) z[j] = s;
    }
    float zmax = -INFINITY, denom = 1.f;
    if (a.scoring == MOE_SCORE_SOFTMAX) {
#pragma unroll
        for (int j = 0; j < MOE_PER_LANE; ++j) zmax = fmaxf(zmax, z[j]);
        zmax = wave_max(zmax);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < MOE_PER_LANE; ++j) sum += z[j] == -INFINITY ? 0.f : expf(z[j] - zmax);
        denom = wave_sum(sum);
    }
    float total = 0.f, mine_w = 0.f;
    int mine_id = 0;
    for (int k = 0; k < a.K; ++k) {
        float best = -INFINITY;
        int at = MOE_MAX_EXPERTS;
#pragma unroll
        for (int j = 0; j < MOE_PER_LANE; ++j)
            if (z[j] > best) { best = z[j]; at = lane + BN_WAVE * j; }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, BN_WAVE);
            const int oa = __shfl_xor(at, o, BN_WAVE);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
#pragma unroll
        for (int j = 0; j < MOE_PER_LANE; ++j)
            if (at == lane + BN_WAVE * j) z[j] = -INFINITY;
        const float score = a.scoring == MOE_SCORE_SOFTMAX ? expf(best - zmax) / denom : 1.0f / (1.0f + expf(-best));
        total += score;
        if (lane == k % BN_WAVE && k < BN_WAVE) { mine_w = score; mine_id = at; }
        if (k >= BN_WAVE && lane == 0) {                  // more choices than lanes: stored as they come
            a.ids[(size_t)t * a.K + k] = at;
            a.wts[(size_t)t * a.K + k] = score;
        }
    }
    const float norm = a.renorm ? 1.0f / total : 1.0f;
    if (lane < a.K) {
        a.ids[(size_t)t * a.K + lane] = mine_id;
        a.wts[(size_t)t * a.K + lane] = mine_w * norm;
    }
    if (a.renorm && a.K > BN_WAVE && lane == 0)
        for (int k = BN_WAVE; k < a.K; ++k) a.wts[(size_t)t * a.K + k] *= norm;
}

extern "C" int bn_moe_route(int dtype, const void* h, int ld, const float* wr, int* ids, float* wts, int n_tokens, int D, int E,
                            int K, int scoring, int renorm, hipStream_t s) {
    if (n_tokens <= 0 || D <= 0 || E <= 0 || E > MOE_MAX_EXPERTS || K <= 0 || K > E || ld < D || !h || !wr || !ids || !wts)
        return BN_ERR_ARG;
    if (scoring != MOE_SCORE_SIGMOID && scoring != MOE_SCORE_SOFTMAX) return BN_ERR_ARG;
    if ((size_t)D * sizeof(float) > 64 * 1024) return BN_ERR_ARG;
    RouteArgs a;
    a.h = h; a.wr = wr; a.ids = ids; a.wts = wts; a.ld = ld; a.D = D; a.E = E; a.K = K; a.scoring = scoring; a.renorm = renorm ? 1 : 0;
    const size_t shm = (size_t)D * sizeof(float);
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(moe_route_kernel<float>, dim3(n_tokens), dim3(BN_WAVE), shm, s, a);
    else if (dtype == BN_DT_BF16) hipLaunchKernelGGL(moe_route_kernel<bf16>, dim3(n_tokens), dim3(BN_WAVE), shm, s, a);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}

// ---- one workgroup a (token, choice) pair -----------------------------------------------------------------------------
#define MOE_PAIR_THREADS 256

struct PairArgs {
    const void* h;            // [T, ld]
    const void* w_up;         // [E, F, D]
    const void* w_down;       // [E, D, F]
    const int* ids;           // [T, K]
    const float* wts;         // [T, K]
    float* y;                 // [K, T, D]
    int ld, T, D, F, K, act, weight_on_input;
};

template <typename T>
__global__ __launch_bounds__(MOE_PAIR_THREADS) void moe_pair_kernel(PairArgs a) {
    extern __shared__ float sh[];                        // x [D], then hidden [F]
    float* xs = sh;
    float* hid = sh + a.D;
    const int pair = blockIdx.x, t = pair / a.K, j = pair - t * a.K;
    const int lane = threadIdx.x & (BN_WAVE - 1), wave = threadIdx.x / BN_WAVE, n_waves = MOE_PAIR_THREADS / BN_WAVE;
    const int e = a.ids[pair];
    const float wt = a.wts[pair];
    const float in_scale = a.weight_on_input ? wt : 1.0f, out_scale = a.weight_on_input ? 1.0f : wt;
    const T* h = reinterpret_cast<const T*>(a.h) + (size_t)t * a.ld;
    for (int d = threadIdx.x; d < a.D; d += MOE_PAIR_THREADS) xs[d] = to_f32(from_f32<T>(to_f32(h[d]) * in_scale));
    __syncthreads();
    const T* wu = reinterpret_cast<const T*>(a.w_up) + (size_t)e * a.F * a.D;
    for (int f = wave; f < a.F; f += n_waves) {
        const T* w = wu + (size_t)f * a.D;
        float s = 0.f;
        for (int d = lane; d < a.D; d += BN_WAVE) s = fmaf(xs[d], to_f32(w[d]), s);
        s = wave_sum(s);
        if (lane == 0) hid[f] = to_f32(from_f32<T>(bn_unary_act(s, a.act)));
    }
    __syncthreads();
    const T* wd = reinterpret_cast<const T*>(a.w_down) + (size_t)e * a.D * a.F;
    float* y = a.y + ((size_t)j * a.T + t) * a.D;
    for (int d = wave; d < a.D; d += n_waves) {
        const T* w = wd + (size_t)d * a.F;
        float s = 0.f;
        for (int f = lane; f < a.F; f += BN_WAVE) s = fmaf(hid[f], to_f32(w[f]), s);
        s = wave_sum(s);
        if (lane == 0) y[d] = s * out_scale;
    }
}

extern "C" int bn_moe_experts(int dtype, const void* h, int ld, const void* w_up, const void* w_down, const int* ids,
                              const float* wts, float* y, int n_tokens, int D, int F, int K, int act, int weight_on_input,
                              hipStream_t s) {
    if (n_tokens <= 0 || D <= 0 || F <= 0 || K <= 0 || ld < D || act < 0 || act >= BN_UNARY_KINDS) return BN_ERR_ARG;
    if (!h || !w_up || !w_down || !ids || !wts || !y || (size_t)(D + F) * sizeof(float) > 64 * 1024) return BN_ERR_ARG;
    PairArgs a;
    a.h = h; a.w_up = w_up; a.w_down = w_down; a.ids = ids; a.wts = wts; a.y = y;
    a.ld = ld; a.T = n_tokens; a.D = D; a.F = F; a.K = K; a.act = act; a.weight_on_input = weight_on_input ? 1 : 0;
    const size_t shm = (size_t)(D + F) * sizeof(float);
    const dim3 grid((unsigned)n_tokens * K), block(MOE_PAIR_THREADS);
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(moe_pair_kernel<float>, grid, block, shm, s, a);
    else if (dtype == BN_DT_BF16) hipLaunchKernelGGL(moe_pair_kernel<bf16>, grid, block, shm, s, a);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}

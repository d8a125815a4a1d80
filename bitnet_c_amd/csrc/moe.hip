// A mixture-of-experts feed-forward whose experts have no gate: expert e is  W_down[e] act(W_up[e] x).
//
//   bn_moe_route     router logits z = W_r h in float32 (one wave a token), scores sigmoid(z) or softmax(z), the top_k
//                    largest (ties: the lower index), optionally divided by their sum -> expert ids and weights [T, top_k]
//   bn_moe_experts   for every (token, choice) pair: y = W_down[e] act(W_up[e] (w h)) when the weight multiplies the
//                    expert's input, w * W_down[e] act(W_up[e] h) when it multiplies the output; a pair reads its expert's
//                    two matrices once, their rows spread over workgroups.  The products accumulate in float32; the scaled
//                    input and the hidden vector are rounded to the activations' type as a product of that type would
//                    see them.
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
        if (at >= a.E) at = k;                           // a row of NaNs (a padding row's garbage): still an expert that exists
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

// ---- a (token, choice) pair at a time ----------------------------------------------------------------------------------
// Steps of few rows: every pair reads its expert's two matrices once, and the rows of a matrix are spread over many
// workgroups so that one pair alone fills the chip (two launches: the hidden vector, then the output).  A workgroup stages
// the pair's input vector in shared memory as float32, each of its waves takes MOE_PAIR_ROWS / 4 rows of the matrix, a row
// as 16-byte loads across the lanes (bf16 rows of whole 8-element groups) or element by element, and sums in float32.
#define MOE_PAIR_THREADS 256
#define MOE_PAIR_ROWS 16

struct PairArgs {
    const void* h;            // [T, ld]
    const void* w_up;         // [E, F, D]
    const void* w_down;       // [E, D, F]
    const int* ids;           // [T, K]
    const float* wts;         // [T, K]
    float* hidden;            // [T K, F] float32 holding values of the activations' type
    float* y;                 // [K, T, D]
    int ld, T, D, F, K, act, weight_on_input;      // T: the rows of a slab of y
};

// sum over n of x[i] w[i]: x in shared memory, w a row in global memory; every lane gets the sum
template <typename T>
__device__ __forceinline__ float moe_row_dot(const T* __restrict__ w, const float* __restrict__ x, int n, int lane) {
    float s = 0.f;
    for (int i = lane; i < n; i += BN_WAVE) s = fmaf(x[i], to_f32(w[i]), s);
    return wave_sum(s);
}
template <>
__device__ __forceinline__ float moe_row_dot<bf16>(const bf16* __restrict__ w, const float* __restrict__ x, int n, int lane) {
    float s = 0.f;
    if (n % 8 == 0 && ((uintptr_t)w & 15) == 0) {
        for (int i = 8 * lane; i < n; i += 8 * BN_WAVE) {
            const uint4 p = *reinterpret_cast<const uint4*>(w + i);
            const float4 a = *reinterpret_cast<const float4*>(x + i), b = *reinterpret_cast<const float4*>(x + i + 4);
            s = fmaf(a.x, bf16lo_to_f32(p.x), s); s = fmaf(a.y, bf16hi_to_f32(p.x), s);
            s = fmaf(a.z, bf16lo_to_f32(p.y), s); s = fmaf(a.w, bf16hi_to_f32(p.y), s);
            s = fmaf(b.x, bf16lo_to_f32(p.z), s); s = fmaf(b.y, bf16hi_to_f32(p.z), s);
            s = fmaf(b.z, bf16lo_to_f32(p.w), s); s = fmaf(b.w, bf16hi_to_f32(p.w), s);
        }
    } else {
        for (int i = lane; i < n; i += BN_WAVE) s = fmaf(x[i], to_f32(w[i]), s);
    }
    return wave_sum(s);
}

// hidden[pair][f] = act(W_up[e][f] . (w h[t])) for the workgroup's rows f
template <typename T>
__global__ __launch_bounds__(MOE_PAIR_THREADS) void moe_pair_up_kernel(PairArgs a) {
    extern __shared__ __align__(16) float xs[];          // [D]
    const int pair = blockIdx.y, t = pair / a.K;
    const int lane = threadIdx.x & (BN_WAVE - 1), wave = threadIdx.x / BN_WAVE;
    const int e = a.ids[pair];
    const float in_scale = a.weight_on_input ? a.wts[pair] : 1.0f;
    const T* h = reinterpret_cast<const T*>(a.h) + (size_t)t * a.ld;
    for (int d = threadIdx.x; d < a.D; d += MOE_PAIR_THREADS) xs[d] = to_f32(from_f32<T>(to_f32(h[d]) * in_scale));
    __syncthreads();
    const T* wu = reinterpret_cast<const T*>(a.w_up) + (size_t)e * a.F * a.D;
    const int f0 = blockIdx.x * MOE_PAIR_ROWS;
    for (int f = f0 + wave; f < min(f0 + MOE_PAIR_ROWS, a.F); f += MOE_PAIR_THREADS / BN_WAVE) {
        const float s = moe_row_dot<T>(wu + (size_t)f * a.D, xs, a.D, lane);
        if (lane == 0) a.hidden[(size_t)pair * a.F + f] = to_f32(from_f32<T>(bn_unary_act(s, a.act)));
    }
}

// y[j][t][d] = W_down[e][d] . hidden[pair] (times w when the weight multiplies the output) for the workgroup's rows d
template <typename T>
__global__ __launch_bounds__(MOE_PAIR_THREADS) void moe_pair_down_kernel(PairArgs a) {
    extern __shared__ __align__(16) float hid[];         // [F]
    const int pair = blockIdx.y, t = pair / a.K, j = pair - t * a.K;
    const int lane = threadIdx.x & (BN_WAVE - 1), wave = threadIdx.x / BN_WAVE;
    const int e = a.ids[pair];
    const float out_scale = a.weight_on_input ? 1.0f : a.wts[pair];
    for (int f = threadIdx.x; f < a.F; f += MOE_PAIR_THREADS) hid[f] = a.hidden[(size_t)pair * a.F + f];
    __syncthreads();
    const T* wd = reinterpret_cast<const T*>(a.w_down) + (size_t)e * a.D * a.F;
    float* y = a.y + ((size_t)j * a.T + t) * a.D;
    const int d0 = blockIdx.x * MOE_PAIR_ROWS;
    for (int d = d0 + wave; d < min(d0 + MOE_PAIR_ROWS, a.D); d += MOE_PAIR_THREADS / BN_WAVE) {
        const float s = moe_row_dot<T>(wd + (size_t)d * a.F, hid, a.F, lane);
        if (lane == 0) y[d] = s * out_scale;
    }
}

// hidden: float32 work space [n_tokens K, F]; y_rows: the rows of a slab of y (>= n_tokens: the call may take a run of a
// step's tokens, y then points at the run's first row of slab 0)
extern "C" int bn_moe_experts(int dtype, const void* h, int ld, const void* w_up, const void* w_down, const int* ids,
                              const float* wts, float* y, float* hidden, int n_tokens, int y_rows, int D, int F, int K, int act,
                              int weight_on_input, hipStream_t s) {
    if (n_tokens <= 0 || y_rows < n_tokens || D <= 0 || F <= 0 || K <= 0 || ld < D || act < 0 || act >= BN_UNARY_KINDS) return BN_ERR_ARG;
    if (!h || !w_up || !w_down || !ids || !wts || !y || !hidden) return BN_ERR_ARG;
    if ((size_t)D * sizeof(float) > 64 * 1024 || (size_t)F * sizeof(float) > 64 * 1024 || (size_t)n_tokens * K > 65535) return BN_ERR_ARG;
    PairArgs a;
    a.h = h; a.w_up = w_up; a.w_down = w_down; a.ids = ids; a.wts = wts; a.y = y; a.hidden = hidden;
    a.ld = ld; a.T = y_rows; a.D = D; a.F = F; a.K = K; a.act = act; a.weight_on_input = weight_on_input ? 1 : 0;
    const dim3 block(MOE_PAIR_THREADS);
    const dim3 up((F + MOE_PAIR_ROWS - 1) / MOE_PAIR_ROWS, n_tokens * K), down((D + MOE_PAIR_ROWS - 1) / MOE_PAIR_ROWS, n_tokens * K);
    if (dtype == BN_DT_F32) {
        hipLaunchKernelGGL(moe_pair_up_kernel<float>, up, block, (size_t)D * sizeof(float), s, a);
        hipLaunchKernelGGL(moe_pair_down_kernel<float>, down, block, (size_t)F * sizeof(float), s, a);
    } else if (dtype == BN_DT_BF16) {
        hipLaunchKernelGGL(moe_pair_up_kernel<bf16>, up, block, (size_t)D * sizeof(float), s, a);
        hipLaunchKernelGGL(moe_pair_down_kernel<bf16>, down, block, (size_t)F * sizeof(float), s, a);
    } else return BN_ERR_DTYPE;
    return bn_launch_status();
}

// ---- grouped products on the matrix cores (bf16) ---------------------------------------------------------------------
// The pairs of a step are ordered by expert and cut into tiles of up to MOE_TILE rows of one expert; a workgroup takes one
// tile and 64 columns of the product, its four waves 16 columns each: a wave loads a 16 x 32 piece of the expert's matrix
// once and uses it for both 16-row halves of the tile (v_mfma_f32_16x16x32_bf16; the matrix as the first operand, so that
// a lane ends up with four consecutive result columns of one row: one store).  Operands come straight from memory, 16 bytes
// a lane; everything that a tile needs to know lies in device memory, so the launches do not depend on the routing.
#define MOE_TILE 32
#define MOE_PLAN_THREADS 1024

typedef __attribute__((ext_vector_type(8))) __bf16 moe_bf16x8;
typedef __attribute__((ext_vector_type(8))) float moe_f32x8;
typedef __attribute__((ext_vector_type(4))) float moe_f32x4;

// order [T K]: the pairs (t K + j) by expert; tiles [max_tiles][3] = expert, first place in `order`, rows; n_tiles [1]
__global__ __launch_bounds__(MOE_PLAN_THREADS) void moe_plan_kernel(const int* __restrict__ ids, int n_pairs, int E,
                                                                    int* __restrict__ order, int* __restrict__ tiles,
                                                                    int* __restrict__ n_tiles) {
    __shared__ int count[MOE_MAX_EXPERTS], first[MOE_MAX_EXPERTS + 1], tile0[MOE_MAX_EXPERTS + 1];
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) atomicAdd(&count[ids[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, tl = 0;
        for (int e = 0; e < E; ++e) {
            first[e] = at; tile0[e] = tl;
            at += count[e];
            tl += (count[e] + MOE_TILE - 1) / MOE_TILE;
        }
        first[E] = at; tile0[E] = tl;
        n_tiles[0] = tl;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        const int n = count[e];
        for (int r = 0, k = tile0[e]; r < n; r += MOE_TILE, ++k) {
            tiles[3 * k] = e; tiles[3 * k + 1] = first[e] + r; tiles[3 * k + 2] = min(MOE_TILE, n - r);
        }
        count[e] = 0;                                    // now the cursor of the scatter
    }
    __syncthreads();
    // the places inside an expert's run are handed out in whatever order the lanes arrive: a row's result does not depend
    // on its place
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const int e = ids[p];
        order[first[e] + atomicAdd(&count[e], 1)] = p;
    }
}

struct GroupedArgs {
    const bf16* x;            // up: h [T, ldx]; down: hidden [pairs, F] in the order of `order`
    const bf16* w;            // up: [E, F, D]; down: [E, D, F]
    bf16* hidden;             // up's result
    float* y;                 // down's result [K, T, D]
    const int* order;
    const int* tiles;
    const int* n_tiles;
    const float* wts;         // [T, K]
    int ldx, T, D, F, K, act, weight_on_input;
};

__device__ __forceinline__ moe_bf16x8 moe_ld16(const bf16* p) {
    return __builtin_bit_cast(moe_bf16x8, *reinterpret_cast<const uint4*>(p));
}

// hidden[place] = act(W_up[e] (w h[t]))  for the rows of a tile; N = F columns, the sum runs over D
__global__ __launch_bounds__(256) void moe_grouped_up_kernel(GroupedArgs a) {
    const int tile = blockIdx.x;
    if (tile >= a.n_tiles[0]) return;
    const int e = a.tiles[3 * tile], start = a.tiles[3 * tile + 1], rows = a.tiles[3 * tile + 2];
    const int lane = threadIdx.x & 63, i = lane & 15, g = lane >> 4;
    const int f0 = blockIdx.y * 64 + 16 * (threadIdx.x >> 6);
    if (f0 >= a.F) return;
    const bf16* wrow = a.w + ((size_t)e * a.F + f0 + i) * a.D + 8 * g;
    const bf16* xrow[2];
    float sc[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        const int pair = a.order[start + min(16 * s + i, rows - 1)];
        xrow[s] = a.x + (size_t)(pair / a.K) * a.ldx + 8 * g;
        sc[s] = a.weight_on_input ? a.wts[pair] : 1.0f;
    }
    moe_f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    for (int c = 0; c < a.D; c += 32) {
        const moe_bf16x8 wf = moe_ld16(wrow + c);
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            if (s == 1 && rows <= 16) break;
            moe_bf16x8 xf = moe_ld16(xrow[s] + c);
            if (a.weight_on_input) {                     // the expert reads w h, rounded to the activations' type
                moe_f32x8 xv = __builtin_convertvector(xf, moe_f32x8);
                xv *= sc[s];
                xf = __builtin_convertvector(xv, moe_bf16x8);
            }
            acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf, acc[s], 0, 0, 0);
        }
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        const int r = 16 * s + i;
        if (r >= rows) continue;
        bf16 o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) o[k] = __float2bfloat16(bn_unary_act(acc[s][k], a.act));
        uint2 pk;
        pk.x = (uint32_t)__builtin_bit_cast(unsigned short, o[0]) | ((uint32_t)__builtin_bit_cast(unsigned short, o[1]) << 16);
        pk.y = (uint32_t)__builtin_bit_cast(unsigned short, o[2]) | ((uint32_t)__builtin_bit_cast(unsigned short, o[3]) << 16);
        *reinterpret_cast<uint2*>(a.hidden + (size_t)(start + r) * a.F + f0 + 4 * g) = pk;
    }
}

// y[j][t] = W_down[e] hidden[place] (times w when the weight multiplies the output); N = D columns, the sum runs over F
__global__ __launch_bounds__(256) void moe_grouped_down_kernel(GroupedArgs a) {
    const int tile = blockIdx.x;
    if (tile >= a.n_tiles[0]) return;
    const int e = a.tiles[3 * tile], start = a.tiles[3 * tile + 1], rows = a.tiles[3 * tile + 2];
    const int lane = threadIdx.x & 63, i = lane & 15, g = lane >> 4;
    const int d0 = blockIdx.y * 64 + 16 * (threadIdx.x >> 6);
    if (d0 >= a.D) return;
    const bf16* wrow = a.w + ((size_t)e * a.D + d0 + i) * a.F + 8 * g;
    const bf16* xrow[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) xrow[s] = a.x + (size_t)(start + min(16 * s + i, rows - 1)) * a.F + 8 * g;
    moe_f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    for (int c = 0; c < a.F; c += 32) {
        const moe_bf16x8 wf = moe_ld16(wrow + c);
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            if (s == 1 && rows <= 16) break;
            acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, moe_ld16(xrow[s] + c), acc[s], 0, 0, 0);
        }
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        const int r = 16 * s + i;
        if (r >= rows) continue;
        const int pair = a.order[start + r], t = pair / a.K, j = pair - t * a.K;
        const float f = a.weight_on_input ? 1.0f : a.wts[pair];
        float4 o = make_float4(acc[s][0] * f, acc[s][1] * f, acc[s][2] * f, acc[s][3] * f);
        *reinterpret_cast<float4*>(a.y + ((size_t)j * a.T + t) * a.D + d0 + 4 * g) = o;
    }
}

// 1 if the grouped products take these sizes (the sums run over whole chunks of 32, the columns come in sixteens)
extern "C" int bn_moe_grouped_supports(int D, int F) { return (D > 0 && F > 0 && D % 32 == 0 && F % 32 == 0) ? 1 : 0; }
extern "C" int bn_moe_grouped_tiles(int n_pairs, int E) { return (n_pairs + MOE_TILE - 1) / MOE_TILE + E; }

// work: int32 [n_pairs + 3 max_tiles + 1] (order, tiles, n_tiles); hidden: bf16 [n_pairs, F]
extern "C" int bn_moe_grouped(const void* h, int ld, const void* w_up, const void* w_down, const int* ids, const float* wts,
                              float* y, int* work, void* hidden, int n_tokens, int D, int F, int E, int K, int act,
                              int weight_on_input, hipStream_t s) {
    if (n_tokens <= 0 || K <= 0 || E <= 0 || E > MOE_MAX_EXPERTS || !bn_moe_grouped_supports(D, F) || ld < D || ld % 8) return BN_ERR_ARG;
    if (act < 0 || act >= BN_UNARY_KINDS || !h || !w_up || !w_down || !ids || !wts || !y || !work || !hidden) return BN_ERR_ARG;
    if ((((uintptr_t)h | (uintptr_t)w_up | (uintptr_t)w_down | (uintptr_t)y | (uintptr_t)hidden) & 15)) return BN_ERR_ARG;
    const int n_pairs = n_tokens * K, max_tiles = bn_moe_grouped_tiles(n_pairs, E);
    int* order = work;
    int* tiles = work + n_pairs;
    int* n_tiles = tiles + 3 * max_tiles;
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(MOE_PLAN_THREADS), 0, s, ids, n_pairs, E, order, tiles, n_tiles);
    GroupedArgs a;
    a.x = (const bf16*)h; a.w = (const bf16*)w_up; a.hidden = (bf16*)hidden; a.y = y; a.order = order; a.tiles = tiles;
    a.n_tiles = n_tiles; a.wts = wts; a.ldx = ld; a.T = n_tokens; a.D = D; a.F = F; a.K = K; a.act = act;
    a.weight_on_input = weight_on_input ? 1 : 0;
    hipLaunchKernelGGL(moe_grouped_up_kernel, dim3(max_tiles, (F + 63) / 64), dim3(256), 0, s, a);
    a.x = (const bf16*)hidden; a.w = (const bf16*)w_down;
    hipLaunchKernelGGL(moe_grouped_down_kernel, dim3(max_tiles, (D + 63) / 64), dim3(256), 0, s, a);
    return bn_launch_status();
}

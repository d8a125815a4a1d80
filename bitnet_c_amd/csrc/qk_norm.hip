// What an attention mixer without a rotation does to its projected heads before they meet: an RMSNorm over each
// query and key head (one weight vector of the head size, shared by the heads; eps inside the root), a query
// temperature that grows with the position, and the write of the new keys and values into the pages.  One kernel
// for prompt and decode steps; all arithmetic in float32, the results stored in the activations' type.
//
//   q_h <- q_h / sqrt(mean(q_h^2) + eps) * wq * (1 + coef * ln(floor((p + 1) / every) + 1))
//   k_g <- k_g / sqrt(mean(k_g^2) + eps) * wk          -> page of position p
//   v_g                                                 -> page of position p
//
// Pages hold a row per position for the keys, [page, kv head, BN_PAGE, hs]; the values lie the same way ("rows" layout,
// [page, kv head, BN_PAGE, vd]) or transposed ([page, kv head, vd, BN_PAGE]), as the caller says.
#include "common.h"
#include <math.h>

struct QkNormArgs {
    void* qkv;                // [T, ld]: q heads (H x hs), k heads (Hkv x hs), v heads (Hkv x vd)
    const int* positions;     // [T]; < 0: a padding row, nothing is written
    const int* seq_index;     // [T] row of the block table
    const int* block_table;   // [n_seqs, bt_stride]
    void* k_pages;
    void* v_pages;            // both null: nothing is stored (the entry reads another entry's cache)
    const float* wq;          // [hs] or null: no norm
    const float* wk;
    int ld, bt_stride, H, Hkv, hs, vd;
    int v_transposed;         // the values' pages are [page, kv head, vd, BN_PAGE]
    float eps, temp_coef;
    int temp_every;           // <= 0: no temperature
};

// one wave per (row, head); heads 0 .. H-1 are queries, then Hkv keys, then Hkv values
template <typename T>
__global__ __launch_bounds__(BN_WAVE) void qk_norm_store_kernel(QkNormArgs a) {
    const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int pos = a.positions[t];
    if (pos < 0) return;
    T* row = reinterpret_cast<T*>(a.qkv) + (size_t)t * a.ld;
    const bool is_q = head < a.H, is_k = !is_q && head < a.H + a.Hkv;
    if (is_q || is_k) {
        T* v = row + (size_t)head * a.hs;
        const float* w = is_q ? a.wq : a.wk;
        float f = 1.0f;
        if (w) {
            float ss = 0.f;
            for (int d = lane; d < a.hs; d += BN_WAVE) { const float x = to_f32(v[d]); ss = fmaf(x, x, ss); }
            ss = wave_sum(ss);
            f = 1.0f / sqrtf(ss / (float)a.hs + a.eps);
        }
        float temp = 1.0f;
        if (is_q && a.temp_every > 0) temp = 1.0f + a.temp_coef * logf((float)((pos + 1) / a.temp_every) + 1.0f);
        T* dst = v;
        if (is_k) {
            if (!a.k_pages) return;
            const int kvh = head - a.H;
            const int page = a.block_table[(size_t)a.seq_index[t] * a.bt_stride + pos / BN_PAGE];
            dst = reinterpret_cast<T*>(a.k_pages) + (((size_t)page * a.Hkv + kvh) * BN_PAGE + pos % BN_PAGE) * a.hs;
        }
        for (int d = lane; d < a.hs; d += BN_WAVE) {
            float x = to_f32(v[d]);
            if (w) x = x * f * w[d];
            dst[d] = from_f32<T>(x * temp);
        }
    } else {
        if (!a.v_pages) return;
        const int kvh = head - a.H - a.Hkv;
        const T* v = row + (size_t)(a.H + a.Hkv) * a.hs + (size_t)kvh * a.vd;
        const int page = a.block_table[(size_t)a.seq_index[t] * a.bt_stride + pos / BN_PAGE];
        if (a.v_transposed) {
            T* dst = reinterpret_cast<T*>(a.v_pages) + ((size_t)page * a.Hkv + kvh) * a.vd * BN_PAGE + pos % BN_PAGE;
            for (int d = lane; d < a.vd; d += BN_WAVE) dst[(size_t)d * BN_PAGE] = v[d];
        } else {
            T* dst = reinterpret_cast<T*>(a.v_pages) + (((size_t)page * a.Hkv + kvh) * BN_PAGE + pos % BN_PAGE) * a.vd;
            for (int d = lane; d < a.vd; d += BN_WAVE) dst[d] = v[d];
        }
    }
}

extern "C" int bn_qk_norm_store(int dtype, void* qkv, int ld, const int* positions, const int* seq_index,
                                const int* block_table, int bt_stride, void* k_pages, void* v_pages, const float* wq,
                                const float* wk, int n_tokens, int H, int Hkv, int hs, int vd, float eps, float temp_coef,
                                int temp_every, int v_transposed, hipStream_t s) {
    if (n_tokens <= 0 || H <= 0 || Hkv <= 0 || hs <= 0 || vd <= 0 || !qkv || !positions) return BN_ERR_ARG;
    if ((k_pages == nullptr) != (v_pages == nullptr) || (k_pages && (!seq_index || !block_table))) return BN_ERR_ARG;
    if ((wq == nullptr) != (wk == nullptr) || ld < H * hs + Hkv * (hs + vd)) return BN_ERR_ARG;
    QkNormArgs a;
    a.qkv = qkv; a.positions = positions; a.seq_index = seq_index; a.block_table = block_table;
    a.k_pages = k_pages; a.v_pages = v_pages; a.wq = wq; a.wk = wk;
    a.ld = ld; a.bt_stride = bt_stride; a.H = H; a.Hkv = Hkv; a.hs = hs; a.vd = vd;
    a.eps = eps; a.temp_coef = temp_coef; a.temp_every = temp_every; a.v_transposed = v_transposed ? 1 : 0;
    const dim3 grid(n_tokens, H + 2 * Hkv);
    if (dtype == BN_DT_F32) hipLaunchKernelGGL(qk_norm_store_kernel<float>, grid, dim3(BN_WAVE), 0, s, a);
    else if (dtype == BN_DT_BF16) hipLaunchKernelGGL(qk_norm_store_kernel<bf16>, grid, dim3(BN_WAVE), 0, s, a);
    else return BN_ERR_DTYPE;
    return bn_launch_status();
}

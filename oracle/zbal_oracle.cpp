/*
 * TEST INFRASTRUCTURE — CPU restatement of the zbal MoE / reduce hot path.
 *
 * This file is the checker that the parity tests, the smoke test and the
 * cpu_baseline leg of the benchmark compare the HIP library against. Nothing
 * in the shipped library includes, links or calls it.
 *
 * Every function restates one reference routine in plain loops with the
 * reference's operation order; the routine is cited above each function
 * (paths relative to /root/reference/app/zbal/src/csrc, OPS =
 * operators/npu/aicore/ops, FDM = OPS/fused_deep_moe). All floating point is
 * IEEE binary32 with no contraction (build with -ffp-contract=off); fused
 * multiply-adds appear only where written as fmaf().
 *
 * The reference's device code (AscendC + Catlass) cannot be built without the
 * CANN toolkit, so there is no compiled reference to compare with; how each
 * function is pinned instead is stated in its comment. "parity unpinned" marks
 * the ones with no reference-held check at all:
 *   - zo_topk_route            parity unpinned (no router in the reference)
 *   - fp8 / W4A8 variants      parity unpinned (extensions; defined here)
 *   - zo_expf inside SwiGLU    parity unpinned against the Ascend Exp unit
 */
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>
#include <algorithm>

#if defined(_OPENMP)
#include <omp.h>
#endif

#define ZO_API extern "C" __attribute__((visibility("default")))

namespace {

/* ---- scalar formats -------------------------------------------------- */

inline float bits_f32(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
inline uint32_t f32_bits(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }

inline float bf16_to_f32(uint16_t h) { return bits_f32(uint32_t(h) << 16); }

/* round-to-nearest-even, NaN kept quiet */
inline uint16_t f32_to_bf16(float f)
{
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return uint16_t((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return uint16_t(u >> 16);
}

inline float fp16_to_f32(uint16_t h)
{
    uint32_t sign = uint32_t(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        float v = float(man) * 5.9604644775390625e-08f; /* 2^-24 */
        return (sign ? -v : v);
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

inline uint16_t f32_to_fp16(float f)
{
    uint32_t u = f32_bits(f);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return uint16_t(sign | 0x7e00u);
    if (a >= 0x477ff000u) { /* >= 65520 rounds to inf */
        return uint16_t(sign | 0x7c00u);
    }
    if (a < 0x38800000u) { /* below 2^-14: subnormal half, RNE via float arithmetic */
        float v = bits_f32(a) * 16777216.0f; /* * 2^24, exact */
        float r = std::nearbyintf(v);
        return uint16_t(sign | uint32_t(r));
    }
    uint32_t man = a & 0x7fffffu;
    uint32_t exp = (a >> 23) - 112u;
    uint32_t m = man >> 13;
    uint32_t rem = man & 0x1fffu;
    uint32_t out = (exp << 10) | m;
    if (rem > 0x1000u || (rem == 0x1000u && (m & 1u))) out += 1;
    return uint16_t(sign | out);
}

/* OCP e4m3fn: bias 7, no inf, 0x7f = NaN, max 448. RNE, saturating. */
inline uint8_t f32_to_e4m3(float f)
{
    uint32_t u = f32_bits(f);
    uint8_t sign = uint8_t((u >> 24) & 0x80u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return uint8_t(sign | 0x7f);
    float af = bits_f32(a);
    if (af >= 448.0f) return uint8_t(sign | 0x7e);
    if (af < 0.015625f) { /* < 2^-6: subnormal, step 2^-9 */
        float q = std::nearbyintf(af * 512.0f);
        return uint8_t(sign | uint8_t(q));
    }
    int32_t exp = int32_t(a >> 23) - 127;
    uint32_t man = a & 0x7fffffu;
    uint32_t m = man >> 20;
    uint32_t rem = man & 0xfffffu;
    uint32_t code = (uint32_t(exp + 7) << 3) | m;
    if (rem > 0x80000u || (rem == 0x80000u && (m & 1u))) code += 1;
    if (code > 0x7eu) code = 0x7eu;
    return uint8_t(sign | code);
}

inline float e4m3_to_f32(uint8_t c)
{
    uint32_t exp = (c >> 3) & 0xfu;
    uint32_t man = c & 7u;
    float v;
    if (exp == 15 && man == 7) return std::nanf("");
    if (exp == 0) v = float(man) * 0.001953125f; /* 2^-9 */
    else v = bits_f32(((exp + 120u) << 23) | (man << 20));
    return (c & 0x80u) ? -v : v;
}

enum { DT_FP16 = 6, DT_FP32 = 7, DT_BF16 = 8 }; /* zbal_datatype_t values */

inline float half_like_to_f32(uint16_t h, int dtype) { return dtype == DT_FP16 ? fp16_to_f32(h) : bf16_to_f32(h); }
inline uint16_t f32_to_half_like(float f, int dtype) { return dtype == DT_FP16 ? f32_to_fp16(f) : f32_to_bf16(f); }

/* round-half-even to integer, then clamp into int8 */
inline int8_t rint_i8(float v)
{
    float r = std::nearbyintf(v);
    if (r > 127.0f) r = 127.0f;
    if (r < -128.0f) r = -128.0f;
    return int8_t(int32_t(r));
}

/*
 * exp() used by the SwiGLU epilogue. The reference calls the Ascend vector
 * unit's Exp, whose bit pattern is not specified; the library fixes this
 * routine instead (Cody-Waite reduction by ln2, degree-6 polynomial evaluated
 * with fmaf, scaling by exact powers of two) and the HIP kernels evaluate the
 * identical sequence, so results agree bit for bit.
 */
inline float pow2i(int n) { return bits_f32(uint32_t(n + 127) << 23); } /* n in [-126, 127] */

inline float zo_expf_impl(float x)
{
    if (!(x == x)) return x;
    if (x > 88.72284f) return INFINITY;
    if (x < -103.97208f) return 0.0f;
    float n = std::nearbyintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693145751953125f, x);       /* ln2 high part (exact in 12 bits) */
    r = fmaf(n, -1.42860682030941723e-06f, r);       /* ln2 low part */
    float p = 1.3888889e-03f;                        /* 1/720 */
    p = fmaf(p, r, 8.3333333e-03f);                  /* 1/120 */
    p = fmaf(p, r, 4.1666668e-02f);                  /* 1/24 */
    p = fmaf(p, r, 1.6666667e-01f);                  /* 1/6 */
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    int ni = int(n);
    int n1 = ni / 2, n2 = ni - n1;                   /* both within [-126, 127] */
    return (p * pow2i(n1)) * pow2i(n2);
}

} // namespace

/* ---- format helpers exported for the tests ----------------------------- */

ZO_API void zo_f32_to_bf16(const float *src, uint16_t *dst, int64_t n) { for (int64_t i = 0; i < n; ++i) dst[i] = f32_to_bf16(src[i]); }
ZO_API void zo_bf16_to_f32(const uint16_t *src, float *dst, int64_t n) { for (int64_t i = 0; i < n; ++i) dst[i] = bf16_to_f32(src[i]); }
ZO_API void zo_f32_to_fp16(const float *src, uint16_t *dst, int64_t n) { for (int64_t i = 0; i < n; ++i) dst[i] = f32_to_fp16(src[i]); }
ZO_API void zo_fp16_to_f32(const uint16_t *src, float *dst, int64_t n) { for (int64_t i = 0; i < n; ++i) dst[i] = fp16_to_f32(src[i]); }
ZO_API void zo_f32_to_e4m3(const float *src, uint8_t *dst, int64_t n) { for (int64_t i = 0; i < n; ++i) dst[i] = f32_to_e4m3(src[i]); }
ZO_API void zo_e4m3_to_f32(const uint8_t *src, float *dst, int64_t n) { for (int64_t i = 0; i < n; ++i) dst[i] = e4m3_to_f32(src[i]); }
ZO_API void zo_expf(const float *src, float *dst, int64_t n) { for (int64_t i = 0; i < n; ++i) dst[i] = zo_expf_impl(src[i]); }
ZO_API int32_t zo_num_threads()
{
#if defined(_OPENMP)
    return omp_get_max_threads();
#else
    return 1;
#endif
}
ZO_API void zo_set_num_threads(int32_t n)
{
#if defined(_OPENMP)
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/*
 * Router. parity unpinned: the reference has none; its tests draw
 * topk_idx with torch.topk and weights at random (test_low_latency.py:68-89).
 * Definition: p = softmax(logits) in fp32 (max-subtracted; exp is the fixed
 * polynomial zo_expf_impl that the GPU router evaluates too, pinned against
 * the float64 exp to 2.5e-7; sum in index order); the K picks are the K largest logits, ties to the lower
 * index, listed in descending order; w_k = p_k / sum of the K picked p.
 * Pinned by brute force and by invariants in the tests.
 */
ZO_API void zo_topk_route(const float *logits, int64_t T, int64_t E, int64_t K, int64_t *topk_idx, float *topk_w)
{
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; ++t) {
        const float *l = logits + t * E;
        float mx = l[0];
        for (int64_t e = 1; e < E; ++e) mx = std::max(mx, l[e]);
        /*
         * Both sums are taken in double and rounded once: the definition is "the fp32 quotient by the correctly rounded
         * sum", which no summation order of an fp32 implementation is more than a few ulps away from (a sequential
         * fp32 sum of a hundred equal terms, by contrast, drifts by a dozen ulps on its own).
         */
        std::vector<float> p(E);
        double sum_d = 0.0;
        for (int64_t e = 0; e < E; ++e) { p[e] = zo_expf_impl(l[e] - mx); sum_d += (double)p[e]; }
        const float sum = (float)sum_d;
        for (int64_t e = 0; e < E; ++e) p[e] = p[e] / sum;
        std::vector<char> used(E, 0);
        double wsum_d = 0.0;
        for (int64_t k = 0; k < K; ++k) {
            int64_t best = -1;
            for (int64_t e = 0; e < E; ++e) {
                if (used[e]) continue;
                if (best < 0 || l[e] > l[best]) best = e;
            }
            used[best] = 1;
            topk_idx[t * K + k] = best;
            topk_w[t * K + k] = p[best];
            wsum_d += (double)p[best];
        }
        const float wsum = (float)wsum_d;
        for (int64_t k = 0; k < K; ++k) topk_w[t * K + k] = topk_w[t * K + k] / wsum;
    }
}

/*
 * Dispatch layout: OPS/dispatch_combine_normal/zbal_kernel_dispatch_layout.h:97-183.
 * Flat (t,k) order; picks outside [0,E) are skipped. The reference leaves
 * their sendTokenIdx slot unwritten (:170-172); this build writes -1.
 * Pinned by an O(n^2) brute-force recount and the reference test's
 * assertions (test_normal.py:95-98,137-149).
 */
ZO_API void zo_dispatch_layout(const int64_t *topk_idx, int64_t T, int64_t K, int64_t E, int64_t R,
                               int32_t *tokens_per_rank, int32_t *tokens_per_expert, int32_t *send_token_idx)
{
    std::vector<int32_t> cnt_e(E, 0), cnt_r(R, 0);
    std::vector<char> seen(R);
    const int64_t e_loc = E / R;
    for (int64_t t = 0; t < T; ++t) {
        std::fill(seen.begin(), seen.end(), 0);
        for (int64_t k = 0; k < K; ++k) {
            int64_t e = topk_idx[t * K + k];
            if (e < 0 || e >= E) { send_token_idx[t * K + k] = -1; continue; }
            send_token_idx[t * K + k] = cnt_e[e]++;
            int64_t r = e / e_loc;
            if (!seen[r]) { seen[r] = 1; cnt_r[r]++; }
        }
    }
    for (int64_t e = 0; e < E; ++e) tokens_per_expert[e] = cnt_e[e];
    for (int64_t r = 0; r < R; ++r) tokens_per_rank[r] = cnt_r[r];
}

/*
 * Notify: OPS/dispatch_combine_normal/zbal_kernel_notify_dispatch.h
 * ReorderRecvDataOutput :356-378, BuildTotalRecvTokens :531-564,
 * BuildRecvTokenPerExp :566-596, BuildBalanceMatrix :421-498 (no re-balancing).
 * counts_all is [R, E]: row s = tokensPerExpert of rank s.
 */
ZO_API void zo_dispatch_notify(const int32_t *counts_all, int64_t R, int64_t E, int64_t K, int64_t me,
                               int32_t *recv_data, int32_t *put_offset, int32_t *total_recv,
                               int64_t *recv_tokens_per_expert, int32_t *balance_matrix)
{
    const int64_t e_loc = E / R;
    for (int64_t i = 0; i < R * E; ++i) recv_data[i] = counts_all[i];
    for (int64_t r = 0; r < R; ++r) {
        int32_t run = 0;
        for (int64_t le = 0; le < e_loc; ++le)
            for (int64_t s = 0; s < R; ++s) {
                put_offset[r * E + le * R + s] = run;
                run += counts_all[s * E + r * e_loc + le];
            }
    }
    int32_t tot = 0;
    for (int64_t le = 0; le < e_loc; ++le) {
        int64_t c = 0;
        for (int64_t s = 0; s < R; ++s) c += counts_all[s * E + me * e_loc + le];
        recv_tokens_per_expert[le] = c;
        tot += int32_t(c);
    }
    *total_recv = tot;
    for (int64_t i = 0; i < R * 2 * R; ++i) balance_matrix[i] = -1;
    for (int64_t i = 0; i < R; ++i) {
        int64_t s = 0;
        for (int64_t e = 0; e < E; ++e) s += counts_all[i * E + e];
        int64_t bs = s / K;
        if (bs > 0) {
            balance_matrix[i * 2 * R + 2 * i] = 0;
            balance_matrix[i * 2 * R + 2 * i + 1] = int32_t(bs - 1);
        }
    }
}

namespace {

/*
 * Per-token symmetric int8 quantisation.
 *   flavour 0: normal mode, s = 127/(amax + 1e-12)   (zbal_kernel_dispatch_normal.h:440-477)
 *   flavour 1: low-latency and fused mode, s = 127/amax
 *              (zbal_kernel_dispatch_low_latency.h:931-969,
 *               FDM/gemm/kernel/grouped_matmul_slice_m_per_token_dequant_swiglu_quant_multistage_workspace.h:952-995);
 *              amax == 0 gives q = 0, scale = 0 here (the reference divides by zero).
 * `smooth` (optional) multiplies the row first (…workspace.h:970-973).
 * Stored scale = 1.0f / s.
 */
inline void quant_row_int8(const uint16_t *x, int dtype, int64_t H, const float *smooth, int flavour, int8_t *q,
                           float *scale)
{
    float amax = 0.0f;
    for (int64_t j = 0; j < H; ++j) {
        float v = half_like_to_f32(x[j], dtype);
        if (smooth) v = v * smooth[j];
        amax = std::max(amax, std::fabs(v));
    }
    if (flavour == 1 && amax == 0.0f) {
        for (int64_t j = 0; j < H; ++j) q[j] = 0;
        *scale = 0.0f;
        return;
    }
    float s = (flavour == 0) ? 127.0f / (amax + 1e-12f) : 127.0f / amax;
    for (int64_t j = 0; j < H; ++j) {
        float v = half_like_to_f32(x[j], dtype);
        if (smooth) v = v * smooth[j];
        q[j] = rint_i8(v * s);
    }
    *scale = 1.0f / s;
}

/*
 * e4m3 quantisation of one row in 1x128 blocks (extension; parity unpinned).
 * Follows the DeepSeek-V3 convention the reference's test helper decodes
 * (test/python/deepep/utils.py:118-126: one fp32 scale per 128 columns):
 * amax = max(|v|, 1e-4); q = e4m3(v * (448/amax)); stored scale = amax * (1/448).
 */
inline void quant_row_fp8(const float *v, int64_t H, uint8_t *q, float *scales)
{
    for (int64_t b = 0; b < H / 128; ++b) {
        float amax = 0.0f;
        for (int64_t j = 0; j < 128; ++j) amax = std::max(amax, std::fabs(v[b * 128 + j]));
        amax = std::max(amax, 1e-4f);
        float mult = 448.0f / amax;
        for (int64_t j = 0; j < 128; ++j) {
            float s = v[b * 128 + j] * mult;
            s = std::min(std::max(s, -448.0f), 448.0f);
            q[b * 128 + j] = f32_to_e4m3(s);
        }
        scales[b] = amax * (1.0f / 448.0f);
    }
}

} // namespace

/*
 * Normal-mode dispatch: OPS/dispatch_combine_normal/zbal_kernel_dispatch_normal.h
 * InputToDstOutput :479-563. quant_mode: 0 copy, 1 int8 (flavour 0),
 * 2 fp8 1x128 (dest_scale is [rows, H/128]). Rows land expert-major in
 * flat-pick order: row = put_offset[e*R + me] + send_token_idx[i].
 * Pinned by: constant rows (q = +-127, scale = |c|/127), |q*scale - x| <=
 * scale/2, and dest[row(i)] == quant(x[t(i)]).
 */
ZO_API void zo_dispatch_normal(const uint16_t *x, int32_t x_dtype, const int32_t *topk_idx,
                               const int32_t *send_token_idx, const int32_t *put_offset, int64_t T, int64_t H,
                               int64_t K, int64_t E, int64_t R, int64_t me, int32_t quant_mode, void *dest,
                               float *dest_scale)
{
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; ++t) {
        std::vector<int8_t> q;
        std::vector<uint8_t> q8;
        std::vector<float> v, sc;
        float scale = 0.0f;
        bool done = false;
        for (int64_t k = 0; k < K; ++k) {
            int64_t e = topk_idx[t * K + k];
            if (e < 0 || e >= E) continue;
            int64_t row = int64_t(put_offset[e * R + me]) + send_token_idx[t * K + k];
            if (quant_mode == 0) {
                std::memcpy(static_cast<uint16_t *>(dest) + row * H, x + t * H, size_t(H) * 2);
            } else if (quant_mode == 1) {
                if (!done) { q.resize(H); quant_row_int8(x + t * H, x_dtype, H, nullptr, 0, q.data(), &scale); done = true; }
                std::memcpy(static_cast<int8_t *>(dest) + row * H, q.data(), size_t(H));
                dest_scale[row] = scale;
            } else {
                if (!done) {
                    v.resize(H); q8.resize(H); sc.resize(H / 128);
                    for (int64_t j = 0; j < H; ++j) v[j] = half_like_to_f32(x[t * H + j], x_dtype);
                    quant_row_fp8(v.data(), H, q8.data(), sc.data());
                    done = true;
                }
                std::memcpy(static_cast<uint8_t *>(dest) + row * H, q8.data(), size_t(H));
                std::memcpy(dest_scale + row * (H / 128), sc.data(), size_t(H / 128) * 4);
            }
        }
    }
}

/*
 * Weighted combine: OPS/dispatch_combine_normal/zbal_kernel_combine_normal.h
 * ReadTokenAndWeightedSum :398-435 — fp32 accumulator, per pick a multiply
 * (Muls :424) then an add (Add :426), one rounding to the element type at the
 * end (:432). Also restates combine_low_latency.h:494-531 and
 * FDM/raw_distributed/zbal_moe_distribute_combine.h:778-813 (same arithmetic);
 * invalid expert ids are skipped in all three here.
 * `base` is the exclusive per-expert row offset.
 * Pinned by the reference's round trip: identity experts give x * sum_k w
 * (test_normal.py:225-236).
 */
ZO_API void zo_combine(const uint16_t *y, int32_t dtype, const int32_t *base, const float *w,
                       const int32_t *topk_idx, const int32_t *send_token_idx, int64_t T, int64_t H, int64_t K,
                       int64_t E, int64_t R, int64_t me, uint16_t *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; ++t) {
        std::vector<float> acc(H, 0.0f);
        for (int64_t k = 0; k < K; ++k) {
            int64_t e = topk_idx[t * K + k];
            if (e < 0 || e >= E) continue;
            int64_t row = int64_t(base[e * R + me]) + send_token_idx[t * K + k];
            const uint16_t *src = y + row * H;
            float wk = w[t * K + k];
            for (int64_t j = 0; j < H; ++j) {
                float tmp = half_like_to_f32(src[j], dtype) * wk;
                acc[j] = acc[j] + tmp;
            }
        }
        for (int64_t j = 0; j < H; ++j) out[t * H + j] = f32_to_half_like(acc[j], dtype);
    }
}

/*
 * Low-latency dispatch at R = 1:
 * OPS/dispatch_combine_low_latency/zbal_kernel_dispatch_low_latency.h
 * LocalLayout :528-568, ReorderRecvDataOutput :641-713, SendToMoeExpert :760-844,
 * QuantProcess :931-969. ep_recv_counts is the INCLUSIVE running sum per
 * expert (:706-708); expert_token_nums is the count (type 1) or the inclusive
 * prefix sum (type 0) (:672-683). expand_idx is the general stable rank (the
 * reference forces token 0's to 0, :796-799, identical when a token's experts
 * are distinct). Rows are packed densely, expert-major.
 * quant_mode: 0 copy, 1 int8 flavour 1, 2 fp8 1x128.
 */
ZO_API void zo_dispatch_low_latency(const uint16_t *x, int32_t x_dtype, const int32_t *expert_ids, int64_t T,
                                    int64_t H, int64_t K, int64_t E, int32_t quant_mode, int32_t token_nums_type,
                                    void *expand_x, float *dynamic_scales, int32_t *expand_idx,
                                    int64_t *expert_token_nums, int32_t *ep_recv_counts)
{
    std::vector<int32_t> cnt(E, 0);
    for (int64_t i = 0; i < T * K; ++i) {
        int64_t e = expert_ids[i];
        if (e < 0 || e >= E) { expand_idx[i] = -1; continue; }
        expand_idx[i] = cnt[e]++;
    }
    int32_t run = 0;
    for (int64_t e = 0; e < E; ++e) {
        run += cnt[e];
        ep_recv_counts[e] = run;
        expert_token_nums[e] = (token_nums_type == 0) ? int64_t(run) : int64_t(cnt[e]);
    }
    std::vector<int8_t> q(H);
    std::vector<uint8_t> q8(H);
    std::vector<float> v(H), sc(H / 128 + 1);
    for (int64_t t = 0; t < T; ++t) {
        bool done = false;
        float scale = 0.0f;
        for (int64_t k = 0; k < K; ++k) {
            int64_t e = expert_ids[t * K + k];
            if (e < 0 || e >= E) continue;
            int64_t row = (e == 0 ? 0 : ep_recv_counts[e - 1]) + expand_idx[t * K + k];
            if (quant_mode == 0) {
                std::memcpy(static_cast<uint16_t *>(expand_x) + row * H, x + t * H, size_t(H) * 2);
            } else if (quant_mode == 1) {
                if (!done) { quant_row_int8(x + t * H, x_dtype, H, nullptr, 1, q.data(), &scale); done = true; }
                std::memcpy(static_cast<int8_t *>(expand_x) + row * H, q.data(), size_t(H));
                dynamic_scales[row] = scale;
            } else {
                if (!done) {
                    for (int64_t j = 0; j < H; ++j) v[j] = half_like_to_f32(x[t * H + j], x_dtype);
                    quant_row_fp8(v.data(), H, q8.data(), sc.data());
                    done = true;
                }
                std::memcpy(static_cast<uint8_t *>(expand_x) + row * H, q8.data(), size_t(H));
                std::memcpy(dynamic_scales + row * (H / 128), sc.data(), size_t(H / 128) * 4);
            }
        }
    }
}

/*
 * Low-latency combine at R = 1: OPS/dispatch_combine_low_latency/
 * zbal_kernel_combine_low_latency.h:426-532; base(e) = e ? counts[e-1] : 0 (:504-506).
 */
ZO_API void zo_combine_low_latency(const uint16_t *expand_x, int32_t dtype, const int32_t *expert_ids,
                                   const int32_t *expand_idx, const int32_t *ep_send_counts, const float *w, int64_t T,
                                   int64_t H, int64_t K, int64_t E, uint16_t *out)
{
    std::vector<int32_t> base(E);
    for (int64_t e = 0; e < E; ++e) base[e] = e ? ep_send_counts[e - 1] : 0;
    zo_combine(expand_x, dtype, base.data(), w, expert_ids, expand_idx, T, H, K, E, 1, 0, out);
}

/*
 * The low-latency pair for a group of R ranks, from the point of view of rank `me`
 * (OPS/dispatch_combine_low_latency/zbal_kernel_dispatch_low_latency.h: counts of all ranks gathered into
 * allExpertTokenNums :344-345; ReorderRecvDataOutput :690-713 builds, per destination rank r, the INCLUSIVE running sum
 * over (local expert le, source rank s) at [r * E + le * R + s]; WaitNotify :641-688 derives the receiving rank's
 * expertTokenNums from its own block; SendToMoeExpert :760-844 puts pick (t, k) of expert e into the window of rank
 * e / E_loc at row start(e * R + me) + expand_idx, start(i) = i % E == 0 ? 0 : counts[i - 1]).
 * ids_all [R][T][K]: every rank's expert ids (all ranks with the same T and K).
 */
ZO_API void zo_ll_counts(const int32_t *ids_all, int64_t R, int64_t me, int64_t T, int64_t K, int64_t E,
                         int32_t token_nums_type, int32_t *all_counts, int32_t *ep_recv_counts,
                         int64_t *expert_token_nums)
{
    const int64_t e_loc = E / R;
    std::fill(all_counts, all_counts + R * E, 0);
    for (int64_t s = 0; s < R; ++s)
        for (int64_t i = 0; i < T * K; ++i) {
            const int64_t e = ids_all[s * T * K + i];
            if (e >= 0 && e < E) all_counts[s * E + e] += 1;
        }
    for (int64_t r = 0; r < R; ++r) {
        int32_t prefix = 0;
        for (int64_t le = 0; le < e_loc; ++le)
            for (int64_t s = 0; s < R; ++s) {
                prefix += all_counts[s * E + r * e_loc + le];
                ep_recv_counts[r * E + le * R + s] = prefix;
            }
    }
    int64_t sums = 0;
    for (int64_t le = 0; le < e_loc; ++le) {
        const int64_t cur = R * (le + 1) - 1;
        const int64_t before = le == 0 ? 0 : ep_recv_counts[me * E + cur - R];
        const int64_t here = ep_recv_counts[me * E + cur] - before;
        sums = (token_nums_type == 0 ? sums : 0) + here;
        expert_token_nums[le] = sums;
    }
}

/*
 * Rank `me` sends its tokens: windows_x / windows_scale are the R receive windows one after the other (rows_cap rows
 * each); only the rows this rank writes are touched. expand_idx = rank of each pick among this rank's earlier picks
 * of the same expert (-1 for an invalid id).
 */
ZO_API void zo_dispatch_low_latency_ranks(const uint16_t *x, int32_t x_dtype, const int32_t *expert_ids, int64_t T,
                                          int64_t H, int64_t K, int64_t E, int64_t R, int64_t me, int32_t quant_mode,
                                          const int32_t *ep_recv_counts, int64_t rows_cap, void *windows_x,
                                          float *windows_scale, int32_t *expand_idx)
{
    const int64_t e_loc = E / R;
    std::vector<int32_t> cnt(E, 0);
    for (int64_t i = 0; i < T * K; ++i) {
        const int64_t e = expert_ids[i];
        if (e < 0 || e >= E) { expand_idx[i] = -1; continue; }
        expand_idx[i] = cnt[e]++;
    }
    std::vector<int8_t> q(H);
    std::vector<uint8_t> q8(H);
    std::vector<float> v(H), sc(H / 128 + 1);
    for (int64_t t = 0; t < T; ++t) {
        bool done = false;
        float scale = 0.0f;
        for (int64_t k = 0; k < K; ++k) {
            const int64_t e = expert_ids[t * K + k];
            if (e < 0 || e >= E) continue;
            const int64_t idx = e * R + me;
            const int64_t start = idx % E == 0 ? 0 : ep_recv_counts[idx - 1];
            const int64_t row = start + expand_idx[t * K + k];
            if (row >= rows_cap) continue;
            const int64_t wrow = (e / e_loc) * rows_cap + row;
            if (quant_mode == 0) {
                std::memcpy(static_cast<uint16_t *>(windows_x) + wrow * H, x + t * H, size_t(H) * 2);
            } else if (quant_mode == 1) {
                if (!done) { quant_row_int8(x + t * H, x_dtype, H, nullptr, 1, q.data(), &scale); done = true; }
                std::memcpy(static_cast<int8_t *>(windows_x) + wrow * H, q.data(), size_t(H));
                windows_scale[wrow] = scale;
            } else {
                if (!done) {
                    for (int64_t j = 0; j < H; ++j) v[j] = half_like_to_f32(x[t * H + j], x_dtype);
                    quant_row_fp8(v.data(), H, q8.data(), sc.data());
                    done = true;
                }
                std::memcpy(static_cast<uint8_t *>(windows_x) + wrow * H, q8.data(), size_t(H));
                std::memcpy(windows_scale + wrow * (H / 128), sc.data(), size_t(H / 128) * 4);
            }
        }
    }
}

/*
 * Rank `me` combines: zbal_kernel_combine_low_latency.h:494-531 (row of pick (t, k) of expert e: window e / E_loc, row
 * start(e * R + me) + expand_idx; Muls then Add in fp32, one rounding). windows_y: the R windows one after the other.
 */
ZO_API void zo_combine_low_latency_ranks(const uint16_t *windows_y, int32_t dtype, const int32_t *expert_ids,
                                         const int32_t *expand_idx, const int32_t *ep_send_counts, const float *w,
                                         int64_t T, int64_t H, int64_t K, int64_t E, int64_t R, int64_t me,
                                         int64_t rows_cap, uint16_t *out)
{
    const int64_t e_loc = E / R;
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; ++t) {
        std::vector<float> acc(H, 0.0f);
        for (int64_t k = 0; k < K; ++k) {
            const int64_t e = expert_ids[t * K + k];
            if (e < 0 || e >= E) continue;
            const int64_t idx = e * R + me;
            const int64_t row = (idx % E == 0 ? 0 : ep_send_counts[idx - 1]) + expand_idx[t * K + k];
            if (row >= rows_cap) continue;
            const uint16_t *src = windows_y + ((e / e_loc) * rows_cap + row) * H;
            const float wk = w[t * K + k];
            for (int64_t j = 0; j < H; ++j) {
                const float tmp = half_like_to_f32(src[j], dtype) * wk;
                acc[j] = acc[j] + tmp;
            }
        }
        for (int64_t j = 0; j < H; ++j) out[t * H + j] = f32_to_half_like(acc[j], dtype);
    }
}

/* ---- grouped GEMMs ------------------------------------------------------ */

/*
 * Weights are given in their LOGICAL layout [E, K, N] (N contiguous), one
 * byte per element (int8, e4m3 code, or an int4 value held in an int8).
 */

namespace {

/* exact int32 row-times-matrix: out[n] = sum_k a[k] * w[k, n] */
inline void row_gemm_i8(const int8_t *a, const int8_t *w, int64_t K, int64_t N, int32_t *out)
{
    std::fill(out, out + N, 0);
    for (int64_t k = 0; k < K; ++k) {
        int32_t av = a[k];
        if (av == 0) continue;
        const int8_t *wr = w + k * N;
        for (int64_t n = 0; n < N; ++n) out[n] += av * int32_t(wr[n]);
    }
}

} // namespace

/*
 * Stand-alone grouped GEMM with per-token / per-channel dequantisation
 * (the GMM2 arithmetic, FDM/epilogue/block/block_epilogue_per_token_dequant.hpp:350-373):
 * y[m,n] = round_to_out( (float(C[m,n]) * wscale[g,n]) * xscale[m] ), C exact int32.
 * wscale is fp32 (wscale_dtype 7) or bf16 (8). Rows of expert g are
 * [off_g, off_g + counts[g]), off = exclusive cumsum of counts.
 * Pinned by comparison with a float64 numpy matmul (exact for these ranges).
 */
ZO_API void zo_grouped_gemm_w8a8_dequant(const int8_t *a, const float *xscale, const int8_t *w, const void *wscale,
                                         int32_t wscale_dtype, const int64_t *counts, int64_t E, int64_t K, int64_t N,
                                         int32_t out_dtype, uint16_t *y)
{
    std::vector<int64_t> off(E + 1, 0);
    for (int64_t g = 0; g < E; ++g) off[g + 1] = off[g] + counts[g];
    for (int64_t g = 0; g < E; ++g) {
#pragma omp parallel for schedule(static)
        for (int64_t m = off[g]; m < off[g + 1]; ++m) {
            std::vector<int32_t> c(N);
            row_gemm_i8(a + m * K, w + g * K * N, K, N, c.data());
            for (int64_t n = 0; n < N; ++n) {
                float ws = (wscale_dtype == DT_FP32) ? static_cast<const float *>(wscale)[g * N + n]
                                                      : bf16_to_f32(static_cast<const uint16_t *>(wscale)[g * N + n]);
                float d = (float(c[n]) * ws) * xscale[m];
                y[m * N + n] = f32_to_half_like(d, out_dtype);
            }
        }
    }
}

/*
 * GMM1 + dequant + SwiGLU + per-token int8 requant, W8A8:
 *   d = (float(C) * w1scale[g,n]) * xs[m]
 *       (FDM/epilogue/block/block_epilogue_per_token_dequant_swiglu.h:256-286)
 *   left = d / (1 + exp(-d)) for n < N1/2, right = d for n >= N1/2 (:273-283)
 *   sgl = left * right; mx = max |sgl|; scale2 = mx * (1/127);
 *   q2 = int8(rint((sgl * 127) * (1/mx)))
 *       (…swiglu_quant_multistage_workspace.h BlockQuant :209-276)
 * A row whose mx is 0 gives q2 = 0, scale2 = 0 (the reference divides by zero).
 * sgl_out (optional) receives the fp32 SwiGLU values.
 */
ZO_API void zo_gmm1_swiglu_quant_w8a8(const int8_t *a, const float *xs, const int8_t *w1, const float *w1scale,
                                      const int64_t *counts, int64_t E, int64_t K, int64_t N1, int8_t *q2,
                                      float *scale2, float *sgl_out)
{
    const int64_t I = N1 / 2;
    std::vector<int64_t> off(E + 1, 0);
    for (int64_t g = 0; g < E; ++g) off[g + 1] = off[g] + counts[g];
    for (int64_t g = 0; g < E; ++g) {
#pragma omp parallel for schedule(static)
        for (int64_t m = off[g]; m < off[g + 1]; ++m) {
            std::vector<int32_t> c(N1);
            std::vector<float> sgl(I);
            row_gemm_i8(a + m * K, w1 + g * K * N1, K, N1, c.data());
            float mx = 0.0f;
            for (int64_t j = 0; j < I; ++j) {
                float dl = (float(c[j]) * w1scale[g * N1 + j]) * xs[m];
                float dr = (float(c[I + j]) * w1scale[g * N1 + I + j]) * xs[m];
                float left = dl / (1.0f + zo_expf_impl(-dl));
                sgl[j] = left * dr;
                mx = std::max(mx, std::fabs(sgl[j]));
            }
            if (sgl_out) std::memcpy(sgl_out + m * I, sgl.data(), size_t(I) * 4);
            if (mx == 0.0f) {
                for (int64_t j = 0; j < I; ++j) q2[m * I + j] = 0;
                scale2[m] = 0.0f;
                continue;
            }
            scale2[m] = mx * (1.0f / 127.0f);
            float inv = 1.0f / mx;
            for (int64_t j = 0; j < I; ++j) q2[m * I + j] = rint_i8((sgl[j] * 127.0f) * inv);
        }
    }
}

/*
 * Block-scaled fp8 grouped GEMM core (extension; parity unpinned):
 *   acc[m,n] = sum over 128-deep K blocks kb of
 *              (sum_{k in kb} a[m,k]*w[k,n]) * (sa[m,kb] * sw[g,kb,n/128])
 * The inner sum is taken in double (the exact product sum up to one rounding),
 * the outer accumulation in fp32 with fmaf, block order ascending.
 * a: e4m3 codes [rows, K]; sa [rows, K/128]; w: e4m3 codes [E, K, N];
 * sw [E, K/128, N/128].
 */
namespace {
inline void row_gemm_fp8_block(const uint8_t *a, const float *sa, const float *wf /* [K,N] decoded */, const float *sw,
                               int64_t K, int64_t N, float *acc)
{
    const int64_t KB = K / 128, NB = N / 128;
    std::vector<double> part(N);
    std::fill(acc, acc + N, 0.0f);
    for (int64_t kb = 0; kb < KB; ++kb) {
        std::fill(part.begin(), part.end(), 0.0);
        for (int64_t k = kb * 128; k < kb * 128 + 128; ++k) {
            double av = e4m3_to_f32(a[k]);
            if (av == 0.0) continue;
            const float *wr = wf + k * N;
            for (int64_t n = 0; n < N; ++n) part[n] += av * double(wr[n]);
        }
        for (int64_t n = 0; n < N; ++n) {
            float s = sa[kb] * sw[kb * NB + n / 128];
            acc[n] = fmaf(float(part[n]), s, acc[n]);
        }
    }
}
} // namespace

/*
 * GMM1 fp8 + SwiGLU + 1x128 e4m3 requant (extension; parity unpinned).
 * gate = acc[:, j], up = acc[:, I + j]; sgl = (gate / (1 + exp(-gate))) * up;
 * then quant_row_fp8 over the I columns. q2 [rows, I], s2 [rows, I/128].
 */
ZO_API void zo_gmm1_swiglu_quant_fp8(const uint8_t *a, const float *sa, const uint8_t *w1, const float *sw1,
                                     const int64_t *counts, int64_t E, int64_t K, int64_t N1, uint8_t *q2, float *s2,
                                     float *sgl_out)
{
    const int64_t I = N1 / 2, KB = K / 128, NB = N1 / 128;
    std::vector<int64_t> off(E + 1, 0);
    for (int64_t g = 0; g < E; ++g) off[g + 1] = off[g] + counts[g];
    std::vector<float> wf(size_t(K) * N1);
    for (int64_t g = 0; g < E; ++g) {
        if (counts[g] == 0) continue;
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < K * N1; ++i) wf[i] = e4m3_to_f32(w1[g * K * N1 + i]);
#pragma omp parallel for schedule(static)
        for (int64_t m = off[g]; m < off[g + 1]; ++m) {
            std::vector<float> acc(N1), sgl(I);
            row_gemm_fp8_block(a + m * K, sa + m * KB, wf.data(), sw1 + g * KB * NB, K, N1, acc.data());
            for (int64_t j = 0; j < I; ++j) {
                float gate = acc[j], up = acc[I + j];
                sgl[j] = (gate / (1.0f + zo_expf_impl(-gate))) * up;
            }
            if (sgl_out) std::memcpy(sgl_out + m * I, sgl.data(), size_t(I) * 4);
            quant_row_fp8(sgl.data(), I, q2 + m * I, s2 + m * (I / 128));
        }
    }
}

/* GMM2 fp8 block-scaled -> bf16/fp16 rows (extension; parity unpinned). */
ZO_API void zo_gmm2_fp8(const uint8_t *a, const float *sa, const uint8_t *w2, const float *sw2, const int64_t *counts,
                        int64_t E, int64_t K, int64_t N, int32_t out_dtype, uint16_t *y)
{
    const int64_t KB = K / 128, NB = N / 128;
    std::vector<int64_t> off(E + 1, 0);
    for (int64_t g = 0; g < E; ++g) off[g + 1] = off[g] + counts[g];
    std::vector<float> wf(size_t(K) * N);
    for (int64_t g = 0; g < E; ++g) {
        if (counts[g] == 0) continue;
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < K * N; ++i) wf[i] = e4m3_to_f32(w2[g * K * N + i]);
#pragma omp parallel for schedule(static)
        for (int64_t m = off[g]; m < off[g + 1]; ++m) {
            std::vector<float> acc(N);
            row_gemm_fp8_block(a + m * K, sa + m * KB, wf.data(), sw2 + g * KB * NB, K, N, acc.data());
            for (int64_t n = 0; n < N; ++n) y[m * N + n] = f32_to_half_like(acc[n], out_dtype);
        }
    }
}

/*
 * W4A8 core (extension; parity unpinned): int8 rows times int4 weights with
 * one fp16 scale per (128-deep K group, column):
 *   acc[m,n] = fmaf(float(sum_{k in group} a*w), float(gs[g,kb,n]), acc) over groups ascending,
 *   d = acc * xs[m].
 * w holds the int4 values as int8 in [-8,7], logical [E, K, N]; gs is fp16 [E, K/128, N].
 */
namespace {
inline void row_gemm_w4a8(const int8_t *a, const int8_t *w, const uint16_t *gs, int64_t K, int64_t N, float *acc)
{
    std::vector<int32_t> part(N);
    std::fill(acc, acc + N, 0.0f);
    for (int64_t kb = 0; kb < K / 128; ++kb) {
        std::fill(part.begin(), part.end(), 0);
        for (int64_t k = kb * 128; k < kb * 128 + 128; ++k) {
            int32_t av = a[k];
            if (av == 0) continue;
            const int8_t *wr = w + k * N;
            for (int64_t n = 0; n < N; ++n) part[n] += av * int32_t(wr[n]);
        }
        for (int64_t n = 0; n < N; ++n) acc[n] = fmaf(float(part[n]), fp16_to_f32(gs[kb * N + n]), acc[n]);
    }
}
} // namespace

ZO_API void zo_gmm1_swiglu_quant_w4a8(const int8_t *a, const float *xs, const int8_t *w1, const uint16_t *gs1,
                                      const int64_t *counts, int64_t E, int64_t K, int64_t N1, int8_t *q2,
                                      float *scale2, float *sgl_out)
{
    const int64_t I = N1 / 2, KB = K / 128;
    std::vector<int64_t> off(E + 1, 0);
    for (int64_t g = 0; g < E; ++g) off[g + 1] = off[g] + counts[g];
    for (int64_t g = 0; g < E; ++g) {
#pragma omp parallel for schedule(static)
        for (int64_t m = off[g]; m < off[g + 1]; ++m) {
            std::vector<float> acc(N1), sgl(I);
            row_gemm_w4a8(a + m * K, w1 + g * K * N1, gs1 + g * KB * N1, K, N1, acc.data());
            float mx = 0.0f;
            for (int64_t j = 0; j < I; ++j) {
                float dl = acc[j] * xs[m];
                float dr = acc[I + j] * xs[m];
                float left = dl / (1.0f + zo_expf_impl(-dl));
                sgl[j] = left * dr;
                mx = std::max(mx, std::fabs(sgl[j]));
            }
            if (sgl_out) std::memcpy(sgl_out + m * I, sgl.data(), size_t(I) * 4);
            if (mx == 0.0f) {
                for (int64_t j = 0; j < I; ++j) q2[m * I + j] = 0;
                scale2[m] = 0.0f;
                continue;
            }
            scale2[m] = mx * (1.0f / 127.0f);
            float inv = 1.0f / mx;
            for (int64_t j = 0; j < I; ++j) q2[m * I + j] = rint_i8((sgl[j] * 127.0f) * inv);
        }
    }
}

ZO_API void zo_gmm2_w4a8(const int8_t *a, const float *xs, const int8_t *w2, const uint16_t *gs2, const int64_t *counts,
                         int64_t E, int64_t K, int64_t N, int32_t out_dtype, uint16_t *y)
{
    const int64_t KB = K / 128;
    std::vector<int64_t> off(E + 1, 0);
    for (int64_t g = 0; g < E; ++g) off[g + 1] = off[g] + counts[g];
    for (int64_t g = 0; g < E; ++g) {
#pragma omp parallel for schedule(static)
        for (int64_t m = off[g]; m < off[g + 1]; ++m) {
            std::vector<float> acc(N);
            row_gemm_w4a8(a + m * K, w2 + g * K * N, gs2 + g * KB * N, K, N, acc.data());
            for (int64_t n = 0; n < N; ++n) y[m * N + n] = f32_to_half_like(acc[n] * xs[m], out_dtype);
        }
    }
}

/*
 * Permute + quantise for the fused operator (QuantToken / LocalQuantFunc,
 * …swiglu_quant_multistage_workspace.h:952-995, 1859-2058): rows expert-major
 * in flat-pick order, int8 flavour 1 with optional per-expert smooth scales
 * [E, H], or fp8 1x128 (mode 2). Outputs counts (int64) as expertTokenNums.
 */
ZO_API void zo_fused_permute_quant(const uint16_t *x, int32_t x_dtype, const int32_t *expert_ids, const float *smooth,
                                   int64_t T, int64_t H, int64_t K, int64_t E, int32_t mode, void *q1, float *xs,
                                   int32_t *expand_idx, int64_t *counts)
{
    std::vector<int64_t> cnt(E, 0), off(E + 1, 0);
    for (int64_t i = 0; i < T * K; ++i) {
        int64_t e = expert_ids[i];
        if (e < 0 || e >= E) { expand_idx[i] = -1; continue; }
        expand_idx[i] = int32_t(cnt[e]++);
    }
    for (int64_t e = 0; e < E; ++e) { off[e + 1] = off[e] + cnt[e]; counts[e] = cnt[e]; }
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; ++t) {
        std::vector<float> v(H);
        for (int64_t k = 0; k < K; ++k) {
            int64_t e = expert_ids[t * K + k];
            if (e < 0 || e >= E) continue;
            int64_t row = off[e] + expand_idx[t * K + k];
            if (mode == 2) {
                for (int64_t j = 0; j < H; ++j) v[j] = half_like_to_f32(x[t * H + j], x_dtype);
                quant_row_fp8(v.data(), H, static_cast<uint8_t *>(q1) + row * H, xs + row * (H / 128));
            } else {
                quant_row_int8(x + t * H, x_dtype, H, smooth ? smooth + e * H : nullptr, 1,
                               static_cast<int8_t *>(q1) + row * H, xs + row);
            }
        }
    }
}

/*
 * N-buffer reduction: the reduce-scatter phase of
 * OPS/classic/zbal_kernel_reducescatter.cpp:94-151 and
 * zbal_kernel_allreduce.cpp:206-260 with the semantics this build fixes:
 * floating types accumulate in fp32 in buffer order 0..N-1 and round once
 * (the reference applies an atomic in the element type per peer, in
 * scheduling order); PROD is a real product (the reference overwrites,
 * aicore/common/zbal_kernel_base.h:211-213). Integer types wrap.
 * op: 0 prod, 1 sum, 2 max, 3 min. dtype: zbal_datatype_t.
 * Pinned by closed forms and the reference's golden rule "sum of all ranks'
 * inputs", rtol 1e-4 (test_zbal_allreduce.py:48-58,148).
 */
namespace {
template <typename A> inline A red_op(A a, A b, int op)
{
    switch (op) {
        case 0: return a * b;
        case 1: return a + b;
        case 2: return a > b ? a : b;
        default: return a < b ? a : b;
    }
}
template <typename T> void reduce_int(const void *const *in, int64_t N, int64_t n, int op, void *out)
{
    typedef typename std::make_unsigned<T>::type U;
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < n; ++j) {
        T acc = static_cast<const T *>(in[0])[j];
        for (int64_t p = 1; p < N; ++p) {
            T v = static_cast<const T *>(in[p])[j];
            if (op == 0) acc = T(U(acc) * U(v));
            else if (op == 1) acc = T(U(acc) + U(v));
            else acc = red_op<T>(acc, v, op);
        }
        static_cast<T *>(out)[j] = acc;
    }
}
} // namespace

ZO_API int32_t zo_reduce(const void *const *in, int64_t N, int64_t n, int32_t dtype, int32_t op, void *out)
{
    switch (dtype) {
        case 0: reduce_int<int8_t>(in, N, n, op, out); return 0;
        case 1: reduce_int<int16_t>(in, N, n, op, out); return 0;
        case 2: reduce_int<int32_t>(in, N, n, op, out); return 0;
        case 3: reduce_int<int64_t>(in, N, n, op, out); return 0;
        case DT_FP32: {
#pragma omp parallel for schedule(static)
            for (int64_t j = 0; j < n; ++j) {
                float acc = static_cast<const float *>(in[0])[j];
                for (int64_t p = 1; p < N; ++p) acc = red_op<float>(acc, static_cast<const float *>(in[p])[j], op);
                static_cast<float *>(out)[j] = acc;
            }
            return 0;
        }
        case DT_FP16:
        case DT_BF16: {
#pragma omp parallel for schedule(static)
            for (int64_t j = 0; j < n; ++j) {
                float acc = half_like_to_f32(static_cast<const uint16_t *>(in[0])[j], dtype);
                for (int64_t p = 1; p < N; ++p)
                    acc = red_op<float>(acc, half_like_to_f32(static_cast<const uint16_t *>(in[p])[j], dtype), op);
                static_cast<uint16_t *>(out)[j] = f32_to_half_like(acc, dtype);
            }
            return 0;
        }
        default: return -2;
    }
}

// Attention whose scores are more than scale * q . k, over paged keys and values of widths of their own.
//
// liyab_qk_prepare: what happens to a step's projected queries, keys and values between the projection
// and the cache. The source is the projection's 32-bit output [q heads | ... | k heads | ... | v heads]
// (values may be the keys' own columns: values that are the keys as projected). Per head, in this
// order: a root-mean-square norm over the head with a weight shared by all heads (queries and keys,
// each optional); the turning of pairs of the first `rot_dims` entries by position * f_i (queries and keys; f from a
// table of doubles; pairs (2i, 2i + 1), or (i, i + rot_dims / 2) with `rot_halves`; cosine and sine times `rot_mag`); a factor on the query that grows with the logarithm of the
// position, 1 + coef * ln(floor((p + 1) / every) + 1). Queries go to a dense buffer in the compute type,
// keys and values to their token's slot of the pages; the rows they go to may be wider than the heads (dk_out, dv_out),
// zeros behind them: keys and values padded to one width are what the matrix-core kernels take. Norms, angles and factors are 32-bit.
// Values may be shared between layers of a step: `v_keep` (float [n, G * dv]) gets this layer's values as projected;
// `v_first` (such rows of an earlier layer) and `v_lam` (one float on the device) make the cached values (1 - lam) v + lam v_first.
//
// liyab_attention_scored: one workgroup a (token, query head). score = scale * q . k, then, each optional:
// a soft cap, cap * tanh(score / cap); a learned bias by distance, table[min(i - j, max_dist), head].
// Causal, with an optional window; ordinary softmax in 32-bit over tiles of 256 keys in position order
// with a running maximum and sum, so that a row's rounding follows from its position alone. Values are
// `dv` wide (keys `dk`). `sinks` (one logit a head, optional): exp(sink) joins the softmax's denominator, with no value.
// The result may be multiplied by the logistic function of a gate's logits before it is rounded to the compute type.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int AS_THREADS = 256;

// position * frequency, taken in double precision and brought into [0, 2 pi) before it is rounded: at position 1,000 a 32-bit
// product is already off by 6e-5 of a turn's radian, which is more than every other rounding of a 32-bit row together
__device__ __forceinline__ float turn_angle(int p, double f) {
    const double a = static_cast<double>(p) * f;
    constexpr double kTwoPi = 6.283185307179586476925286766559;
    return static_cast<float>(a - kTwoPi * floor(a / kTwoPi));
}

template <typename T>
__global__ void __launch_bounds__(kWave)
qk_prepare_kernel(const float* __restrict__ src, int64_t ld, int q_off, int k_off, int v_off, int H, int G, int dk, int dv, int dk_out,
                  int dv_out, T* __restrict__ q_out, T* __restrict__ kc, T* __restrict__ vc, const int* __restrict__ slots, int page_size,
                  int num_pages, const float* __restrict__ q_norm, const float* __restrict__ k_norm, float eps,
                  const double* __restrict__ freqs, int rot_dims, float temp_coef, int temp_every, const int* __restrict__ positions,
                  int rot_halves, float rot_mag, float* __restrict__ v_keep, const float* __restrict__ v_first, const float* __restrict__ v_lam) {
    const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
    const int p = positions[t];
    const float* row = src + static_cast<int64_t>(t) * ld;
    if (hh < H + G) {
        const bool is_q = hh < H;
        const int head = is_q ? hh : hh - H;
        const float* x = row + (is_q ? q_off : k_off) + head * dk;
        const float* nw = is_q ? q_norm : k_norm;
        float factor = 1.0f;
        if (nw != nullptr) {
            float ss = 0.0f;
            for (int i = lane; i < dk; i += kWave) ss = fmaf(x[i], x[i], ss);
            factor = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(dk) + eps);
        }
        float temp = 1.0f;
        if (is_q && temp_every > 0) temp = 1.0f + temp_coef * logf(static_cast<float>((p + 1) / temp_every) + 1.0f);
        T* dst;
        if (is_q) {
            dst = q_out + static_cast<int64_t>(t) * H * dk_out + head * dk_out;
        } else {
            const int64_t slot = slots[t];
            if (slot < 0 || slot >= static_cast<int64_t>(num_pages) * page_size) return;
            dst = kc + (((slot / page_size) * G + head) * page_size + slot % page_size) * dk_out;
        }
        for (int i = dk + lane; i < dk_out; i += kWave) dst[i] = from_float<T>(0.0f);  // rows wider than the head: zeros behind it
        if (rot_halves) {
            // pairs (i, i + rot_dims / 2): a lane takes a pair at a time, then the entries behind the turned ones
            const int half = rot_dims / 2;
            for (int i = lane; i < half; i += kWave) {
                const float a = x[i] * factor * (nw != nullptr ? nw[i] : 1.0f);
                const float b = x[i + half] * factor * (nw != nullptr ? nw[i + half] : 1.0f);
                const float angle = turn_angle(p, freqs[i]);
                const float c = cosf(angle) * rot_mag, s = sinf(angle) * rot_mag;
                dst[i] = from_float<T>((a * c - b * s) * temp);
                dst[i + half] = from_float<T>((b * c + a * s) * temp);
            }
            for (int i = rot_dims + lane; i < dk; i += kWave) dst[i] = from_float<T>(x[i] * factor * (nw != nullptr ? nw[i] : 1.0f) * temp);
            return;
        }
        // pairs of entries: a lane takes a pair at a time
        for (int i2 = lane; 2 * i2 < dk; i2 += kWave) {
            const int e0 = 2 * i2, e1 = e0 + 1;
            float a = x[e0] * factor * (nw != nullptr ? nw[e0] : 1.0f);
            float b = e1 < dk ? x[e1] * factor * (nw != nullptr ? nw[e1] : 1.0f) : 0.0f;
            if (freqs != nullptr && e1 < rot_dims) {
                const float angle = turn_angle(p, freqs[i2]);
                const float c = cosf(angle) * rot_mag, s = sinf(angle) * rot_mag;
                const float ra = a * c - b * s, rb = b * c + a * s;
                a = ra;
                b = rb;
            }
            dst[e0] = from_float<T>(a * temp);
            if (e1 < dk) dst[e1] = from_float<T>(b * temp);
        }
    } else {
        const int head = hh - H - G;
        const int64_t slot = slots[t];
        const float* x = row + v_off + head * dv;
        // values kept for later layers of the step (v_keep), or mixed with the values an earlier layer kept:
        // v <- (1 - lam) v + lam v_first, in 32 bits, before they are rounded for the pages
        const int64_t at = (static_cast<int64_t>(t) * G + head) * dv;
        if (v_keep != nullptr)
            for (int i = lane; i < dv; i += kWave) v_keep[at + i] = x[i];
        if (slot < 0 || slot >= static_cast<int64_t>(num_pages) * page_size) return;
        T* dst = vc + (((slot / page_size) * G + head) * page_size + slot % page_size) * dv_out;
        const float lam = v_first != nullptr ? v_lam[0] : 0.0f;
        for (int i = lane; i < dv_out; i += kWave) {
            float v = i < dv ? x[i] : 0.0f;
            if (v_first != nullptr && i < dv) v = (1.0f - lam) * v + lam * v_first[at + i];
            dst[i] = from_float<T>(v);
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(AS_THREADS)
attention_scored_kernel(T* __restrict__ out, int64_t out_stride, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ kc,
                        const T* __restrict__ vc, const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ tok_seq,
                        const int* __restrict__ tok_pos, float scale, float softcap, int window, const float* __restrict__ bias_table,
                        int max_dist, const float* __restrict__ gate, int64_t gate_stride, int n_head, int n_kv_head, int dk, int dv,
                        int page_size, int num_pages, const float* __restrict__ sinks) {
    extern __shared__ float smem[];
    float* qs = smem;                          // [dk]
    float* sc = qs + dk;                       // [AS_THREADS]
    float* red = sc + AS_THREADS;              // [AS_THREADS / kWave]
    float* accs = red + AS_THREADS / kWave;    // [G][dv]

    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave;
    const int pos = static_cast<int>(min(static_cast<int64_t>(max(tok_pos[t], 0)), static_cast<int64_t>(max_blocks) * page_size - 1));
    const int* bt = block_tables + static_cast<int64_t>(tok_seq[t]) * max_blocks;
    const int hkv = h / (n_head / n_kv_head);
    const int first = window > 0 ? max(0, pos - window + 1) : 0;
    const T* qrow = q + static_cast<int64_t>(t) * q_stride + static_cast<int64_t>(h) * dk;
    for (int e = tid; e < dk; e += AS_THREADS) qs[e] = to_float<T>(qrow[e]);
    __syncthreads();

    const int G = AS_THREADS / dv;  // groups of dv threads sharing the keys of a tile
    const int g = tid / dv, e = tid % dv;
    const bool vthread = g < G;
    const float inv_cap = softcap > 0.0f ? 1.0f / softcap : 0.0f;
    float m = -INFINITY, l = 0.0f, acc = 0.0f;

    for (int j0 = first; j0 <= pos; j0 += AS_THREADS) {
        const int j = j0 + tid;
        float s = -INFINITY;
        if (j <= pos) {
            const int64_t page = min(max(bt[j / page_size], 0), num_pages - 1);
            const T* kr = kc + ((page * n_kv_head + hkv) * page_size + j % page_size) * dk;
            float dot = 0.0f;
            for (int i = 0; i < dk; ++i) dot = fmaf(to_float<T>(kr[i]), qs[i], dot);
            s = dot * scale;
            if (softcap > 0.0f) s = softcap * tanhf(s * inv_cap);
            if (bias_table != nullptr) s += bias_table[static_cast<int64_t>(min(pos - j, max_dist)) * n_head + h];
        }
        float tm = wave_max(s);
        if (lane == 0) red[wave] = tm;
        __syncthreads();
        tm = red[0];
#pragma unroll
        for (int i = 1; i < AS_THREADS / kWave; ++i) tm = fmaxf(tm, red[i]);
        const float m_new = fmaxf(m, tm);
        const float p = j <= pos ? expf(s - m_new) : 0.0f;
        sc[tid] = p;
        float ps = wave_sum(p);
        __syncthreads();
        if (lane == 0) red[wave] = ps;
        __syncthreads();
        ps = 0.0f;
#pragma unroll
        for (int i = 0; i < AS_THREADS / kWave; ++i) ps += red[i];
        const float corr = expf(m - m_new);
        l = l * corr + ps;
        acc *= corr;
        m = m_new;
        if (vthread) {
            const int len = min(AS_THREADS, pos - j0 + 1);
            for (int jj = g; jj < len; jj += G) {
                const int jv = j0 + jj;
                const int64_t page = min(max(bt[jv / page_size], 0), num_pages - 1);
                const T* vr = vc + ((page * n_kv_head + hkv) * page_size + jv % page_size) * dv;
                acc = fmaf(sc[jj], to_float<T>(vr[e]), acc);
            }
        }
        __syncthreads();
    }
    if (vthread) accs[g * dv + e] = acc;
    __syncthreads();
    if (tid < dv) {
        float o = 0.0f;
        for (int i = 0; i < G; ++i) o += accs[i * dv + tid];
        if (sinks != nullptr) {
            // a sink: exp(sink) joins the denominator, both rescaled to the larger of the row's maximum and the sink
            const float M = fmaxf(m, sinks[h]);
            const float w = expf(m - M);
            l = l * w + expf(sinks[h] - M);
            o *= w;
        }
        o /= l;
        if (gate != nullptr) o *= 1.0f / (1.0f + expf(-gate[static_cast<int64_t>(t) * gate_stride + static_cast<int64_t>(h) * dv + tid]));
        out[static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * dv + tid] = from_float<T>(o);
    }
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_qk_prepare(const float* src, int64_t ld, int q_off, int k_off, int v_off, int H, int G, int dk, int dv, int dk_out,
                                int dv_out, void* q_out, void* kc, void* vc, int dtype, const int* slots, int page_size, int num_pages, const float* q_norm,
                                const float* k_norm, float eps, const double* freqs, int rot_dims, float temp_coef, int temp_every,
                                const int* positions, int n, int rot_halves, float rot_mag, float* v_keep, const float* v_first,
                                const float* v_lam, hipStream_t stream) {
    LIYAB_REQUIRE(src && q_out && kc && vc && slots && positions, "qk_prepare: null pointer");
    LIYAB_REQUIRE(n >= 0 && H > 0 && G > 0 && dk > 0 && dv > 0 && page_size > 0 && num_pages > 0, "qk_prepare: bad sizes");
    LIYAB_REQUIRE(H + 2 * G <= 65535, "qk_prepare: too many heads");
    LIYAB_REQUIRE(dk_out >= dk && dv_out >= dv, "qk_prepare: rows of %d / %d do not hold heads of %d / %d", dk_out, dv_out, dk, dv);
    LIYAB_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + static_cast<int64_t>(H) * dk <= ld && k_off + static_cast<int64_t>(G) * dk <= ld &&
                      v_off + static_cast<int64_t>(G) * dv <= ld,
                  "qk_prepare: the heads' columns pass the source's rows");
    LIYAB_REQUIRE(rot_dims >= 0 && rot_dims <= dk && rot_dims % 2 == 0 && (rot_dims == 0 || freqs != nullptr), "qk_prepare: %d turned entries of heads of %d", rot_dims, dk);
    LIYAB_REQUIRE(temp_every >= 0, "qk_prepare: bad query factor");
    LIYAB_REQUIRE((v_first == nullptr) == (v_lam == nullptr) && !(v_keep != nullptr && v_first != nullptr), "qk_prepare: values are kept, or mixed with kept ones and a rate");
    if (n == 0) return 0;
    dim3 grid(n, H + 2 * G);
    const double* fr = rot_dims > 0 ? freqs : nullptr;
    if (dtype == kF32)
        qk_prepare_kernel<float><<<grid, kWave, 0, stream>>>(src, ld, q_off, k_off, v_off, H, G, dk, dv, dk_out, dv_out, static_cast<float*>(q_out), static_cast<float*>(kc),
                                                             static_cast<float*>(vc), slots, page_size, num_pages, q_norm, k_norm, eps, fr, rot_dims,
                                                             temp_coef, temp_every, positions, rot_halves, rot_mag, v_keep, v_first, v_lam);
    else if (dtype == kBF16)
        qk_prepare_kernel<bf16_t><<<grid, kWave, 0, stream>>>(src, ld, q_off, k_off, v_off, H, G, dk, dv, dk_out, dv_out, static_cast<bf16_t*>(q_out),
                                                              static_cast<bf16_t*>(kc), static_cast<bf16_t*>(vc), slots, page_size, num_pages, q_norm,
                                                              k_norm, eps, fr, rot_dims, temp_coef, temp_every, positions, rot_halves, rot_mag, v_keep,
                                                              v_first, v_lam);
    else return fail(1, "qk_prepare: unknown dtype %d", dtype);
    return check_launch("qk_prepare");
}

extern "C" int liyab_attention_scored(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc, const void* vc, int dtype,
                                      const int* block_tables, int max_blocks, const int* tok_seq, const int* tok_pos, int n, float scale,
                                      float softcap, int window, const float* bias_table, int max_dist, const float* gate, int64_t gate_stride,
                                      int n_head, int n_kv_head, int dk, int dv, int page_size, int num_pages, const float* sinks, hipStream_t stream) {
    LIYAB_REQUIRE(out && q && kc && vc && block_tables && tok_seq && tok_pos, "attention_scored: null pointer");
    LIYAB_REQUIRE(num_pages > 0 && n >= 0 && n_head > 0 && n_kv_head > 0 && page_size > 0 && max_blocks > 0, "attention_scored: bad sizes");
    LIYAB_REQUIRE(n_head % n_kv_head == 0, "attention_scored: %d query heads are no multiple of %d key/value heads", n_head, n_kv_head);
    LIYAB_REQUIRE(dk > 0 && dk <= 512 && dv > 0 && dv <= AS_THREADS, "attention_scored: heads of %d / %d are outside 1..512 / 1..256", dk, dv);
    LIYAB_REQUIRE(out_stride >= static_cast<int64_t>(n_head) * dv && q_stride >= static_cast<int64_t>(n_head) * dk, "attention_scored: row strides are shorter than the heads");
    LIYAB_REQUIRE(window >= 0 && softcap >= 0.0f, "attention_scored: negative window or cap");
    LIYAB_REQUIRE(bias_table == nullptr || max_dist >= 0, "attention_scored: a bias table needs its largest distance");
    LIYAB_REQUIRE(gate == nullptr || gate_stride >= static_cast<int64_t>(n_head) * dv, "attention_scored: the gate's rows are shorter than the heads");
    LIYAB_REQUIRE(n_head <= 65535, "attention_scored: too many heads");
    if (n == 0) return 0;
    const int G = AS_THREADS / dv;
    const size_t smem = sizeof(float) * (dk + AS_THREADS + AS_THREADS / kWave + static_cast<size_t>(G) * dv);
    dim3 grid(n, n_head);
    if (dtype == kF32)
        attention_scored_kernel<float><<<grid, AS_THREADS, smem, stream>>>(
            static_cast<float*>(out), out_stride, static_cast<const float*>(q), q_stride, static_cast<const float*>(kc), static_cast<const float*>(vc),
            block_tables, max_blocks, tok_seq, tok_pos, scale, softcap, window, bias_table, max_dist, gate, gate_stride, n_head, n_kv_head, dk, dv,
            page_size, num_pages, sinks);
    else if (dtype == kBF16)
        attention_scored_kernel<bf16_t><<<grid, AS_THREADS, smem, stream>>>(
            static_cast<bf16_t*>(out), out_stride, static_cast<const bf16_t*>(q), q_stride, static_cast<const bf16_t*>(kc), static_cast<const bf16_t*>(vc),
            block_tables, max_blocks, tok_seq, tok_pos, scale, softcap, window, bias_table, max_dist, gate, gate_stride, n_head, n_kv_head, dk, dv,
            page_size, num_pages, sinks);
    else return fail(1, "attention_scored: unknown dtype %d", dtype);
    return check_launch("attention_scored");
}

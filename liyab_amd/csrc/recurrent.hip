// Mixers that carry a matrix of state from token to token instead of keys: the recurrence itself and
// what stands around it.
//
// Both recurrences here keep, a head, a matrix S [rows, cols] of 32-bit floats a request:
//   decayed outer products with a bonus (a "wkv" head; rows = key channels, cols = value channels):
//       o_t = (S + diag(u) k_t v_t^T)^T r_t,      S <- diag(w_t) S + k_t v_t^T,   w_t = exp(-exp(wraw_t + w0))
//   a selective state space (rows = state size, cols = the head's channels), a = exp(-exp(A_log) dt_t):
//       S <- a S + dt_t B_t x_t^T,                y_t = S^T C_t + D x_t,          dt_t = softplus(dtraw_t + dt_bias)
// One kernel serves both: a workgroup a (request, head) walks the request's tokens of the step in order.
// A thread owns one column of a block of rows of S in registers, so nothing of the state moves between
// threads; a token's vectors are staged through LDS sixteen tokens at a time (one trip to memory a
// chunk, not a token), the threads leave partial sums of the outputs in LDS, and after the chunk the
// workgroup adds them up and finishes the rows (a wkv head: unit root mean square over the head, the
// weight, the gate silu(g); a state-space head: + D x). The state comes from the request's slot (zeros
// at position 0 whatever the slot still holds) and goes back to it. The workgroup of head 0 also keeps
// the request's last input rows for the next step (the previous token's input of a token shift, the last
// taps - 1 inputs of a short convolution), at ring place position % ring: after every read of them, since
// the kernels that read them ran before this one.
// A step with a long portion runs the same kernel over segments of the portions side by side (seg_tokens > 0), in three
// launches: every segment from a zero state for its end state and the product of its decays; scan_combine_kernel, which
// strings a request's segments together and leaves each the state it starts from; every segment again from that state,
// with outputs. Decays are only ever multiplied, and the grids follow from the step's rows and requests alone.
//
// liyab_token_shift: m_c[t] = h[t] + (h[t - 1] - h[t]) * mu_c for each of n_mix learned mixes (a token's mixes side by side
//   in its row of the output, [n, n_mix * d]), the previous
//   row taken from the step's rows, from the request's slot, or zero at position 0.
// liyab_conv_act: out[t, c] = silu(bias[c] + sum_j w[c, j] * in[t - taps + 1 + j, c]) over a request's
//   own rows in time (the last column of w is the current row's), earlier rows from the ring; act = 0: without the silu.
// liyab_gated_group_norm: out = unit_rms_g(y * silu(z)) * w, the root mean square taken over each of
//   `groups` equal parts of a row.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int SCAN_THREADS = 512;  // eight waves, two a SIMD: one wave's waits for LDS and for its own results hide behind the other's work
constexpr int SCAN_CHUNK = 16;  // tokens staged through LDS together
constexpr size_t SCAN_MAX_LDS = 128 * 1024;

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

struct ScanArgs {
    // common
    float* state;           // [n_slots, state_stride]; the heads' matrices first, [H, rows, cols]
    int64_t state_stride;
    int n_slots;
    const int* seq_starts;  // [n_seqs + 1]
    const int* positions;   // [n]
    const int* state_slots; // [n_seqs]
    int H, rows, cols;
    int col_lanes;          // a power of two >= cols (threads side by side a block of rows)
    int rows_per;           // rows a thread holds
    // the rows kept for the next step
    const void* keep_src;
    int keep_bf16;
    int64_t keep_ld;
    int keep_width, keep_ring;
    int64_t keep_off;       // floats from the slot's start
    // wkv
    const float *r, *k, *v, *wraw, *gate;
    int64_t ld;
    const float *w0, *u, *norm_w;
    float eps;
    void* out;              // wkv: rows in the compute type [n, H * cols]; ssd: float [n, ldy]
    // ssd
    const float* xbc;       // [n, ldx]: x at 0, B at inner, C at inner + G * rows
    int64_t ldx;
    const float* dtraw;     // [n, ldp], one a head
    int64_t ldp;
    const float *dt_bias, *A_log, *Dskip;
    int64_t ldy;
    int G, inner;
    // long portions in segments (seg_tokens > 0): a workgroup a (segment, head) instead of a (request, head), in three passes
    int n_seqs, seg_tokens, max_segs, phase;  // phase 0: the whole portion by one workgroup; 1: each segment from a zero state, for its end; 3: each segment from its true start
    float* seg_state;       // [segments][H][rows][cols]: after pass 1 a segment's own end state, after the combining pass the state it starts from
    float* seg_decay;       // [segments][H][rows]: the product of a segment's decays, a row
};

// PF: elements a thread fetches ahead of each staged array (0: none are fetched ahead; the staging loop takes any size).
// With PF > 0 the next chunk's values are asked for before the current chunk is computed and written to LDS after it, so
// that a chunk's trip to memory hides behind the chunk before.
template <int MODE, int REG, int PF, typename OutT>
__global__ void __launch_bounds__(SCAN_THREADS)
scan_kernel(ScanArgs a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int h = blockIdx.y, tid = threadIdx.x;
    int s = blockIdx.x, seg_begin = -1, seg_end = -1;
    bool last_seg = true;
    if (a.seg_tokens > 0) {
        // segment blockIdx.x in the order of the requests: which request's, and which of its segments (a workgroup past the last exits)
        int g = blockIdx.x;
        for (s = 0; s < a.n_seqs; ++s) {
            const int b = a.seq_starts[s], len = a.seq_starts[s + 1] - b;
            const int n_seg = (len + a.seg_tokens - 1) / a.seg_tokens;
            if (g < n_seg) {
                seg_begin = b + g * a.seg_tokens;
                seg_end = min(seg_begin + a.seg_tokens, b + len);
                last_seg = g == n_seg - 1;
                break;
            }
            g -= n_seg;
        }
        if (seg_begin < 0 || (a.phase == 1 && last_seg)) return;  // (nobody needs the end state of a request's last segment from zero)
    }
    const int R = a.rows, C = a.cols, CL = a.col_lanes;
    const int n_rb = SCAN_THREADS / CL;
    const int Rp = n_rb * a.rows_per;  // rows as staged: zeros behind the last (rows_per is a multiple of 4)
    float* decay = lds;                           // [CHUNK][Rp]
    float* inr = decay + SCAN_CHUNK * Rp;         // [CHUNK][Rp]
    float* qr = inr + SCAN_CHUNK * Rp;            // [CHUNK][Rp]
    float* val = qr + SCAN_CHUNK * Rp;            // [CHUNK][CL]
    float* part = val + SCAN_CHUNK * CL;          // [CHUNK][n_rb][CL]

    const int begin = seg_begin >= 0 ? seg_begin : a.seq_starts[s], end = seg_begin >= 0 ? seg_end : a.seq_starts[s + 1];
    const int slot = a.state_slots[s];
    const bool slot_ok = slot >= 0 && slot < a.n_slots;
    const int cl_shift = __builtin_ctz(CL);  // (CL is a power of two)
    const int j = tid & (CL - 1), rb = tid >> cl_shift;
    const int i0 = rb * a.rows_per;
    float* S_glob = a.state + static_cast<int64_t>(slot_ok ? slot : 0) * a.state_stride + static_cast<int64_t>(h) * R * C;
    const bool fresh = a.positions[begin] == 0;
    float* S_seg = a.seg_state + (static_cast<int64_t>(blockIdx.x) * a.H + h) * R * C;  // (read or written in passes 1 and 3 only)

    float S[REG], bonus[MODE == 0 ? REG : 1], prod[REG];
#pragma unroll
    for (int ii = 0; ii < REG; ++ii) {
        const int i = i0 + ii;
        const bool mine = ii < a.rows_per && i < R && j < C;
        prod[ii] = 1.0f;
        if (a.phase == 0) S[ii] = (mine && slot_ok && !fresh) ? S_glob[static_cast<int64_t>(i) * C + j] : 0.0f;
        else S[ii] = (mine && a.phase == 3) ? S_seg[static_cast<int64_t>(i) * C + j] : 0.0f;
        if (MODE == 0) bonus[ii] = (ii < a.rows_per && i < R) ? a.u[h * R + i] : 0.0f;
    }
    const int g = MODE == 1 ? h / (a.H / a.G) : 0;
    const float neg_A = MODE == 1 ? -expf(a.A_log[h]) : 0.0f;
    const float dskip = MODE == 1 ? a.Dskip[h] : 0.0f;
    const float dtb = MODE == 1 ? a.dt_bias[h] : 0.0f;

    // What a chunk's staged element (token tt of the chunk, row i / column jj) is made of, as it lies in memory. The loads stand
    // under no branch (a load under a branch is waited for where the branch ends): a token or a row past the end is fetched
    // from the last one's address and masked when it is staged.
    auto raw_rows = [&](int c0, int len, int tt, int i, float& d, float& x, float& q) {
        const int64_t t = c0 + min(tt, len - 1);
        const int ic = min(i, R - 1);
        if (MODE == 0) {
            const int64_t at = t * a.ld + h * R + ic;
            d = a.wraw[at] + a.w0[h * R + ic];
            x = a.k[at];
            q = a.r[at];
        } else {
            d = a.dtraw[t * a.ldp + h];
            x = a.xbc[t * a.ldx + a.inner + g * R + ic];
            q = a.xbc[t * a.ldx + a.inner + a.G * R + g * R + ic];
        }
    };
    auto raw_val = [&](int c0, int len, int tt, int jj) {
        const int64_t t = c0 + min(tt, len - 1);
        const int jc = min(jj, C - 1);
        return MODE == 0 ? a.v[t * a.ld + h * C + jc] : a.xbc[t * a.ldx + h * C + jc];
    };
    auto raw_gate = [&](int c0, int len, int tt, int jj) {
        return a.gate[static_cast<int64_t>(c0 + min(tt, len - 1)) * a.ld + h * C + min(jj, C - 1)];
    };
    auto put_rows = [&](int len, int tt, int i, float d, float x, float q) {
        if (tt < len) {
            const int e = tt * Rp + i;
            const bool real = i < R;
            if (MODE == 0) {
                decay[e] = real ? expf(-expf(d)) : 0.0f;
                inr[e] = real ? x : 0.0f;
            } else {
                const float dt = softplus_f(d + dtb);
                decay[e] = real ? expf(neg_A * dt) : 0.0f;
                inr[e] = real ? dt * x : 0.0f;
            }
            qr[e] = real ? q : 0.0f;
        }
    };
    constexpr int NPF = PF > 0 ? PF : 1;
    float pd[NPF], px[NPF], pq[NPF], pv[NPF], pg[NPF];
    // where this thread's elements of a chunk lie (token, row) and (token, column): the same for every chunk
    int rt[NPF], ri[NPF], vt[NPF], vc[NPF];
#pragma unroll
    for (int k = 0; k < NPF; ++k) {
        const int e = tid + k * SCAN_THREADS;
        rt[k] = e / Rp;
        ri[k] = e % Rp;
        vt[k] = e >> cl_shift;
        vc[k] = e & (CL - 1);
    }
    float* gates = part + SCAN_CHUNK * SCAN_THREADS;  // [CHUNK][CL] (wkv): silu of the gate's logits
    auto fetch = [&](int from) {  // (past the request's last token: its last token once more, never staged)
        const int c0 = min(from, end - 1);
        const int len = min(SCAN_CHUNK, end - c0);
#pragma unroll
        for (int k = 0; k < NPF; ++k) {
            raw_rows(c0, len, rt[k], ri[k], pd[k], px[k], pq[k]);
            pv[k] = raw_val(c0, len, vt[k], vc[k]);
            if (MODE == 0) pg[k] = raw_gate(c0, len, vt[k], vc[k]);
        }
    };
    if (PF > 0) fetch(begin);

    for (int c0 = begin; c0 < end; c0 += SCAN_CHUNK) {
        const int len = min(SCAN_CHUNK, end - c0);
        __syncthreads();  // the chunk before has been read
        if (PF > 0) {
#pragma unroll
            for (int k = 0; k < NPF; ++k) {
                put_rows(len, rt[k], ri[k], pd[k], px[k], pq[k]);
                if (vt[k] < len) {
                    val[vt[k] * CL + vc[k]] = vc[k] < C ? pv[k] : 0.0f;
                    if (MODE == 0) gates[vt[k] * CL + vc[k]] = silu_f(pg[k]);
                }
            }
        } else {
            for (int e = tid; e < len * Rp; e += SCAN_THREADS) {
                float d, x, q;
                raw_rows(c0, len, e / Rp, e % Rp, d, x, q);
                put_rows(len, e / Rp, e % Rp, d, x, q);
            }
            for (int e = tid; e < len * CL; e += SCAN_THREADS) {
                val[e] = (e & (CL - 1)) < C ? raw_val(c0, len, e >> cl_shift, e & (CL - 1)) : 0.0f;
                if (MODE == 0) gates[e] = silu_f(raw_gate(c0, len, e >> cl_shift, e & (CL - 1)));
            }
        }
        __syncthreads();
        if (PF > 0) fetch(c0 + SCAN_CHUNK);  // on their way while this chunk is computed
        // A token's operands are asked for while the token before is computed: the reads of LDS stand ahead of the store of
        // the partial sums in the program's order (the compiler cannot move them past it by itself), and with one wave a SIMD
        // nothing else hides their way.
        float4 nd[REG / 4], nk[REG / 4], nq[REG / 4];
        float nv;
        auto operands = [&](int tt) {
            nv = val[tt * CL + j];
            const float4* dr = reinterpret_cast<const float4*>(decay + tt * Rp + i0);
            const float4* ir = reinterpret_cast<const float4*>(inr + tt * Rp + i0);
            const float4* qq = reinterpret_cast<const float4*>(qr + tt * Rp + i0);
#pragma unroll
            for (int i4 = 0; i4 < REG / 4; ++i4) {
                const int at = 4 * i4 < a.rows_per ? i4 : 0;  // (rows this thread does not hold: its first four once more)
                nd[i4] = dr[at];
                nk[i4] = ir[at];
                nq[i4] = qq[at];
            }
        };
        operands(0);
        auto tokens = [&](auto first_pass) {
            constexpr bool kEndOnly = decltype(first_pass)::value;  // pass 1: the state and the decays' product, no outputs
            for (int tt = 0; tt < len; ++tt) {
                float4 cd[REG / 4], ck[REG / 4], cq[REG / 4];
                const float vj = nv;
#pragma unroll
                for (int i4 = 0; i4 < REG / 4; ++i4) {
                    cd[i4] = nd[i4];
                    ck[i4] = nk[i4];
                    cq[i4] = nq[i4];
                }
                operands(min(tt + 1, len - 1));
                float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll
                for (int i4 = 0; i4 < REG / 4; ++i4) {
                    if (4 * i4 < a.rows_per) {
                        const float dd[4] = {cd[i4].x, cd[i4].y, cd[i4].z, cd[i4].w}, kk[4] = {ck[i4].x, ck[i4].y, ck[i4].z, ck[i4].w},
                                    qv[4] = {cq[i4].x, cq[i4].y, cq[i4].z, cq[i4].w};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int ii = 4 * i4 + e;
                            const float kin = kk[e] * vj;
                            float& acc = e % 2 ? acc1 : acc0;
                            if constexpr (kEndOnly) {
                                S[ii] = fmaf(dd[e], S[ii], kin);
                                prod[ii] *= dd[e];
                            } else if (MODE == 0) {
                                acc = fmaf(qv[e], fmaf(bonus[ii], kin, S[ii]), acc);
                                S[ii] = fmaf(dd[e], S[ii], kin);
                            } else {
                                S[ii] = fmaf(dd[e], S[ii], kin);
                                acc = fmaf(qv[e], S[ii], acc);
                            }
                        }
                    }
                }
                if constexpr (!kEndOnly) part[(tt * n_rb + rb) * CL + j] = acc0 + acc1;
            }
        };
        if (a.phase == 1) tokens(std::true_type{});
        else tokens(std::false_type{});
        __syncthreads();
        if (a.phase == 1) continue;  // (no outputs in pass 1)
        if (MODE == 0) {
            // a wave a token: the head's outputs, their root mean square, the weight and the gate
            const int wave = tid / kWave, lane = tid % kWave;
            for (int tt = wave; tt < len; tt += SCAN_THREADS / kWave) {
                const int64_t t = c0 + tt;
                float ss = 0.0f;
                for (int jj = lane; jj < C; jj += kWave) {
                    float o = 0.0f;
                    for (int b = 0; b < n_rb; ++b) o += part[(tt * n_rb + b) * CL + jj];
                    ss = fmaf(o, o, ss);
                }
                const float rinv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(C) + a.eps);
                for (int jj = lane; jj < C; jj += kWave) {
                    float o = 0.0f;
                    for (int b = 0; b < n_rb; ++b) o += part[(tt * n_rb + b) * CL + jj];
                    const int col = h * C + jj;
                    const float y = o * rinv * a.norm_w[col] * gates[tt * CL + jj];
                    static_cast<OutT*>(a.out)[t * (static_cast<int64_t>(a.H) * C) + col] = from_float<OutT>(y);
                }
            }
        } else {
            for (int e = tid; e < len * CL; e += SCAN_THREADS) {
                const int tt = e >> cl_shift, jj = e & (CL - 1);
                if (jj >= C) continue;
                float o = 0.0f;
                for (int b = 0; b < n_rb; ++b) o += part[(tt * n_rb + b) * CL + jj];
                static_cast<float*>(a.out)[(c0 + tt) * a.ldy + h * C + jj] = fmaf(dskip, val[tt * CL + jj], o);
            }
        }
    }
    if (a.phase == 1) {
        // the segment's end state from zero and the product of its decays, for the pass that strings the segments together
        float* P_seg = a.seg_decay + (static_cast<int64_t>(blockIdx.x) * a.H + h) * R;
#pragma unroll
        for (int ii = 0; ii < REG; ++ii) {
            const int i = i0 + ii;
            if (ii < a.rows_per && i < R && j < C) S_seg[static_cast<int64_t>(i) * C + j] = S[ii];
            if (ii < a.rows_per && i < R && j == 0) P_seg[i] = prod[ii];
        }
        return;
    }
    if (slot_ok && last_seg) {
#pragma unroll
        for (int ii = 0; ii < REG; ++ii) {
            const int i = i0 + ii;
            if (ii < a.rows_per && i < R && j < C) S_glob[static_cast<int64_t>(i) * C + j] = S[ii];
        }
        if (h == 0 && a.keep_src != nullptr && a.keep_ring > 0) {
            float* dst = a.state + static_cast<int64_t>(slot) * a.state_stride + a.keep_off;
            const int first = max(a.seq_starts[s], end - a.keep_ring);  // (of the request's rows, not of its last segment's only)
            for (int t = first; t < end; ++t) {
                const int place = a.positions[t] % a.keep_ring;
                for (int c = tid; c < a.keep_width; c += SCAN_THREADS) {
                    const int64_t at = static_cast<int64_t>(t) * a.keep_ld + c;
                    dst[static_cast<int64_t>(place) * a.keep_width + c] =
                        a.keep_bf16 ? bf16_to_float(static_cast<const bf16_t*>(a.keep_src)[at]) : static_cast<const float*>(a.keep_src)[at];
                }
            }
        }
    }
}

// Between the two passes over a long portion's segments: the state each segment starts from. A workgroup a (request, head)
// walks the request's segments in order, S <- decays' product * S + the segment's own end state, and leaves in seg_state what
// each segment starts from (the first: the slot's state, or zeros at position 0).
__global__ void __launch_bounds__(256)
scan_combine_kernel(ScanArgs a) {
    const int s = blockIdx.x, h = blockIdx.y;
    int g0 = 0;
    for (int q = 0; q < s; ++q) g0 += (a.seq_starts[q + 1] - a.seq_starts[q] + a.seg_tokens - 1) / a.seg_tokens;
    const int begin = a.seq_starts[s];
    const int n_seg = (a.seq_starts[s + 1] - begin + a.seg_tokens - 1) / a.seg_tokens;
    const int slot = a.state_slots[s];
    const bool from_slot = slot >= 0 && slot < a.n_slots && a.positions[begin] != 0;
    const int R = a.rows, C = a.cols;
    const int e = blockIdx.z * 256 + threadIdx.x;  // an element of the state a thread
    if (e >= R * C) return;
    const int i = e / C;
    const float* S0 = a.state + static_cast<int64_t>(from_slot ? slot : 0) * a.state_stride + static_cast<int64_t>(h) * R * C;
    float S = from_slot ? S0[e] : 0.0f;
    // eight segments' values are asked for together, ahead of the chain that uses them (a load behind a store to the same
    // array is not moved ahead of it by the compiler)
    constexpr int kBatch = 8;
    for (int c0 = 0; c0 < n_seg; c0 += kBatch) {
        float own[kBatch], dec[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const int64_t g = g0 + min(c0 + u, n_seg - 1);
            own[u] = a.seg_state[(g * a.H + h) * R * C + e];  // (a request's last segment has none: read and dropped)
            dec[u] = a.seg_decay[(g * a.H + h) * R + i];
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            if (c0 + u < n_seg) {
                a.seg_state[(static_cast<int64_t>(g0 + c0 + u) * a.H + h) * R * C + e] = S;
                if (c0 + u + 1 < n_seg) S = fmaf(dec[u], S, own[u]);
            }
        }
    }
}

// rows a thread holds (a multiple of 4), lanes side by side, elements a thread fetches ahead, and the dynamic LDS for a
// state of rows x cols; false when the kernel does not take the size
static bool scan_shape(int rows, int cols, int* col_lanes, int* rows_per, int* reg, int* pf, size_t* smem) {
    if (rows <= 0 || cols <= 0 || cols > SCAN_THREADS) return false;
    int cl = 1;
    while (cl < cols) cl *= 2;
    // no more blocks of rows than the rows fill four at a time (few columns of many rows: lanes idle rather than rows staged as zeros)
    while (SCAN_THREADS / cl > 1 && (SCAN_THREADS / cl) * 4 > (rows + 3) / 4 * 4) cl *= 2;
    const int n_rb = SCAN_THREADS / cl;
    const int rp = ((rows + n_rb - 1) / n_rb + 3) / 4 * 4;
    if (rp > 64) return false;
    *col_lanes = cl;
    *rows_per = rp;
    *reg = rp <= 8 ? 8 : rp <= 16 ? 16 : rp <= 32 ? 32 : 64;
    const int Rp = n_rb * rp;
    const int ahead = (SCAN_CHUNK * (Rp > cl ? Rp : cl) + SCAN_THREADS - 1) / SCAN_THREADS;
    *pf = ahead <= 4 ? 4 : ahead <= 8 ? 8 : 0;
    *smem = sizeof(float) * (static_cast<size_t>(3) * SCAN_CHUNK * Rp + 2 * SCAN_CHUNK * cl + SCAN_CHUNK * SCAN_THREADS);
    return *smem <= SCAN_MAX_LDS;
}

template <int MODE, int REG, int PF, typename OutT>
static void launch_scan_one(const ScanArgs& a, int n_seqs, size_t smem, hipStream_t stream) {
    auto kern = scan_kernel<MODE, REG, PF, OutT>;
    if (smem > 48 * 1024) {
        static bool allowed = false;  // (once a kernel: more dynamic LDS than the default limit)
        if (!allowed) allowed = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(SCAN_MAX_LDS)) == hipSuccess;
    }
    if (a.seg_tokens > 0) {
        // segments side by side: each from a zero state for its end, the ends strung together, each again from its true start
        ScanArgs p = a;
        p.phase = 1;
        kern<<<dim3(a.max_segs, a.H), SCAN_THREADS, smem, stream>>>(p);
        scan_combine_kernel<<<dim3(n_seqs, a.H, (a.rows * a.cols + 255) / 256), 256, 0, stream>>>(p);
        p.phase = 3;
        kern<<<dim3(a.max_segs, a.H), SCAN_THREADS, smem, stream>>>(p);
        return;
    }
    kern<<<dim3(n_seqs, a.H), SCAN_THREADS, smem, stream>>>(a);
}

template <int MODE, typename OutT, int PF>
static void launch_scan_pf(const ScanArgs& a, int n_seqs, int reg, size_t smem, hipStream_t stream) {
    switch (reg) {
        case 8: launch_scan_one<MODE, 8, PF, OutT>(a, n_seqs, smem, stream); break;
        case 16: launch_scan_one<MODE, 16, PF, OutT>(a, n_seqs, smem, stream); break;
        case 32: launch_scan_one<MODE, 32, PF, OutT>(a, n_seqs, smem, stream); break;
        default: launch_scan_one<MODE, 64, PF, OutT>(a, n_seqs, smem, stream); break;
    }
}

template <int MODE, typename OutT>
static void launch_scan(const ScanArgs& a, int n_seqs, int reg, int pf, size_t smem, hipStream_t stream) {
    if (pf == 4) launch_scan_pf<MODE, OutT, 4>(a, n_seqs, reg, smem, stream);
    else if (pf == 8) launch_scan_pf<MODE, OutT, 8>(a, n_seqs, reg, smem, stream);
    else launch_scan_pf<MODE, OutT, 0>(a, n_seqs, reg, smem, stream);
}

template <typename T>
__global__ void __launch_bounds__(256)
token_shift_kernel(T* __restrict__ out, const T* __restrict__ h, const float* __restrict__ mu, int n_mix, const float* __restrict__ state,
                   int64_t state_stride, int n_slots, const int* __restrict__ tok_seq, const int* __restrict__ positions,
                   const int* __restrict__ seq_starts, const int* __restrict__ state_slots, int n, int d) {
    const int t = blockIdx.x;
    const int s = tok_seq[t], p = positions[t];
    const int slot = state_slots[s];
    const bool from_step = t > seq_starts[s];
    const bool from_state = !from_step && p > 0 && slot >= 0 && slot < n_slots;
    const float* prev_state = state + static_cast<int64_t>(from_state ? slot : 0) * state_stride;
    for (int i = threadIdx.x; i < d; i += 256) {
        const float cur = to_float<T>(h[static_cast<int64_t>(t) * d + i]);
        // both candidates are asked for under no branch (a load under a branch is waited for where the branch ends)
        const float before = to_float<T>(h[static_cast<int64_t>(max(t - 1, 0)) * d + i]);
        const float kept = prev_state[i];
        const float prev = p > 0 ? (from_step ? before : (from_state ? kept : 0.0f)) : 0.0f;
        const float diff = prev - cur;
        for (int c = 0; c < n_mix; ++c)
            out[(static_cast<int64_t>(t) * n_mix + c) * d + i] = from_float<T>(fmaf(diff, mu[c * d + i], cur));
    }
}

__global__ void __launch_bounds__(256)
conv_act_kernel(float* __restrict__ out, int64_t ldo, const float* __restrict__ in, int64_t ldi, const float* __restrict__ w,
                const float* __restrict__ bias, int taps, const float* __restrict__ state, int64_t state_stride, int n_slots,
                const int* __restrict__ tok_seq, const int* __restrict__ positions, const int* __restrict__ seq_starts,
                const int* __restrict__ state_slots, int C, int act) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int s = tok_seq[t], p = positions[t];
    const int begin = seq_starts[s];
    const int slot = state_slots[s];
    const bool slot_ok = slot >= 0 && slot < n_slots;
    const float* ring = state + static_cast<int64_t>(slot_ok ? slot : 0) * state_stride;
    float acc = bias != nullptr ? bias[c] : 0.0f;
    for (int jt = 0; jt < taps; ++jt) {
        const int back = taps - 1 - jt;  // rows before this one
        const int sp = p - back;
        if (sp < 0) continue;
        float x;
        if (t - back >= begin) x = in[static_cast<int64_t>(t - back) * ldi + c];
        else x = slot_ok ? ring[static_cast<int64_t>(sp % (taps - 1)) * C + c] : 0.0f;
        acc = fmaf(w[static_cast<int64_t>(c) * taps + jt], x, acc);
    }
    out[static_cast<int64_t>(t) * ldo + c] = act ? silu_f(acc) : acc;
}

template <typename T>
__global__ void __launch_bounds__(256)
gated_group_norm_kernel(T* __restrict__ out, const float* __restrict__ y, int64_t ldy, const float* __restrict__ z, int64_t ldz,
                        const float* __restrict__ w, float eps, int inner, int groups) {
    __shared__ float red[256 / kWave];
    const int t = blockIdx.x, g = blockIdx.y;
    const int width = inner / groups;
    const float* yr = y + static_cast<int64_t>(t) * ldy + g * width;
    const float* zr = z + static_cast<int64_t>(t) * ldz + g * width;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < width; i += 256) {
        const float v = yr[i] * silu_f(zr[i]);
        ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = ss;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < 256 / kWave; ++i) total += red[i];
    const float rinv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
    for (int i = threadIdx.x; i < width; i += 256) {
        const float v = yr[i] * silu_f(zr[i]) * rinv * w[g * width + i];
        out[static_cast<int64_t>(t) * inner + g * width + i] = from_float<T>(v);
    }
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_scan_takes(int rows, int cols) {
    int cl, rp, reg, pf;
    size_t smem;
    return scan_shape(rows, cols, &cl, &rp, &reg, &pf, &smem) ? 1 : 0;
}

extern "C" int liyab_wkv_scan(void* out, int out_dtype, const float* r, const float* k, const float* v, const float* wraw, const float* gate,
                              int64_t ld, const float* w0, const float* u, const float* norm_w, float eps, float* state, int64_t state_stride,
                              int n_slots, const void* keep_src, int keep_dtype, int64_t keep_ld, int keep_width, int64_t keep_off,
                              const int* seq_starts, const int* positions, const int* state_slots, int n_seqs, int H, int D,
                              int seg_tokens, int max_segs, float* seg_state, float* seg_decay, hipStream_t stream) {
    LIYAB_REQUIRE(out && r && k && v && wraw && gate && w0 && u && norm_w && state && seq_starts && positions && state_slots, "wkv_scan: null pointer");
    LIYAB_REQUIRE(n_seqs >= 0 && H > 0 && D > 0 && n_slots > 0, "wkv_scan: bad sizes");
    LIYAB_REQUIRE(ld >= static_cast<int64_t>(H) * D, "wkv_scan: rows shorter than heads x head size");
    LIYAB_REQUIRE(state_stride >= static_cast<int64_t>(H) * D * D + (keep_src ? keep_off - static_cast<int64_t>(H) * D * D + keep_width : 0) &&
                      (keep_src == nullptr || keep_off >= static_cast<int64_t>(H) * D * D),
                  "wkv_scan: a slot of %lld floats does not hold the state", static_cast<long long>(state_stride));
    ScanArgs a = {};
    size_t smem;
    int reg, pf;
    LIYAB_REQUIRE(scan_shape(D, D, &a.col_lanes, &a.rows_per, &reg, &pf, &smem), "wkv_scan: heads of %d are not taken", D);
    if (n_seqs == 0) return 0;
    LIYAB_REQUIRE(seg_tokens >= 0 && (seg_tokens == 0 || (max_segs > 0 && seg_state && seg_decay)), "scan: segments need their count and scratch");
    a.n_seqs = n_seqs; a.seg_tokens = seg_tokens; a.max_segs = max_segs; a.seg_state = seg_state; a.seg_decay = seg_decay;
    a.state = state; a.state_stride = state_stride; a.n_slots = n_slots;
    a.seq_starts = seq_starts; a.positions = positions; a.state_slots = state_slots;
    a.H = H; a.rows = D; a.cols = D;
    a.keep_src = keep_src; a.keep_bf16 = keep_dtype == kBF16; a.keep_ld = keep_ld; a.keep_width = keep_width; a.keep_ring = 1; a.keep_off = keep_off;
    a.r = r; a.k = k; a.v = v; a.wraw = wraw; a.gate = gate; a.ld = ld; a.w0 = w0; a.u = u; a.norm_w = norm_w; a.eps = eps; a.out = out;
    if (out_dtype == kF32) launch_scan<0, float>(a, n_seqs, reg, pf, smem, stream);
    else if (out_dtype == kBF16) launch_scan<0, bf16_t>(a, n_seqs, reg, pf, smem, stream);
    else return fail(1, "wkv_scan: unknown dtype %d", out_dtype);
    return check_launch("wkv_scan");
}

extern "C" int liyab_ssd_scan(float* y, int64_t ldy, const float* xbc, int64_t ldx, const float* dtraw, int64_t ldp, const float* dt_bias,
                              const float* A_log, const float* Dskip, float* state, int64_t state_stride, int n_slots, const float* keep_src,
                              int64_t keep_ld, int keep_width, int keep_ring, int64_t keep_off, const int* seq_starts, const int* positions,
                              const int* state_slots, int n_seqs, int H, int P, int N, int G, int seg_tokens, int max_segs, float* seg_state,
                              float* seg_decay, hipStream_t stream) {
    LIYAB_REQUIRE(y && xbc && dtraw && dt_bias && A_log && Dskip && state && seq_starts && positions && state_slots, "ssd_scan: null pointer");
    LIYAB_REQUIRE(n_seqs >= 0 && H > 0 && P > 0 && N > 0 && G > 0 && H % G == 0 && n_slots > 0, "ssd_scan: bad sizes");
    const int64_t inner = static_cast<int64_t>(H) * P;
    LIYAB_REQUIRE(ldy >= inner && ldx >= inner + 2 * static_cast<int64_t>(G) * N && ldp >= H, "ssd_scan: rows shorter than their parts");
    LIYAB_REQUIRE(state_stride >= inner * N && (keep_src == nullptr || (keep_off >= inner * N && state_stride >= keep_off + static_cast<int64_t>(keep_ring) * keep_width)),
                  "ssd_scan: a slot of %lld floats does not hold the state", static_cast<long long>(state_stride));
    ScanArgs a = {};
    size_t smem;
    int reg, pf;
    LIYAB_REQUIRE(scan_shape(N, P, &a.col_lanes, &a.rows_per, &reg, &pf, &smem), "ssd_scan: a state of %d x %d a head is not taken", N, P);
    if (n_seqs == 0) return 0;
    LIYAB_REQUIRE(seg_tokens >= 0 && (seg_tokens == 0 || (max_segs > 0 && seg_state && seg_decay)), "scan: segments need their count and scratch");
    a.n_seqs = n_seqs; a.seg_tokens = seg_tokens; a.max_segs = max_segs; a.seg_state = seg_state; a.seg_decay = seg_decay;
    a.state = state; a.state_stride = state_stride; a.n_slots = n_slots;
    a.seq_starts = seq_starts; a.positions = positions; a.state_slots = state_slots;
    a.H = H; a.rows = N; a.cols = P;
    a.keep_src = keep_src; a.keep_bf16 = 0; a.keep_ld = keep_ld; a.keep_width = keep_width; a.keep_ring = keep_ring; a.keep_off = keep_off;
    a.out = y; a.ldy = ldy; a.xbc = xbc; a.ldx = ldx; a.dtraw = dtraw; a.ldp = ldp; a.dt_bias = dt_bias; a.A_log = A_log; a.Dskip = Dskip;
    a.G = G; a.inner = static_cast<int>(inner);
    launch_scan<1, float>(a, n_seqs, reg, pf, smem, stream);
    return check_launch("ssd_scan");
}

extern "C" int liyab_token_shift(void* out, int dtype, const void* h, const float* mu, int n_mix, const float* state, int64_t state_stride,
                                 int n_slots, const int* tok_seq, const int* positions, const int* seq_starts, const int* state_slots, int n,
                                 int d, hipStream_t stream) {
    LIYAB_REQUIRE(out && h && mu && state && tok_seq && positions && seq_starts && state_slots, "token_shift: null pointer");
    LIYAB_REQUIRE(n >= 0 && d > 0 && n_mix > 0 && n_slots > 0 && state_stride >= d, "token_shift: bad sizes");
    if (n == 0) return 0;
    if (dtype == kF32)
        token_shift_kernel<float><<<n, 256, 0, stream>>>(static_cast<float*>(out), static_cast<const float*>(h), mu, n_mix, state, state_stride,
                                                          n_slots, tok_seq, positions, seq_starts, state_slots, n, d);
    else if (dtype == kBF16)
        token_shift_kernel<bf16_t><<<n, 256, 0, stream>>>(static_cast<bf16_t*>(out), static_cast<const bf16_t*>(h), mu, n_mix, state, state_stride,
                                                           n_slots, tok_seq, positions, seq_starts, state_slots, n, d);
    else return fail(1, "token_shift: unknown dtype %d", dtype);
    return check_launch("token_shift");
}

extern "C" int liyab_conv_act(float* out, int64_t ldo, const float* in, int64_t ldi, const float* w, const float* bias, int taps,
                              const float* state, int64_t state_stride, int n_slots, const int* tok_seq, const int* positions,
                              const int* seq_starts, const int* state_slots, int n, int C, int act, hipStream_t stream) {
    LIYAB_REQUIRE(out && in && w && tok_seq && positions && seq_starts && state_slots, "conv_act: null pointer");
    LIYAB_REQUIRE(n >= 0 && n <= 65535 && C > 0 && taps >= 1 && ldo >= C && ldi >= C, "conv_act: bad sizes");
    LIYAB_REQUIRE(taps == 1 || (state != nullptr && n_slots > 0 && state_stride >= static_cast<int64_t>(taps - 1) * C),
                  "conv_act: %d taps need the last %d rows of a request in its slot", taps, taps - 1);
    if (n == 0) return 0;
    dim3 grid((C + 255) / 256, n);
    conv_act_kernel<<<grid, 256, 0, stream>>>(out, ldo, in, ldi, w, bias, taps, state, state_stride, taps > 1 ? n_slots : 0, tok_seq, positions,
                                              seq_starts, state_slots, C, act);
    return check_launch("conv_act");
}

extern "C" int liyab_gated_group_norm(void* out, int out_dtype, const float* y, int64_t ldy, const float* z, int64_t ldz, const float* w,
                                      float eps, int n, int inner, int groups, hipStream_t stream) {
    LIYAB_REQUIRE(out && y && z && w, "gated_group_norm: null pointer");
    LIYAB_REQUIRE(n >= 0 && inner > 0 && groups > 0 && groups <= 65535 && inner % groups == 0 && ldy >= inner && ldz >= inner, "gated_group_norm: bad sizes");
    if (n == 0) return 0;
    dim3 grid(n, groups);
    if (out_dtype == kF32) gated_group_norm_kernel<float><<<grid, 256, 0, stream>>>(static_cast<float*>(out), y, ldy, z, ldz, w, eps, inner, groups);
    else if (out_dtype == kBF16) gated_group_norm_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), y, ldy, z, ldz, w, eps, inner, groups);
    else return fail(1, "gated_group_norm: unknown dtype %d", out_dtype);
    return check_launch("gated_group_norm");
}

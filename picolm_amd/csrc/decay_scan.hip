// A matrix state whose every element decays by a factor of its own (mixers.h, picolm_call_decay_scan):
// the walk of a selective state-space layer (decays exp(dt A) per channel and state) and of linear
// attention with a forget gate per key channel.  All of it is float arithmetic, token by token.
//
// A column of the state lies in the registers of R lanes, up to DS_KPT rows each (row i R + r with
// lane r), so that the read-out along q is a short chain in a lane and a few steps across lanes.
// A decode step and short prompts walk whole sequences from and to the slot's state.  A longer
// prompt is walked in chunks side by side: the update is  S <- a S + k w^T  element by element, so a
// chunk's effect on a state is  S_end = P S_start + N  with P the product of the chunk's decays and
// N the chunk walked from zero; pass 1 leaves (N, P) of every chunk, a second kernel takes the
// states from chunk to chunk, pass 2 walks every chunk again from its start state and writes the
// outputs.  The result equals the unchunked walk up to the order of a few products and sums.
#include "mixers.h"

#include "api.h"
#include "common.h"

#define VIEW_REQUIRE(who, v)                                                                                      \
    PICOLM_REQUIRE((v) && (v)->struct_bytes == (int32_t)sizeof(picolm_step_view), "%s: the step view is of another version", who)

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// e^x for x <= 0 through the hardware's 2^y, with the rounding of y = x log2(e) carried along:
// y = hi + lo, e^x = 2^hi (1 + lo ln 2).  Within two units in the last place, at a tenth of the
// library function's instructions; a walk takes it once per state element and token.
__device__ __forceinline__ float exp_of_decay(float x) {
    const float log2e_hi = 1.44269502162933349609375f, log2e_lo = 1.925963033500011e-8f;
    const float hi = x * log2e_hi;
    const float lo = fmaf(x, log2e_hi, -hi) + x * log2e_lo;
    return __builtin_amdgcn_exp2f(hi) * fmaf(lo, 0.693147182464599609375f, 1.f);
}

#define DS_TB 16         // tokens whose q, k, decays and inputs wait in LDS at a time
#define DS_KPT 16        // rows of the state a thread keeps in registers
#define DS_MAX_KEY_DIM 256

struct DecayScan {
    const float* qk;
    const float* x;
    const float* dt;
    float* out;
    float* state;
    const float* dt_bias;
    const float* A;
    const float* skip;
    const int32_t* cu_seqlens;
    const int32_t* seq_slot;
    int64_t slot_floats;
    int qk_stride, q_off, k_off, a_off, x_stride, x_off, dt_stride, dt_off;
    int kind, heads, key_heads, key_dim, value_dim;
    int R, kpt, n_waves, n_cb;
    int mode, chunk_len, chunks_per_seq;      // mode 0: whole sequences; 1: (N, P) of every chunk; 3: outputs from the chunks' start states
    float* ws;                                // [sequence][chunk][head][N | P | S_start][key_dim][value_dim]
};

__device__ __forceinline__ float* ds_ws(const DecayScan& a, int seq, int chunk, int head, int part) {
    return a.ws + ((((size_t)seq * a.chunks_per_seq + chunk) * a.heads + head) * 3 + part) * a.key_dim * a.value_dim;
}

// KIND: 1 a decay per row, 2 exp(dt A) per element; TRACK: pass 1 of the chunked walk (no outputs, the decays' products kept)
template <int R, int KIND, bool TRACK>
__global__ __launch_bounds__(256) void decay_scan_kernel(DecayScan a) {
    extern __shared__ float ds_lds[];
    constexpr int CW = WAVE / R;
    constexpr int kpt = DS_KPT, kd = kpt * R;      // rows past key_dim are zeros that stay zeros: no test per row in the walk
    const int CB = a.n_waves * CW;
    float* ks = ds_lds;                      // [TB][kd]
    float* qs = ks + DS_TB * kd;             // [TB][kd]
    float* as = qs + DS_TB * kd;             // [TB][kd]   (kind 1)
    float* xs = as + DS_TB * kd;             // [TB][CB]
    float* dts = xs + DS_TB * CB;            // [TB][CB]   (kind 2)
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int cb = blockIdx.x % a.n_cb, head = (blockIdx.x / a.n_cb) % a.heads, unit = blockIdx.x / (a.n_cb * a.heads);
    const int seq = a.mode ? unit / a.chunks_per_seq : unit, chunk = a.mode ? unit % a.chunks_per_seq : 0;
    int row0 = a.cu_seqlens[seq], row1 = a.cu_seqlens[seq + 1];
    if (a.mode) {
        row0 += chunk * a.chunk_len;
        if (row0 >= row1) return;               // (the whole workgroup: the sequence has fewer chunks)
        row1 = min(row1, row0 + a.chunk_len);
    }
    const int r = lane / CW, col = wave * CW + lane % CW, j = cb * CB + col;
    const bool valid = j < a.value_dim;
    const int kh = head / (a.heads / a.key_heads);
    const size_t channel = (size_t)head * a.value_dim + j;
    float* st = a.state + (size_t)a.seq_slot[seq] * a.slot_floats + (size_t)head * a.key_dim * a.value_dim;
    float S[DS_KPT], P[DS_KPT], Ar[DS_KPT];
#pragma unroll
    for (int i = 0; i < DS_KPT; ++i) {
        const int kr = i * R + r;
        const bool in = i < kpt && valid && kr < a.key_dim;
        if (a.mode == 0) S[i] = in ? st[(size_t)kr * a.value_dim + j] : 0.f;
        else if (TRACK) S[i] = 0.f;
        else S[i] = in ? ds_ws(a, seq, chunk, head, 2)[(size_t)kr * a.value_dim + j] : 0.f;
        P[i] = 1.f;
        Ar[i] = in && KIND == 2 ? a.A[channel * a.key_dim + kr] : 0.f;
    }
    const float skip = a.skip && valid ? a.skip[channel] : 0.f;
    for (int b0 = row0; b0 < row1; b0 += DS_TB) {
        const int nb = min(DS_TB, row1 - b0);
        __syncthreads();
        for (int idx = tid; idx < nb * kd; idx += blockDim.x) {
            const int t = idx / kd, i = idx % kd;
            const float* src = a.qk + (size_t)(b0 + t) * a.qk_stride + (size_t)kh * a.key_dim + i;
            const bool in = i < a.key_dim;
            ks[idx] = in ? src[a.k_off] : 0.f;
            qs[idx] = in ? src[a.q_off] : 0.f;
            if (KIND == 1) as[idx] = in ? src[a.a_off] : 0.f;
        }
        for (int idx = tid; idx < nb * CB; idx += blockDim.x) {
            const int t = idx / CB, c = cb * CB + idx % CB;
            const bool in = c < a.value_dim;
            const size_t ch = (size_t)head * a.value_dim + c;
            xs[idx] = in ? a.x[(size_t)(b0 + t) * a.x_stride + a.x_off + ch] : 0.f;
            if (KIND == 2)
                dts[idx] = in ? softplus_f(a.dt[(size_t)(b0 + t) * a.dt_stride + a.dt_off + ch] + (a.dt_bias ? a.dt_bias[ch] : 0.f)) : 0.f;
        }
        __syncthreads();
        for (int t = 0; t < nb; ++t) {
            const float xv = xs[t * CB + col];
            const float dtv = KIND == 2 ? dts[t * CB + col] : 1.f;
            const float wv = dtv * xv;
            const float* k = ks + t * kd + r;
            const float* q = qs + t * kd + r;
            const float* ar = as + t * kd + r;
            float o = 0.f;
#pragma unroll
            for (int i = 0; i < DS_KPT; ++i) {
                const float decay = KIND == 2 ? exp_of_decay(dtv * Ar[i]) : ar[i * R];
                S[i] = decay * S[i] + k[i * R] * wv;
                if (TRACK) P[i] *= decay;
                else o += S[i] * q[i * R];
            }
            if (TRACK) continue;
            for (int off = CW; off < WAVE; off <<= 1) o += __shfl_xor(o, off, WAVE);
            if (r == 0 && valid) a.out[(size_t)(b0 + t) * a.heads * a.value_dim + channel] = o + skip * xv;
        }
    }
    if (a.mode == 3) return;
    float* n_out = a.mode == 0 ? st : ds_ws(a, seq, chunk, head, 0);
    float* p_out = TRACK ? ds_ws(a, seq, chunk, head, 1) : nullptr;
#pragma unroll
    for (int i = 0; i < DS_KPT; ++i) {
        const int kr = i * R + r;
        if (i < kpt && valid && kr < a.key_dim) {
            n_out[(size_t)kr * a.value_dim + j] = S[i];
            if (p_out) p_out[(size_t)kr * a.value_dim + j] = P[i];
        }
    }
}

// From chunk to chunk, a thread an element of the state: S_start of every chunk, and the state after
// the last one to the slot.
__global__ void decay_carry_kernel(DecayScan a) {
    const int64_t per_seq = (int64_t)a.heads * a.key_dim * a.value_dim;
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int seq = blockIdx.y;
    if (e >= per_seq) return;
    const int head = (int)(e / ((int64_t)a.key_dim * a.value_dim));
    const size_t within = (size_t)(e % ((int64_t)a.key_dim * a.value_dim));
    const int n = a.cu_seqlens[seq + 1] - a.cu_seqlens[seq];
    const int n_chunks = (n + a.chunk_len - 1) / a.chunk_len;
    float* st = a.state + (size_t)a.seq_slot[seq] * a.slot_floats + (size_t)e;
    float s = *st;
    for (int c = 0; c < n_chunks; ++c) {
        ds_ws(a, seq, c, head, 2)[within] = s;
        s = ds_ws(a, seq, c, head, 1)[within] * s + ds_ws(a, seq, c, head, 0)[within];
    }
    *st = s;
}

// scratch of the chunked walk: one allocation of the process that grows to the largest request
// (prefill steps are not recorded, so it never changes under a recorded step)
static float* g_ds_ws = nullptr;
static size_t g_ds_ws_floats = 0;
static int ds_workspace(size_t floats, float** out) {
    if (floats > g_ds_ws_floats) {
        hipError_t e = g_ds_ws ? hipFree(g_ds_ws) : hipSuccess;
        g_ds_ws = nullptr, g_ds_ws_floats = 0;
        if (e == hipSuccess) e = hipMalloc((void**)&g_ds_ws, floats * sizeof(float));
        PICOLM_REQUIRE(e == hipSuccess, "decay_scan: %zu bytes of scratch for the chunked walk: %s", floats * sizeof(float), hipGetErrorString(e));
        g_ds_ws_floats = floats;
    }
    *out = g_ds_ws;
    return 0;
}
#define DS_CHUNK_TOKENS 64              // a chunk of the chunked walk, doubled while the scratch would pass the limit
#define DS_CHUNKED_FROM 256             // new tokens of a sequence from which a step is walked in chunks
#define DS_WS_LIMIT_FLOATS ((size_t)1 << 30)

extern "C" int picolm_call_decay_scan(void* user, const picolm_step_view* v) {
    const picolm_decay_scan_args* a = (const picolm_decay_scan_args*)user;
    VIEW_REQUIRE("decay_scan", v);
    PICOLM_REQUIRE(a && v->in && v->out && v->extra[0] && v->state, "decay_scan: buffers or state are missing");
    const int heads = a->n_heads, kh = a->n_key_heads, kd = a->key_dim, vd = a->value_dim;
    PICOLM_REQUIRE((a->kind == 1 || a->kind == 2) && heads > 0 && kh > 0 && heads % kh == 0 && kd > 0 && kd <= DS_MAX_KEY_DIM && vd > 0,
                   "decay_scan: kind %d, %d heads over %d, keys of %d (up to %d), values of %d", a->kind, heads, kh, kd, DS_MAX_KEY_DIM, vd);
    const int64_t channels = (int64_t)heads * vd;
    PICOLM_REQUIRE(a->q_off >= 0 && a->q_off + kh * kd <= a->qk_stride && a->k_off >= 0 && a->k_off + kh * kd <= a->qk_stride &&
                       (a->kind != 1 || (a->a_off >= 0 && a->a_off + kh * kd <= a->qk_stride)) && v->extra_row_bytes[0] >= a->qk_stride * 4,
                   "decay_scan: the rows of %d floats do not hold q, k and the decays at the offsets named", a->qk_stride);
    PICOLM_REQUIRE(a->x_off >= 0 && a->x_off + channels <= a->x_stride && v->in_row_bytes >= (int64_t)a->x_stride * 4 &&
                       v->out_row_bytes >= channels * 4,
                   "decay_scan: input or output rows too short for %lld channels", (long long)channels);
    PICOLM_REQUIRE(a->kind != 2 || (a->A && v->extra[1] && a->dt_off >= 0 && a->dt_off + channels <= a->dt_stride &&
                                    v->extra_row_bytes[1] >= (int64_t)a->dt_stride * 4),
                   "decay_scan: decays of the exponential kind need A and a step size per channel");
    const int64_t need = (a->state_off + channels * kd) * 4;
    PICOLM_REQUIRE(a->state_off >= 0 && need <= v->state_bytes_per_slot, "decay_scan: the state of a slot has %lld bytes, the matrices need %lld",
                   (long long)v->state_bytes_per_slot, (long long)need);
    if (v->n_tokens <= 0) return 0;
    DecayScan s;
    s.qk = (const float*)v->extra[0];
    s.x = (const float*)v->in;
    s.dt = (const float*)v->extra[1];
    s.out = (float*)v->out;
    s.state = (float*)v->state + a->state_off;
    s.dt_bias = a->dt_bias, s.A = a->A, s.skip = a->skip;
    s.cu_seqlens = v->cu_seqlens, s.seq_slot = v->seq_slot;
    s.slot_floats = v->state_bytes_per_slot / 4;
    s.qk_stride = a->qk_stride, s.q_off = a->q_off, s.k_off = a->k_off, s.a_off = a->a_off;
    s.x_stride = a->x_stride, s.x_off = a->x_off, s.dt_stride = a->dt_stride, s.dt_off = a->dt_off;
    s.kind = a->kind, s.heads = heads, s.key_heads = kh, s.key_dim = kd, s.value_dim = vd;
    int R = 1;
    while (R * DS_KPT < kd) R *= 2;
    s.R = R;
    s.kpt = DS_KPT;
    s.mode = 0, s.chunk_len = 0, s.chunks_per_seq = 1, s.ws = nullptr;
    const int CW = WAVE / R;
    auto launch = [&](int units) -> int {
        // few units: one wave a workgroup, so that more workgroups share the walk; many: up to four
        int n_waves = std::min(4, ceil_div(vd, CW));
        if ((int64_t)units * heads * ceil_div(vd, n_waves * CW) < 1024) n_waves = 1;
        s.n_waves = n_waves;
        s.n_cb = ceil_div(vd, n_waves * CW);
        const int64_t blocks = (int64_t)units * heads * s.n_cb;
        PICOLM_REQUIRE(blocks < (1ll << 31), "decay_scan: %lld workgroups exceed the grid", (long long)blocks);
        const size_t lds = sizeof(float) * DS_TB * ((size_t)3 * s.kpt * R + 2 * n_waves * CW);
        const dim3 grid((unsigned)blocks), block(n_waves * WAVE);
#define DS_LAUNCH(RR)                                                                                              \
    do {                                                                                                          \
        if (s.kind == 1 && s.mode == 1) decay_scan_kernel<RR, 1, true><<<grid, block, lds, v->stream>>>(s);       \
        else if (s.kind == 1) decay_scan_kernel<RR, 1, false><<<grid, block, lds, v->stream>>>(s);                \
        else if (s.mode == 1) decay_scan_kernel<RR, 2, true><<<grid, block, lds, v->stream>>>(s);                 \
        else decay_scan_kernel<RR, 2, false><<<grid, block, lds, v->stream>>>(s);                                 \
    } while (0)
        if (R == 1) DS_LAUNCH(1);
        else if (R == 2) DS_LAUNCH(2);
        else if (R == 4) DS_LAUNCH(4);
        else if (R == 8) DS_LAUNCH(8);
        else DS_LAUNCH(16);
#undef DS_LAUNCH
        PICOLM_LAUNCH_CHECK("decay_scan");
        return 0;
    };
    int most_new = 0;
    if (!v->is_decode && !v->recording && v->n_new)
        for (int i = 0; i < v->n_seq; ++i) most_new = std::max(most_new, v->n_new[i]);
    if (most_new < DS_CHUNKED_FROM) return launch(v->n_seq);
    s.chunk_len = DS_CHUNK_TOKENS;
    auto ws_floats = [&]() { return (size_t)v->n_seq * ceil_div(most_new, s.chunk_len) * heads * 3 * kd * vd; };
    while (ws_floats() > DS_WS_LIMIT_FLOATS && s.chunk_len < most_new) s.chunk_len *= 2;
    s.chunks_per_seq = ceil_div(most_new, s.chunk_len);
    if (s.chunks_per_seq < 2) return launch(v->n_seq);
    if (ds_workspace(ws_floats(), &s.ws)) return -1;
    PICOLM_REQUIRE((int64_t)v->n_seq * s.chunks_per_seq < (1 << 24) && v->n_seq <= 65535, "decay_scan: %d sequences of %d chunks", v->n_seq,
                   s.chunks_per_seq);
    s.mode = 1;
    if (launch(v->n_seq * s.chunks_per_seq)) return -1;
    const int64_t per_seq = channels * kd;
    decay_carry_kernel<<<dim3((unsigned)ceil_div64(per_seq, 256), v->n_seq), 256, 0, v->stream>>>(s);
    PICOLM_LAUNCH_CHECK("decay_scan (carry)");
    s.mode = 3;
    return launch(v->n_seq * s.chunks_per_seq);
}

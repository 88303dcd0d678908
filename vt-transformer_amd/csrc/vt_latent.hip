// Attention over a low-rank cache ("latent attention"): a token leaves one vector c of R elements (RMS-normed) and one
// rotated key part of Dr elements in the cache, shared by all heads; a head's unrotated key is Wk_h c and its value
// Wv_h c.  Neither is ever formed here.  With q = [qn (Dn) | qr (Dr)] per head,
//     score = qn . (Wk_h c) + qr . kr = (Wk_h^T qn) . c + qr . kr
//     out_h = Wv_h (sum_j p_j c_j)
// so the attention itself runs over one key/value head whose keys are [c | kr] (R + Dr) and whose values are c (R),
// with queries [Wk_h^T qn | qr], through the kernels of vt_attn_masked*.hip; this file holds what stands around it:
//
//   vt_latent_prepare: per token, from the input projection's row: c = rmsnorm(first R of the low-rank part) * w into
//                      the key page's first R elements and, transposed, into the value page; the last Dr elements,
//                      rotated (the first `rot` of them, element i with element i + rot/2), into the key page behind
//                      c; every head's qr, rotated alike, into the query row's elements R .. R + Dr.
//                      K [page][1][slot][R + Dr], V [page][1][R][slot].
//   vt_head_linear:    y[t, h, :] = W_h x[t, h, :] or W_h^T x[t, h, :], one small matrix per head, optionally times
//                      sigmoid(gate[t, h, :]) element by element.  Float32 sums in an order that depends on the
//                      matrix's shape only.
//   vt_head_linear_mfma: the same for the 16-bit types on the matrix cores, a wave per (16 tokens, head, 16 outputs).
#include "vt_common.h"
#include <math.h>

VT_DEFINE_LAST_ERROR()

struct LatentPrepArgs {
    const void* x;          // [n][ldx]
    const float* norm_w;    // [R]
    const float* cos_t;     // [max_pos][rot/2]
    const float* sin_t;
    const int* positions;
    const int* tok_entry;
    const int* block_table;
    void* q_out;            // [n][H][R + Dr]
    void* k_pages;
    void* v_pages;
    long long ldx;
    int q_col, c_col;       // columns of the first head's query and of the low-rank part in a row of x
    int H, Dn, Dr, R, rot, max_pos, page_size, max_blocks, num_pages;
    float eps;
};

// the rotated part of a vector: element d of Dr, the first `rot` rotated in half-split pairs
template <typename TI>
__device__ __forceinline__ float rotated_at(const TI* src, int d, int rot, const float* c, const float* s, bool in_table) {
    float v = load_f32<TI>(src, d);
    if (d < rot && in_table) {
        const int half = rot >> 1;
        const bool low = d < half;
        const int p = low ? d : d - half;
        v = rotate_pair(c[p], s[p], v, load_f32<TI>(src, low ? d + half : d - half), low);
    }
    return v;
}

template <typename TI, typename TC>
__global__ __launch_bounds__(256) void latent_prepare_kernel(LatentPrepArgs a) {
    const int t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    const TI* x = (const TI*)a.x + (size_t)t * a.ldx;
    const int pos = a.positions[t];
    const float* c = a.cos_t + (size_t)pos * (a.rot >> 1);
    const float* s = a.sin_t + (size_t)pos * (a.rot >> 1);
    const bool in_table = pos < a.max_pos;
    const int blk = pos / a.page_size;
    const int pg = blk < a.max_blocks ? a.block_table[(size_t)a.tok_entry[t] * a.max_blocks + blk] : -1;
    const bool page_ok = pg >= 0 && pg < a.num_pages;
    const int slot = pos - blk * a.page_size;
    const int DK = a.R + a.Dr;
    for (int u = blockIdx.y * nw + wave; u < a.H + 2; u += nw * gridDim.y) {
        if (u < a.H) {
            const TI* src = x + a.q_col + (size_t)u * (a.Dn + a.Dr) + a.Dn;
            TC* dst = (TC*)a.q_out + ((size_t)t * a.H + u) * DK + a.R;
            for (int d = lane; d < a.Dr; d += 64) store_f32<TC>(dst, d, rotated_at<TI>(src, d, a.rot, c, s, in_table));
        } else if (!page_ok) {
            continue;
        } else if (u == a.H) {
            const TI* src = x + a.c_col;
            float ss = 0.f;
            for (int d = lane; d < a.R; d += 64) {
                const float v = load_f32<TI>(src, d);
                ss += v * v;
            }
            ss = wave_sum(ss);
            const float r = 1.0f / sqrtf(ss / (float)a.R + a.eps);
            TC* kd = (TC*)a.k_pages + ((size_t)pg * a.page_size + slot) * DK;
            TC* vd = (TC*)a.v_pages + (size_t)pg * a.R * a.page_size + slot;
            for (int d = lane; d < a.R; d += 64) {
                const float v = load_f32<TI>(src, d) * r * a.norm_w[d];
                store_f32<TC>(kd, d, v);
                store_f32<TC>(vd, (size_t)d * a.page_size, v);
            }
        } else {
            const TI* src = x + a.c_col + a.R;
            TC* kd = (TC*)a.k_pages + ((size_t)pg * a.page_size + slot) * DK + a.R;
            for (int d = lane; d < a.Dr; d += 64) store_f32<TC>(kd, d, rotated_at<TI>(src, d, a.rot, c, s, in_table));
        }
    }
}

extern "C" int vt_latent_prepare(const void* x, int x_dtype, long long ldx, int q_col, int c_col, const float* norm_w,
                                 float eps, const float* cos_t, const float* sin_t, int rot, int max_pos,
                                 const int* positions, const int* tok_entry, const int* block_table, int max_blocks,
                                 void* q_out, void* k_pages, void* v_pages, int cache_dtype, int page_size, int num_pages,
                                 int n, int H, int Dn, int Dr, int R, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && H > 0 && Dn > 0 && Dr >= 0 && R > 0, "vt_latent_prepare: bad sizes H=%d Dn=%d Dr=%d R=%d", H, Dn, Dr, R);
    VT_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= Dr, "vt_latent_prepare: %d rotated elements of %d", rot, Dr);
    VT_REQUIRE(rot == 0 || (cos_t && sin_t && max_pos > 0), "vt_latent_prepare: no table of angles");
    VT_REQUIRE(q_col >= 0 && c_col >= 0 && ldx >= (long long)q_col + (long long)H * (Dn + Dr) && ldx >= (long long)c_col + R + Dr,
               "vt_latent_prepare: rows of %lld elements are too short", ldx);
    VT_REQUIRE(page_size > 0 && max_blocks > 0 && num_pages > 0 && block_table && k_pages && v_pages && norm_w,
               "vt_latent_prepare: bad cache sizes");
    if (n == 0) return 0;
    LatentPrepArgs a;
    a.x = x; a.norm_w = norm_w; a.cos_t = cos_t; a.sin_t = sin_t; a.positions = positions; a.tok_entry = tok_entry;
    a.block_table = block_table; a.q_out = q_out; a.k_pages = k_pages; a.v_pages = v_pages; a.ldx = ldx; a.q_col = q_col;
    a.c_col = c_col; a.H = H; a.Dn = Dn; a.Dr = Dr; a.R = R; a.rot = rot; a.max_pos = max_pos; a.page_size = page_size;
    a.max_blocks = max_blocks; a.num_pages = num_pages; a.eps = eps;
    const dim3 grid(n, n >= 1024 ? 1 : (H + 2 + 3) / 4);
    if (x_dtype == VT_F32 && cache_dtype == VT_F32) latent_prepare_kernel<float, float><<<grid, 256, 0, stream>>>(a);
    else if (x_dtype == VT_F32 && cache_dtype == VT_BF16) latent_prepare_kernel<float, bf16_t><<<grid, 256, 0, stream>>>(a);
    else if (x_dtype == VT_BF16 && cache_dtype == VT_BF16) latent_prepare_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>(a);
    else return vt_fail("vt_latent_prepare: dtypes %d -> %d are not handled", x_dtype, cache_dtype);
    VT_CHECK_LAUNCH("vt_latent_prepare");
    return 0;
}

// ---------------------------------------------------------------------------
struct HeadLinArgs {
    const void* x;          // x[t * ldx + h * x_head + i]
    const void* w;          // [H][out][in], or with `transposed` [H][in][out]
    const void* gate;       // gate[t * ldg + h * out + o], or null
    void* y;                // y[t * ldy + h * y_head + o]
    long long ldx, ldy, ldg;
    int x_head, y_head, n, H, in, out, transposed, gate_f32;
};

__device__ __forceinline__ float gated(float v, const HeadLinArgs& a, int t, int h, int o) {
    if (a.gate) {
        const size_t gi = (size_t)t * a.ldg + (size_t)h * a.out + o;
        const float z = a.gate_f32 ? ((const float*)a.gate)[gi] : bf16_to_f32(((const bf16_t*)a.gate)[gi]);
        v *= 1.0f / (1.0f + expf(-z));
    }
    return v;
}

// One block per (token, head): the head's input in LDS; W_h^T x: a thread per output walks the inputs in order (the
// matrix's rows are read side by side); W_h x: a wave per output, its lanes over the inputs, then the wave's sum.
template <typename TX, typename TC>
__global__ __launch_bounds__(256) void head_linear_kernel(HeadLinArgs a) {
    extern __shared__ float xs[];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const TX* x = (const TX*)a.x + (size_t)t * a.ldx + (size_t)h * a.x_head;
    for (int i = tid; i < a.in; i += 256) xs[i] = load_f32<TX>(x, i);
    __syncthreads();
    const TC* w = (const TC*)a.w + (size_t)h * a.in * a.out;
    TC* y = (TC*)a.y + (size_t)t * a.ldy + (size_t)h * a.y_head;
    if (a.transposed) {
        for (int o = tid; o < a.out; o += 256) {
            float acc = 0.f;
            for (int i = 0; i < a.in; ++i) acc = fmaf(xs[i], load_f32<TC>(w, (size_t)i * a.out + o), acc);
            store_f32<TC>(y, o, gated(acc, a, t, h, o));
        }
    } else {
        const int wave = tid >> 6, lane = tid & 63;
        for (int o = wave; o < a.out; o += 4) {
            const TC* wr = w + (size_t)o * a.in;
            float acc = 0.f;
            for (int i = lane; i < a.in; i += 64) acc = fmaf(xs[i], load_f32<TC>(wr, i), acc);
            acc = wave_sum(acc);
            if (lane == 0) store_f32<TC>(y, o, gated(acc, a, t, h, o));
        }
    }
}

// The 16-bit product on the matrix cores: a wave takes 16 tokens, one head and 16 outputs; Y^T = W_h X^T
// [16 outputs x 16 tokens] by v_mfma_f32_16x16x16 over the inputs.  A = W_h: a lane holds 4 consecutive inputs of its
// output's row (W_h x) or gathers them from 4 rows (W_h^T x); B = X: 4 consecutive inputs of the lane's token.
// Inputs beyond `in` and rows beyond n are zeros.  y is 16-bit, x 16-bit or float32 (rounded on its way in); `in` is a
// multiple of 4.
typedef __attribute__((ext_vector_type(4))) float hl_f32x4;
__device__ __forceinline__ vt_lowp4_t load_x4(const bf16_t* p) { return *(const vt_lowp4_t*)p; }
__device__ __forceinline__ vt_lowp4_t load_x4(const float* p) {
    const float4 v = *(const float4*)p;
    struct { unsigned a, b; } u = {vt_pack2(v.x, v.y), vt_pack2(v.z, v.w)};
    return __builtin_bit_cast(vt_lowp4_t, u);
}
template <typename TX>
__global__ __launch_bounds__(256) void head_linear_mfma_kernel(HeadLinArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, grp = lane >> 4;
    const int otiles = (a.out + 15) / 16;
    const int item = blockIdx.x * 4 + wave;             // (token tile, head, output tile); output tiles fastest
    const int ttiles = (a.n + 15) / 16;
    if (item >= ttiles * a.H * otiles) return;
    const int ot = item % otiles, h = (item / otiles) % a.H, tt = item / (otiles * a.H);
    const int t = tt * 16 + r, o = ot * 16 + r;
    const bool t_ok = t < a.n, o_ok = o < a.out;
    const TX* x = (const TX*)a.x + (size_t)(t_ok ? t : 0) * a.ldx + (size_t)h * a.x_head;
    const bf16_t* w = (const bf16_t*)a.w + (size_t)h * a.in * a.out;
    hl_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    const vt_lowp4_t zero = {0, 0, 0, 0};
    for (int k0 = 0; k0 < a.in; k0 += 16) {
        const int k = k0 + grp * 4;
        const bool k_ok = k < a.in;                     // (in is a multiple of 4: a lane's four inputs are all in or all out)
        vt_lowp4_t xb = zero, wa = zero;
        if (k_ok && t_ok) xb = load_x4(x + k);
        if (k_ok && o_ok) {
            if (a.transposed) {
                struct { bf16_t e[4]; } g;
#pragma unroll
                for (int e = 0; e < 4; ++e) g.e[e] = w[(size_t)(k + e) * a.out + o];
                wa = __builtin_bit_cast(vt_lowp4_t, g);
            } else {
                wa = *(const vt_lowp4_t*)(w + (size_t)o * a.in + k);
            }
        }
        acc = VT_MFMA_16X16X16(wa, xb, acc);
    }
    // the lane holds outputs ot * 16 + grp * 4 + e of token tt * 16 + r
    if (!t_ok) return;
    bf16_t* y = (bf16_t*)a.y + (size_t)t * a.ldy + (size_t)h * a.y_head;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int oo = ot * 16 + grp * 4 + e;
        if (oo < a.out) y[oo] = f32_to_bf16(gated(acc[e], a, t, h, oo));
    }
}

// Many tokens: a wave takes 32 tokens and one head, keeps their inputs in registers (KS steps of 16: in <= 16 KS) and
// goes through the head's output tiles, so that the tokens are read once and a row of W_h once per 32 tokens.
// W_h as [out][in] only.
template <typename TX, int KS>
__global__ __launch_bounds__(256) void head_linear_mfma_rows_kernel(HeadLinArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, grp = lane >> 4;
    const int item = blockIdx.x * 4 + wave;             // (pair of token tiles, head); heads fastest
    const int tpairs = (a.n + 31) / 32;
    if (item >= tpairs * a.H) return;
    const int h = item % a.H, t0 = (item / a.H) * 32;
    const vt_lowp4_t zero = {0, 0, 0, 0};
    vt_lowp4_t xb[2][KS];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int t = t0 + 16 * u + r;
        const TX* x = (const TX*)a.x + (size_t)(t < a.n ? t : 0) * a.ldx + (size_t)h * a.x_head;
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            const int k = kk * 16 + grp * 4;
            xb[u][kk] = (t < a.n && k < a.in) ? load_x4(x + k) : zero;
        }
    }
    const bf16_t* w = (const bf16_t*)a.w + (size_t)h * a.in * a.out;
    for (int ot = 0; ot * 16 < a.out; ++ot) {
        const int o = ot * 16 + r;
        vt_lowp4_t wa[KS];
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            const int k = kk * 16 + grp * 4;
            wa[kk] = (o < a.out && k < a.in) ? *(const vt_lowp4_t*)(w + (size_t)o * a.in + k) : zero;
        }
        hl_f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            acc0 = VT_MFMA_16X16X16(wa[kk], xb[0][kk], acc0);
            acc1 = VT_MFMA_16X16X16(wa[kk], xb[1][kk], acc1);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int t = t0 + 16 * u + r;
            if (t >= a.n) continue;
            bf16_t* y = (bf16_t*)a.y + (size_t)t * a.ldy + (size_t)h * a.y_head;
            const int oo = ot * 16 + grp * 4;
            const hl_f32x4 acc = u ? acc1 : acc0;
            if (oo + 3 < a.out && ((a.ldy | a.y_head) & 3) == 0 && (((uintptr_t)a.y) & 7) == 0) {
                struct { unsigned lo, hi; } pk = {vt_pack2(gated(acc[0], a, t, h, oo), gated(acc[1], a, t, h, oo + 1)),
                                                  vt_pack2(gated(acc[2], a, t, h, oo + 2), gated(acc[3], a, t, h, oo + 3))};
                *(uint2*)(y + oo) = __builtin_bit_cast(uint2, pk);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (oo + e < a.out) y[oo + e] = f32_to_bf16(gated(acc[e], a, t, h, oo + e));
            }
        }
    }
}

template <typename TX>
static bool launch_head_rows(const HeadLinArgs& a, hipStream_t stream) {
    // (worth it from a few hundred waves on; below that the kernel with a wave per output tile fills the GPU better)
    const long long items = (long long)((a.n + 31) / 32) * a.H;
    if (a.transposed || a.in > 256 || items < 512) return false;
    const unsigned blocks = (unsigned)((items + 3) / 4);
    if (a.in <= 64) head_linear_mfma_rows_kernel<TX, 4><<<blocks, 256, 0, stream>>>(a);
    else if (a.in <= 128) head_linear_mfma_rows_kernel<TX, 8><<<blocks, 256, 0, stream>>>(a);
    else if (a.in <= 192) head_linear_mfma_rows_kernel<TX, 12><<<blocks, 256, 0, stream>>>(a);
    else head_linear_mfma_rows_kernel<TX, 16><<<blocks, 256, 0, stream>>>(a);
    return true;
}

extern "C" int vt_head_linear(const void* x, int x_dtype, long long ldx, int x_head, const void* w, const void* gate,
                              int gate_dtype, long long ldg, void* y, int y_dtype, long long ldy, int y_head, int n,
                              int H, int in, int out, int transposed, int matrix_cores, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && H > 0 && in > 0 && out > 0, "vt_head_linear: bad sizes n=%d H=%d in=%d out=%d", n, H, in, out);
    VT_REQUIRE(in <= 8192, "vt_head_linear: %d inputs per head (up to 8192)", in);
    VT_REQUIRE(H <= 65535, "vt_head_linear: too many heads (%d)", H);
    VT_REQUIRE(x_head >= 0 && y_head >= 0 && ldx >= (long long)(H - 1) * x_head + in && ldy >= (long long)(H - 1) * y_head + out,
               "vt_head_linear: rows are too short for %d heads", H);
    VT_REQUIRE(!gate || gate_dtype == VT_F32 || gate_dtype == VT_BF16, "vt_head_linear: gate dtype %d", gate_dtype);
    VT_REQUIRE(!gate || ldg >= (long long)H * out, "vt_head_linear: gate rows are too short");
    if (n == 0) return 0;
    HeadLinArgs a;
    a.x = x; a.w = w; a.gate = gate; a.y = y; a.ldx = ldx; a.ldy = ldy; a.ldg = ldg; a.x_head = x_head; a.y_head = y_head;
    a.n = n; a.H = H; a.in = in; a.out = out; a.transposed = transposed; a.gate_f32 = gate_dtype == VT_F32;
    if (matrix_cores) {
        VT_REQUIRE(y_dtype == VT_BF16, "vt_head_linear: the matrix cores give 16-bit results");
        VT_REQUIRE(in % 4 == 0 && ldx % 4 == 0 && x_head % 4 == 0 && ((uintptr_t)x & (x_dtype == VT_F32 ? 15 : 7)) == 0 &&
                   ((uintptr_t)w & 7) == 0, "vt_head_linear: the matrix cores take inputs in aligned groups of four");
        if (x_dtype == VT_F32 ? launch_head_rows<float>(a, stream) : launch_head_rows<bf16_t>(a, stream)) {
            VT_CHECK_LAUNCH("vt_head_linear(rows)");
            return 0;
        }
        const long long items = (long long)((n + 15) / 16) * H * ((out + 15) / 16);
        if (x_dtype == VT_F32) head_linear_mfma_kernel<float><<<(unsigned)((items + 3) / 4), 256, 0, stream>>>(a);
        else head_linear_mfma_kernel<bf16_t><<<(unsigned)((items + 3) / 4), 256, 0, stream>>>(a);
        VT_CHECK_LAUNCH("vt_head_linear");
        return 0;
    }
    const dim3 grid(n, H);
    const size_t shmem = (size_t)in * sizeof(float);
    if (x_dtype == VT_F32 && y_dtype == VT_F32) head_linear_kernel<float, float><<<grid, 256, shmem, stream>>>(a);
    else if (x_dtype == VT_F32 && y_dtype == VT_BF16) head_linear_kernel<float, bf16_t><<<grid, 256, shmem, stream>>>(a);
    else if (x_dtype == VT_BF16 && y_dtype == VT_BF16) head_linear_kernel<bf16_t, bf16_t><<<grid, 256, shmem, stream>>>(a);
    else return vt_fail("vt_head_linear: dtypes %d -> %d are not handled", x_dtype, y_dtype);
    VT_CHECK_LAUNCH("vt_head_linear");
    return 0;
}

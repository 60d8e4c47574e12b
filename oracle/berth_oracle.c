/*
 * berth_oracle.c — CPU restatement of the EXL3 trellis-linear and MoE hot path.
 * TEST INFRASTRUCTURE ONLY; see berth_oracle.h for the parity status of each
 * function and the reference file:line each one follows.
 */
#include "berth_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ fp16 */

float bo_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* double -> binary16, one rounding (nearest even), handles subnormals/inf/nan */
uint16_t bo_f64_to_f16(double d)
{
    uint64_t u;
    memcpy(&u, &d, 8);
    uint16_t sign = (uint16_t)((u >> 48) & 0x8000u);
    int exp = (int)((u >> 52) & 0x7ff);
    uint64_t man = u & 0xfffffffffffffull;
    if (exp == 0x7ff) return (uint16_t)(sign | 0x7c00u | (man ? 0x200u : 0));
    if (exp == 0 && man == 0) return sign;
    /* value = 1.man * 2^(exp-1023) (doubles that are subnormal are far below
     * the fp16 range and round to zero below) */
    int e = exp - 1023;
    if (exp == 0) return sign;
    if (e > 15) return (uint16_t)(sign | 0x7c00u);
    uint64_t full = man | (1ull << 52);         /* 53-bit significand */
    int shift;                                  /* bits to drop */
    int hexp;
    if (e >= -14) { shift = 42; hexp = e + 15; }
    else { shift = 42 + (-14 - e); hexp = 0; }
    if (shift > 63) return sign;
    uint64_t kept = full >> shift;
    uint64_t rem = full & ((1ull << shift) - 1);
    uint64_t half = 1ull << (shift - 1);
    if (rem > half || (rem == half && (kept & 1))) kept++;
    uint32_t out;
    if (hexp == 0) {
        out = (uint32_t)kept;                   /* may carry into exp = 1 */
    } else {
        out = ((uint32_t)hexp << 10) + (uint32_t)(kept - 0x400u);
    }
    if (out >= 0x7c00u) out = 0x7c00u;
    return (uint16_t)(sign | out);
}

uint16_t bo_f32_to_f16(float f)
{
    return bo_f64_to_f16((double)f);            /* float -> double is exact */
}

/* ---------------------------------------------------------------- format */

/* [A] upstream lays the 256 weights of a tile out in the order the 32 lanes of
 * an m16n8k16 MMA hold two B fragments: lane L owns 8 consecutive stream
 * positions; k = 2*(L%4) + {0,1,8,9}, n = L/4 (+8 for the second fragment). */
void bo_tile_perm(int perm[256])
{
    for (int lane = 0; lane < 32; ++lane) {
        int r0 = (lane % 4) * 2;
        int c0 = lane / 4;
        const int dr[4] = {0, 1, 8, 9};
        for (int e = 0; e < 8; ++e) {
            int r = r0 + dr[e & 3];
            int c = c0 + ((e >> 2) ? 8 : 0);
            perm[lane * 8 + e] = r * 16 + c;
        }
    }
}

/* Tile bitstream: the 16*bits u16 words in index order, most significant bit of
 * each word first.  Each stream position t appends `bits` new bits; its state is
 * the 16 bits that END with them, i.e. stream bits [(t+1)*bits-16, (t+1)*bits),
 * wrapping around the tile (tail-biting, docs/exl3.md:13).  [A] for the phase. */
uint32_t bo_trellis_state(const uint16_t* w, int bits, int t)
{
    int total = 256 * bits;
    int start = ((t + 1) * bits - 16) % total;
    if (start < 0) start += total;
    uint32_t s = 0;
    for (int i = 0; i < 16; ++i) {
        int p = start + i;
        if (p >= total) p -= total;
        uint32_t bit = (w[p >> 4] >> (15 - (p & 15))) & 1u;
        s = (s << 1) | bit;
    }
    return s;
}

uint16_t bo_decode_state(uint32_t state, int cb)
{
    uint32_t x = state & 0xffffu;
    if (cb == 2) {
        /* MUL1: multiplier pinned by ptx/sm86_probes.cu:248, byte sum :143 */
        x *= 0x83DCD12Du;
        uint32_t t = (x & 0xff) + ((x >> 8) & 0xff) + ((x >> 16) & 0xff) + (x >> 24);
        uint16_t hbits = (uint16_t)(0x6400u | t);       /* fp16 value 1024 + t */
        double h = (double)bo_f16_to_f32(hbits);
        double kinv = (double)bo_f16_to_f32(0x1EEE);    /* [A] */
        double kbias = (double)bo_f16_to_f32(0xC931);   /* [A] */
        return bo_f64_to_f16(h * kinv + kbias);         /* one rounding = fp16 fma */
    }
    if (cb == 0) x = x * 89226354u + 64248484u;         /* [A] 3INST */
    else x = x * 0xCBAC1FEDu;                           /* [A] MCG   */
    x = (x & 0x8FFF8FFFu) ^ 0x3B603B60u;                /* ptx/sm86_probes.cu:157 */
    double lo = (double)bo_f16_to_f32((uint16_t)(x & 0xffff));
    double hi = (double)bo_f16_to_f32((uint16_t)(x >> 16));
    return bo_f64_to_f16(lo + hi);                      /* one fp16 add */
}

int bo_dequant(const uint16_t* trellis, int size_k, int size_n, int bits, int cb,
               uint16_t* w_out)
{
    if (size_k < 16 || size_n < 16 || size_k % 16 || size_n % 16) return -1;
    if (bits < 1 || bits > 8 || cb < 0 || cb > 2) return -1;
    int perm[256];
    bo_tile_perm(perm);
    int tk = size_k / 16, tn = size_n / 16;
    size_t tile_words = (size_t)16 * bits;
#pragma omp parallel for collapse(2) schedule(static)
    for (int kt = 0; kt < tk; ++kt) {
        for (int nt = 0; nt < tn; ++nt) {
            const uint16_t* w = trellis + ((size_t)kt * tn + nt) * tile_words;
            for (int t = 0; t < 256; ++t) {
                uint16_t v = bo_decode_state(bo_trellis_state(w, bits, t), cb);
                int r = perm[t] >> 4, c = perm[t] & 15;
                w_out[(size_t)(kt * 16 + r) * size_n + nt * 16 + c] = v;
            }
        }
    }
    return 0;
}

/* crates/berth-exl3/src/signs.rs:25-46 */
long bo_unpack_signs(const uint8_t* p, size_t nbytes, uint16_t* out)
{
    if (nbytes % 2) return -1;
    size_t words = nbytes / 2;
    for (size_t i = 0; i < words; ++i) {
        uint16_t word = (uint16_t)(p[2 * i] | (p[2 * i + 1] << 8));
        for (int b = 0; b < 16; ++b)
            out[i * 16 + b] = ((word >> b) & 1) ? 0xBC00 : 0x3C00;
    }
    return (long)(words * 16);
}

/* -------------------------------------------------------------- Hadamard */

#define BO_RSQRT128 0.088388347648f /* crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:44 */

void bo_had128(float v[128])
{
    for (int h = 1; h < 128; h <<= 1)
        for (int i = 0; i < 128; ++i)
            if (!(i & h)) {
                float a = v[i], b = v[i + h];
                v[i] = a + b;
                v[i + h] = a - b;
            }
}

int bo_had_rows_f16(const uint16_t* in, uint16_t* out, const uint16_t* scale,
                    int pre, int rows, int cols)
{
    if (rows < 1 || cols < 128 || cols % 128) return -1;
#pragma omp parallel for schedule(static)
    for (long blk = 0; blk < (long)rows * (cols / 128); ++blk) {
        int r = (int)(blk / (cols / 128)), cb = (int)(blk % (cols / 128));
        const uint16_t* src = in + (size_t)r * cols + cb * 128;
        uint16_t* dst = out + (size_t)r * cols + cb * 128;
        const uint16_t* sc = scale ? scale + cb * 128 : NULL;
        float v[128];
        for (int i = 0; i < 128; ++i) {
            v[i] = bo_f16_to_f32(src[i]);
            if (pre && sc) v[i] *= bo_f16_to_f32(sc[i]);
        }
        bo_had128(v);
        for (int i = 0; i < 128; ++i) {
            float o = v[i] * BO_RSQRT128;
            if (!pre && sc) o *= bo_f16_to_f32(sc[i]);
            dst[i] = bo_f32_to_f16(o);
        }
    }
    return 0;
}

int bo_had_rows_f32(const float* in, float* out, const uint16_t* scale,
                    int pre, int rows, int cols)
{
    if (rows < 1 || cols < 128 || cols % 128) return -1;
#pragma omp parallel for schedule(static)
    for (long blk = 0; blk < (long)rows * (cols / 128); ++blk) {
        int r = (int)(blk / (cols / 128)), cb = (int)(blk % (cols / 128));
        const float* src = in + (size_t)r * cols + cb * 128;
        float* dst = out + (size_t)r * cols + cb * 128;
        const uint16_t* sc = scale ? scale + cb * 128 : NULL;
        float v[128];
        for (int i = 0; i < 128; ++i) {
            v[i] = src[i];
            if (pre && sc) v[i] *= bo_f16_to_f32(sc[i]);
        }
        bo_had128(v);
        for (int i = 0; i < 128; ++i) {
            float o = v[i] * BO_RSQRT128;
            if (!pre && sc) o *= bo_f16_to_f32(sc[i]);
            dst[i] = o;
        }
    }
    return 0;
}

/* Effective weight: both 128-block Hadamards and both sign scales folded into the decoded
 * weight, per 128 x 128 block W_eff = diag(suh) Hh W Hh diag(svh)
 * (crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:96-123; the kernel body is in the
 * absent fork, so the rounding contract is this build's: fp32 butterflies down the columns,
 * then along the rows, ((v / sqrt(128)) / sqrt(128)) * suh[k] * svh[n], one rounding to
 * fp16).  Pinned by the operator identity a @ W_eff == bo_linear(a). */
int bo_reconstruct_had(const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh,
                       int size_k, int size_n, int bits, int cb, uint16_t* w_out)
{
    if (size_k < 128 || size_n < 128 || size_k % 128 || size_n % 128) return -1;
    uint16_t* w = (uint16_t*)malloc((size_t)size_k * size_n * 2);
    if (!w) return -2;
    int rc = bo_dequant(trellis, size_k, size_n, bits, cb, w);
    if (rc) { free(w); return rc; }
#pragma omp parallel for collapse(2) schedule(static)
    for (int kb = 0; kb < size_k / 128; ++kb) {
        for (int nb = 0; nb < size_n / 128; ++nb) {
            float* blk = (float*)malloc(128 * 128 * sizeof(float));
            float v[128];
            for (int k = 0; k < 128; ++k)
                for (int n = 0; n < 128; ++n)
                    blk[k * 128 + n] = bo_f16_to_f32(w[(size_t)(kb * 128 + k) * size_n + nb * 128 + n]);
            for (int n = 0; n < 128; ++n) {
                for (int k = 0; k < 128; ++k) v[k] = blk[k * 128 + n];
                bo_had128(v);
                for (int k = 0; k < 128; ++k) blk[k * 128 + n] = v[k];
            }
            for (int k = 0; k < 128; ++k) {
                bo_had128(blk + k * 128);
                float su = bo_f16_to_f32(suh[kb * 128 + k]);
                for (int n = 0; n < 128; ++n) {
                    float o = blk[k * 128 + n] * BO_RSQRT128;
                    o = o * BO_RSQRT128;
                    o = o * su;
                    o = o * bo_f16_to_f32(svh[nb * 128 + n]);
                    w_out[(size_t)(kb * 128 + k) * size_n + nb * 128 + n] = bo_f32_to_f16(o);
                }
            }
            free(blk);
        }
    }
    free(w);
    return 0;
}

/* ---------------------------------------------------------------- linear */

static void finish_rows(const float* z, void* c_out, const uint16_t* svh,
                        int m, int n, int out_fp32)
{
    /* y = H(z)/sqrt(128) * svh, then cast (linear.cu(prefill):220) */
#pragma omp parallel for schedule(static)
    for (long blk = 0; blk < (long)m * (n / 128); ++blk) {
        int r = (int)(blk / (n / 128)), cb = (int)(blk % (n / 128));
        float v[128];
        memcpy(v, z + (size_t)r * n + cb * 128, sizeof v);
        bo_had128(v);
        for (int i = 0; i < 128; ++i) {
            float o = v[i] * BO_RSQRT128;
            o *= bo_f16_to_f32(svh[cb * 128 + i]);
            size_t at = (size_t)r * n + cb * 128 + i;
            if (out_fp32) ((float*)c_out)[at] = o;
            else ((uint16_t*)c_out)[at] = bo_f32_to_f16(o);
        }
    }
}

int bo_linear_w(const uint16_t* a, const uint16_t* w, void* c_out,
                const uint16_t* suh, uint16_t* a_had_out, const uint16_t* svh,
                int m, int K, int N, int out_fp32, int acc64)
{
    if (m < 1 || K < 128 || N < 128 || K % 128 || N % 128) return -1;
    uint16_t* ah = (uint16_t*)malloc((size_t)m * K * 2);
    float* ahf = (float*)malloc((size_t)m * K * 4);
    float* wf = (float*)malloc((size_t)K * N * 4);
    float* z = (float*)malloc((size_t)m * N * 4);
    if (!ah || !ahf || !wf || !z) { free(ah); free(ahf); free(wf); free(z); return -1; }
    bo_had_rows_f16(a, ah, suh, 1, m, K);
    if (a_had_out) memcpy(a_had_out, ah, (size_t)m * K * 2);
    for (size_t i = 0; i < (size_t)m * K; ++i) ahf[i] = bo_f16_to_f32(ah[i]);
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)K * N; ++i) wf[i] = bo_f16_to_f32(w[i]);
    /* z = a_had @ W, accumulated over k ascending */
#pragma omp parallel for schedule(static)
    for (long rn = 0; rn < (long)m * (N / 128); ++rn) {
        int r = (int)(rn / (N / 128)), nb = (int)(rn % (N / 128)) * 128;
        const float* xr = ahf + (size_t)r * K;
        if (acc64) {
            double acc[128];
            for (int j = 0; j < 128; ++j) acc[j] = 0.0;
            for (int k = 0; k < K; ++k) {
                double xv = xr[k];
                const float* wr = wf + (size_t)k * N + nb;
                for (int j = 0; j < 128; ++j) acc[j] += xv * (double)wr[j];
            }
            for (int j = 0; j < 128; ++j) z[(size_t)r * N + nb + j] = (float)acc[j];
        } else {
            float acc[128];
            for (int j = 0; j < 128; ++j) acc[j] = 0.0f;
            for (int k = 0; k < K; ++k) {
                float xv = xr[k];
                const float* wr = wf + (size_t)k * N + nb;
                for (int j = 0; j < 128; ++j) acc[j] = fmaf(xv, wr[j], acc[j]);
            }
            memcpy(z + (size_t)r * N + nb, acc, sizeof acc);
        }
    }
    finish_rows(z, c_out, svh, m, N, out_fp32);
    free(ah); free(ahf); free(wf); free(z);
    return 0;
}

int bo_linear(const uint16_t* a, const uint16_t* trellis, void* c_out,
              const uint16_t* suh, uint16_t* a_had_out, const uint16_t* svh,
              int m, int K, int N, int bits, int cb, int out_fp32, int acc64)
{
    if (m < 1 || K < 128 || N < 128 || K % 128 || N % 128) return -1;
    uint16_t* w = (uint16_t*)malloc((size_t)K * N * 2);
    if (!w) return -1;
    int rc = bo_dequant(trellis, K, N, bits, cb, w);
    if (rc == 0) rc = bo_linear_w(a, w, c_out, suh, a_had_out, svh, m, K, N, out_fp32, acc64);
    free(w);
    return rc;
}

/* 65536-entry state -> fp32 weight table for one codebook (built on demand) */
static float* g_lut[3];
static const float* state_lut(int cb)
{
    float* t;
#pragma omp critical(bo_lut)
    {
        t = g_lut[cb];
        if (!t) {
            t = (float*)malloc(65536 * sizeof(float));
            for (uint32_t s = 0; s < 65536; ++s)
                t[s] = bo_f16_to_f32(bo_decode_state(s, cb));
            g_lut[cb] = t;
        }
    }
    return t;
}

int bo_gemv_fused(const uint16_t* a, const uint16_t* trellis, void* c_out,
                  const uint16_t* suh, uint16_t* a_had_out, const uint16_t* svh,
                  int K, int N, int bits, int cb, int out_fp32)
{
    if (K < 128 || N < 128 || K % 128 || N % 128) return -1;
    if (bits < 1 || bits > 8 || cb < 0 || cb > 2) return -1;
    const float* lut = state_lut(cb);
    int perm[256];
    bo_tile_perm(perm);
    uint16_t* ah = (uint16_t*)malloc((size_t)K * 2);
    float* xh = (float*)malloc((size_t)K * 4);
    float* z = (float*)malloc((size_t)N * 4);
    bo_had_rows_f16(a, ah, suh, 1, 1, K);
    if (a_had_out) memcpy(a_had_out, ah, (size_t)K * 2);
    for (int i = 0; i < K; ++i) xh[i] = bo_f16_to_f32(ah[i]);
    int tk = K / 16, tn = N / 16;
    size_t tile_words = (size_t)16 * bits;
    int total = 256 * bits;
    /* one thread owns a column of tiles, walks k ascending: per output column
     * the accumulation order is k-tile ascending, stream order inside a tile */
#pragma omp parallel for schedule(static)
    for (int nt = 0; nt < tn; ++nt) {
        float acc[16];
        for (int j = 0; j < 16; ++j) acc[j] = 0.0f;
        for (int kt = 0; kt < tk; ++kt) {
            const uint16_t* w = trellis + ((size_t)kt * tn + nt) * tile_words;
            const float* xk = xh + kt * 16;
            /* rolling 16-bit state: start at stream position 0 */
            uint32_t s = bo_trellis_state(w, bits, 0);
            int pos = bits;                      /* next unread stream bit */
            for (int t = 0; t < 256; ++t) {
                float wv = lut[s];
                acc[perm[t] & 15] = fmaf(xk[perm[t] >> 4], wv, acc[perm[t] & 15]);
                /* shift in the next `bits` bits */
                uint32_t nb = 0;
                for (int i = 0; i < bits; ++i) {
                    int p = pos + i;
                    if (p >= total) p -= total;
                    nb = (nb << 1) | ((w[p >> 4] >> (15 - (p & 15))) & 1u);
                }
                pos += bits;
                s = ((s << bits) | nb) & 0xffffu;
            }
        }
        memcpy(z + nt * 16, acc, sizeof acc);
    }
    finish_rows(z, c_out, svh, 1, N, out_fp32);
    free(ah); free(xh); free(z);
    return 0;
}

int bo_hgemm(const uint16_t* a, const uint16_t* b, void* c, int m, int k, int n,
             int ldc, int c_fp32)
{
    if (m < 1 || k < 1 || n < 1 || ldc < n) return -1;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < m; ++r) {
        float* acc = (float*)calloc((size_t)n, sizeof(float));
        for (int kk = 0; kk < k; ++kk) {
            float xv = bo_f16_to_f32(a[(size_t)r * k + kk]);
            const uint16_t* br = b + (size_t)kk * n;
            for (int j = 0; j < n; ++j) acc[j] = fmaf(xv, bo_f16_to_f32(br[j]), acc[j]);
        }
        for (int j = 0; j < n; ++j) {
            if (c_fp32) ((float*)c)[(size_t)r * ldc + j] = acc[j];
            else ((uint16_t*)c)[(size_t)r * ldc + j] = bo_f32_to_f16(acc[j]);
        }
        free(acc);
    }
    return 0;
}

/* ----------------------------------------------------------- elementwise */

/* crates/berth-kernels/csrc/ops/act.cu:35-69; caller crates/berth-engine/src/mlp.rs:128-148.
 * The reference's fixture (testdata/kernels/ops/silu.*) is reproduced bit for
 * bit by half-precision arithmetic with every step rounded to fp16:
 *   e = f16(exp(-g)); s = f16(1 + e); r = f16(1 / s); t = f16(g * r); out = f16(t * u) */
int bo_silu_mul_f16(const uint16_t* gate, const uint16_t* up, uint16_t* out,
                    int64_t numel, float act_limit)
{
    if (numel < 2 || (numel & 1)) return -1;
    for (int64_t i = 0; i < numel; ++i) {
        double g = (double)bo_f16_to_f32(gate[i]);
        double u = (double)bo_f16_to_f32(up[i]);
        if (act_limit != 0.0f) {                 /* [A] clamp form of upstream */
            g = fmin(g, (double)act_limit);
            u = fmax(fmin(u, (double)act_limit), -(double)act_limit);
        }
        double e = (double)bo_f16_to_f32(bo_f64_to_f16(exp(-g)));
        double s = (double)bo_f16_to_f32(bo_f64_to_f16(1.0 + e));
        double r = (double)bo_f16_to_f32(bo_f64_to_f16(1.0 / s));
        double t = (double)bo_f16_to_f32(bo_f64_to_f16(g * r));
        out[i] = bo_f64_to_f16(t * u);
    }
    return 0;
}

int bo_add_f32(const float* a, const float* b, float* c, int n)
{
    if (n < 1) return -1;
    for (int i = 0; i < n; ++i) c[i] = a[i] + b[i];
    return 0;
}

/* ------------------------------------------------------------------- MoE */

#define BO_ROUTE_SEG 64 /* rows of the router weight per partial sum */

int bo_moe_route(const uint16_t* x, const uint16_t* wr, const float* bias,
                 int T, int H, int E, int k, int renorm,
                 int32_t* idx, float* w, float* logits_out)
{
    if (T < 1 || H < 1 || E < 1 || k < 1 || k > E) return -1;
#pragma omp parallel for schedule(static)
    for (int t = 0; t < T; ++t) {
        float* logit = (float*)malloc((size_t)E * sizeof(float));
        float* part = (float*)malloc((size_t)E * sizeof(float));
        char* taken = (char*)calloc((size_t)E, 1);
        for (int e = 0; e < E; ++e) logit[e] = 0.0f;
        /* partial sums over segments of 64 rows, each accumulated in row
         * order; segments are then added in order */
        for (int h0 = 0; h0 < H; h0 += BO_ROUTE_SEG) {
            int h1 = h0 + BO_ROUTE_SEG < H ? h0 + BO_ROUTE_SEG : H;
            for (int e = 0; e < E; ++e) part[e] = 0.0f;
            for (int h = h0; h < h1; ++h) {
                float xv = bo_f16_to_f32(x[(size_t)t * H + h]);
                const uint16_t* row = wr + (size_t)h * E;
                for (int e = 0; e < E; ++e)
                    part[e] = fmaf(xv, bo_f16_to_f32(row[e]), part[e]);
            }
            for (int e = 0; e < E; ++e) logit[e] += part[e];
        }
        if (bias) for (int e = 0; e < E; ++e) logit[e] += bias[e];
        if (logits_out) memcpy(logits_out + (size_t)t * E, logit, (size_t)E * sizeof(float));
        /* top-k on the logits (softmax is monotone): largest first, ties to
         * the lowest expert index */
        for (int j = 0; j < k; ++j) {
            int best = -1;
            for (int e = 0; e < E; ++e) {
                if (taken[e]) continue;
                if (best < 0 || logit[e] > logit[best]) best = e;
            }
            taken[best] = 1;
            idx[(size_t)t * k + j] = best;
        }
        float mx = logit[idx[(size_t)t * k]];
        float denom = 0.0f;
        if (renorm) {
            for (int j = 0; j < k; ++j) {
                float ev = expf(logit[idx[(size_t)t * k + j]] - mx);
                w[(size_t)t * k + j] = ev;
                denom += ev;
            }
        } else {
            for (int e = 0; e < E; ++e) denom += expf(logit[e] - mx);
            for (int j = 0; j < k; ++j)
                w[(size_t)t * k + j] = expf(logit[idx[(size_t)t * k + j]] - mx);
        }
        for (int j = 0; j < k; ++j) w[(size_t)t * k + j] /= denom;
        free(logit); free(part); free(taken);
    }
    return 0;
}

int bo_moe_permute(const int32_t* idx, int T, int k, int E,
                   int32_t* offsets, int32_t* perm)
{
    if (T < 1 || k < 1 || E < 1) return -1;
    for (int e = 0; e <= E; ++e) offsets[e] = 0;
    for (int p = 0; p < T * k; ++p) {
        if (idx[p] < 0 || idx[p] >= E) return -1;
        offsets[idx[p] + 1]++;
    }
    for (int e = 0; e < E; ++e) offsets[e + 1] += offsets[e];
    int32_t* cur = (int32_t*)malloc((size_t)E * sizeof(int32_t));
    memcpy(cur, offsets, (size_t)E * sizeof(int32_t));
    for (int p = 0; p < T * k; ++p) perm[cur[idx[p]]++] = p;
    free(cur);
    return 0;
}

int bo_expert_ffn(const uint16_t* x, int m, int H, int I, int bits, int cb,
                  const bo_lin_t* gate, const bo_lin_t* up, const bo_lin_t* down,
                  float* out)
{
    uint16_t* g = (uint16_t*)malloc((size_t)m * I * 2);
    uint16_t* u = (uint16_t*)malloc((size_t)m * I * 2);
    int rc = bo_linear(x, gate->trellis, g, gate->suh, NULL, gate->svh, m, H, I, bits, cb, 0, 0);
    if (!rc) rc = bo_linear(x, up->trellis, u, up->suh, NULL, up->svh, m, H, I, bits, cb, 0, 0);
    if (!rc) rc = bo_silu_mul_f16(g, u, u, (int64_t)m * I, 0.0f);
    if (!rc) rc = bo_linear(u, down->trellis, out, down->suh, NULL, down->svh, m, I, H, bits, cb, 1, 0);
    free(g); free(u);
    return rc;
}

/* scale[t] = 1 / (1 + exp(-z)), z = x[t] . wg: an fp32 fma chain in row order over every
 * 64-row segment, the segment sums added in segment order (the routing's arithmetic). */
int bo_moe_shared_gate(const uint16_t* x, const float* wg, int T, int H, float* scale)
{
    if (T < 1 || H < 1) return 1;
    for (int t = 0; t < T; ++t) {
        float z = 0.0f;
        for (int h0 = 0; h0 < H; h0 += 64) {
            float part = 0.0f;
            for (int h = h0; h < H && h < h0 + 64; ++h) part = fmaf(bo_f16_to_f32(x[(size_t)t * H + h]), wg[h], part);
            z += part;
        }
        scale[t] = 1.0f / (1.0f + expf(-z));
    }
    return 0;
}

int bo_moe_layer(const uint16_t* x, int T, int H, int E, int k, int I, int bits,
                 int cb, const uint16_t* wr, const float* bias, int renorm,
                 const bo_lin_t* experts, const bo_lin_t* shared, int shared_I,
                 float* out, int32_t* idx_out, float* w_out)
{
    return bo_moe_layer_gated(x, T, H, E, k, I, bits, cb, wr, bias, renorm, experts, shared, shared_I, NULL, out,
                              idx_out, w_out);
}

int bo_moe_layer_gated(const uint16_t* x, int T, int H, int E, int k, int I, int bits,
                       int cb, const uint16_t* wr, const float* bias, int renorm,
                       const bo_lin_t* experts, const bo_lin_t* shared, int shared_I,
                       const float* shared_gate, float* out, int32_t* idx_out, float* w_out)
{
    int32_t* idx = (int32_t*)malloc((size_t)T * k * sizeof(int32_t));
    float* w = (float*)malloc((size_t)T * k * sizeof(float));
    int32_t* offsets = (int32_t*)malloc((size_t)(E + 1) * sizeof(int32_t));
    int32_t* perm = (int32_t*)malloc((size_t)T * k * sizeof(int32_t));
    float* slot_out = (float*)malloc((size_t)T * k * H * sizeof(float));
    int rc = bo_moe_route(x, wr, bias, T, H, E, k, renorm, idx, w, NULL);
    if (!rc) rc = bo_moe_permute(idx, T, k, E, offsets, perm);
    for (int e = 0; e < E && !rc; ++e) {
        int m = offsets[e + 1] - offsets[e];
        if (!m) continue;
        uint16_t* xe = (uint16_t*)malloc((size_t)m * H * 2);
        float* oe = (float*)malloc((size_t)m * H * sizeof(float));
        for (int r = 0; r < m; ++r) {
            int t = perm[offsets[e] + r] / k;
            memcpy(xe + (size_t)r * H, x + (size_t)t * H, (size_t)H * 2);
        }
        rc = bo_expert_ffn(xe, m, H, I, bits, cb, &experts[3 * e], &experts[3 * e + 1],
                           &experts[3 * e + 2], oe);
        for (int r = 0; r < m; ++r)
            memcpy(slot_out + (size_t)perm[offsets[e] + r] * H, oe + (size_t)r * H,
                   (size_t)H * sizeof(float));
        free(xe); free(oe);
    }
    if (!rc) {
        if (shared) rc = bo_expert_ffn(x, T, H, shared_I, bits, cb, &shared[0], &shared[1],
                                       &shared[2], out);
        else memset(out, 0, (size_t)T * H * sizeof(float));
        if (!rc && shared && shared_gate) {
            float* scale = (float*)malloc((size_t)T * sizeof(float));
            rc = bo_moe_shared_gate(x, shared_gate, T, H, scale);
            for (int t = 0; t < T && !rc; ++t)
                for (int h = 0; h < H; ++h) out[(size_t)t * H + h] *= scale[t];
            free(scale);
        }
    }
    if (!rc) {
        for (int t = 0; t < T; ++t)
            for (int j = 0; j < k; ++j) {
                float wj = w[(size_t)t * k + j];
                const float* so = slot_out + ((size_t)t * k + j) * H;
                for (int h = 0; h < H; ++h)
                    out[(size_t)t * H + h] = fmaf(wj, so[h], out[(size_t)t * H + h]);
            }
        if (idx_out) memcpy(idx_out, idx, (size_t)T * k * sizeof(int32_t));
        if (w_out) memcpy(w_out, w, (size_t)T * k * sizeof(float));
    }
    free(idx); free(w); free(offsets); free(perm); free(slot_out);
    return rc;
}

int bo_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void bo_set_num_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ---- glue ops around the MLP (crates/berth-kernels/src/ops.rs:398-552) ------------
 * rms_norm: y[row] = fp16( (x * rmf) * (w + constant_bias) * constant_scale ), rmf =
 * 1/sqrt(mean(x^2) + epsilon) rounded to fp32, products in fp32.  With `residual` the
 * row is first residual += x (fp32, in place) and the norm runs on the sum.  weight
 * is bf16 (weight_bf16 = 1) or fp16 bits. */
static float bo_bf16_to_f32(uint16_t h)
{
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

int bo_rms_norm(const float* x, const uint16_t* weight, uint16_t* y, float* residual, int rows, int dim,
                float epsilon, float constant_bias, float constant_scale, int weight_bf16)
{
    if (!x || !weight || !y || rows < 1 || dim < 1 || dim % 4) return -1;
    for (int r = 0; r < rows; ++r) {
        const float* xr = x + (size_t)r * dim;
        float* rr = residual ? residual + (size_t)r * dim : NULL;
        double ss = 0.0;
        for (int i = 0; i < dim; ++i) {
            float v = xr[i];
            if (rr) { v = rr[i] + v; rr[i] = v; }
            ss += (double)v * (double)v;
        }
        const float rmf = (float)(1.0 / sqrt(ss / dim + (double)epsilon));
        for (int i = 0; i < dim; ++i) {
            const float v = rr ? rr[i] : xr[i];
            const float w = weight_bf16 ? bo_bf16_to_f32(weight[i]) : bo_f16_to_f32(weight[i]);
            float t = v * rmf;
            t = t * (w + constant_bias);
            t = t * constant_scale;
            y[(size_t)r * dim + i] = bo_f64_to_f16((double)t);
        }
    }
    return 0;
}


/* Integer-only C restatement of the LL128 codec, of the element addition and
 * of the ring reduce-scatter walked hop by hop through the wire format.
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/liboracle_c.so by oracle/Makefile
 * and loaded by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg
 * of bench.py.  The shipped library never links or loads it.
 *
 * It is written line by line (no index tables) so that it is an independent
 * derivation from oracle/ll128.py, which is table driven.
 *
 * Reference semantics restated:
 *   line format      protocol.py:42-48   (128 B = 120 B payload + 8 B flag)
 *   pair layout      protocol.py:57-100,132-137 (load/save/send_ll128)
 *   line numbers     2_sendrecv_indirect.py:61,76-77,93
 *   fp16 addition    primitive.py:232-247 (add.f16x2: RNE, subnormals kept)
 *   reduce order     7_reducescatter.py:54-73, protocol.py:150-155
 * The wave64 layout is the 64-lane redesign described in oracle/ll128.py.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>

enum { LAYOUT_PAIR = 0, LAYOUT_WAVE64 = 1 };
enum { DT_F16 = 0, DT_BF16 = 1, DT_F32 = 2 };

static size_t ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }

size_t ref_line_count(size_t n, int layout) {
    return layout == LAYOUT_PAIR ? ceil_div(n, 120) : ceil_div(n, 960) * 8;
}

/* copy raw[off, off+len) into dst, zero beyond n */
static void take(const uint8_t *raw, size_t n, size_t off, size_t len, uint8_t *dst) {
    size_t have = off < n ? (n - off < len ? n - off : len) : 0;
    if (have) memcpy(dst, raw + off, have);
    if (have < len) memset(dst + have, 0, len - have);
}

/* write src[0,len) to raw[off, off+len), dropping what lies beyond n */
static void give(uint8_t *raw, size_t n, size_t off, size_t len, const uint8_t *src) {
    size_t have = off < n ? (n - off < len ? n - off : len) : 0;
    if (have) memcpy(raw + off, src, have);
}

/* pair layout: 8-byte flag after 120 payload bytes.  wave64 layout: the low
 * 32 bits of the flag after the 60 payload bytes of each 64-byte sector. */
static void put_flag(uint8_t *line, uint64_t f, int layout) {
    if (layout == LAYOUT_PAIR) {
        for (int i = 0; i < 8; ++i) line[120 + i] = (uint8_t)(f >> (8 * i));
    } else {
        for (int i = 0; i < 4; ++i) line[60 + i] = line[124 + i] = (uint8_t)(f >> (8 * i));
    }
}
static int flag_ok(const uint8_t *line, uint64_t want, int layout) {
    if (layout == LAYOUT_PAIR) {
        uint64_t f = 0;
        for (int i = 0; i < 8; ++i) f |= (uint64_t)line[120 + i] << (8 * i);
        return f == want;
    }
    uint32_t a = 0, b = 0;
    for (int i = 0; i < 4; ++i) {
        a |= (uint32_t)line[60 + i] << (8 * i);
        b |= (uint32_t)line[124 + i] << (8 * i);
    }
    return a == (uint32_t)want && b == (uint32_t)want;
}

void ref_pack(const uint8_t *raw, size_t n, uint64_t flag_base, uint64_t flag_stride,
              int layout, uint8_t *msg) {
    size_t lines = ref_line_count(n, layout);
    for (size_t L = 0; L < lines; ++L) {
        uint8_t *line = msg + L * 128;
        if (layout == LAYOUT_PAIR) {
            size_t base = (L / 2) * 240;
            if (L % 2 == 0) {
                take(raw, n, base, 120, line);
            } else {
                take(raw, n, base + 128, 112, line);
                take(raw, n, base + 120, 8, line + 112);
            }
        } else {
            size_t base = (L / 8) * 960;
            for (size_t h = 0; h < 2; ++h) {           /* the line's two sectors */
                size_t i = (L % 8) * 2 + h;
                take(raw, n, base + 48 * i, 48, line + 64 * h);
                take(raw, n, base + 768 + 12 * i, 12, line + 64 * h + 48);
            }
        }
        put_flag(line, flag_base + L * flag_stride, layout);
    }
}

size_t ref_unpack(const uint8_t *msg, size_t n, uint64_t flag_base, uint64_t flag_stride,
                  int layout, uint8_t *raw) {
    size_t lines = ref_line_count(n, layout), bad = 0;
    for (size_t L = 0; L < lines; ++L) {
        const uint8_t *line = msg + L * 128;
        if (!flag_ok(line, flag_base + L * flag_stride, layout)) ++bad;
        if (layout == LAYOUT_PAIR) {
            size_t base = (L / 2) * 240;
            if (L % 2 == 0) {
                give(raw, n, base, 120, line);
            } else {
                give(raw, n, base + 128, 112, line);
                give(raw, n, base + 120, 8, line + 112);
            }
        } else {
            size_t base = (L / 8) * 960;
            for (size_t h = 0; h < 2; ++h) {
                size_t i = (L % 8) * 2 + h;
                give(raw, n, base + 48 * i, 48, line + 64 * h);
                give(raw, n, base + 768 + 12 * i, 12, line + 64 * h + 48);
            }
        }
    }
    return bad;
}

/* Soft-float addition, round to nearest even, for a binary format with E
 * exponent bits and M fraction bits (binary16: 5/10, bfloat16: 8/7).
 * NaN results are the canonical quiet NaN (sign 0). */
static uint32_t sf_add(uint32_t a, uint32_t b, int E, int M) {
    const uint32_t emax = (1u << E) - 1, fmask = (1u << M) - 1;
    uint32_t sa = a >> (E + M), ea = (a >> M) & emax, fa = a & fmask;
    uint32_t sb = b >> (E + M), eb = (b >> M) & emax, fb = b & fmask;
    const uint32_t qnan = (emax << M) | (1u << (M - 1));
    if ((ea == emax && fa) || (eb == emax && fb)) return qnan;
    if (ea == emax) return (eb == emax && sa != sb) ? qnan : a;
    if (eb == emax) return b;
    int xa = ea ? (int)ea : 1, xb = eb ? (int)eb : 1;
    uint64_t va = (uint64_t)(ea ? fa | (1u << M) : fa) << 3;
    uint64_t vb = (uint64_t)(eb ? fb | (1u << M) : fb) << 3;
    if (xa < xb || (xa == xb && va < vb)) {
        int tx = xa; xa = xb; xb = tx;
        uint64_t tv = va; va = vb; vb = tv;
        uint32_t ts = sa; sa = sb; sb = ts;
    }
    int d = xa - xb;
    if (d > 0) {
        if (d >= 40) vb = vb != 0;
        else vb = (vb >> d) | ((vb & ((1ull << d) - 1)) != 0);
    }
    uint64_t v = sa == sb ? va + vb : va - vb;
    int x = xa;
    if (v == 0) return sa == sb ? sa << (E + M) : 0;
    if (v >> (M + 4)) { v = (v >> 1) | (v & 1); ++x; }
    while (x > 1 && !(v >> (M + 3))) { v <<= 1; --x; }
    uint32_t g = (uint32_t)(v & 7), lsb = (uint32_t)(v >> 3) & 1;
    v >>= 3;
    if (g > 4 || (g == 4 && lsb)) ++v;
    if (v >> (M + 1)) { v >>= 1; ++x; }
    uint32_t e = (v >> M) ? (uint32_t)x : 0;
    if (e >= emax) return (sa << (E + M)) | (emax << M);
    return (sa << (E + M)) | (e << M) | ((uint32_t)v & fmask);
}

uint16_t ref_add_f16(uint16_t a, uint16_t b) { return (uint16_t)sf_add(a, b, 5, 10); }
uint16_t ref_add_bf16(uint16_t a, uint16_t b) { return (uint16_t)sf_add(a, b, 8, 7); }

/* out = rn(a + b) elementwise; nelem elements of the given dtype */
void ref_add(const void *a, const void *b, void *out, size_t nelem, int dtype) {
    if (dtype == DT_F32) {
        const float *x = a, *y = b; float *o = out;
        for (size_t i = 0; i < nelem; ++i) o[i] = x[i] + y[i];
    } else {
        const uint16_t *x = a, *y = b; uint16_t *o = out;
        int E = dtype == DT_F16 ? 5 : 8, M = dtype == DT_F16 ? 10 : 7;
        for (size_t i = 0; i < nelem; ++i) o[i] = (uint16_t)sf_add(x[i], y[i], E, M);
    }
}

/* ---- CPU baseline: ring reduce-scatter walked through the wire format -------
 * xs[r] points at rank r's (world x row_bytes) buffer.  For every chunk c the
 * walk of 7_reducescatter.py:54-73 is done block by block (960 raw bytes): the
 * root's block is packed into a 1 KiB wave64 message with the step tag, the
 * next rank checks the 16 sector tags, unpacks, adds its own block
 * (protocol.py:142-156) and packs again; after world hops the root unpacks
 * into its row c.  In place, like the reference.  Element addition uses the
 * host FPU (binary32 add, one rounding back) - see oracle/ring.py for why that
 * equals one correctly rounded addition - and OpenMP over (chunk, block).
 * Returns the number of messages whose tags were wrong (always 0). */
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static float half_to_float(uint16_t h) {
    uint32_t s = (uint32_t)(h >> 15) << 31, e = (h >> 10) & 31, f = h & 1023, u;
    if (e == 0) {
        if (!f) { u = s; }
        else { int sh = 0; while (!(f & 1024)) { f <<= 1; ++sh; }
               u = s | ((uint32_t)(113 - sh) << 23) | ((f & 1023) << 13); }
    } else if (e == 31) { u = s | 0x7F800000u | (f << 13); }
    else { u = s | ((e + 112) << 23) | (f << 13); }
    float r; memcpy(&r, &u, 4); return r;
}
static uint16_t float_to_half(float x) {       /* round to nearest even */
    uint32_t u; memcpy(&u, &x, 4);
    uint32_t s = (u >> 16) & 0x8000u, a = u & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) return (uint16_t)(s | 0x7C00u | (a > 0x7F800000u ? 0x200u : 0));
    if (a >= 0x477FF000u) return (uint16_t)(s | 0x7C00u);           /* rounds to inf */
    if (a < 0x38800000u) {                                           /* subnormal half */
        if (a < 0x33000000u) return (uint16_t)s;                     /* below half of 2^-24 */
        uint32_t e = a >> 23, m = (a & 0x7FFFFFu) | 0x800000u, sh = 126 - e;   /* 14..24 */
        uint32_t q = m >> sh, rem = m & ((1u << sh) - 1), half = 1u << (sh - 1);
        if (rem > half || (rem == half && (q & 1))) ++q;
        return (uint16_t)(s | q);
    }
    uint32_t q = (a - 0x38000000u) >> 13, rem = a & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1))) ++q;
    return (uint16_t)(s | q);
}
static uint16_t float_to_bf16(float x) {
    uint32_t u; memcpy(&u, &x, 4);
    if (x != x) return 0x7FC0;
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
static void add_block(const uint8_t *own, const uint8_t *recv, uint8_t *out, size_t nbytes,
                      int dtype) {
    if (dtype == DT_F32) {
        for (size_t i = 0; i + 4 <= nbytes; i += 4) {
            float a, b; memcpy(&a, own + i, 4); memcpy(&b, recv + i, 4);
            a = a + b; memcpy(out + i, &a, 4);
        }
    } else if (dtype == DT_F16) {
        for (size_t i = 0; i + 2 <= nbytes; i += 2) {
            uint16_t a, b; memcpy(&a, own + i, 2); memcpy(&b, recv + i, 2);
            uint16_t r = float_to_half(half_to_float(a) + half_to_float(b));
            memcpy(out + i, &r, 2);
        }
    } else {
        for (size_t i = 0; i + 2 <= nbytes; i += 2) {
            uint16_t a, b; memcpy(&a, own + i, 2); memcpy(&b, recv + i, 2);
            uint32_t ua = (uint32_t)a << 16, ub = (uint32_t)b << 16; float fa, fb;
            memcpy(&fa, &ua, 4); memcpy(&fb, &ub, 4);
            uint16_t r = float_to_bf16(fa + fb);
            memcpy(out + i, &r, 2);
        }
    }
}

size_t ref_reducescatter_wire(uint8_t *const *xs, int world, size_t row_bytes, int dtype,
                              const int *ring, uint32_t epoch, int threads) {
    size_t nblocks = ceil_div(row_bytes, 960), bad = 0;
#ifdef _OPENMP
    if (threads > 0) omp_set_num_threads(threads);
#else
    (void)threads;
#endif
    long total = (long)world * (long)nblocks;
#pragma omp parallel for schedule(static) reduction(+ : bad)
    for (long t = 0; t < total; ++t) {
        int c = (int)(t / (long)nblocks);
        size_t g = (size_t)(t % (long)nblocks);
        size_t off = g * 960, len = row_bytes - off < 960 ? row_bytes - off : 960;
        int start = 0;
        for (int i = 0; i < world; ++i) if (ring[i] == c) start = i;
        uint8_t acc[960], recv[960], msg[1024];
        uint64_t tag = ((uint64_t)epoch << 20) | (uint64_t)(g + 1);
        memcpy(acc, xs[c] + (size_t)c * row_bytes + off, len);
        for (int k = 1; k <= world; ++k) {
            ref_pack(acc, len, tag, 0, LAYOUT_WAVE64, msg);
            bad += ref_unpack(msg, len, tag, 0, LAYOUT_WAVE64, recv);
            int r = ring[(start + k) % world];
            if (k < world)
                add_block(xs[r] + (size_t)c * row_bytes + off, recv, acc, len, dtype);
            else
                memcpy(xs[c] + (size_t)c * row_bytes + off, recv, len);
        }
    }
    return bad;
}

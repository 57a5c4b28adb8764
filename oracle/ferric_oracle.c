/*
 * CPU oracle for the quantized-GGUF matmul path (Q8_0 / Q4_K / Q6_K, and the further block formats of the same reader).
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is a plain-C restatement of the reference's own CPU
 * algorithms, used only as the checker in tests, the smoke check and the CPU-baseline leg of the
 * benchmark. The shipped library never links or calls it.
 *
 * Every function cites the reference source it follows (paths are under the reference checkout).
 * The reference is Rust: every f32 operation there is individually rounded and Rust never
 * contracts a*b+c into an FMA, so this file MUST be compiled with -ffp-contract=off (the Makefile
 * does) to reproduce the same bits.
 *
 * Pinning status (what independent evidence each restatement is checked against in tests/):
 *   f16 -> f32            exhaustive 65536 patterns vs numpy.float16 + reference landmarks
 *                         (crates/ferric-tensor/src/cpu_simd.rs:203-213)
 *   deq_q8_0              closed form; reference ground-truth generator cpu_simd.rs:136-156
 *   deq_q4_k              reference known-answer block crates/ferric-gguf/examples/roundtrip.rs:54-87,
 *                         pack/unpack identity over all 8x64x64 (sc,m) values, second (random-access)
 *                         formulation from crates/ferric-tensor/src/dtype.rs:2078-2086, single-field
 *                         perturbations, numpy twin
 *   deq_q6_k              second formulation dtype.rs:1236-1246, single-field perturbations, numpy twin
 *                         (the reference holds no known-answer vector for Q6_K)
 *   row_q8_0/matvec       reference tests cpu_simd.rs:162-200 restated (ground truth built beside the
 *                         bytes, partition invariance, span composition)
 *   deq_q4_0/q4_1/q5_0/q5_1/q5_k, deq_iq4_nl/iq4_xs
 *                         second formulation from the reference's GPU kernel bodies, numpy twin, closed-form relations
 *                         between formats and single-field perturbations (tests/test_oracle_formats.py); the IQ4
 *                         codebook constant is restated from crates/ferric-gguf/src/lib.rs:751
 *   deq_mxfp4             ggml-captured known answers held by the reference's tests (lib.rs:1099-1222: 10 scale bytes
 *                         x 16 codes, 8 blocks of a released checkpoint), all 256 x 16 (scale, code) pairs vs ldexp
 *   parity with ggml itself is pinned for MXFP4 only (through those captured answers); for the other formats it is
 *   not pinned anywhere in the reference tree.
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define GGML_F32 0u
#define GGML_F16 1u
#define GGML_BF16 30u
#define GGML_Q4_0 2u
#define GGML_Q4_1 3u
#define GGML_Q5_0 6u
#define GGML_Q5_1 7u
#define GGML_Q8_0 8u
#define GGML_Q4_K 12u
#define GGML_Q5_K 13u
#define GGML_Q6_K 14u
#define GGML_IQ4_NL 20u
#define GGML_IQ4_XS 23u
#define GGML_MXFP4 39u

/* ---------------------------------------------------------------- f16 <-> f32 */

/* IEEE binary16 -> f32, exact, including subnormals / inf / nan.
 * Follows the hand decoder crates/ferric-tensor/src/cpu_simd.rs:29-48 (same result as
 * half::f16::to_f32 used by crates/ferric-gguf/src/lib.rs:605). */
float fo_f16_to_f32(uint16_t bits) {
    uint32_t sign = (bits >> 15) & 1u, exp = (bits >> 10) & 0x1Fu, man = bits & 0x3FFu, out;
    if (exp == 0) {
        if (man == 0) {
            out = sign << 31;
        } else {
            uint32_t m = man, k = 0;
            while ((m & 0x400u) == 0) { m <<= 1; k++; }
            out = (sign << 31) | ((113u - k) << 23) | ((m & 0x3FFu) << 13);
        }
    } else if (exp == 0x1F) {
        out = (sign << 31) | 0x7F800000u | (man << 13);
    } else {
        out = (sign << 31) | ((exp + 127u - 15u) << 23) | (man << 13);
    }
    float f; memcpy(&f, &out, 4); return f;
}

/* All 65536 decodings as raw f32 bit patterns (a float return value passed through a foreign-call
 * layer may have a signalling NaN quieted; a bit table cannot).
 * NaN inputs: this decoder keeps the payload (cpu_simd.rs:45), half::f16::to_f32 additionally sets
 * the quiet bit; the two reference decoders agree on every non-NaN pattern, and tests compare NaN
 * patterns by NaN-ness only. */
void fo_f16_table_bits(uint32_t* out) {
    for (uint32_t b = 0; b < 65536; b++) { float f = fo_f16_to_f32((uint16_t)b); memcpy(&out[b], &f, 4); }
}

/* f32 -> binary16, round-to-nearest-even (what half::f16::from_f32 does; only the test-data
 * generators need it: crates/ferric-tensor/examples/q4_k.rs:17-18, q6_k.rs:14,
 * crates/ferric-gguf/src/lib.rs:990). */
uint16_t fo_f32_to_f16(float f) {
    uint32_t x; memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u, man = x & 0x7FFFFFu;
    int32_t exp = (int32_t)((x >> 23) & 0xFF);
    if (exp == 0xFF) return (uint16_t)(sign | 0x7C00u | (man ? (0x200u | (man >> 13)) : 0));
    int32_t e = exp - 127 + 15;
    if (e >= 0x1F) return (uint16_t)(sign | 0x7C00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half_man = man >> shift, rem = man & ((1u << shift) - 1), halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t h = ((uint32_t)e << 10) | (man >> 13), rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) h++;
    return (uint16_t)(sign | h);
}

static inline uint16_t rd_u16(const uint8_t* b) { return (uint16_t)(b[0] | (b[1] << 8)); }

/* ---------------------------------------------------------------- sizes */

/* crates/ferric-gguf/src/lib.rs:471-494 (type_size), the three in-scope rows; 0 = unsupported.
 * Integer division truncates exactly as the reference's `n / 32 * 34`. */
size_t fo_type_size(uint32_t ty, size_t n) {
    switch (ty) {
        case GGML_F32: return n * 4;
        case GGML_F16: return n * 2;
        case GGML_BF16: return n * 2;
        case GGML_Q8_0: return n / 32 * 34;
        case GGML_Q4_K: return n / 256 * 144;
        case GGML_Q6_K: return n / 256 * 210;
        case GGML_Q4_0: return n / 32 * 18;
        case GGML_Q4_1: return n / 32 * 20;
        case GGML_Q5_0: return n / 32 * 22;
        case GGML_Q5_1: return n / 32 * 24;
        case GGML_Q5_K: return n / 256 * 176;
        case GGML_IQ4_NL: return n / 32 * 18;
        case GGML_IQ4_XS: return n / 256 * 136;
        case GGML_MXFP4: return n / 32 * 17;
        default: return 0;
    }
}

/* crates/ferric-tensor/src/dtype.rs:873-889 (QMatrix::block_bytes): (values, bytes) per block. */
int fo_block_bytes(uint32_t ty, size_t* vals, size_t* bytes) {
    switch (ty) {
        case GGML_Q8_0: *vals = 32; *bytes = 34; return 1;
        case GGML_Q4_K: *vals = 256; *bytes = 144; return 1;
        case GGML_Q6_K: *vals = 256; *bytes = 210; return 1;
        case GGML_Q4_0: *vals = 32; *bytes = 18; return 1;
        case GGML_Q4_1: *vals = 32; *bytes = 20; return 1;
        case GGML_Q5_0: *vals = 32; *bytes = 22; return 1;
        case GGML_Q5_1: *vals = 32; *bytes = 24; return 1;
        case GGML_Q5_K: *vals = 256; *bytes = 176; return 1;
        case GGML_IQ4_NL: *vals = 32; *bytes = 18; return 1;
        case GGML_IQ4_XS: *vals = 256; *bytes = 136; return 1;
        case GGML_MXFP4: *vals = 32; *bytes = 17; return 1;
        default: return 0;
    }
}

/* ---------------------------------------------------------------- dequantizers (sequential form) */

/* crates/ferric-gguf/src/lib.rs:608-615. Returns the number of f32 written: whole blocks only,
 * limited both by n/32 and by the bytes present (chunks_exact(34).take(n/32)), so a ragged tail
 * yields a SHORTER output, as in the reference. Operand order q*d. */
size_t fo_deq_q8_0(const uint8_t* raw, size_t raw_len, size_t n, float* out) {
    size_t nb = n / 32, have = raw_len / 34, w = 0;
    if (have < nb) nb = have;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t* blk = raw + b * 34;
        float d = fo_f16_to_f32(rd_u16(blk));
        for (int j = 0; j < 32; j++) out[w++] = (float)(int8_t)blk[2 + j] * d;
    }
    return w;
}

/* crates/ferric-gguf/src/lib.rs:795-804 (closure get_sc_min). */
static inline void get_sc_min(const uint8_t* s, int j, uint8_t* sc, uint8_t* m) {
    if (j < 4) {
        *sc = s[j] & 63; *m = s[j + 4] & 63;
    } else {
        *sc = (uint8_t)((s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4));
        *m = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
}
void fo_q4k_get_sc_min(const uint8_t* scales12, int j, uint8_t* sc, uint8_t* m) { get_sc_min(scales12, j, sc, m); }

/* crates/ferric-gguf/src/lib.rs:793-825. out is pre-zeroed to n (`vec![0.0; n]`), whole blocks
 * present in both n and raw are filled; y = (d*sc)*q - (dmin*m), each op rounded. Returns n. */
size_t fo_deq_q4_k(const uint8_t* raw, size_t raw_len, size_t n, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    size_t nb = n / 256, have = raw_len / 144;
    if (have < nb) nb = have;
    for (size_t bi = 0; bi < nb; bi++) {
        const uint8_t* blk = raw + bi * 144;
        float d = fo_f16_to_f32(rd_u16(blk)), dmin = fo_f16_to_f32(rd_u16(blk + 2));
        const uint8_t* scales = blk + 4; const uint8_t* qs = blk + 16;
        size_t y = bi * 256, q = 0; int is = 0;
        for (int it = 0; it < 4; it++) {
            uint8_t sc1, m1, sc2, m2;
            get_sc_min(scales, is, &sc1, &m1);
            get_sc_min(scales, is + 1, &sc2, &m2);
            float d1 = d * (float)sc1, mm1 = dmin * (float)m1;
            float d2 = d * (float)sc2, mm2 = dmin * (float)m2;
            for (int l = 0; l < 32; l++) out[y + l] = d1 * (float)(qs[q + l] & 0x0F) - mm1;
            for (int l = 0; l < 32; l++) out[y + l + 32] = d2 * (float)(qs[q + l] >> 4) - mm2;
            y += 64; q += 32; is += 2;
        }
    }
    return n;
}

/* crates/ferric-gguf/src/lib.rs:721-746. y = d * sc * q evaluated left to right: (d*sc)*q. */
size_t fo_deq_q6_k(const uint8_t* raw, size_t raw_len, size_t n, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    size_t nb = n / 256, have = raw_len / 210;
    if (have < nb) nb = have;
    for (size_t bi = 0; bi < nb; bi++) {
        const uint8_t* blk = raw + bi * 210;
        float d = fo_f16_to_f32(rd_u16(blk + 208));
        const uint8_t* ql = blk; const uint8_t* qh = blk + 128; const int8_t* sc = (const int8_t*)(blk + 192);
        size_t y = bi * 256;
        for (int half = 0; half < 2; half++) {
            const uint8_t* qlh = ql + half * 64; const uint8_t* qhh = qh + half * 32; const int8_t* sch = sc + half * 8;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int q1 = (int)((qlh[l] & 0xF) | (((qhh[l] >> 0) & 3) << 4)) - 32;
                int q2 = (int)((qlh[l + 32] & 0xF) | (((qhh[l] >> 2) & 3) << 4)) - 32;
                int q3 = (int)((qlh[l] >> 4) | (((qhh[l] >> 4) & 3) << 4)) - 32;
                int q4 = (int)((qlh[l + 32] >> 4) | (((qhh[l] >> 6) & 3) << 4)) - 32;
                out[y + l] = d * (float)sch[is] * (float)q1;
                out[y + l + 32] = d * (float)sch[is + 2] * (float)q2;
                out[y + l + 64] = d * (float)sch[is + 4] * (float)q3;
                out[y + l + 96] = d * (float)sch[is + 6] * (float)q4;
            }
            y += 128;
        }
    }
    return n;
}

/* ---- the other block formats of the same reader (the "next" formats of the path) ----
 * Pinning: each sequential form is checked bit for bit against its element formula taken from the
 * reference's GPU kernels (second formulation, below), against a numpy twin written from the layout, and
 * against closed-form relations to the formats pinned above (Q5_K with qh = 0 is Q4_K on the same bytes;
 * Q5_1 with qh = 0 is Q4_1; Q5_0 = Q4_0 - 8d when qh = 0; Q4_1 with m = -8d is Q4_0 where -8d is exact).
 * The reference tree holds no known-answer vectors for these five. */

static inline uint32_t rd_u32(const uint8_t* b) { return (uint32_t)b[0] | ((uint32_t)b[1] << 8) | ((uint32_t)b[2] << 16) | ((uint32_t)b[3] << 24); }

/* crates/ferric-gguf/src/lib.rs:618-629: x = (nibble - 8) * d, low nibbles then high. */
size_t fo_deq_q4_0(const uint8_t* raw, size_t raw_len, size_t n, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    size_t nb = n / 32, have = raw_len / 18;
    if (have < nb) nb = have;
    for (size_t bi = 0; bi < nb; bi++) {
        const uint8_t* blk = raw + bi * 18;
        float d = fo_f16_to_f32(rd_u16(blk));
        for (int i = 0; i < 16; i++) {
            uint8_t byte = blk[2 + i];
            out[bi * 32 + i] = (float)((int)(byte & 0x0F) - 8) * d;
            out[bi * 32 + i + 16] = (float)((int)(byte >> 4) - 8) * d;
        }
    }
    return n;
}

/* crates/ferric-gguf/src/lib.rs:633-645: x = nibble * d + m. */
size_t fo_deq_q4_1(const uint8_t* raw, size_t raw_len, size_t n, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    size_t nb = n / 32, have = raw_len / 20;
    if (have < nb) nb = have;
    for (size_t bi = 0; bi < nb; bi++) {
        const uint8_t* blk = raw + bi * 20;
        float d = fo_f16_to_f32(rd_u16(blk)), m = fo_f16_to_f32(rd_u16(blk + 2));
        for (int i = 0; i < 16; i++) {
            uint8_t byte = blk[4 + i];
            out[bi * 32 + i] = (float)(byte & 0x0F) * d + m;
            out[bi * 32 + i + 16] = (float)(byte >> 4) * d + m;
        }
    }
    return n;
}

/* crates/ferric-gguf/src/lib.rs:650-665: x = ((nibble | bit << 4) - 16) * d, bit i of qh for value i, bit i+16 for i+16. */
size_t fo_deq_q5_0(const uint8_t* raw, size_t raw_len, size_t n, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    size_t nb = n / 32, have = raw_len / 22;
    if (have < nb) nb = have;
    for (size_t bi = 0; bi < nb; bi++) {
        const uint8_t* blk = raw + bi * 22;
        float d = fo_f16_to_f32(rd_u16(blk));
        uint32_t qh = rd_u32(blk + 2);
        for (int i = 0; i < 16; i++) {
            uint8_t byte = blk[6 + i];
            uint32_t xh0 = ((qh >> i) & 1u) << 4, xh1 = ((qh >> (i + 16)) & 1u) << 4;
            out[bi * 32 + i] = (float)((int)((uint32_t)(byte & 0x0F) | xh0) - 16) * d;
            out[bi * 32 + i + 16] = (float)((int)((uint32_t)(byte >> 4) | xh1) - 16) * d;
        }
    }
    return n;
}

/* crates/ferric-gguf/src/lib.rs:669-684: x = (nibble | bit << 4) * d + m. */
size_t fo_deq_q5_1(const uint8_t* raw, size_t raw_len, size_t n, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    size_t nb = n / 32, have = raw_len / 24;
    if (have < nb) nb = have;
    for (size_t bi = 0; bi < nb; bi++) {
        const uint8_t* blk = raw + bi * 24;
        float d = fo_f16_to_f32(rd_u16(blk)), m = fo_f16_to_f32(rd_u16(blk + 2));
        uint32_t qh = rd_u32(blk + 4);
        for (int i = 0; i < 16; i++) {
            uint8_t byte = blk[8 + i];
            uint32_t xh0 = ((qh >> i) & 1u) << 4, xh1 = ((qh >> (i + 16)) & 1u) << 4;
            out[bi * 32 + i] = (float)((uint32_t)(byte & 0x0F) | xh0) * d + m;
            out[bi * 32 + i + 16] = (float)((uint32_t)(byte >> 4) | xh1) * d + m;
        }
    }
    return n;
}

/* crates/ferric-gguf/src/lib.rs:692-716: Q4_K plus one high bit per value, y = (d*sc)*(nibble + 16*bit) - dmin*m. */
size_t fo_deq_q5_k(const uint8_t* raw, size_t raw_len, size_t n, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    size_t nb = n / 256, have = raw_len / 176;
    if (have < nb) nb = have;
    for (size_t bi = 0; bi < nb; bi++) {
        const uint8_t* blk = raw + bi * 176;
        float d = fo_f16_to_f32(rd_u16(blk)), dmin = fo_f16_to_f32(rd_u16(blk + 2));
        const uint8_t* scales = blk + 4; const uint8_t* qh = blk + 16; const uint8_t* qs = blk + 48;
        size_t y = bi * 256, q = 0; int is = 0;
        for (int jg = 0; jg < 4; jg++) {
            uint8_t sc1, m1, sc2, m2;
            get_sc_min(scales, is, &sc1, &m1);
            get_sc_min(scales, is + 1, &sc2, &m2);
            float d1 = d * (float)sc1, mm1 = dmin * (float)m1;
            float d2 = d * (float)sc2, mm2 = dmin * (float)m2;
            uint8_t b1 = (uint8_t)(1u << (2 * jg)), b2 = (uint8_t)(1u << (2 * jg + 1));
            for (int l = 0; l < 32; l++) out[y + l] = d1 * (float)((qs[q + l] & 0x0F) + ((qh[l] & b1) ? 16 : 0)) - mm1;
            for (int l = 0; l < 32; l++) out[y + l + 32] = d2 * (float)((qs[q + l] >> 4) + ((qh[l] & b2) ? 16 : 0)) - mm2;
            y += 64; q += 32; is += 2;
        }
    }
    return n;
}

/* crates/ferric-gguf/src/lib.rs:751: the 16 signed levels of the IQ4 non-linear codebook (llama.cpp kvalues_iq4nl). */
static const int FO_KVALUES_IQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

/* crates/ferric-gguf/src/lib.rs:755-767: 18-byte block [f16 d][qs[16]], value = d * kvalues[index]. */
size_t fo_deq_iq4_nl(const uint8_t* raw, size_t raw_len, size_t n, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    size_t nb = n / 32, have = raw_len / 18;
    if (have < nb) nb = have;
    for (size_t bi = 0; bi < nb; bi++) {
        const uint8_t* blk = raw + bi * 18;
        float d = fo_f16_to_f32(rd_u16(blk));
        for (int j = 0; j < 16; j++) {
            out[bi * 32 + j] = d * (float)FO_KVALUES_IQ4NL[blk[2 + j] & 0x0F];
            out[bi * 32 + j + 16] = d * (float)FO_KVALUES_IQ4NL[blk[2 + j] >> 4];
        }
    }
    return n;
}

/* crates/ferric-gguf/src/lib.rs:772-791: 136-byte super-block [f16 d][u16 scales_h][scales_l[4]][qs[128]]; sub-block ib
 * has the 6-bit scale ls = nibble ib of scales_l | bits 2ib, 2ib+1 of scales_h << 4; dl = d * (ls - 32). */
size_t fo_deq_iq4_xs(const uint8_t* raw, size_t raw_len, size_t n, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    size_t nb = n / 256, have = raw_len / 136;
    if (have < nb) nb = have;
    for (size_t bi = 0; bi < nb; bi++) {
        const uint8_t* blk = raw + bi * 136;
        float d = fo_f16_to_f32(rd_u16(blk));
        uint32_t scales_h = rd_u16(blk + 2);
        const uint8_t* scales_l = blk + 4; const uint8_t* qs = blk + 8;
        for (int ib = 0; ib < 8; ib++) {
            int ls = (int)(((uint32_t)(scales_l[ib / 2] >> (4 * (ib % 2))) & 0x0Fu) | (((scales_h >> (2 * ib)) & 3u) << 4));
            float dl = d * (float)(ls - 32);
            const uint8_t* q = qs + ib * 16;
            for (int j = 0; j < 16; j++) {
                out[bi * 256 + ib * 32 + j] = dl * (float)FO_KVALUES_IQ4NL[q[j] & 0x0F];
                out[bi * 256 + ib * 32 + j + 16] = dl * (float)FO_KVALUES_IQ4NL[q[j] >> 4];
            }
        }
    }
    return n;
}

/* crates/ferric-gguf/src/lib.rs:857-860: the E2M1 value table, doubled ({0, .5, 1, 1.5, 2, 3, 4, 6} * 2); code 8 is +0.0. */
static const float FO_KVALUES_MXFP4_2X[16] = {0.0f, 1.0f, 2.0f, 3.0f, 4.0f, 6.0f, 8.0f, 12.0f,
                                              0.0f, -1.0f, -2.0f, -3.0f, -4.0f, -6.0f, -8.0f, -12.0f};
/* crates/ferric-gguf/src/lib.rs:880-886: 2^(e - 128) from the E8M0 byte; e = 0 and e = 1 are subnormal bit patterns. */
float fo_e8m0_half(uint8_t e) {
    uint32_t bits = e == 0 ? (1u << 21) : e == 1 ? (1u << 22) : ((uint32_t)e - 1u) << 23;
    float f; memcpy(&f, &bits, 4); return f;
}
/* crates/ferric-gguf/src/lib.rs:896-908: 17-byte block [u8 e][qs[16]], value = table[code] * 2^(e - 128); element i is the
 * low nibble of qs[i], element i + 16 the high nibble. */
size_t fo_deq_mxfp4(const uint8_t* raw, size_t raw_len, size_t n, float* out) {
    for (size_t i = 0; i < n; i++) out[i] = 0.0f;
    size_t nb = n / 32, have = raw_len / 17;
    if (have < nb) nb = have;
    for (size_t bi = 0; bi < nb; bi++) {
        const uint8_t* blk = raw + bi * 17;
        float d = fo_e8m0_half(blk[0]);
        for (int i = 0; i < 16; i++) {
            out[bi * 32 + i] = FO_KVALUES_MXFP4_2X[blk[1 + i] & 0x0F] * d;
            out[bi * 32 + i + 16] = FO_KVALUES_MXFP4_2X[blk[1 + i] >> 4] * d;
        }
    }
    return n;
}

/* crates/ferric-gguf/src/lib.rs:497-520 (deq_raw), in-scope types. Returns the number of f32 the
 * reference's Vec would hold, or (size_t)-1 for "unsupported ggml type". */
/* The unquantized arms (lib.rs:499-501) slice raw[..n * size] first, which panics when the bytes are short:
 * (size_t)-2 stands for that panic. F32: little-endian bytes as they are; F16: the exact decode; BF16: the 16
 * bits become the top half of the f32 pattern. */
size_t fo_deq_raw(const uint8_t* raw, size_t raw_len, size_t n, uint32_t ty, float* out) {
    switch (ty) {
        case GGML_F32:
            if (raw_len < n * 4) return (size_t)-2;
            for (size_t i = 0; i < n; i++) {
                uint32_t b = (uint32_t)raw[4 * i] | ((uint32_t)raw[4 * i + 1] << 8) | ((uint32_t)raw[4 * i + 2] << 16) | ((uint32_t)raw[4 * i + 3] << 24);
                memcpy(out + i, &b, 4);
            }
            return n;
        case GGML_F16:
            if (raw_len < n * 2) return (size_t)-2;
            for (size_t i = 0; i < n; i++) out[i] = fo_f16_to_f32(rd_u16(raw + 2 * i));
            return n;
        case GGML_BF16:
            if (raw_len < n * 2) return (size_t)-2;
            for (size_t i = 0; i < n; i++) {
                uint32_t b = (uint32_t)rd_u16(raw + 2 * i) << 16;
                memcpy(out + i, &b, 4);
            }
            return n;
        case GGML_Q8_0: return fo_deq_q8_0(raw, raw_len, n, out);
        case GGML_Q4_K: return fo_deq_q4_k(raw, raw_len, n, out);
        case GGML_Q6_K: return fo_deq_q6_k(raw, raw_len, n, out);
        case GGML_Q4_0: return fo_deq_q4_0(raw, raw_len, n, out);
        case GGML_Q4_1: return fo_deq_q4_1(raw, raw_len, n, out);
        case GGML_Q5_0: return fo_deq_q5_0(raw, raw_len, n, out);
        case GGML_Q5_1: return fo_deq_q5_1(raw, raw_len, n, out);
        case GGML_Q5_K: return fo_deq_q5_k(raw, raw_len, n, out);
        case GGML_IQ4_NL: return fo_deq_iq4_nl(raw, raw_len, n, out);
        case GGML_IQ4_XS: return fo_deq_iq4_xs(raw, raw_len, n, out);
        case GGML_MXFP4: return fo_deq_mxfp4(raw, raw_len, n, out);
        default: return (size_t)-1;
    }
}

/* ---------------------------------------------------------------- dequantizers (random-access form)
 * A second, independent formulation: value of element v of one block, as the reference's
 * matrix-unit prefill kernels address it. Tests demand bit-equality with the sequential form. */

/* crates/ferric-tensor/src/dtype.rs:2078-2086 (Q4_K element -> (byte, shift)); scale/min from
 * the same 6-bit split as dtype.rs:2272-2279. */
float fo_q4k_elem(const uint8_t* blk, int v) {
    float d = fo_f16_to_f32(rd_u16(blk)), dmin = fo_f16_to_f32(rd_u16(blk + 2));
    const uint8_t* s = blk + 4; const uint8_t* qs = blk + 16;
    int sb = v / 32, l = v % 32;
    uint32_t sc, m;
    if (sb < 4) { sc = s[sb] & 63u; m = s[sb + 4] & 63u; }
    else { sc = (s[sb + 4] & 15u) | ((uint32_t)(s[sb - 4] >> 6) << 4); m = (uint32_t)(s[sb + 4] >> 4) | ((uint32_t)(s[sb] >> 6) << 4); }
    uint8_t byte = qs[32 * (sb >> 1) + l];
    uint32_t nib = (sb & 1) ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 15);
    float d1 = d * (float)sc, mm = dmin * (float)m;
    return d1 * (float)nib - mm;
}

/* crates/ferric-tensor/src/dtype.rs:1236-1246 (Q6_K element formula). */
float fo_q6k_elem(const uint8_t* blk, int v) {
    float d = fo_f16_to_f32(rd_u16(blk + 208));
    int hf = v / 128, within = v % 128, g = within / 32, l = within % 32, is = l >> 4;
    int8_t sc = (int8_t)blk[192 + 8 * hf + is + 2 * g];
    uint32_t h = blk[128 + 32 * hf + l];
    uint32_t qlbyte = blk[64 * hf + l + (g & 1) * 32];
    uint32_t nib = (g >= 2) ? (qlbyte >> 4) : (qlbyte & 0xFu);
    int q = (int)(nib | (((h >> (2 * g)) & 3u) << 4)) - 32;
    return d * (float)sc * (float)q;
}

/* crates/ferric-tensor/src/dtype.rs:1351-1356 (Q8_0 element formula). */
float fo_q8_0_elem(const uint8_t* blk, int v) {
    return (float)(int8_t)blk[2 + v] * fo_f16_to_f32(rd_u16(blk));
}

/* crates/ferric-tensor/src/dtype.rs:3548-3555 (Q4_0: word w of a block holds values 4w..4w+3 in its low nibbles and
 * 16+4w.. in its high nibbles) and :3613-3620 (Q4_1, the same words with + m). */
float fo_q4_0_elem(const uint8_t* blk, int v) {
    uint32_t word = rd_u32(blk + 2 + 4 * ((v & 15) >> 2));
    int nib = (int)((word >> (8 * (v & 3) + (v >= 16 ? 4 : 0))) & 0xFu);
    return (float)(nib - 8) * fo_f16_to_f32(rd_u16(blk));
}
float fo_q4_1_elem(const uint8_t* blk, int v) {
    uint32_t word = rd_u32(blk + 4 + 4 * ((v & 15) >> 2));
    uint32_t nib = (word >> (8 * (v & 3) + (v >= 16 ? 4 : 0))) & 0xFu;
    return (float)nib * fo_f16_to_f32(rd_u16(blk)) + fo_f16_to_f32(rd_u16(blk + 2));
}
/* crates/ferric-tensor/src/dtype.rs:3778-3792 (Q5_0: fifth bit of value base+c is qh bit base+c, of 16+base+c bit
 * base+16+c) and :3858-3874 (Q5_1). */
float fo_q5_0_elem(const uint8_t* blk, int v) {
    uint32_t qh = rd_u32(blk + 2), word = rd_u32(blk + 6 + 4 * ((v & 15) >> 2));
    uint32_t nib = (word >> (8 * (v & 3) + (v >= 16 ? 4 : 0))) & 0xFu;
    return (float)((int)(nib | (((qh >> v) & 1u) << 4)) - 16) * fo_f16_to_f32(rd_u16(blk));
}
float fo_q5_1_elem(const uint8_t* blk, int v) {
    uint32_t qh = rd_u32(blk + 4), word = rd_u32(blk + 8 + 4 * ((v & 15) >> 2));
    uint32_t nib = (word >> (8 * (v & 3) + (v >= 16 ? 4 : 0))) & 0xFu;
    return (float)(nib | (((qh >> v) & 1u) << 4)) * fo_f16_to_f32(rd_u16(blk)) + fo_f16_to_f32(rd_u16(blk + 2));
}
/* crates/ferric-tensor/src/dtype.rs:1108-1121 (Q5_K element of the matrix-unit kernel: sub-block s = v/32, l = v%32,
 * nibble from qs word 8*(s/2) + l/4, fifth bit = bit s of qh byte l), in raw-block offsets (qh at 16, qs at 48). */
float fo_q5k_elem(const uint8_t* blk, int v) {
    float d = fo_f16_to_f32(rd_u16(blk)), dmin = fo_f16_to_f32(rd_u16(blk + 2));
    const uint8_t* s = blk + 4;
    int sb = v / 32, l = v % 32;
    uint32_t sc, m;
    if (sb < 4) { sc = s[sb] & 63u; m = s[sb + 4] & 63u; }
    else { sc = (s[sb + 4] & 15u) | ((uint32_t)(s[sb - 4] >> 6) << 4); m = (uint32_t)(s[sb + 4] >> 4) | ((uint32_t)(s[sb] >> 6) << 4); }
    uint32_t qsw = rd_u32(blk + 48 + 4 * (8 * (sb >> 1) + (l >> 2)));
    uint32_t nib = (qsw >> (8 * (l & 3) + ((sb & 1) ? 4 : 0))) & 0xFu;
    uint32_t qhw = rd_u32(blk + 16 + 4 * (l >> 2));
    uint32_t bit = (qhw >> (8 * (l & 3) + sb)) & 1u;
    float ds = d * (float)sc, mm = dmin * (float)m;
    return ds * (float)(nib + bit * 16u) - mm;
}

/* crates/ferric-tensor/src/dtype.rs:3205-3214 (IQ4_NL body): byte j of the block's four code words, codebook value of
 * its low nibble for element j and of its high nibble for element j + 16. */
float fo_iq4_nl_elem(const uint8_t* blk, int v) {
    int j = v & 15;
    uint32_t b = (rd_u32(blk + 2 + 4 * (j >> 2)) >> (8 * (j & 3))) & 0xFFu;
    return fo_f16_to_f32(rd_u16(blk)) * (float)FO_KVALUES_IQ4NL[v >= 16 ? (b >> 4) : (b & 0x0Fu)];
}
/* crates/ferric-tensor/src/dtype.rs:3119-3145 (IQ4_XS body): scales_l read as one u32, the sub-block's four code words. */
float fo_iq4_xs_elem(const uint8_t* blk, int v) {
    uint32_t scales_h = rd_u16(blk + 2), scales_l = rd_u32(blk + 4);
    uint32_t ib = (uint32_t)v >> 5; int j = v & 15;
    uint32_t sl = (scales_l >> (8 * (ib >> 1))) & 0xFFu;
    uint32_t lo = (sl >> (4 * (ib & 1))) & 0x0Fu, hi = (scales_h >> (2 * ib)) & 3u;
    float dl = fo_f16_to_f32(rd_u16(blk)) * (float)((int)(lo | (hi << 4)) - 32);
    uint32_t b = (rd_u32(blk + 8 + 4 * (ib * 4 + (uint32_t)(j >> 2))) >> (8 * (j & 3))) & 0xFFu;
    return dl * (float)FO_KVALUES_IQ4NL[(v & 16) ? (b >> 4) : (b & 0x0Fu)];
}
/* crates/ferric-tensor/src/dtype.rs:3318-3344 (MXFP4 helpers + body): the integral table and the scale split in two
 * factors 2^(a - 64) * 2^(b - 64), a = e >> 1, b = e - a, applied one after the other. */
float fo_mxfp4_elem(const uint8_t* blk, int v) {
    static const int KM[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};
    uint32_t e = blk[0], a = e >> 1, b2 = e - a;
    uint32_t xa = (a + 63u) << 23, xb = (b2 + 63u) << 23;
    float dx, dy; memcpy(&dx, &xa, 4); memcpy(&dy, &xb, 4);
    int j = v & 15;
    uint32_t b = (rd_u32(blk + 1 + 4 * (j >> 2)) >> (8 * (j & 3))) & 0xFFu;
    return ((float)KM[v >= 16 ? (b >> 4) : (b & 0x0Fu)] * dx) * dy;
}

void fo_deq_elemwise(const uint8_t* raw, size_t n, uint32_t ty, float* out) {
    size_t vals, bytes;
    if (!fo_block_bytes(ty, &vals, &bytes)) return;
    for (size_t i = 0; i < n; i++) {
        const uint8_t* blk = raw + (i / vals) * bytes; int v = (int)(i % vals);
        switch (ty) {
            case GGML_Q8_0: out[i] = fo_q8_0_elem(blk, v); break;
            case GGML_Q4_K: out[i] = fo_q4k_elem(blk, v); break;
            case GGML_Q6_K: out[i] = fo_q6k_elem(blk, v); break;
            case GGML_Q4_0: out[i] = fo_q4_0_elem(blk, v); break;
            case GGML_Q4_1: out[i] = fo_q4_1_elem(blk, v); break;
            case GGML_Q5_0: out[i] = fo_q5_0_elem(blk, v); break;
            case GGML_Q5_1: out[i] = fo_q5_1_elem(blk, v); break;
            case GGML_Q5_K: out[i] = fo_q5k_elem(blk, v); break;
            case GGML_IQ4_NL: out[i] = fo_iq4_nl_elem(blk, v); break;
            case GGML_IQ4_XS: out[i] = fo_iq4_xs_elem(blk, v); break;
            case GGML_MXFP4: out[i] = fo_mxfp4_elem(blk, v); break;
            default: break;
        }
    }
}

/* ---------------------------------------------------------------- Q8_0 CPU mat-vec */

/* crates/ferric-tensor/src/cpu_simd.rs:57-72 (row_q8_0): per block part = sum_j x_j*q_j in order,
 * then acc += part*d; blocks in order. */
static float row_q8_0(const float* x, const uint8_t* blocks, size_t cols) {
    size_t nblk = cols / 32;
    float acc = 0.0f;
    for (size_t b = 0; b < nblk; b++) {
        const uint8_t* blk = blocks + b * 34;
        float d = fo_f16_to_f32(rd_u16(blk));
        const float* xs = x + b * 32;
        float part = 0.0f;
        for (int j = 0; j < 32; j++) part += xs[j] * (float)(int8_t)blk[2 + j];
        acc += part * d;
    }
    return acc;
}

/* crates/ferric-tensor/src/cpu_simd.rs:79-86 (matvec_q8_0). Returns 0 on the reference's assert
 * failures (cols % 32, byte length), 1 on success. */
int fo_matvec_q8_0(const float* x, const uint8_t* w, size_t w_len, size_t rows, size_t cols, float* y) {
    if (cols % 32 != 0) return 0;
    size_t row_bytes = cols / 32 * 34;
    if (w_len != rows * row_bytes) return 0;
    for (size_t r = 0; r < rows; r++) y[r] = row_q8_0(x, w + r * row_bytes, cols);
    return 1;
}

typedef struct {
    const float* x; const uint8_t* w; size_t row_bytes, cols, lo, hi; uint32_t ty; int direct_q8; float* y; size_t xrows, xstride, ystride;
} span_job;

static void* span_worker(void* p) {
    span_job* j = (span_job*)p;
    float* scratch = j->direct_q8 ? NULL : (float*)malloc(j->cols * sizeof(float));
    for (size_t r = j->lo; r < j->hi; r++) {
        const uint8_t* row = j->w + r * j->row_bytes;
        if (j->direct_q8) {
            for (size_t t = 0; t < j->xrows; t++) j->y[t * j->ystride + r] = row_q8_0(j->x + t * j->xstride, row, j->cols);
        } else {
            /* The reference's CPU route for K-quants: deq_raw (crates/ferric-gguf/src/lib.rs:497) then the
             * sequential-k f32 dot of crates/ferric-core/src/lib.rs:428-440 / crates/ferric-tensor/src/cpu.rs:72-92
             * (`s += a[..]*b[..]`, activation operand first). The row is dequantized once and reused for
             * every activation row. */
            fo_deq_raw(row, j->row_bytes, j->cols, j->ty, scratch);
            for (size_t t = 0; t < j->xrows; t++) {
                const float* xr = j->x + t * j->xstride; float s = 0.0f;
                for (size_t l = 0; l < j->cols; l++) s += xr[l] * scratch[l];
                j->y[t * j->ystride + r] = s;
            }
        }
    }
    free(scratch);
    return NULL;
}

/* Row-span threading of crates/ferric-tensor/src/cpu_simd.rs:92-112 (matvec_q8_0_threaded):
 * threads clamped to [1, rows], per = ceil(rows/threads), thread t owns rows [t*per, min(rows,(t+1)*per)).
 * direct_q8 = 1 uses row_q8_0 (the Q8_0 CPU mat-vec); 0 uses dequant-then-dot (K-quants, or Q8_0
 * checked the way the reference examples check the GPU: deq_raw + dense matmul).
 * x is [xrows, cols] row-major, y is [xrows, rows] row-major (y = x * W^T). */
int fo_matmul_threaded(const float* x, size_t xrows, const uint8_t* w, size_t w_len, uint32_t ty, size_t rows, size_t cols,
                       int direct_q8, size_t threads, float* y) {
    size_t vals, bytes;
    if (!fo_block_bytes(ty, &vals, &bytes)) return 0;
    if (cols % vals != 0) return 0;
    size_t row_bytes = cols / vals * bytes;
    if (w_len != rows * row_bytes) return 0;
    if (direct_q8 && ty != GGML_Q8_0) return 0;
    if (threads < 1) threads = 1;
    if (threads > (rows ? rows : 1)) threads = rows ? rows : 1;
    size_t per = (rows + threads - 1) / threads;
    if (per == 0) return 1;
    size_t nt = (rows + per - 1) / per;
    span_job* jobs = (span_job*)calloc(nt, sizeof(span_job));
    pthread_t* th = (pthread_t*)calloc(nt, sizeof(pthread_t));
    for (size_t t = 0; t < nt; t++) {
        size_t lo = t * per, hi = lo + per; if (hi > rows) hi = rows;
        span_job j = { x, w, row_bytes, cols, lo, hi, ty, direct_q8, y, xrows, cols, rows };
        jobs[t] = j;
        if (nt == 1) span_worker(&jobs[t]); else pthread_create(&th[t], NULL, span_worker, &jobs[t]);
    }
    if (nt > 1) for (size_t t = 0; t < nt; t++) pthread_join(th[t], NULL);
    free(jobs); free(th);
    return 1;
}

/* crates/ferric-tensor/src/cpu_simd.rs:92-112. */
int fo_matvec_q8_0_threaded(const float* x, const uint8_t* w, size_t w_len, size_t rows, size_t cols, size_t threads, float* y) {
    if (cols % 32 != 0) return 0;
    return fo_matmul_threaded(x, 1, w, w_len, GGML_Q8_0, rows, cols, 1, threads, y);
}

/* crates/ferric-tensor/src/cpu_simd.rs:118-122 (matvec_q8_0_span): rows [lo,hi) only; y has hi-lo entries. */
int fo_matvec_q8_0_span(const float* x, const uint8_t* w, size_t cols, size_t lo, size_t hi, size_t threads, float* y) {
    if (lo > hi || cols % 32 != 0) return 0;
    size_t row_bytes = cols / 32 * 34;
    return fo_matvec_q8_0_threaded(x, w + lo * row_bytes, (hi - lo) * row_bytes, hi - lo, cols, threads, y);
}

/* ---------------------------------------------------------------- SwiGLU + f64 checker */

/* crates/ferric-tensor/src/dtype.rs:2406-2408 and crates/ferric-tensor/src/lib.rs:2611-2616:
 * gu is [t, 2*n_ff] = [gate | up] per row; out[t, n_ff] = (g / (1 + exp(-g))) * u in f32. */
void fo_swiglu(const float* gu, size_t t, size_t n_ff, float* out) {
    for (size_t r = 0; r < t; r++)
        for (size_t c = 0; c < n_ff; c++) {
            float g = gu[r * 2 * n_ff + c], u = gu[r * 2 * n_ff + n_ff + c];
            out[r * n_ff + c] = (g / (1.0f + expf(-g))) * u;
        }
}

/* Tolerance checker, not a reference function: y64 = x * W^T accumulated in f64 over the
 * oracle-dequantized weights, plus ||w_row||_2 per output row, for the bound
 * |dy| <= 1e-3 * ||w_row|| * ||x||. */
int fo_matmul_f64(const float* x, size_t xrows, const uint8_t* w, size_t w_len, uint32_t ty, size_t rows, size_t cols,
                  double* y64, double* wnorm) {
    size_t vals, bytes;
    if (!fo_block_bytes(ty, &vals, &bytes) || cols % vals != 0) return 0;
    size_t row_bytes = cols / vals * bytes;
    if (w_len != rows * row_bytes) return 0;
    float* scratch = (float*)malloc(cols * sizeof(float));
    for (size_t r = 0; r < rows; r++) {
        fo_deq_raw(w + r * row_bytes, row_bytes, cols, ty, scratch);
        double nn = 0.0;
        for (size_t l = 0; l < cols; l++) nn += (double)scratch[l] * (double)scratch[l];
        if (wnorm) wnorm[r] = sqrt(nn);
        for (size_t t = 0; t < xrows; t++) {
            double s = 0.0; const float* xr = x + t * cols;
            for (size_t l = 0; l < cols; l++) s += (double)xr[l] * (double)scratch[l];
            y64[t * rows + r] = s;
        }
    }
    free(scratch);
    return 1;
}

/* ---------------------------------------------------------------- the reference's test-data generators
 * All integer arithmetic is u32 wrapping (release-mode Rust). */

/* crates/ferric-tensor/examples/q4_k.rs:13-37 (q4k_block). */
void fo_gen_q4k_block(uint32_t seed, uint8_t* b) {
    float d = 0.05f + 0.01f * (float)(seed % 7), dmin = 0.02f + 0.005f * (float)(seed % 5);
    uint16_t dh = fo_f32_to_f16(d), mh = fo_f32_to_f16(dmin);
    b[0] = dh & 0xFF; b[1] = dh >> 8; b[2] = mh & 0xFF; b[3] = mh >> 8;
    uint8_t* s = b + 4; memset(s, 0, 12);
    for (uint32_t j = 0; j < 8; j++) {
        uint8_t scv = (uint8_t)((seed * 2654435761u + j * 40503u) % 64u);
        uint8_t mnv = (uint8_t)((seed * 40503u + j * 2654435761u) % 64u);
        if (j < 4) { s[j] |= scv & 63; s[j + 4] |= mnv & 63; }
        else { s[j + 4] |= (scv & 0x0F) | ((mnv & 0x0F) << 4); s[j - 4] |= (scv >> 4) << 6; s[j] |= (mnv >> 4) << 6; }
    }
    for (uint32_t i = 0; i < 128; i++) b[16 + i] = (uint8_t)((seed + i * 2246822519u) % 256u);
}

/* crates/ferric-tensor/examples/q6_k.rs:9-17 (q6k_block). */
void fo_gen_q6k_block(uint32_t seed, uint8_t* b) {
    for (uint32_t i = 0; i < 128; i++) b[i] = (uint8_t)((seed + i * 2246822519u) % 256u);
    for (uint32_t i = 0; i < 64; i++) b[128 + i] = (uint8_t)((seed * 40503u + i * 97u) % 256u);
    for (uint32_t i = 0; i < 16; i++) b[192 + i] = (uint8_t)(int8_t)((int32_t)((seed + i * 7u) % 64u) - 32);
    uint16_t dh = fo_f32_to_f16(0.04f + 0.01f * (float)(seed % 6));
    b[208] = dh & 0xFF; b[209] = dh >> 8;
}

/* Weight builders used by the reference examples: block seed = r*nblk + blk + 1
 * (q4_k.rs:46, q6_k.rs:25). ty 12 or 14. */
void fo_gen_kquant_matrix(uint32_t ty, size_t rows, size_t cols, uint8_t* out) {
    size_t nblk = cols / 256, bytes = ty == GGML_Q4_K ? 144 : 210;
    for (size_t r = 0; r < rows; r++)
        for (size_t b = 0; b < nblk; b++) {
            uint32_t seed = (uint32_t)(r * nblk + b) + 1u;
            uint8_t* dst = out + (r * nblk + b) * bytes;
            if (ty == GGML_Q4_K) fo_gen_q4k_block(seed, dst); else fo_gen_q6k_block(seed, dst);
        }
}

/* crates/ferric-gguf/src/lib.rs:985-997 (quant_q8_0): d = amax/127 kept in f32 for the division,
 * stored as f16; q = clamp(round_half_away(v/d), -127, 127). len must be a multiple of 32 here. */
void fo_quant_q8_0(const float* x, size_t len, uint8_t* out) {
    for (size_t b = 0; b < len / 32; b++) {
        const float* blk = x + b * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) { float a = fabsf(blk[i]); if (a > amax) amax = a; }
        float d = amax / 127.0f;
        uint16_t dh = fo_f32_to_f16(d);
        uint8_t* o = out + b * 34;
        o[0] = dh & 0xFF; o[1] = dh >> 8;
        for (int i = 0; i < 32; i++) {
            int8_t q = 0;
            if (d != 0.0f) { float r = roundf(blk[i] / d); if (r < -127.0f) r = -127.0f; if (r > 127.0f) r = 127.0f; q = (int8_t)r; }
            o[2 + i] = (uint8_t)q;
        }
    }
}

/* crates/ferric-tensor/src/cpu_simd.rs:136-156 (test helper synth): raw Q8_0 bytes plus the exact
 * f32 values they encode, built beside the bytes and not through the dequantizer. */
void fo_gen_q8_0_synth(size_t rows, size_t cols, uint32_t seed, uint8_t* raw, float* vals) {
    uint32_t s = seed * 2654435761u + 1u;
    size_t nblk = cols / 32, w = 0;
    for (size_t r = 0; r < rows; r++)
        for (size_t b = 0; b < nblk; b++) {
            s = s * 1664525u + 1013904223u;
            uint16_t dbits = (uint16_t)(0x1C00u | ((uint16_t)(s >> 16) & 0x3Fu));
            raw[w++] = dbits & 0xFF; raw[w++] = dbits >> 8;
            float d = fo_f16_to_f32(dbits);
            for (int j = 0; j < 32; j++) {
                s = s * 1664525u + 1013904223u;
                uint8_t c = (uint8_t)((uint16_t)(s >> 16) & 0xFF);
                raw[w++] = c;
                vals[r * cols + b * 32 + j] = (float)(int8_t)c * d;
            }
        }
}

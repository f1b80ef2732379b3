// CPU oracle for the speculative-verify hot path.  TEST INFRASTRUCTURE ONLY: see shadow_oracle.h.
//
// Compiled with `g++ -O2 -std=c++17 -ffp-contract=off` so that no multiply-add is fused: the dequantizers must give the
// same bits as the reference's unfused f32 arithmetic.  Paths in comments are relative to the reference checkout.
//
// How each function is pinned (tests/test_oracle_*.py):
//   f16 <-> f32            numpy.float16 over all 65,536 patterns; known values of half.rs:76-93.
//   F16 / BF16 matrices    numpy.float16 / the f32 whose upper half the bf16 is, over all 65,536 patterns.
//   Q8_0 dequant           closed form d * q (one f32 rounding) against numpy for every q and a sweep of scales.
//   IQ3_S dequant          the 8 real IQ3_S blocks with ggml's expected bits (tests/golden/iq3_s_blocks.txt).
//   EXL3 codebooks         independent numpy float16 arithmetic over all 65,536 states; unit-Gaussian statistics.
//   EXL3 tile decode       bit-loop decode == 64-bit-window decode (two independent statements), K = 1..8 and halves;
//                          tile_pos is a bijection.  The K + 1/2 rates (exl3.rs:150-170): PARITY UNPINNED - the reference
//                          holds no tensor and no known answer at such a rate; the agreement of the two statements is all there is.
//   EXL3 reconstruct       recorded sum of squares and first four values of the two real tensors in
//                          tests/golden/exl3_sample.safetensors.
//   EXL3 matvec_blob       equals x times the reconstructed matrix (dense f64 product) within 2e-4 of the largest output.
//   GGUF matvec            dense f64 product of the dequantized matrix (numpy), bitwise.
//   rmsnorm / hc_read      numpy f64 restatement on small shapes (closed forms: a constant row, unit weights; inject off).
//   route                  full stable sort by (ex descending, index ascending) with numpy, ties included.
//   moe_token              recomputed in numpy from orc_backend_matvec outputs; special cases (k = 1, zero shared gate).
//   int8 activations       closed form in numpy; int32 dots exact against numpy int64.
//   argmax/topk/accept     numpy sort on adversarial rows (ties, all equal, -inf, NaN); all four outcomes of K = 3.
//   2-bit head screen      the gates of the reference's own test (crates/shadowzero-cuda/tests/head_proxy.rs:176-232) on its
//                          shape: cosine of the block maxima with the exact ones above 0.85, the best row's block chosen,
//                          the number of chosen blocks in range; a float64 restatement of the scores from the levels'
//                          values; the rotated matrix against the exact product; the textbook distortion of the optimal
//                          uniform four-level quantizer of a Gaussian (0.1188 of the variance at a step of 0.9957 sigma);
//                          the choice of blocks against a plain top-k wherever no residue class holds five of them.

#include "shadow_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

namespace {

const uint32_t IQ3S_GRID[512] = {
#include "iq3s_grid.inc"
};

inline float bits_f32(uint32_t b) {
    float f;
    std::memcpy(&f, &b, 4);
    return f;
}
inline uint32_t f32_bits(float f) {
    uint32_t b;
    std::memcpy(&b, &f, 4);
    return b;
}

int hw_threads() {
    unsigned n = std::thread::hardware_concurrency();
    return n ? (int) n : 4;   // forward.rs:205-207
}

inline float f16_at(const uint8_t* b, size_t i) {
    return orc_f16_to_f32((uint16_t) (b[i] | (b[i + 1] << 8)));
}

// quant.rs:174-179
void q8_0_block(const uint8_t* b, float* y) {
    const float d = f16_at(b, 0);
    for (int i = 0; i < 32; i++) y[i] = d * (float) (int8_t) b[2 + i];
}

// quant.rs:148-159
void iq3_s_block(const uint8_t* b, float* y) {
    const float d = f16_at(b, 0);
    const uint8_t *qs = b + 2, *qh = b + 66, *signs = b + 74, *scales = b + 106;
    for (int e = 0; e < 256; e++) {
        const int j = e / 4;
        const unsigned idx = qs[j] | (((qh[j / 8] >> (j % 8)) & 1u) << 8);
        const int g = e / 32;
        const unsigned s = (scales[g / 2] >> (4 * (g % 2))) & 0x0f;
        const float db = d * (float) (1 + 2 * s);
        const float grid = (float) ((IQ3S_GRID[idx] >> (8 * (e % 4))) & 0xff);
        const float sg = ((signs[e / 8] >> (e % 8)) & 1) ? -1.0f : 1.0f;
        y[e] = db * grid * sg;
    }
}

template <class F>
void parallel_chunks(size_t n, size_t per, F&& f) {
    // rows (or blocks) split into chunks of `per`, one thread a chunk, as forward.rs:214-226 / exl3.rs:569-578
    std::vector<std::thread> th;
    for (size_t first = 0; first < n; first += per) {
        const size_t last = std::min(n, first + per);
        th.emplace_back([=, &f] { f(first, last); });
    }
    for (auto& t : th) t.join();
}

struct Rate {
    int bits;
    bool half;
    int ring_words() const { return half ? 4 * (2 * bits + 1) : 8 * bits; }   // exl3.rs:153
    int tile_words() const { return 2 * ring_words(); }                       // exl3.rs:158
    int end_bit(int t) const {                                                // exl3.rs:164
        if (!half) return (t + 1) * bits;
        const int b2 = 2 * bits + 1;
        return (t & 1) ? (t / 2 + 1) * b2 : (t / 2) * b2 + bits;
    }
};

inline uint32_t stream_bit(const uint16_t* tile, int s) {                     // exl3.rs:126
    const int w = s / 32;
    const uint32_t word = (uint32_t) tile[2 * w] | ((uint32_t) tile[2 * w + 1] << 16);
    return (word >> (31 - s % 32)) & 1u;
}

float two_halves_sum(uint32_t x) {                                            // exl3.rs:70
    x = (x & 0x8fff8fffu) ^ 0x3b603b60u;
    return orc_round_f16((double) orc_f16_to_f32((uint16_t) (x & 0xffff)) + (double) orc_f16_to_f32((uint16_t) (x >> 16)));
}

const float* codebook_table(int cb) {                                         // exl3.rs:354
    static std::vector<float> tabs[3];
    static std::once_flag once[3];
    cb = std::min(std::max(cb, 0), 2);
    std::call_once(once[cb], [cb] {
        tabs[cb].resize(65536);
        for (uint32_t s = 0; s < 65536; s++) tabs[cb][s] = orc_exl3_codebook(cb, s);
    });
    return tabs[cb].data();
}

struct TilePos {
    uint8_t row[256], col[256];
    TilePos() {
        for (int p = 0; p < 256; p++) {
            int r, c;
            orc_exl3_tile_pos(p, &r, &c);
            row[p] = (uint8_t) r;
            col[p] = (uint8_t) c;
        }
    }
};
const TilePos& tile_pos_table() {
    static TilePos t;
    return t;
}

void decode_tile_fast(const uint16_t* tile, Rate rate, const float* lut, float* out) {   // exl3.rs:375-386
    const int nw = rate.ring_words();
    const int n = nw * 32;
    auto word = [&](int i) { return (uint32_t) tile[2 * i] | ((uint32_t) tile[2 * i + 1] << 16); };
    for (int t = 0; t < 256; t++) {
        const int s = (rate.end_bit(t) + n - 16) % n;
        const int wi = s / 32, sh = s % 32;
        const uint64_t merged = ((uint64_t) word(wi) << 32) | (uint64_t) word((wi + 1) % nw);
        out[t] = lut[(merged >> (48 - sh)) & 0xffff];
    }
}

bool exl3_type(int ty, int* bits, bool* half, int* cb) {                       // gguf.rs exl3()/exl3_half()
    if (ty >= 1031 && ty <= 1033) { *bits = ty - 1030; *half = true; *cb = 2; return true; }
    if (ty >= 1001 && ty <= 1028 && (ty % 10) >= 1 && (ty % 10) <= 8) {
        *bits = ty % 10; *half = false; *cb = (ty - 1000) / 10; return true;
    }
    return false;
}

}   // namespace

extern "C" {

int orc_hardware_threads(void) { return hw_threads(); }

// ---------------------------------------------------------------------------------------------------------- half.rs
float orc_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t) (h >> 15) << 31;
    const uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ff;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        // subnormal m * 2^-24: normalise
        int top = 31 - __builtin_clz(man);              // position of the highest set bit, 0..9
        const uint32_t m = (man << (10 - top)) & 0x3ff;
        return bits_f32(sign | ((uint32_t) (127 - 24 + top) << 23) | (m << 13));
    }
    if (exp == 31) return bits_f32(sign | (man ? 0x7fc00000u | (man << 13) : 0x7f800000u));
    return bits_f32(sign | ((exp + 112) << 23) | (man << 13));
}

uint16_t orc_f32_to_f16(float f) {
    const uint32_t x = f32_bits(f);
    const uint16_t sign = (uint16_t) ((x >> 16) & 0x8000);
    const int exp = (int) ((x >> 23) & 0xff);
    const uint32_t man = x & 0x7fffff;
    if (exp == 0xff) return sign | (man == 0 ? 0x7c00 : (uint16_t) (0x7e00 | ((man >> 13) & 0x1ff)));
    const int e = exp - 127 + 15;
    if (e >= 31) return sign | 0x7c00;
    if (e <= 0) {
        if (e < -10) return sign;
        const uint32_t m = man | 0x800000;
        const uint32_t shift = (uint32_t) (14 - e);
        const uint32_t halfway = 1u << (shift - 1);
        const uint32_t rem = m & ((1u << shift) - 1);
        uint32_t r = m >> shift;
        if (rem > halfway || (rem == halfway && (r & 1))) r++;
        return sign | (uint16_t) r;
    }
    uint32_t r = ((uint32_t) e << 10) | (man >> 13);
    const uint32_t rem = man & 0x1fff;
    if (rem > 0x1000 || (rem == 0x1000 && (r & 1))) r++;   // a carry into the exponent (and into infinity) is right
    return sign | (uint16_t) r;
}

// exl3.rs:32-63, restated on the bits of the double (one rounding, ties to even)
uint16_t orc_f64_to_f16_bits(double x) {
    if (std::isnan(x)) return 0x7e00;
    uint64_t b;
    std::memcpy(&b, &x, 8);
    const uint16_t sign = (uint16_t) ((b >> 48) & 0x8000);
    const double a = std::fabs(x);
    if (a >= 65520.0) return sign | 0x7c00;
    if (a < 6.103515625e-5) {
        // multiples of 2^-24: a * 2^24 is exact in f64, round to nearest even integer
        const double s = a * 16777216.0;
        double r = std::floor(s);
        const double frac = s - r;
        if (frac > 0.5 || (frac == 0.5 && std::fmod(r, 2.0) == 1.0)) r += 1.0;
        return sign | (uint16_t) r;
    }
    const int e = (int) ((b >> 52) & 0x7ff) - 1023;          // a in [2^e, 2^(e+1)), e in [-14, 15]
    const uint64_t man = b & 0xfffffffffffffull;             // 52 bits
    uint32_t m = (uint32_t) (man >> 42);                     // top 10 bits
    const uint64_t rem = man & ((1ull << 42) - 1), halfway = 1ull << 41;
    int ee = e;
    if (rem > halfway || (rem == halfway && (m & 1))) m++;
    if (m == 1024) { m = 0; ee++; }
    if (ee + 15 >= 31) return sign | 0x7c00;
    return sign | (uint16_t) ((ee + 15) << 10) | (uint16_t) m;
}

float orc_round_f16(double x) { return orc_f16_to_f32(orc_f64_to_f16_bits(x)); }

// --------------------------------------------------------------------------------------------------------- quant.rs
int orc_block_layout(int ty, uint64_t* elems, uint64_t* bytes) {
    uint64_t e = 0, b = 0;
    switch (ty) {
        case ORC_TYPE_F32: e = 1; b = 4; break;
        case ORC_TYPE_F16: case ORC_TYPE_BF16: e = 1; b = 2; break;
        case ORC_TYPE_Q8_0: e = 32; b = 34; break;
        case ORC_TYPE_IQ3_S: e = 256; b = 110; break;
        default: return 1;
    }
    if (elems) *elems = e;
    if (bytes) *bytes = b;
    return 0;
}

int orc_dequantize(int ty, const uint8_t* data, size_t nbytes, float* out, size_t nout) {
    uint64_t e, b;
    if (orc_block_layout(ty, &e, &b)) return 1;
    if (nbytes % b != 0 || nout != nbytes / b * e) return 2;
    const size_t nb = nbytes / b;
    for (size_t i = 0; i < nb; i++) {
        const uint8_t* blk = data + i * b;
        float* y = out + i * e;
        switch (ty) {
            case ORC_TYPE_F32: std::memcpy(y, blk, 4); break;                                   // quant.rs:237
            case ORC_TYPE_F16: y[0] = f16_at(blk, 0); break;                                    // quant.rs:238
            case ORC_TYPE_BF16: y[0] = bits_f32((uint32_t) (blk[0] | (blk[1] << 8)) << 16); break;   // quant.rs:239, half.rs bf16_to_f32
            case ORC_TYPE_Q8_0: q8_0_block(blk, y); break;
            case ORC_TYPE_IQ3_S: iq3_s_block(blk, y); break;
        }
    }
    return 0;
}

// ------------------------------------------------------------------------------------------- forward.rs: matvec/Backend
static int gguf_matvec(const orc_tensor* t, const float* x, float* y, int threads) {       // forward.rs:210-228
    uint64_t e, b;
    if (orc_block_layout(t->ggml_type, &e, &b)) return 1;
    if (t->cols % e) return 2;
    const size_t cols = t->cols, rb = cols / e * b;
    if (rb == 0 || t->nbytes % rb) return 2;
    const size_t rows = t->nbytes / rb;
    if (t->rows && rows != t->rows) return 2;
    const int nt = threads > 0 ? threads : hw_threads();
    const size_t per = std::max<size_t>((rows + nt - 1) / nt, 16);
    const int ty = t->ggml_type;
    const uint8_t* bytes = t->bytes;
    parallel_chunks(rows, per, [=](size_t first, size_t last) {
        std::vector<float> w(cols);
        for (size_t r = first; r < last; r++) {
            orc_dequantize(ty, bytes + r * rb, rb, w.data(), cols);
            double acc = 0.0;
            for (size_t i = 0; i < cols; i++) acc += (double) w[i] * (double) x[i];
            y[r] = (float) acc;
        }
    });
    return 0;
}

int orc_backend_matvec(const orc_tensor* t, const float* x, float* y, int threads) {       // forward.rs:239-249
    int bits, cb;
    bool half;
    if (exl3_type(t->ggml_type, &bits, &half, &cb))
        return orc_exl3_matvec_blob(t->cols, t->rows, bits, half, cb, t->bytes, t->nbytes, x, y, threads > 0 ? threads : hw_threads());
    return gguf_matvec(t, x, y, threads);
}

// ---------------------------------------------------------------------------------------------------------- exl3.rs
float orc_exl3_codebook(int cb, uint32_t state) {
    if (cb == 0) return two_halves_sum(state * 89226354u + 64248484u);                     // exl3.rs:76
    if (cb == 1) return two_halves_sum(state * 0xCBAC1FEDu);                               // exl3.rs:81
    const uint32_t x = state * 0x83DCD12Du;                                                // exl3.rs:87-94
    const uint32_t sum = 0x6400u + (x & 0xff) + ((x >> 8) & 0xff) + ((x >> 16) & 0xff) + (x >> 24);
    const double h = (double) orc_f16_to_f32((uint16_t) sum);
    const double k_inv = (double) orc_f16_to_f32(0x1eee), k_bias = (double) orc_f16_to_f32(0xc931);
    return orc_round_f16(h * k_inv + k_bias);
}

void orc_exl3_tile_pos(int p, int* row, int* col) {
    const int l = p / 8, j = p % 8;
    *row = 2 * (l % 4) + (j & 1) + 8 * ((j >> 1) & 1);
    *col = 2 * (l >> 3) + ((l >> 2) & 1) + 8 * (j >> 2);
}

uint32_t orc_exl3_state(const uint16_t* tile, int bits, int half, int t) {
    const Rate rate{bits, half != 0};
    const int n = rate.ring_words() * 32;
    const int end = rate.end_bit(t);
    uint32_t w = 0;
    for (int b = 0; b < 16; b++) w = (w << 1) | stream_bit(tile, (end + n - 16 + b) % n);
    return w;
}

void orc_exl3_decode_tile(const uint16_t* tile, int bits, int half, int cb, float* out) {
    for (int t = 0; t < 256; t++) out[t] = orc_exl3_codebook(cb, orc_exl3_state(tile, bits, half, t));
}

void orc_exl3_decode_tile_fast(const uint16_t* tile, int bits, int half, int cb, float* out) {
    decode_tile_fast(tile, Rate{bits, half != 0}, codebook_table(cb), out);
}

uint64_t orc_exl3_blob_len(uint64_t in_f, uint64_t out_f, int bits, int half) {
    return 2 * in_f + 2 * out_f + 4 + in_f * out_f * (uint64_t) (2 * bits + (half ? 1 : 0)) / 16;
}

void orc_wht128(float* v) {
    for (int h = 1; h < 128; h *= 2)
        for (int i = 0; i < 128; i += 2 * h)
            for (int j = i; j < i + h; j++) {
                const float a = v[j], b = v[j + h];
                v[j] = a + b;
                v[j + h] = a - b;
            }
    const float s = 0.08838835f;
    for (int i = 0; i < 128; i++) v[i] *= s;
}

int orc_exl3_reconstruct(uint64_t ni, uint64_t no, int bits, int half, int cb, const uint8_t* blob, uint64_t nbytes,
                         int inner_only, float* w) {
    if (ni % 128 || no % 128 || nbytes != orc_exl3_blob_len(ni, no, bits, half)) return 2;
    const Rate rate{bits, half != 0};
    const size_t osv = 2 * ni, otr = 2 * ni + 2 * no + 4;
    std::vector<float> suh(ni), svh(no);
    for (size_t i = 0; i < ni; i++) suh[i] = f16_at(blob, 2 * i);
    for (size_t i = 0; i < no; i++) svh[i] = f16_at(blob, osv + 2 * i);
    std::vector<uint16_t> trellis((nbytes - otr) / 2);
    std::memcpy(trellis.data(), blob + otr, nbytes - otr);
    const size_t kt = ni / 16, nt = no / 16, tw = rate.tile_words();
    float vals[256];
    for (size_t k = 0; k < kt; k++)                                          // exl3.rs:242-256
        for (size_t n = 0; n < nt; n++) {
            orc_exl3_decode_tile(&trellis[(k * nt + n) * tw], bits, half, cb, vals);
            for (int p = 0; p < 256; p++) {
                int r, c;
                orc_exl3_tile_pos(p, &r, &c);
                w[(k * 16 + r) * no + n * 16 + c] = vals[p];
            }
        }
    if (inner_only) return 0;
    float col[128];                                                          // exl3.rs:259-293
    for (size_t b = 0; b < ni / 128; b++)
        for (size_t c = 0; c < no; c++) {
            for (int i = 0; i < 128; i++) col[i] = w[(b * 128 + i) * no + c];
            orc_wht128(col);
            for (int i = 0; i < 128; i++) w[(b * 128 + i) * no + c] = col[i];
        }
    for (size_t i = 0; i < ni; i++)
        for (size_t c = 0; c < no; c++) w[i * no + c] *= suh[i];
    for (size_t r = 0; r < ni; r++)
        for (size_t b = 0; b < no / 128; b++) orc_wht128(&w[r * no + b * 128]);
    for (size_t r = 0; r < ni; r++)
        for (size_t c = 0; c < no; c++) w[r * no + c] *= svh[c];
    return 0;
}

int orc_exl3_matvec_blob(uint64_t ni, uint64_t no, int bits, int half, int cb, const uint8_t* blob, uint64_t nbytes,
                         const float* x, float* y, int threads) {            // exl3.rs:528-580
    if (ni % 128 || no % 128 || nbytes != orc_exl3_blob_len(ni, no, bits, half)) return 2;
    const Rate rate{bits, half != 0};
    const size_t osv = 2 * ni, otr = 2 * ni + 2 * no + 4;
    std::vector<float> svh(no), xr(ni);
    for (size_t i = 0; i < ni; i++) xr[i] = x[i] * f16_at(blob, 2 * i);
    for (size_t i = 0; i < no; i++) svh[i] = f16_at(blob, osv + 2 * i);
    for (size_t b = 0; b < ni / 128; b++) orc_wht128(&xr[b * 128]);
    std::vector<uint16_t> trellis((nbytes - otr) / 2);
    std::memcpy(trellis.data(), blob + otr, nbytes - otr);
    const size_t kt = ni / 16, nt = no / 16, tw = rate.tile_words();
    const float* lut = codebook_table(cb);
    const TilePos& pos = tile_pos_table();
    const size_t nb = no / 128;
    const size_t nthreads = threads > 0 ? threads : 1;
    const size_t per = std::max<size_t>((nb + nthreads - 1) / nthreads, 1);
    parallel_chunks(nb, per, [&](size_t first, size_t last) {
        float vals[256];
        for (size_t ob = first; ob < last; ob++) {
            double acc[128] = {0};
            for (size_t c = 0; c < 8; c++) {
                const size_t n = ob * 8 + c;
                for (size_t k = 0; k < kt; k++) {
                    decode_tile_fast(&trellis[(k * nt + n) * tw], rate, lut, vals);
                    const float* xk = &xr[k * 16];
                    for (int p = 0; p < 256; p++) acc[c * 16 + pos.col[p]] += (double) xk[pos.row[p]] * (double) vals[p];
                }
            }
            float o[128];
            for (int i = 0; i < 128; i++) o[i] = (float) acc[i];
            orc_wht128(o);
            for (int i = 0; i < 128; i++) y[ob * 128 + i] = o[i] * svh[ob * 128 + i];
        }
    });
    return 0;
}

// ------------------------------------------------------------------------------------- forward.rs: router, MoE layer
int orc_route(const float* logits, int ne, int k, uint32_t* idx, double* w) {               // forward.rs:1088-1153
    if (k <= 0 || ne <= 0) return 0;
    float mx = -3.40282347e+38f;                                                            // f32::MIN
    for (int i = 0; i < ne; i++) mx = std::max(mx, logits[i]);                              // f32::max: NaN ignored
    std::vector<double> ex(ne);
    double z = 0.0;
    for (int i = 0; i < ne; i++) {
        ex[i] = std::exp((double) (logits[i] - mx));
        z += ex[i];
    }
    // the first k of a full sort by (ex descending, index ascending), kept by insertion
    std::vector<int> top;
    auto before = [&](int a, int b) { return ex[a] > ex[b] || (ex[a] == ex[b] && a < b); };
    for (int i = 0; i < ne; i++) {
        if ((int) top.size() == k && !before(i, top[k - 1])) continue;
        size_t at = 0;
        while (at < top.size() && before(top[at], i)) at++;
        top.insert(top.begin() + at, i);
        if ((int) top.size() > k) top.resize(k);
    }
    double tz = 0.0;
    for (int e : top) tz += ex[e] / z;
    for (size_t t = 0; t < top.size(); t++) {
        idx[t] = (uint32_t) top[t];
        w[t] = (ex[top[t]] / z) / tz;
    }
    return (int) top.size();
}

float orc_sigmoid(float x) { return (float) (1.0 / (1.0 + std::exp(-(double) x))); }        // forward.rs:262
float orc_silu(float x) { return x * orc_sigmoid(x); }                                      // forward.rs:266

void orc_rmsnorm_groups(const float* x, const float* w, size_t n, size_t group, float eps, float* out) {   // forward.rs:251-260
    for (size_t g0 = 0; g0 < n; g0 += group) {
        const size_t len = std::min(group, n - g0);
        double ms = 0.0;
        for (size_t i = 0; i < len; i++) ms += (double) x[g0 + i] * (double) x[g0 + i];
        ms /= (double) len;
        const double r = 1.0 / std::sqrt(ms + (double) eps);
        for (size_t i = 0; i < len; i++) out[g0 + i] = (float) ((double) x[g0 + i] * r) * w[g0 + i];
    }
}

int orc_hc_read(const float* r, size_t h, size_t cs, size_t rank, float eps, const float* norm_w, const orc_tensor* down,
                const orc_tensor* up, const orc_tensor* inject, float* u, float* g, int threads) {         // forward.rs:797-817
    const size_t ch = h * cs;
    std::vector<float> rn(ch), dn(rank), mix(ch);
    orc_rmsnorm_groups(r, norm_w, ch, h, eps, rn.data());
    if (int e = orc_backend_matvec(down, rn.data(), dn.data(), threads)) return e;
    for (size_t i = 0; i < rank; i++) dn[i] = orc_silu(dn[i] / (float) cs);
    if (int e = orc_backend_matvec(up, dn.data(), mix.data(), threads)) return e;
    for (size_t i = 0; i < ch; i++) mix[i] = orc_sigmoid(mix[i]);
    for (size_t i = 0; i < h; i++) u[i] = 0.0f;
    for (size_t s = 0; s < cs; s++)
        for (size_t i = 0; i < h; i++) u[i] += mix[s * h + i] * rn[s * h + i];
    for (size_t i = 0; i < h; i++) u[i] /= (float) cs;
    if (inject && g) {
        std::vector<float> gi(cs);
        if (int e = orc_backend_matvec(inject, rn.data(), gi.data(), threads)) return e;
        for (size_t s = 0; s < cs; s++) g[s] = 2.0f * orc_sigmoid(gi[s] / (float) cs);
    }
    return 0;
}

void orc_hc_write(float* r, const float* g, const float* y, size_t h, size_t cs) {                           // forward.rs:1078-1084
    for (size_t s = 0; s < cs; s++)
        for (size_t i = 0; i < h; i++) r[s * h + i] += g[s] * y[i];
}

static void expert_tensors(const orc_expert_shape* s, const uint8_t* blob, orc_tensor* g, orc_tensor* u, orc_tensor* d) {
    *g = orc_tensor{s->gate_up_type, s->hidden, s->ff, blob, s->gate_bytes};
    *u = orc_tensor{s->gate_up_type, s->hidden, s->ff, blob + s->gate_bytes, s->up_bytes};
    *d = orc_tensor{s->down_type, s->ff, s->hidden, blob + s->gate_bytes + s->up_bytes, s->down_bytes};
}

static int expert_forward(const orc_expert_shape* s, const uint8_t* blob, const float* u, float* out, int threads) {
    orc_tensor tg, tu, td;
    expert_tensors(s, blob, &tg, &tu, &td);
    std::vector<float> g(s->ff), up(s->ff), act(s->ff);
    if (int r = orc_backend_matvec(&tg, u, g.data(), threads)) return r;
    if (int r = orc_backend_matvec(&tu, u, up.data(), threads)) return r;
    for (size_t i = 0; i < s->ff; i++) act[i] = orc_silu(g[i]) * up[i];                     // forward.rs:1020
    return orc_backend_matvec(&td, act.data(), out, threads);
}

int orc_moe_token(const orc_expert_shape* shape, const uint8_t* const* experts, int ne, int k, const float* logits,
                  const orc_expert_shape* shared_shape, const uint8_t* shared, float shared_gate_logit,
                  const float* u, float* y, uint32_t* route_idx, float* route_w, int threads) {   // forward.rs:1009-1034
    const size_t h = shape->hidden;
    std::vector<uint32_t> idx(k);
    std::vector<double> w(k);
    const int n = orc_route(logits, ne, k, idx.data(), w.data());
    for (int t = 0; t < n; t++) {
        if (route_idx) route_idx[t] = idx[t];
        if (route_w) route_w[t] = (float) w[t];
    }
    std::vector<double> acc(h, 0.0);
    std::vector<float> out(h);
    for (int t = 0; t < n; t++) {
        if (int r = expert_forward(shape, experts[idx[t]], u, out.data(), threads)) return r;
        for (size_t i = 0; i < h; i++) acc[i] += w[t] * (double) out[i];
    }
    if (shared) {
        if (int r = expert_forward(shared_shape, shared, u, out.data(), threads)) return r;
        const float sg = orc_sigmoid(shared_gate_logit);
        for (size_t i = 0; i < h; i++) y[i] = (float) (acc[i] + (double) (sg * out[i]));
    } else {
        for (size_t i = 0; i < h; i++) y[i] = (float) acc[i];
    }
    return 0;
}

// ------------------------------------------------------------------------------- cpu_expert*.rs: int8 activations
void orc_quantize_act(const float* x, size_t n, size_t blk, int8_t* q, float* d, int32_t* sums) {   // avx512.rs:25-42
    for (size_t b = 0; b < n / blk; b++) {
        const float* xb = x + b * blk;
        float amax = 0.0f;
        for (size_t i = 0; i < blk; i++) amax = std::max(amax, std::fabs(xb[i]));
        const float dd = amax / 127.0f;
        const float id = dd > 0.0f ? 1.0f / dd : 0.0f;
        int32_t s = 0;
        for (size_t i = 0; i < blk; i++) {
            float r = std::round(xb[i] * id);          // half away from zero, as f32::round
            r = std::min(127.0f, std::max(-127.0f, r));
            q[b * blk + i] = (int8_t) r;
            s += (int32_t) r;
        }
        d[b] = dd;
        if (sums) sums[b] = s;
    }
}

void orc_iq3s_int8(const uint8_t* b, int8_t* q, float* s) {                                  // cpu_expert.rs:99-110
    const float d = f16_at(b, 0);
    const uint8_t *qs = b + 2, *qh = b + 66, *signs = b + 74, *scales = b + 106;
    for (int e = 0; e < 256; e++) {
        const int j = e / 4;
        const unsigned idx = qs[j] | (((qh[j / 8] >> (j % 8)) & 1u) << 8);
        const int mag = (int) ((IQ3S_GRID[idx] >> (8 * (e % 4))) & 0xff);
        q[e] = (int8_t) (((signs[e / 8] >> (e % 8)) & 1) ? -mag : mag);
    }
    for (int g = 0; g < 8; g++) s[g] = d * (float) (1 + 2 * ((scales[g / 2] >> (4 * (g % 2))) & 0x0f));
}

float orc_iq3s_row_dot_q8(const uint8_t* row, size_t cols, const int8_t* q, const float* d, int32_t* isums) {
    float total = 0.0f;
    int8_t wq[256];
    float ws[8];
    for (size_t b = 0; b < cols / 256; b++) {
        orc_iq3s_int8(row + b * 110, wq, ws);
        for (int g = 0; g < 8; g++) {
            int32_t acc = 0;
            for (int i = 0; i < 32; i++) acc += (int32_t) wq[g * 32 + i] * (int32_t) q[b * 256 + g * 32 + i];
            if (isums) isums[b * 8 + g] = acc;
            total += (ws[g] * d[b * 8 + g]) * (float) acc;
        }
    }
    return total;
}

int orc_expert_int8(const uint8_t* expert, uint64_t hidden, uint64_t ff, const int8_t* x_q, const float* x_d, float* out,
                    float* act_out) {                                                       // cpu_expert.rs:243-339
    if (hidden % 256 || ff % 256) return 2;
    const size_t grow = hidden / 256 * 110, drow = ff / 256 * 110;
    const uint8_t *gate = expert, *up = expert + ff * grow, *down = expert + 2 * ff * grow;
    std::vector<float> act(ff);
    for (size_t r = 0; r < ff; r++) {
        const float g = orc_iq3s_row_dot_q8(gate + r * grow, hidden, x_q, x_d, nullptr);
        const float u = orc_iq3s_row_dot_q8(up + r * grow, hidden, x_q, x_d, nullptr);
        act[r] = (g / (1.0f + std::exp(-g))) * u;                                           // cpu_expert.rs:217
    }
    if (act_out) std::memcpy(act_out, act.data(), ff * 4);
    std::vector<int8_t> aq(ff);
    std::vector<float> ad(ff / 32);
    orc_quantize_act(act.data(), ff, 32, aq.data(), ad.data(), nullptr);
    for (size_t r = 0; r < hidden; r++) out[r] = orc_iq3s_row_dot_q8(down + r * drow, ff, aq.data(), ad.data(), nullptr);
    return 0;
}

// ---------------------------------------------------------------------------------- sampler.rs / engine.rs
uint32_t orc_argmax(const float* v, size_t n) {                                             // sampler.rs:99-107
    size_t best = 0;
    for (size_t i = 0; i < n; i++)
        if (v[i] > v[best]) best = i;
    return (uint32_t) best;
}

void orc_topk(const float* row, size_t n, int k, float* vals, uint32_t* ids) {
    std::vector<uint32_t> order(n);
    for (size_t i = 0; i < n; i++) order[i] = (uint32_t) i;
    auto val = [&](uint32_t i) { return std::isnan(row[i]) ? -INFINITY : row[i]; };
    const size_t kk = std::min<size_t>(k, n);
    std::partial_sort(order.begin(), order.begin() + kk, order.end(), [&](uint32_t a, uint32_t b) {
        const float va = val(a), vb = val(b);
        return va > vb || (va == vb && a < b);
    });
    for (size_t t = 0; t < kk; t++) {
        vals[t] = val(order[t]);
        ids[t] = order[t];
    }
}

// lookup_from, crates/shadowzero-serve/src/engine.rs:828-839: the match lengths longest first; the first that the history's tail
// matches at an earlier place (the most recent such place) gives the draft.  Returns the number of drafted tokens.
int orc_lookup_draft(const uint32_t* hist, size_t n_hist, int k, const uint32_t* lens, int n_lens, uint32_t* out) {
    for (int li = 0; li < n_lens; li++) {
        const size_t n = lens[li];
        if (k == 0 || n_hist <= n) break;
        bool found = false;
        size_t at = 0;
        for (size_t i = 0; i + n < n_hist; i++) {          // every earlier start; keep the last that matches
            bool same = true;
            for (size_t j = 0; j < n; j++) same = same && hist[i + j] == hist[n_hist - n + j];
            if (same) {
                found = true;
                at = i;
            }
        }
        if (found) {
            int c = 0;
            for (size_t j = at + n; j < n_hist && c < k; j++) out[c++] = hist[j];
            return c;
        }
    }
    return 0;
}

int orc_accept(const uint32_t* want, const uint32_t* drafts, int n_drafts) {                // engine.rs:2377-2408
    int keep = 1;
    for (int i = 0; i < n_drafts; i++) {
        if (want[i] != drafts[i]) break;
        keep++;
    }
    return keep;
}

// --------------------------------------------------------- the inexact 2-bit lm_head screen (kernels/exl3.cu:916-987,
// kernels/forward.cu:4371-4622).  The reference holds this path as CUDA kernels only (off in its exact mode,
// crates/shadowzero-cuda/src/session.rs:786); what follows restates those kernels' arithmetic operation by operation:
// the same f32 operations in the same order, fused where they call fmaf, the integer parts as integers.

// One 128-point transform without the 1 / sqrt(128) factor, stages h = 1 .. 64 (exl3.cu:21-30).
static void wht128_raw(float* v) {
    for (int h = 1; h < 128; h *= 2)
        for (int i = 0; i < 128; i += 2 * h)
            for (int j = i; j < i + h; j++) {
                const float a = v[j], b = v[j + h];
                v[j] = a + b;
                v[j + h] = a - b;
            }
}

// exl3_build_q2_proxy (exl3.cu:919-987): every 128 x 128 block (output block ob, input block b) of the matrix in the
// rotated basis, W_rot[i][c] = (row i of the decoded block, transformed over its 128 outputs) / 128 * svh[c], rounded to
// f16, is cut to the four levels {-3, -1, 1, 3} * sh with sh = f16(0.5 * 0.9957 * rms) of the output's 128 values of the
// block.  w_q2 holds 16-byte groups [(ob * 2 n_b + 2 b + hb) * 128 + r] of four words; code of input hb * 64 + wi * 16 +
// 4 sl + bi sits in word wi at bit 8 bi + 2 sl.  w_sc[(ob * n_b + b) * 128 + r] = sh.
int orc_q2_proxy_build(uint64_t ni, uint64_t no, int bits, const uint8_t* blob, uint64_t nbytes, uint32_t* w_q2, uint16_t* w_sc) {
    if (ni % 128 || no % 128 || nbytes != orc_exl3_blob_len(ni, no, bits, 0)) return 2;
    std::vector<float> w(ni * no);
    if (orc_exl3_reconstruct(ni, no, bits, 0, 2, blob, nbytes, 1, w.data())) return 2;
    const size_t n_b = ni / 128, n_ob = no / 128;
    std::vector<float> svh(no);
    for (size_t i = 0; i < no; i++) svh[i] = f16_at(blob, 2 * ni + 2 * i);
    parallel_chunks(n_ob, std::max<size_t>((n_ob + hw_threads() - 1) / hw_threads(), 1), [&](size_t first, size_t last) {
        std::vector<uint16_t> wh(128 * 128);   // [output][input]
        float row[128];
        for (size_t ob = first; ob < last; ob++)
            for (size_t b = 0; b < n_b; b++) {
                for (size_t i = 0; i < 128; i++) {
                    for (size_t c = 0; c < 128; c++) row[c] = w[(b * 128 + i) * no + ob * 128 + c];
                    wht128_raw(row);
                    for (size_t c = 0; c < 128; c++) wh[c * 128 + i] = orc_f32_to_f16(row[c] * 0.0078125f * svh[ob * 128 + c]);
                }
                for (size_t r = 0; r < 128; r++) {
                    float sq = 0.0f;
                    for (size_t c = 0; c < 128; c++) {
                        const float fv = orc_f16_to_f32(wh[r * 128 + c]);
                        sq = std::fmaf(fv, fv, sq);
                    }
                    const float delta = 0.9957f * std::sqrt(sq * 0.0078125f);
                    const uint16_t sh = orc_f32_to_f16(0.5f * delta);
                    const float thr = 2.0f * orc_f16_to_f32(sh);
                    w_sc[(ob * n_b + b) * 128 + r] = sh;
                    for (size_t hb = 0; hb < 2; hb++)
                        for (size_t wi = 0; wi < 4; wi++) {
                            uint32_t pw = 0;
                            for (size_t sl = 0; sl < 4; sl++)
                                for (size_t bi = 0; bi < 4; bi++) {
                                    const float fv = orc_f16_to_f32(wh[r * 128 + hb * 64 + wi * 16 + sl * 4 + bi]);
                                    const uint32_t q = fv >= 0.0f ? (fv >= thr ? 3u : 2u) : (fv <= -thr ? 0u : 1u);
                                    pw |= q << (bi * 8 + sl * 2);
                                }
                            w_q2[((ob * (n_b * 2) + b * 2 + hb) * 128 + r) * 4 + wi] = pw;
                        }
                }
            }
    });
    return 0;
}

// exl3_rotate_rows_f32 + proxy_q2_quant_x (exl3.cu:610-625, forward.cu:4376-4420) for one input row: (x * suh) transformed
// without the 1 / sqrt(128) factor, every 128-block to int8 codes with the scale amax / 127 (round half to even), four codes
// a word; x_corr = -3 * (sum of the block's codes) * scale.
void orc_q2_proxy_quant_x(const uint8_t* blob, const float* x, uint64_t ni, uint32_t* xq, float* x_sc, float* x_corr) {
    float v[128];
    for (size_t b = 0; b < ni / 128; b++) {
        for (size_t i = 0; i < 128; i++) v[i] = x[b * 128 + i] * f16_at(blob, 2 * (b * 128 + i));
        wht128_raw(v);
        float amax = 0.0f;
        for (size_t i = 0; i < 128; i++) amax = std::fmax(amax, std::fabs(v[i]));
        const float sc = amax > 0.0f ? amax / 127.0f : 0.0f;
        const float inv = sc > 0.0f ? 1.0f / sc : 0.0f;
        int tot = 0;
        for (size_t k = 0; k < 32; k++) {
            uint32_t p4 = 0;
            for (size_t e = 0; e < 4; e++) {
                const int q = (int) std::nearbyint(std::fmax(-127.0f, std::fmin(127.0f, v[4 * k + e] * inv)));
                tot += q;
                p4 |= (uint32_t) (uint8_t) (int8_t) q << (8 * e);
            }
            xq[b * 32 + k] = p4;
        }
        x_sc[b] = sc;
        x_corr[b] = -3.0f * (float) tot * sc;
    }
}

// proxy_q2_dp4a_bmax (forward.cu:4428-4497) for one input row: the score of output r is the sum over the input blocks, in
// order, of fma(sh, fma(2 x_sc, sum of code * u, x_corr), acc) with u = 0..3 the stored level (the level's value is
// 2 u - 3, which is what the correction term restores); bmax[ob] = the largest score of the block's 128 outputs.
void orc_q2_proxy_bmax(const uint32_t* w_q2, const uint16_t* w_sc, const uint32_t* xq, const float* x_sc, const float* x_corr,
                       uint64_t n_ob, uint64_t ni, float* bmax) {
    const size_t n_b = ni / 128;
    parallel_chunks(n_ob, std::max<size_t>((n_ob + hw_threads() - 1) / hw_threads(), 1), [&](size_t first, size_t last) {
        for (size_t ob = first; ob < last; ob++) {
            float best = 0.0f;
            for (size_t r = 0; r < 128; r++) {
                float acc = 0.0f;
                for (size_t b = 0; b < n_b; b++) {
                    int ia = 0;
                    for (size_t hb = 0; hb < 2; hb++)
                        for (size_t wi = 0; wi < 4; wi++) {
                            const uint32_t word = w_q2[((ob * (n_b * 2) + b * 2 + hb) * 128 + r) * 4 + wi];
                            for (size_t sl = 0; sl < 4; sl++) {
                                const uint32_t xw = xq[b * 32 + hb * 16 + wi * 4 + sl];
                                for (size_t bi = 0; bi < 4; bi++)
                                    ia += (int) (int8_t) (xw >> (8 * bi)) * (int) ((word >> (8 * bi + 2 * sl)) & 3u);
                            }
                        }
                    const float wsc = orc_f16_to_f32(w_sc[(ob * n_b + b) * 128 + r]);
                    acc = std::fmaf(wsc, std::fmaf(2.0f * x_sc[b], (float) ia, x_corr[b]), acc);
                }
                best = r == 0 ? acc : std::fmax(best, acc);
            }
            bmax[ob] = best;
        }
    });
}

// proxy_pick_rows + proxy_compact_seen (forward.cu:4519-4622): for each of the m rows of bmax[m][n_ob], the blocks i = t,
// t + 256, .. of each t < 256 give their four best (strictly larger replaces the fourth, equal values keep the earlier
// block; NaN counts as -3e38), the 1024 candidates are ordered by value descending then block ascending, and the first
// k_blk that are blocks are marked.  The union of the rows' marks, ascending, goes to sel[1 ..]; sel[0] = their number, at
// most max_sel.  Returns the number of marked blocks.
uint32_t orc_q2_proxy_pick(const float* bmax, uint32_t m, uint32_t n_ob, uint32_t k_blk, uint32_t max_sel, uint32_t* sel) {
    std::vector<uint8_t> seen(n_ob, 0);
    for (uint32_t row = 0; row < m; row++) {
        std::vector<std::pair<float, uint32_t>> cand;
        for (uint32_t t = 0; t < 256; t++) {
            float lv[4] = {-3.0e38f, -3.0e38f, -3.0e38f, -3.0e38f};
            uint32_t li[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
            for (uint32_t i = t; i < n_ob; i += 256) {
                float v = bmax[(size_t) row * n_ob + i];
                if (v != v) v = -3.0e38f;
                if (v > lv[3]) {
                    lv[3] = v;
                    li[3] = i;
                    for (int k = 3; k > 0; k--)
                        if (lv[k] > lv[k - 1] || (lv[k] == lv[k - 1] && li[k] < li[k - 1])) {
                            std::swap(lv[k], lv[k - 1]);
                            std::swap(li[k], li[k - 1]);
                        }
                }
            }
            for (int k = 0; k < 4; k++) cand.push_back({lv[k], li[k]});
        }
        std::sort(cand.begin(), cand.end(), [](const std::pair<float, uint32_t>& a, const std::pair<float, uint32_t>& b) {
            return a.first > b.first || (a.first == b.first && a.second < b.second);
        });
        for (uint32_t t = 0; t < k_blk && t < n_ob && t < cand.size(); t++)
            if (cand[t].second < n_ob) seen[cand[t].second] = 1;
    }
    uint32_t n = 0;
    for (uint32_t ob = 0; ob < n_ob; ob++)
        if (seen[ob]) {
            if (n < max_sel) sel[1 + n] = ob;
            n++;
        }
    sel[0] = n < max_sel ? n : max_sel;
    return n;
}

}   // extern "C"

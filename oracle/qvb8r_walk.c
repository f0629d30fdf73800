/* CPU restatement of the QVB8R tile walk and of its inverse.  TEST INFRASTRUCTURE: only tests, the smoke check and the
 * CPU-baseline leg of the benchmark may load this; the product never does.
 *
 * qvb8r_walk follows the decoder of the reference, src/qv_band/formats/qvb8r/backends/cuda_qvb8r/qvb8r_cpu.cpp:35-47
 * (the same order as the GPU walk, qvb8r_cuda.cu:51-75): per tile 32 lanes, lane j holds a 64-bit state; per pair of
 * steps every lane decodes two symbols (slot = x & 4095, entry E = tab[slot]: symbol = E & 2047, offset d =
 * (E >> 11) & 2047, frequency f = (E >> 22) + 1; x' = f * (x >> 12) + d), then the lanes whose state fell below 2^32 take
 * the next 32-bit word of the tile's stream in lane order.  Step s covers columns 32 s .. 32 s + 31, lane j = column j.
 *
 * qvb8r_encode_tile follows the encoder, qvb8r_cpu.cpp:76-96 (pairs walked backwards, lanes 31 .. 0, a word emitted
 * BEFORE the pair when x >= (f1 * f2) << 40, the buffer reversed at the end).
 *
 * Pinned by: round trip encode -> walk on random symbols, a single-lane closed-form rANS check in the tests, equality of
 * this encoder's words / states with the reference's own compiled encoder (oracle/_ref, where that builds), and the
 * reference's compiled row decoder reading this encoder's streams. */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* Decodes all rows of tiles [0, nt) into out_sym[(first row + r) * P + column].  Returns 0, or -(tile + 1) when a tile
 * reads past its stream (tile_off[tile + 1]) or past n_words. */
int64_t qvb8r_walk(const uint32_t* words, int64_t n_words, const int64_t* tile_off, const uint64_t* states,
                   const int64_t* tiles, int64_t nt, const uint32_t* tab, int64_t P, int16_t* out_sym) {
    const int64_t S = P / 32;
    for (int64_t t = 0; t < nt; ++t) {
        const uint32_t* tb = tab + tiles[3 * t] * 4096;
        const int64_t r0 = tiles[3 * t + 1], nr = tiles[3 * t + 2];
        uint64_t x[32];
        for (int j = 0; j < 32; ++j) x[j] = states[t * 32 + j];
        int64_t ptr = tile_off[t];
        for (int64_t rr = 0; rr < nr; ++rr) {
            int16_t* y = out_sym + (r0 + rr) * P;
            for (int64_t s0 = 0; s0 < S; s0 += 2) {
                for (int j = 0; j < 32; ++j) {
                    for (int h = 0; h < 2; ++h) {
                        const uint32_t E = tb[x[j] & 4095u], s = E & 2047u;
                        x[j] = (uint64_t)((E >> 22) + 1u) * (x[j] >> 12) + ((E >> 11) & 2047u);
                        y[(s0 + h) * 32 + j] = (int16_t)s;
                    }
                    if (x[j] < (1ull << 32)) {
                        if (ptr >= tile_off[t + 1] || ptr >= n_words) return -(t + 1);
                        x[j] = (x[j] << 32) | words[ptr++];
                    }
                }
            }
        }
        if (ptr != tile_off[t + 1]) return -(t + 1);          /* a conforming stream is consumed exactly */
    }
    return 0;
}

/* Encodes one tile: sym = first row of the tile (nr rows of P int16 symbols), f / c = the class's frequencies and
 * exclusive cumulative sums (N entries).  Writes at most cap words to out_words (stream order) and 32 final states.
 * Returns the number of words, or -1 when cap is too small or a symbol has zero frequency. */
int64_t qvb8r_encode_tile(const int16_t* sym, int64_t nr, int64_t P, const int64_t* f, const int64_t* c,
                          uint32_t* out_words, int64_t cap, uint64_t* out_states) {
    const int64_t S = P / 32;
    uint64_t x[32];
    for (int l = 0; l < 32; ++l) x[l] = 1ull << 32;
    int64_t n = 0;
    for (int64_t p = nr * S / 2 - 1; p >= 0; --p) {
        const int64_t a = 2 * p, b = a + 1;
        const int16_t* s1p = sym + (a / S) * P + (a % S) * 32;
        const int16_t* s2p = sym + (b / S) * P + (b % S) * 32;
        for (int l = 31; l >= 0; --l) {
            const uint64_t f1 = (uint64_t)f[s1p[l]], c1 = (uint64_t)c[s1p[l]], f2 = (uint64_t)f[s2p[l]], c2 = (uint64_t)c[s2p[l]];
            if (f1 == 0 || f2 == 0) return -1;
            uint64_t v = x[l];
            if (v >= ((f1 * f2) << 40)) {
                if (n >= cap) return -1;
                out_words[n++] = (uint32_t)v;
                v >>= 32;
            }
            v = ((v / f2) << 12) + v % f2 + c2;
            v = ((v / f1) << 12) + v % f1 + c1;
            x[l] = v;
        }
    }
    for (int64_t i = 0; i < n / 2; ++i) { const uint32_t tmp = out_words[i]; out_words[i] = out_words[n - 1 - i]; out_words[n - 1 - i] = tmp; }
    for (int l = 0; l < 32; ++l) out_states[l] = x[l];
    return n;
}

// Host entropy codec for packed ternary tensors: a static three-symbol range coder with a 16-bit
// probability table and bytewise renormalisation, wrapped in a 26-byte big-endian container.
// Byte-compatible with the reference's compress_ternary / decompress_ternary
// (tmq/tmq_native.cpp:50-140, tmq/rangecoder.h:41-193, tmq/bitstream.h:31-177). Runs on the
// host by design; no GPU is involved.
//
// Container: [u64 symbols][u64 payload bits][u32 total bytes][3 x u16 probabilities] payload,
// where the payload carries one trailing zero byte that is counted in `total bytes` but not in
// `payload bits`. Symbol order is (-1, 0, +1).
#include <cstdint>
#include <cstring>
#include <vector>

#include "tmq_hip.h"

namespace {

constexpr size_t kHeader = 8 + 8 + 4 + 6;

struct Model {
    uint16_t pmf[3];
    uint32_t cum[3];
    uint32_t total;
    void finish() {
        cum[0] = 0;
        cum[1] = pmf[0];
        cum[2] = cum[1] + pmf[1];
        total = cum[2] + pmf[2];
    }
};

// The carry-less range coder state; `settle` tells whether another byte must move.
struct RangeState {
    uint32_t low = 0;
    uint32_t range = 0xFFFFFFFFu;
    void narrow(const Model &m, int sym) {
        range /= m.total;
        low += m.cum[sym] * range;
        range *= m.pmf[sym];
    }
    bool settle() {
        if (((low ^ (low + range)) >> 24) == 0) return true;   // top byte decided
        if (range < 0x10000u) {                                // underflow: cut to the next 64 Ki boundary
            range = (0u - low) & 0xFFFFu;
            return true;
        }
        return false;
    }
    void shift() {
        range <<= 8;
        low <<= 8;
    }
};

inline int lanes_in_word(int64_t columns, int64_t qc) {
    const int64_t left = columns - qc * 16;
    return left < 16 ? (int)left : 16;
}

template <typename T>
void store_be(uint8_t *p, T v) {
    for (size_t i = 0; i < sizeof(T); i++) p[i] = (uint8_t)(v >> (8 * (sizeof(T) - 1 - i)));
}
template <typename T>
T load_be(const uint8_t *p) {
    T v = 0;
    for (size_t i = 0; i < sizeof(T); i++) v = (T)((v << 8) | p[i]);
    return v;
}

constexpr uint8_t kSymOfCode[4] = {1, 2, 0, 3};   // code 00 (0) -> 1, 01 (+1) -> 2, 10 (-1) -> 0
constexpr uint8_t kCodeOfSym[3] = {2, 0, 1};

}  // namespace

extern "C" {

size_t tmq_compress_bound(int64_t rows, int64_t columns) {
    if (rows < 0 || columns < 0) return 0;
    // log2(65535/1) = 16 bits per symbol at worst for a symbol of minimal probability, plus flush.
    return kHeader + (size_t)rows * (size_t)columns * 2 + 16;
}

int tmq_compress_ternary(const uint32_t *words, int64_t rows, int64_t columns, uint8_t *out, size_t out_cap,
                         size_t *out_size) {
    if (!words || !out || !out_size || rows <= 0 || columns <= 0) return TMQ_ERR_INVALID_ARG;
    const int64_t qcols = (columns + 15) / 16;
    int64_t histo[4] = {0, 0, 0, 0};
    for (int64_t r = 0; r < rows; r++)
        for (int64_t qc = 0; qc < qcols; qc++) {
            const uint32_t w = words[r * qcols + qc];
            for (int i = 0, n = lanes_in_word(columns, qc); i < n; i++) histo[kSymOfCode[(w >> (30 - 2 * i)) & 3u]]++;
        }
    if (histo[3] != 0) return TMQ_ERR_BAD_DATA;   // code 11 is not a ternary value
    const int64_t total = histo[0] + histo[1] + histo[2];
    const float scale = 65535.f / (float)total;
    Model m;
    for (int i = 0; i < 3; i++) {
        m.pmf[i] = (uint16_t)((float)histo[i] * scale);
        // A symbol that occurs but rounds to probability 0 cannot be coded (the reference coder
        // would never terminate on it); report it instead.
        if (histo[i] > 0 && m.pmf[i] == 0) return TMQ_ERR_UNSUPPORTED;
    }
    m.finish();

    std::vector<uint8_t> payload;
    payload.reserve((size_t)(total / 4) + 64);
    RangeState st;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t qc = 0; qc < qcols; qc++) {
            const uint32_t w = words[r * qcols + qc];
            for (int i = 0, n = lanes_in_word(columns, qc); i < n; i++) {
                st.narrow(m, kSymOfCode[(w >> (30 - 2 * i)) & 3u]);
                while (st.settle()) {
                    payload.push_back((uint8_t)(st.low >> 24));
                    st.shift();
                }
            }
        }
    for (int i = 0; i < 4; i++) {
        payload.push_back((uint8_t)(st.low >> 24));
        st.low <<= 8;
    }
    const uint64_t bits = (uint64_t)payload.size() * 8u;
    payload.push_back(0);   // the stream object of the reference always ends in a spare zero byte
    const size_t total_size = kHeader + payload.size();
    if (total_size > 0xFFFFFFFFull) return TMQ_ERR_TOO_LARGE;
    *out_size = total_size;
    if (total_size > out_cap) return TMQ_ERR_INVALID_ARG;
    store_be<uint64_t>(out, (uint64_t)(rows * columns));
    store_be<uint64_t>(out + 8, bits);
    store_be<uint32_t>(out + 16, (uint32_t)total_size);
    for (int i = 0; i < 3; i++) store_be<uint16_t>(out + 20 + 2 * i, m.pmf[i]);
    std::memcpy(out + kHeader, payload.data(), payload.size());
    return TMQ_OK;
}

int tmq_decompress_ternary(const uint8_t *in, size_t in_size, uint32_t *words, int64_t rows, int64_t columns) {
    if (!in || !words || rows <= 0 || columns <= 0) return TMQ_ERR_INVALID_ARG;
    if (in_size < kHeader) return TMQ_ERR_BAD_DATA;
    const uint64_t symbols = load_be<uint64_t>(in);
    if (symbols == 0) return TMQ_ERR_BAD_DATA;
    if (symbols != (uint64_t)rows * (uint64_t)columns) return TMQ_ERR_BAD_DATA;
    const uint64_t bits = load_be<uint64_t>(in + 8);
    const uint32_t total_size = load_be<uint32_t>(in + 16);
    if (total_size < kHeader) return TMQ_ERR_BAD_DATA;
    Model m;
    for (int i = 0; i < 3; i++) m.pmf[i] = load_be<uint16_t>(in + 20 + 2 * i);
    m.finish();
    if (m.total == 0) return TMQ_ERR_BAD_DATA;
    const uint8_t *pay = in + kHeader;
    const size_t nbytes = (size_t)((bits + 7) / 8);
    if (nbytes > in_size - kHeader) return TMQ_ERR_BAD_DATA;
    size_t pos = 0;
    auto next = [&]() -> uint32_t { return pos < nbytes ? pay[pos++] : 0u; };   // reads past the end give zeros

    RangeState st;
    uint32_t window = 0;
    for (int i = 0; i < 4; i++) window = (window << 8) | next();
    const int64_t qcols = (columns + 15) / 16;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t qc = 0; qc < qcols; qc++) {
            uint32_t w = 0;
            const int n = lanes_in_word(columns, qc);
            for (int i = 0; i < n; i++) {
                const uint32_t step = st.range / m.total;
                if (step == 0) return TMQ_ERR_BAD_DATA;
                const uint32_t freq = (window - st.low) / step;
                // Largest symbol whose cumulative count does not exceed freq; symbols of zero
                // probability are skipped because their interval is empty.
                int sym = 0;
                if (m.cum[1] <= freq) sym = (m.cum[2] <= freq) ? 2 : 1;
                if (m.pmf[sym] == 0) return TMQ_ERR_BAD_DATA;
                st.narrow(m, sym);
                while (st.settle()) {
                    window = (window << 8) | next();
                    st.shift();
                }
                w = (w << 2) | kCodeOfSym[sym];
            }
            if (n != 16) w <<= 2 * (16 - n);
            words[r * qcols + qc] = w;
        }
    return TMQ_OK;
}

}  // extern "C"

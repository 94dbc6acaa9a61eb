// Lyndon words and the Lyndon (standard-bracketing) basis of the free Lie algebra, prepared on the host for the
// compressed log-signature coordinates (siglib/shared/preparation/log_sig/lyndon_words.cpp,
// siglib/cpsig/cp_tensor_log.h:140-170):
//   method 1: the expanded log signature read off at the Lyndon words;
//   method 2: beta = M^-1 x, x the Lyndon-word coefficients, M[i][j] = coefficient of Lyndon word i in the bracket
//             P_j = [P_u, P_v] (j = uv, v the longest proper Lyndon suffix).  P_j is j plus lexicographically larger
//             words of the same letters, so M is unit lower triangular in the enumeration order (lengths ascending,
//             lexicographic inside a length) and integer; so is its inverse, which is what the device applies.
#pragma once
#include <cstdint>
#include <map>
#include <stdexcept>
#include <unordered_map>
#include <vector>

namespace sigamd {

struct LyndonTables {
    uint64_t dimension = 0, degree = 0;
    int method = 0;                          // 1: word positions only; 2: with the inverse projection
    std::vector<uint64_t> index;             // position of every Lyndon word in a scalar-free signature row
    // strictly lower part of M^-1 (unit diagonal implicit), CSR over rows, and of its transpose
    std::vector<uint64_t> row_ptr, t_row_ptr;
    std::vector<uint32_t> col, t_col;
    std::vector<int32_t> val, t_val;
};

namespace lyndon_detail {

using Word = std::vector<uint32_t>;

inline bool is_lyndon(const Word& w, size_t from)        // is the suffix w[from:] a Lyndon word?
{
    const size_t n = w.size() - from;
    for (size_t i = 1; i < n; ++i) {
        // strictly smaller than every proper suffix of itself
        bool less = false, decided = false;
        for (size_t a = 0; a + i < n; ++a) {
            if (w[from + a] != w[from + i + a]) {
                less = w[from + a] < w[from + i + a];
                decided = true;
                break;
            }
        }
        if (!decided) less = false;     // the suffix is a prefix of the word: the (shorter) suffix is smaller
        if (!less) return false;
    }
    return true;
}

// Duval's successor rule, one length at a time
template <typename F>
void for_each_lyndon_word(uint64_t n, uint64_t d, F&& f)
{
    Word w{0};
    while (!w.empty()) {
        const size_t m = w.size();
        if (m == n) f(w);
        while (w.size() < n) w.push_back(w[w.size() - m]);
        while (!w.empty() && w.back() == d - 1) w.pop_back();
        if (!w.empty()) ++w.back();
    }
}

// index of a word among ALL words (the empty word is 0): idx(w a) = idx(w) * d + a + 1
inline uint64_t flat_index(const Word& w, uint64_t d)
{
    uint64_t idx = 0;
    for (uint32_t a : w) {
        if (idx > (UINT64_MAX - a - 1) / d) throw std::overflow_error("Lyndon word index overflows 64 bits");
        idx = idx * d + a + 1;
    }
    return idx;
}

}  // namespace lyndon_detail

inline LyndonTables build_lyndon_tables(uint64_t d, uint64_t degree, int method)
{
    using namespace lyndon_detail;
    if (d == 0) throw std::invalid_argument("prepare_log_sig_cuda received dimension 0");
    LyndonTables t;
    t.dimension = d;
    t.degree = degree;
    t.method = method;
    std::vector<Word> words;
    for (uint64_t n = 1; n <= degree; ++n)
        for_each_lyndon_word(n, d, [&](const Word& w) {
            words.push_back(w);
            if (words.size() > (uint64_t(1) << 26)) throw std::runtime_error("prepare_log_sig_cuda: too many Lyndon words");
        });
    const size_t m = words.size();
    t.index.resize(m);
    std::vector<uint64_t> flat(m);
    for (size_t i = 0; i < m; ++i) {
        flat[i] = flat_index(words[i], d);
        t.index[i] = flat[i] - 1;            // scalar-free rows drop the empty word
    }
    t.row_ptr.assign(m + 1, 0);
    t.t_row_ptr.assign(m + 1, 0);
    if (method < 2) return t;

    std::unordered_map<uint64_t, uint32_t> pos;
    pos.reserve(m * 2);
    for (size_t i = 0; i < m; ++i) pos[flat[i]] = uint32_t(i);
    std::vector<uint64_t> pw(degree + 1, 1);         // d^k, saturating
    for (uint64_t k = 1; k <= degree; ++k) pw[k] = pw[k - 1] > UINT64_MAX / d ? UINT64_MAX : pw[k - 1] * d;

    // bracket polynomials over all words, keyed by flat index
    std::vector<std::map<uint64_t, int64_t>> poly(m);
    std::vector<std::vector<std::pair<uint32_t, int64_t>>> m_rows(m);       // strictly lower part of M, by row
    for (size_t j = 0; j < m; ++j) {
        const Word& w = words[j];
        if (w.size() == 1) {
            poly[j][flat[j]] = 1;
            continue;
        }
        size_t split = 1;
        while (!is_lyndon(w, split)) ++split;        // longest proper Lyndon suffix = smallest such start
        const Word u(w.begin(), w.begin() + split), v(w.begin() + split, w.end());
        const auto& pu = poly[pos.at(flat_index(u, d))];
        const auto& pv = poly[pos.at(flat_index(v, d))];
        const uint64_t len_u = u.size(), len_v = v.size();
        // offsets: flat(xy) = flat(x) * d^|y| + flat(y)
        auto& acc = poly[j];
        for (const auto& eu : pu)
            for (const auto& ev : pv) {
                const int64_t c = eu.second * ev.second;
                acc[eu.first * pw[len_v] + ev.first] += c;
                acc[ev.first * pw[len_u] + eu.first] -= c;
            }
        for (auto it = acc.begin(); it != acc.end();) it = it->second == 0 ? acc.erase(it) : std::next(it);
        for (const auto& e : acc) {
            auto hit = pos.find(e.first);
            if (hit == pos.end() || hit->second == j) continue;
            if (hit->second < j) throw std::logic_error("Lyndon projection is not lower triangular");
            m_rows[hit->second].push_back({uint32_t(j), e.second});
        }
    }
    poly.clear();
    // X = M^-1 row by row: X_i = e_i - sum_{j < i} M[i][j] X_j (strictly lower parts kept)
    std::vector<std::map<uint32_t, int64_t>> inv(m);
    uint64_t nnz = 0;
    for (size_t i = 0; i < m; ++i) {
        auto& row = inv[i];
        for (const auto& e : m_rows[i]) {
            row[e.first] -= e.second;
            for (const auto& x : inv[e.first]) row[x.first] -= e.second * x.second;
        }
        for (auto it = row.begin(); it != row.end();) it = it->second == 0 ? row.erase(it) : std::next(it);
        nnz += row.size();
        if (nnz > (uint64_t(1) << 28)) throw std::runtime_error("prepare_log_sig_cuda: Lyndon basis projection too large");
    }
    t.col.reserve(nnz);
    t.val.reserve(nnz);
    std::vector<uint64_t> t_count(m, 0);
    for (size_t i = 0; i < m; ++i) {
        for (const auto& x : inv[i]) {
            if (x.second > INT32_MAX || x.second < INT32_MIN) throw std::overflow_error("Lyndon projection entry overflows");
            t.col.push_back(x.first);
            t.val.push_back(int32_t(x.second));
            ++t_count[x.first];
        }
        t.row_ptr[i + 1] = t.col.size();
    }
    for (size_t i = 0; i < m; ++i) t.t_row_ptr[i + 1] = t.t_row_ptr[i] + t_count[i];
    t.t_col.resize(nnz);
    t.t_val.resize(nnz);
    std::vector<uint64_t> fill(t.t_row_ptr.begin(), t.t_row_ptr.end() - 1);
    for (size_t i = 0; i < m; ++i)
        for (uint64_t k = t.row_ptr[i]; k < t.row_ptr[i + 1]; ++k) {
            const uint64_t dst = fill[t.col[k]]++;
            t.t_col[dst] = uint32_t(i);
            t.t_val[dst] = t.val[k];
        }
    return t;
}

}  // namespace sigamd

// Host-side analysis of an EinsumDense equation "lhs,kernel->rhs"
// (include/fdeep/layers/einsum_dense_layer.hpp:51-79, 125-168): which characters are summed,
// the extent of every character, and whether the contraction is a plain row-major GEMM.
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace fdx {

struct EinsumSpec {
    std::string lhs, ker, rhs, summed, bias_chars; // bias_chars: the bias axes in rhs order (:204-207)
    std::map<char, int64_t> size;

    // false with a message when the equation cannot be evaluated
    bool parse(const std::string& equation, const std::string& bias_axes, std::string& err)
    {
        const size_t comma = equation.find(','), arrow = equation.find("->");
        if (comma == std::string::npos || arrow == std::string::npos || arrow < comma) {
            err = "EinsumDense: equation must have the form lhs,kernel->rhs";
            return false;
        }
        lhs = equation.substr(0, comma);
        ker = equation.substr(comma + 1, arrow - comma - 1);
        rhs = equation.substr(arrow + 2);
        auto unique = [](const std::string& s) {
            for (size_t i = 0; i < s.size(); ++i)
                if (s.find(s[i], i + 1) != std::string::npos)
                    return false;
            return true;
        };
        if (!unique(lhs) || !unique(ker) || !unique(rhs)) {
            err = "EinsumDense: repeated characters inside one operand are not supported";
            return false;
        }
        if (rhs.size() < 2) {
            err = "EinsumDense output equation must have at least a batch char and one feature char.";
            return false;
        }
        summed.clear();
        for (char c : lhs) {
            const bool in_rhs = rhs.find(c) != std::string::npos, in_ker = ker.find(c) != std::string::npos;
            if (!in_rhs && in_ker)
                summed.push_back(c);
            else if (!in_rhs) { // the reference never assigns a position to such a character
                err = "EinsumDense: an input character that is neither summed nor in the output";
                return false;
            }
        }
        for (char c : ker)
            if (lhs.find(c) == std::string::npos && rhs.find(c) == std::string::npos) {
                err = "EinsumDense: a kernel character that is neither in the input nor in the output";
                return false;
            }
        bias_chars.clear();
        for (char c : rhs)
            if (bias_axes.find(c) != std::string::npos)
                bias_chars.push_back(c);
        if (rhs.size() > 6 || summed.size() > 4) {
            err = "EinsumDense: at most 6 output and 4 summed characters";
            return false;
        }
        return true;
    }

    // Extents: kernel characters from the trailing kernel dims, input characters from the trailing
    // input dims (missing leading ones are 1), output-only characters from full_output_shape
    // (one entry per rhs character, <= 0 when unknown).  einsum_dense_layer.hpp:125-168.
    bool derive_sizes(const std::vector<int64_t>& kernel_dims, const std::vector<int64_t>& in_dims,
        const std::vector<int64_t>& full_output_shape, std::string& err)
    {
        size.clear();
        if (ker.size() > kernel_dims.size()) {
            err = "EinsumDense: kernel chars exceed kernel dimensions.";
            return false;
        }
        const size_t ko = kernel_dims.size() - ker.size();
        for (size_t i = 0; i < ker.size(); ++i)
            size[ker[i]] = kernel_dims[ko + i];
        if (lhs.size() < in_dims.size()) {
            err = "EinsumDense: input rank exceeds lhs char count.";
            return false;
        }
        const size_t lead = lhs.size() - in_dims.size();
        for (size_t i = 0; i < lhs.size(); ++i) {
            const int64_t sz = i >= lead ? in_dims[i - lead] : 1;
            auto it = size.find(lhs[i]);
            if (it != size.end()) {
                if (it->second != sz) {
                    err = "EinsumDense: inconsistent char size in equation.";
                    return false;
                }
            } else
                size[lhs[i]] = sz;
        }
        for (size_t i = 0; i < rhs.size(); ++i)
            if (!size.count(rhs[i])) {
                const int64_t d = i < full_output_shape.size() ? full_output_shape[i] : -1;
                if (d <= 0) {
                    err = "EinsumDense: cannot infer size of output-only char.";
                    return false;
                }
                size[rhs[i]] = d;
            }
        return true;
    }

    int64_t volume_of(const std::string& chars) const
    {
        int64_t v = 1;
        for (char c : chars)
            v *= size.at(c);
        return v;
    }

    // row-major stride of character c inside an operand laid out as `chars` (0 when absent)
    int64_t stride_in(const std::string& chars, char c) const
    {
        const size_t p = chars.find(c);
        if (p == std::string::npos)
            return 0;
        int64_t s = 1;
        for (size_t i = p + 1; i < chars.size(); ++i)
            s *= size.at(chars[i]);
        return s;
    }

    // True when, with the first lhs / rhs character as the row-batch, the contraction is
    // out[rows][N] = in[rows][K] * kernel[K][N]: lhs = a M K, kernel = K N, rhs = a M N with the
    // character groups in the same order on both sides, and the bias (if any) only over N.
    bool gemm_form(std::string* n_chars = nullptr) const
    {
        if (summed.empty() || lhs.size() < summed.size() + 1)
            return false;
        const size_t m_len = lhs.size() - summed.size();
        if (lhs.substr(m_len) != summed || ker.substr(0, summed.size()) != summed)
            return false;
        const std::string m = lhs.substr(0, m_len), n = ker.substr(summed.size());
        if (n.empty() || rhs != m + n)
            return false;
        for (char c : m)
            if (ker.find(c) != std::string::npos)
                return false;
        for (char c : bias_chars)
            if (n.find(c) == std::string::npos)
                return false;
        if (n_chars)
            *n_chars = n;
        return true;
    }
};

} // namespace fdx

// TEST INFRASTRUCTURE ONLY — CPU restatement of crates/maidenx_cpu/src/nn/conv.rs.
// Metadata: 12 slots  B, C, H, W, kh, kw, oh, ow, pad_h, pad_w, stride_h, stride_w
// in the order the kernel READS them (conv.rs:20-34); the reference's caller fills slots
// 8-11 as stride_h, stride_w, pad_h, pad_w, which only agrees when stride == pad.
#include <algorithm>

#include "common.hpp"

using namespace orc;

namespace {

template <typename T> inline T zero_of() { return T(0); }
template <> inline bf16 zero_of<bf16>() { return bf16::from_f32(0.0f); }
template <> inline f16 zero_of<f16>() { return f16::from_f32(0.0f); }

struct CV { size_t B, C, H, W, kh, kw, oh, ow, ph, pw, sh, sw; };
inline CV parse(const size_t* m) { return CV{m[0], m[1], m[2], m[3], m[4], m[5], m[6], m[7], m[8], m[9], m[10], m[11]}; }

// conv2d_im2col (conv.rs:13-73): col[b][(c*kh+i)*kw+j][h_out*ow+w_out]
template <typename T>
void im2col(size_t num_els, const size_t* md, const T* input, T* col) {
    if (!md || !input || !col) return;
    CV p = parse(md);
    size_t ksz = p.kh * p.kw, osz = p.oh * p.ow, chunk = p.C * ksz * osz;
    size_t nchunks = chunk ? (num_els + chunk - 1) / chunk : 0;
    ORC_PAR_FOR
    for (size_t b = 0; b < nchunks; ++b) {
        T* cc = col + b * chunk;
        for (size_t c = 0; c < p.C; ++c)
            for (size_t i = 0; i < p.kh; ++i)
                for (size_t j = 0; j < p.kw; ++j) {
                    size_t in_off = b * p.C * p.H * p.W + c * p.H * p.W;
                    size_t col_off = (c * ksz + i * p.kw + j) * osz;
                    for (size_t ho = 0; ho < p.oh; ++ho) {
                        long hi = (long)ho * (long)p.sh - (long)p.ph + (long)i;
                        for (size_t wo = 0; wo < p.ow; ++wo) {
                            long wi = (long)wo * (long)p.sw - (long)p.pw + (long)j;
                            bool ok = hi >= 0 && hi < (long)p.H && wi >= 0 && wi < (long)p.W;
                            cc[col_off + ho * p.ow + wo] = ok ? input[in_off + (size_t)hi * p.W + (size_t)wi] : zero_of<T>();
                        }
                    }
                }
    }
}

// conv2d_col2im (conv.rs:84-149): gather form, h_out then w_out ascending, indices at or
// beyond num_els skipped (:135).
template <typename T>
void col2im(size_t num_els, const size_t* md, const T* col, T* output) {
    if (!md || !col || !output) return;
    CV p = parse(md);
    if (p.sh == 0 || p.sw == 0) return;      // the reference panics here (usize division by zero, conv.rs:121-124)
    size_t chunk = p.C * p.H * p.W;
    ORC_PAR_FOR
    for (size_t b = 0; b < p.B; ++b) {
        T* oc = output + b * chunk;
        for (size_t c = 0; c < p.C; ++c)
            for (size_t h = 0; h < p.H; ++h) {
                size_t h_pad = h + p.ph;
                for (size_t w = 0; w < p.W; ++w) {
                    size_t w_pad = w + p.pw;
                    size_t hs = h_pad > p.kh - 1 ? h_pad - (p.kh - 1) : 0;   // saturating_sub
                    size_t ws = w_pad > p.kw - 1 ? w_pad - (p.kw - 1) : 0;
                    size_t h_start = (hs + p.sh - 1) / p.sh, w_start = (ws + p.sw - 1) / p.sw;   // div_ceil
                    size_t h_end = std::min(h_pad / p.sh + 1, p.oh), w_end = std::min(w_pad / p.sw + 1, p.ow);
                    T sum = zero_of<T>();
                    for (size_t ho = h_start; ho < h_end; ++ho)
                        for (size_t wo = w_start; wo < w_end; ++wo) {
                            size_t i = h_pad - ho * p.sh, j = w_pad - wo * p.sw;
                            if (i < p.kh && j < p.kw) {
                                size_t ci = (((b * p.C + c) * p.kh * p.kw + i * p.kw + j) * p.oh + ho) * p.ow + wo;
                                if (ci < num_els) sum += col[ci];
                            }
                        }
                    oc[(c * p.H + h) * p.W + w] = sum;
                }
            }
    }
}

}  // namespace

#define ORC_CONV_FOR(T, SUF)                                                                               \
    extern "C" void oracle_conv2d_im2col_##SUF(size_t num_els, const size_t* md, const T* in, T* col) {    \
        im2col<T>(num_els, md, in, col);                                                                   \
    }                                                                                                      \
    extern "C" void oracle_conv2d_col2im_##SUF(size_t num_els, const size_t* md, const T* col, T* out) {   \
        col2im<T>(num_els, md, col, out);                                                                  \
    }

ORC_CONV_FOR(float, f32)
ORC_CONV_FOR(double, f64)
ORC_CONV_FOR(bf16, bf16)
ORC_CONV_FOR(f16, f16)

// Host-side index tables of a TAGI convolution, in closed form.
//
// The reference derives the tables by sorting the receptive-field matrix
// (src/indices.cpp:267-464 and 514-696, driven by get_conv2d_idx,
// src/conv2d_layer.cpp:656-719). Their content has a direct description, which
// is what this file computes in O(wo*ho*k*k):
//
//   Fmwa_2[o][t]  1-based id of the input pixel under kernel tap t = ky*k + kx
//                 of output pixel o = oy*wo + ox, or -1 on padding;
//   for every input pixel p that occurs at all (w of them, ascending), the list
//   of its (o, t) occurrences in row-major order of Fmwa_2 (h = longest list):
//   FCzwa_1[c][j] tap id (1-based) of the j-th occurrence of the c-th pixel,
//                 param_pad_idx beyond the end of its list;      layout [w][h]
//   Szz_ud[j][c]  output-pixel id (1-based) of that occurrence, -1 beyond the
//                 end;                                            layout [h][w]
//
// pad_type 1 pads all four sides, pad_type 2 only right and bottom
// (src/indices.cpp:63-103).
#include <vector>

#include "tagi_internal.h"

namespace tagi {

int conv2d_out_size(int kernel, int stride, int wi, int hi, int pad, int pad_type, int *wo,
                    int *ho) {
    // A negative stride is what the pooling layers pass by default ("stride =
    // kernel"); the reference's formula then only works out for a window that
    // covers the whole image (nom = 0), which is how global pooling is written.
    if (kernel <= 0 || stride == 0 || wi <= 0 || hi <= 0 || pad < 0) return -1;
    const int extra = pad_type == 1 ? 2 * pad : pad_type == 2 ? pad : 0;
    const int nom_w = wi - kernel + extra, nom_h = hi - kernel + extra;
    if (nom_w < 0 || nom_h < 0 || nom_w % stride != 0 || nom_h % stride != 0) return -1;
    *wo = nom_w / stride + 1;
    *ho = nom_h / stride + 1;
    if (*wo < 1 || *ho < 1) return -1;
    return 0;
}

int conv2d_build_idx(int kernel, int stride, int wi, int hi, int pad, int pad_type,
                     int param_pad_idx, int *Fmwa_2, int *FCzwa_1, int *Szz_ud, int *w_out,
                     int *h_out) {
    int wo = 0, ho = 0;
    if (conv2d_out_size(kernel, stride, wi, hi, pad, pad_type, &wo, &ho) != 0) return -1;
    if (wi != hi) return -1;                             // square images only
    if (pad > 0 && pad_type != 1 && pad_type != 2) return -1;
    const int k2 = kernel * kernel;
    const int shift = (pad > 0 && pad_type == 1) ? pad : 0;
    const int npix = wi * hi;

    std::vector<int> count(npix, 0);
    for (int oy = 0; oy < ho; oy++)
        for (int ox = 0; ox < wo; ox++)
            for (int ky = 0; ky < kernel; ky++)
                for (int kx = 0; kx < kernel; kx++) {
                    const int iy = oy * stride + ky - shift, ix = ox * stride + kx - shift;
                    const bool inside = iy >= 0 && iy < hi && ix >= 0 && ix < wi;
                    const int o = oy * wo + ox, t = ky * kernel + kx;
                    Fmwa_2[(size_t)o * k2 + t] = inside ? iy * wi + ix + 1 : -1;
                    if (inside) count[iy * wi + ix]++;
                }

    // dense numbering of the pixels that occur, and the longest occurrence list
    std::vector<int> slot(npix, -1);
    int w = 0, h = 0;
    for (int p = 0; p < npix; p++)
        if (count[p] > 0) {
            slot[p] = w++;
            if (count[p] > h) h = count[p];
        }
    if (w == 0) return -1;

    for (size_t i = 0; i < (size_t)w * h; i++) {
        FCzwa_1[i] = param_pad_idx;
        Szz_ud[i] = -1;
    }
    std::vector<int> filled(w, 0);
    for (int o = 0; o < wo * ho; o++)
        for (int t = 0; t < k2; t++) {
            const int p = Fmwa_2[(size_t)o * k2 + t];
            if (p < 0) continue;
            const int c = slot[p - 1], j = filled[c]++;
            FCzwa_1[(size_t)c * h + j] = t + 1;
            Szz_ud[(size_t)j * w + c] = o + 1;
        }
    *w_out = w;
    *h_out = h;
    return 0;
}

// Pooling tables (reference: get_pool_index, src/pooling_layer.cpp:453-484, as
// AvgPool2d::lazy_index_init calls it): the receptive-field table transposed to
// [tap][output pixel], and -- only for overlapping windows -- the per-input-pixel
// list of output pixels [h][w].
int avgpool2d_build_idx(int kernel, int stride, int wi, int hi, int pad, int pad_type,
                        int *pool_idx, int *z_ud_idx, int *w_out, int *h_out, int *overlap) {
    int wo = 0, ho = 0;
    if (conv2d_out_size(kernel, stride, wi, hi, pad, pad_type, &wo, &ho) != 0) return -1;
    const int k2 = kernel * kernel;
    std::vector<int> fm((size_t)wo * ho * k2), zw((size_t)wi * hi * k2), zud((size_t)wi * hi * k2);
    int w = 0, h = 0;
    if (conv2d_build_idx(kernel, stride, wi, hi, pad, pad_type, k2 + 1, fm.data(), zw.data(),
                         zud.data(), &w, &h) != 0)
        return -1;
    for (int o = 0; o < wo * ho; o++)
        for (int t = 0; t < k2; t++) pool_idx[(size_t)t * wo * ho + o] = fm[(size_t)o * k2 + t];
    *overlap = !(kernel == stride || kernel == wi);
    if (*overlap) {
        for (int i = 0; i < w * h; i++) z_ud_idx[i] = zud[i];
        *w_out = w;
        *h_out = h;
    } else {
        *w_out = 0;
        *h_out = 0;
    }
    return 0;
}

}  // namespace tagi

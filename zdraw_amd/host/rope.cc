// Host-side rope tables and token positions that feed the fused attention
// entry: the counterparts of klein/zflux2_dit.zig:102-170 (Rope, buildRope,
// buildRopeRef), zimage/zrope.zig:29-106 (Cache.init/fill), zimage/zseq.zig:15-34
// (padLen, paddedLen, grid) and zimage/zstep_shape.zig:58-66 (imgStart, capGrid).
#include "zdraw_host.hpp"

#include <cmath>
#include <vector>

namespace zdraw {
namespace rope {

// Klein: ids (T, H, W, L) per token; four 32-wide axes, 16 frequencies each,
// evaluated in double and narrowed once; both columns of a pair get the value.
// cos_out / sin_out: [txt_len + grid_h*grid_w + ref_h*ref_w][128].
void kleinBuildRopeRef(float* cos_out, float* sin_out, size_t txt_len, size_t grid_h, size_t grid_w,
                       size_t ref_h, size_t ref_w, double theta) {
    double freq[16];
    for (int i = 0; i < 16; i++) freq[i] = 1.0 / std::pow(theta, (double)(2 * i) / 32.0);
    const size_t img = grid_h * grid_w;
    const size_t total = txt_len + img + ref_h * ref_w;
    for (size_t t = 0; t < total; t++) {
        double id[4] = {0.0, 0.0, 0.0, 0.0};
        if (t < txt_len) {
            id[3] = (double)t;
        } else if (t < txt_len + img) {
            const size_t p = t - txt_len;
            id[1] = (double)(p / grid_w);
            id[2] = (double)(p % grid_w);
        } else {
            const size_t p = t - txt_len - img;
            id[0] = 10.0;
            id[1] = (double)(p / ref_w);
            id[2] = (double)(p % ref_w);
        }
        float* c = cos_out + t * 128;
        float* s = sin_out + t * 128;
        for (int ax = 0; ax < 4; ax++) {
            for (int i = 0; i < 16; i++) {
                const double arg = id[ax] * freq[i];
                const float cv = (float)std::cos(arg);
                const float sv = (float)std::sin(arg);
                c[ax * 32 + 2 * i] = c[ax * 32 + 2 * i + 1] = cv;
                s[ax * 32 + 2 * i] = s[ax * 32 + 2 * i + 1] = sv;
            }
        }
    }
}

// Z-Image: per axis a table [len][dim/2] of (cos, sin), angle = pos * theta^(-2*pair/dim)
// computed in fp32 as exp(-ln(theta) * (2*pair/dim)). Returns false for a
// config the reference rejects (zrope.zig:82-87).
bool zimageFill(float* values, const size_t dims[3], const size_t lens[3], float theta) {
    if (!(theta > 0.0f)) return false;
    for (int a = 0; a < 3; a++)
        if (dims[a] == 0 || lens[a] == 0 || dims[a] % 2 != 0) return false;
    const float neg_ln = -std::log(theta);
    float* dst = values;
    for (int a = 0; a < 3; a++) {
        const size_t pairs = dims[a] / 2;
        std::vector<float> rate(pairs);
        for (size_t p = 0; p < pairs; p++) rate[p] = std::exp(neg_ln * (2.0f * (float)p / (float)dims[a]));
        for (size_t pos = 0; pos < lens[a]; pos++) {
            const float fpos = (float)pos;
            for (size_t p = 0; p < pairs; p++) {
                const float ang = fpos * rate[p];
                *dst++ = std::cos(ang);
                *dst++ = std::sin(ang);
            }
        }
    }
    return true;
}

size_t zseqPadLen(size_t len) { return (32 - len % 32) % 32; }
size_t zseqPaddedLen(size_t len) { return len + zseqPadLen(len); }

// Row-major (frame, row, column) positions from `start`.
bool zseqGrid(size_t* out, size_t out_len, const size_t size[3], const size_t start[3]) {
    if (out_len != size[0] * size[1] * size[2]) return false;
    size_t n = 0;
    for (size_t f = 0; f < size[0]; f++)
        for (size_t r = 0; r < size[1]; r++)
            for (size_t c = 0; c < size[2]; c++) {
                out[n++] = start[0] + f;
                out[n++] = start[1] + r;
                out[n++] = start[2] + c;
            }
    return true;
}

// The joint sequence of one Z-Image step: image tokens then caption tokens
// (zunify.zig:31-34). The image grid starts at (cap_total + 1, 0, 0) and its
// pad slots sit at the origin; the caption grid spans its padded length from
// (1, 0, 0). pos: [img_total + cap_total][3].
bool zimageSequencePositions(size_t* pos, size_t pos_len, size_t grid_h, size_t grid_w, size_t cap_tokens) {
    const size_t img_raw = grid_h * grid_w;
    const size_t img_total = zseqPaddedLen(img_raw);
    const size_t cap_total = zseqPaddedLen(cap_tokens);
    if (pos_len != img_total + cap_total || img_raw == 0 || cap_tokens == 0) return false;
    const size_t isz[3] = {1, grid_h, grid_w};
    const size_t ist[3] = {cap_total + 1, 0, 0};
    zseqGrid(pos, img_raw, isz, ist);
    for (size_t t = img_raw; t < img_total; t++) pos[3 * t] = pos[3 * t + 1] = pos[3 * t + 2] = 0;
    const size_t csz[3] = {cap_total, 1, 1};
    const size_t cst[3] = {1, 0, 0};
    zseqGrid(pos + 3 * img_total, cap_total, csz, cst);
    return true;
}

} // namespace rope
} // namespace zdraw

extern "C" {
void zh_klein_build_rope_ref(float* c, float* s, size_t txt_len, size_t gh, size_t gw, size_t rh, size_t rw,
                             double theta) {
    zdraw::rope::kleinBuildRopeRef(c, s, txt_len, gh, gw, rh, rw, theta);
}
int zh_zimage_rope_fill(float* values, const size_t* dims, const size_t* lens, float theta) {
    return zdraw::rope::zimageFill(values, dims, lens, theta) ? 0 : 2;
}
size_t zh_zseq_padded_len(size_t len) { return zdraw::rope::zseqPaddedLen(len); }
int zh_zseq_grid(size_t* out, size_t out_len, const size_t* size, const size_t* start) {
    return zdraw::rope::zseqGrid(out, out_len, size, start) ? 0 : 2;
}
int zh_zimage_sequence_positions(size_t* pos, size_t pos_len, size_t gh, size_t gw, size_t cap_tokens) {
    return zdraw::rope::zimageSequencePositions(pos, pos_len, gh, gw, cap_tokens) ? 0 : 2;
}
}

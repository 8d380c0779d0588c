// Host-only sanitizer run of the tile model and the weight packing (no GPU code involved).
#include <cstdio>
#include <random>
#include <vector>
#include "tdc_internal.hpp"
using namespace tdc;
int main() {
    std::mt19937 rng(1);
    long long tiles_checked = 0, packed = 0;
    const int shapes[][8] = {  // batch C N H W K stride pad
        {1, 128, 128, 56, 56, 3, 1, 1}, {1, 64, 64, 28, 28, 3, 1, 1}, {2, 13, 20, 9, 11, 3, 1, 1}, {1, 3, 64, 224, 224, 7, 2, 3},
        {1, 40, 24, 13, 13, 3, 2, 1},   {1, 512, 128, 28, 28, 1, 1, 0}, {1, 7, 5, 5, 7, 3, 1, 0},   {1, 96, 96, 14, 14, 3, 1, 1},
        {1, 16, 16, 7, 7, 3, 1, 1},     {3, 5, 7, 1, 300, 3, 1, 1},     {1, 2048, 256, 7, 7, 1, 1, 0}, {1, 32, 48, 6, 6, 5, 1, 2}};
    for (const auto &sh : shapes) {
        tdc_conv_desc d{sh[0], sh[1], sh[2], sh[3], sh[4], sh[5], sh[5], sh[6], sh[7], 1, 0, 0};
        std::vector<tdc_tile> tiles = model_enumerate(d, 0);
        std::vector<float> w((size_t)d.N * d.C * d.KH * d.KW);
        for (float &v : w) v = (float)(rng() % 17) - 8.0f;
        tdc_tile_info best{};
        std::string why;
        if (!model_select(d, best, &why, 0)) { std::printf("no tile: %s\n", why.c_str()); return 1; }
        const size_t step = tiles.size() / 400 + 1;
        for (size_t i = 0; i < tiles.size(); i += step) {
            tdc_tile_info info;
            Geometry g;
            if (!model_evaluate(d, tiles[i], info, &why, 0)) { std::printf("enumerated tile fails: %s\n", why.c_str()); return 1; }
            if (!make_geometry(d, tiles[i], g, &why, 0)) return 1;
            ++tiles_checked;
            if (i % (step * 8) == 0) {   // pack into an exactly sized buffer: any overrun is caught
                std::vector<float> buf(packed_weight_floats(g));
                pack_weights(d, tiles[i], g, w.data(), buf.data());
                ++packed;
            }
        }
        std::printf("shape C%d N%d %dx%d K%d s%d: %zu tiles, pick alg %d\n", d.C, d.N, d.H, d.W, d.KH, d.stride, tiles.size(), best.tile.alg);
    }
    std::printf("checked %lld tiles, packed %lld weight sets\n", tiles_checked, packed);
    return 0;
}

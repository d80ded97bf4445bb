// Runs the CPU oracle (test infrastructure) over small seeded frames under the address and
// undefined-behaviour sanitizers: `make -C oracle asan` builds this file together with
// fgs_oracle.cpp into _build/oracle_sanitize_check.  The frames include what the oracle must
// survive: Gaussians behind the camera, zero and huge covariances, NaN inputs, a key buffer that
// is too small, an image that is not a multiple of the tile, an empty scene.  Exit status 0 and
// "oracle sanitize check ok" on success; the sanitizers abort the run otherwise.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <limits>
#include <vector>

#include "fgs_oracle.h"

namespace {

uint64_t g_state = 0x9e3779b97f4a7c15ull;
double uniform()        // xorshift64*, [0, 1)
{
    g_state ^= g_state >> 12; g_state ^= g_state << 25; g_state ^= g_state >> 27;
    return (double)((g_state * 0x2545f4914f6cdd1dull) >> 11) / 9007199254740992.0;
}

int frame(int n, int W, int H, int bx, int by, int64_t capacity, bool poison)
{
    std::vector<float> pos(3 * (size_t)n + 1), shs(48 * (size_t)n + 1), op(n + 1), scale(3 * (size_t)n + 1), rot(4 * (size_t)n + 1),
        cov(6 * (size_t)n + 1);
    for (int i = 0; i < n; i++) {
        for (int k = 0; k < 3; k++) pos[3 * i + k] = (float)(uniform() * 10.0 - 5.0);
        for (int k = 0; k < 48; k++) shs[48 * i + k] = (float)(uniform() - 0.5);
        op[i] = (float)uniform();
        for (int k = 0; k < 3; k++) scale[3 * i + k] = (float)std::exp(-4.0 + 3.0 * uniform());
        float q[4], norm = 0.f;
        for (int k = 0; k < 4; k++) { q[k] = (float)(uniform() - 0.5); norm += q[k] * q[k]; }
        for (int k = 0; k < 4; k++) rot[4 * i + k] = q[k] / std::sqrt(norm);
    }
    fgs_oracle_cov3d(n, scale.data(), rot.data(), cov.data());
    if (poison && n >= 8) {
        const float nan = std::numeric_limits<float>::quiet_NaN(), inf = std::numeric_limits<float>::infinity();
        pos[0] = nan; op[1] = nan; cov[6 * 2] = nan; cov[6 * 3] = inf; cov[6 * 3 + 3] = inf; cov[6 * 3 + 5] = inf;
        for (int k = 0; k < 6; k++) cov[6 * 4 + k] = 0.f;
        pos[3 * 5 + 2] = -14.9f;                       // right in front of the camera: a screen-filling splat
        for (int k = 0; k < 6; k++) cov[6 * 5 + k] = (k == 0 || k == 3 || k == 5) ? 1e6f : 0.f;
        op[6] = 0.0f; op[7] = 1e-9f;
        shs[48 * 7] = inf;
    }
    const float cam_pos[3] = {0.f, 0.f, -15.f};
    const float cam_rot[9] = {1, 0, 0, 0, 1, 0, 0, 0, 1};
    const float f = (float)(H / (2.0 * std::tan(25.0 * 3.14159265358979 / 180.0)));
    std::vector<float> xy(2 * (size_t)n + 1, -1.f), rgbd(4 * (size_t)n + 1, -1.f), co(4 * (size_t)n + 1, -1.f);
    std::vector<uint64_t> keys((size_t)capacity + 1), ks((size_t)capacity + 1);
    std::vector<uint32_t> vals((size_t)capacity + 1), vs((size_t)capacity + 1);
    int offset = 0;
    int64_t counts[4] = {0, 0, 0, 0};
    const int rc = fgs_oracle_preprocess(n, pos.data(), shs.data(), op.data(), cov.data(), W, H, bx, by, cam_pos, cam_rot, f, f,
                                         100.f, 0.01f, xy.data(), rgbd.data(), co.data(), keys.data(), vals.data(), capacity,
                                         &offset, counts, 2);
    if (rc != 0) return rc;       // the key buffer was too small: nothing beyond it may have been written (the sanitizer watches)
    const int K = offset;
    fgs_oracle_sort(K, W, H, bx, by, keys.data(), vals.data(), ks.data(), vs.data(), 2);
    for (int i = 1; i < K; i++)
        if (ks[i - 1] > ks[i]) { std::fprintf(stderr, "sorted keys out of order at %d\n", i); std::exit(1); }
    const int tiles = ((W + bx - 1) / bx) * ((H + by - 1) / by);
    std::vector<int> ranges(2 * (size_t)tiles);
    fgs_oracle_ranges(K, ks.data(), ranges.data(), tiles);
    std::vector<uint8_t> u8(3 * (size_t)W * H);
    std::vector<float> f32(3 * (size_t)W * H);
    const float bg[3] = {0.1f, 0.2f, 0.3f};
    int64_t walked = 0;
    fgs_oracle_render(W, H, bx, by, xy.data(), rgbd.data(), co.data(), vs.data(), ranges.data(), bg, u8.data(), f32.data(), &walked, 2);
    return 0;
}

} // namespace

int main()
{
    int rc = 0;
    rc |= frame(3000, 200, 120, 16, 16, 1 << 18, false);
    rc |= frame(3000, 203, 117, 16, 16, 1 << 20, true);       // partial tiles, poisoned inputs
    rc |= frame(500, 130, 70, 32, 16, 1 << 18, true);
    rc |= frame(500, 130, 70, 32, 32, 1 << 18, true);
    rc |= frame(0, 64, 64, 16, 16, 16, false);                // empty scene
    if (rc != 0) { std::fprintf(stderr, "a frame that fits its key buffer reported an overflow\n"); return 1; }
    if (frame(3000, 200, 120, 16, 16, 100, false) == 0) {     // the key buffer is too small: reported, not overrun
        std::fprintf(stderr, "an overflowing frame was not reported\n");
        return 1;
    }
    float view[16], proj[16];
    const float pos[3] = {1.f, 2.f, 3.f}, rot[9] = {0, 1, 0, -1, 0, 0, 0, 0, 1};
    fgs_oracle_view_proj(pos, rot, 7680, 4320, 3000.f, 3000.f, 100.f, 0.01f, view, proj);
    int rmin[2], rmax[2];
    fgs_oracle_rect(-1e30f, 1e30f, 1 << 30, 1 << 30, 100, 100, 16, 16, rmin, rmax);   // float -> int saturation
    (void)fgs_oracle_higher_msb(0u); (void)fgs_oracle_higher_msb(0xffffffffu);
    (void)fgs_oracle_log2f(1e-38f); (void)fgs_oracle_log2f(3e38f);
    std::puts("oracle sanitize check ok");
    return 0;
}

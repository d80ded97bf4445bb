// Host-side self-check of libflashgs_hip, meant to be built with the address and
// undefined-behaviour sanitizers on the host code (`python -m flashgs_amd.build --asan-host`) and
// run on the CPU: it never launches a kernel and needs no GPU.
//
//  * ply_reader.h against the files an untrusted caller can hand to loadPly: headers that claim
//    more vertices than the file holds (nothing may be allocated for them), missing or malformed
//    headers, truncated data, plus a well-formed file whose rows are checked.
//  * every entry point of the C ABI with the arguments that must be refused before any HIP call:
//    the status is FGS_E_INVALID / FGS_E_WORKSPACE and fgs_last_error() says why.
//  * the host arithmetic: camera matrices, workspace sizes up to the largest count.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

#include "flashgs_hip.h"
#include "ply_reader.h"

namespace {

int g_failures = 0;

void expect(bool ok, const char* what)
{
    if (!ok) {
        std::fprintf(stderr, "host check failed: %s\n", what);
        g_failures++;
    }
}

std::string header(const std::string& vertex_line)
{
    return "ply\nformat binary_little_endian 1.0\n" + vertex_line + "property float x\nend_header\n";
}

// parses `bytes` as a .ply the way loadPly does; returns "" or the error text
std::string parse(const std::string& bytes, int* n_out, std::vector<float>* rows)
{
    std::istringstream file(bytes, std::ios::binary);
    try {
        const int n = fgs_ply::read_header(file, bytes.size());
        *n_out = n;
        std::vector<float> position(3 * (size_t)n), shs(48 * (size_t)n), opacity((size_t)n), cov3d(6 * (size_t)n);
        fgs_ply::read_records(file, n, position.data(), shs.data(), opacity.data(), cov3d.data());
        if (rows) {
            rows->clear();
            rows->insert(rows->end(), position.begin(), position.end());
            rows->insert(rows->end(), shs.begin(), shs.end());
            rows->insert(rows->end(), opacity.begin(), opacity.end());
            rows->insert(rows->end(), cov3d.begin(), cov3d.end());
        }
    } catch (const std::exception& e) {
        return e.what();
    }
    return "";
}

void check_ply()
{
    int n = -1;
    std::vector<float> rows;
    // two well-formed records
    std::vector<float> rec(2 * fgs_ply::kPlyFloats);
    for (size_t i = 0; i < rec.size(); i++) rec[i] = 0.01f * (float)i - 0.5f;
    for (int v = 0; v < 2; v++) { float* q = rec.data() + v * fgs_ply::kPlyFloats + 58; q[0] = 1.f; q[1] = q[2] = q[3] = 0.f; }
    std::string good = header("element vertex 2\n");
    good.append(reinterpret_cast<const char*>(rec.data()), rec.size() * sizeof(float));
    expect(parse(good, &n, &rows).empty() && n == 2, "a well-formed file parses");
    expect(rows.size() == 2 * (3 + 48 + 1 + 6), "all rows are returned");
    expect(rows[0] == rec[0] && rows[3] == rec[fgs_ply::kPlyFloats], "positions are the first three floats of a record");
    // identity rotation: Sigma = diag(exp(2 s))
    const float s0 = std::exp(rec[55]);
    expect(std::fabs(rows[2 * 3 + 2 * 48 + 2] - s0 * s0) <= 1e-6f * s0 * s0, "cov3d xx = exp(scale)^2 under the identity rotation");
    expect(rows[2 * 3 + 3] == rec[6 + 3] && rows[2 * 3 + 4] == rec[6 + 3 + 15], "rest coefficients are interleaved per channel");

    // the header claims what the file cannot hold: refused before anything is sized by it
    for (const char* claim : {"element vertex 3\n", "element vertex 2147483647\n", "element vertex 99999999999999\n"}) {
        std::string lie = header(claim);
        lie.append(reinterpret_cast<const char*>(rec.data()), rec.size() * sizeof(float));
        const std::string err = parse(lie, &n, nullptr);
        expect(err.find("exceeds") != std::string::npos || err.find("not positive") != std::string::npos, claim);
    }
    expect(parse(good.substr(0, good.size() - 5), &n, nullptr).find("exceeds") != std::string::npos, "a truncated last record is refused");
    expect(parse(header("element vertex 0\n"), &n, nullptr) == "Vertex number is not positive", "vertex 0");
    expect(parse(header("element vertex -4\n"), &n, nullptr) == "Vertex number is not positive", "negative vertex count");
    expect(parse(header("element vertex many\n"), &n, nullptr) == "Vertex number is not positive", "vertex count that is no number");
    expect(parse("ply\nelement vertex 2\n", &n, nullptr) == "Cannot find end of header", "no end_header");
    expect(parse("", &n, nullptr) == "Cannot find end of header", "empty file");
    expect(parse(std::string(4096, '\xff'), &n, nullptr) == "Cannot find end of header", "binary noise");
    expect(parse(header(""), &n, nullptr).empty() && n == 0, "a header without a vertex element yields no rows, as in the reference");
}

void check_arguments()
{
    const float pos[3] = {0, 0, 0}, rot[9] = {1, 0, 0, 0, 1, 0, 0, 0, 1}, bg[3] = {0, 0, 0};
    float* const f = reinterpret_cast<float*>(0x1000);              // never dereferenced: every call below is refused first
    uint64_t* const k = reinterpret_cast<uint64_t*>(0x1000);
    uint32_t* const v = reinterpret_cast<uint32_t*>(0x1000);
    int* const i32 = reinterpret_cast<int*>(0x1000);
    uint8_t* const u8 = reinterpret_cast<uint8_t*>(0x1000);
    char* const ws = reinterpret_cast<char*>(0x1000);
    auto refused = [&](int rc, const char* what) {
        expect(rc == FGS_E_INVALID && std::strlen(fgs_last_error()) > 0, what);
    };
    for (int is_static = 0; is_static < 2; is_static++) {
        auto pre = is_static ? fgs_preprocess_static : fgs_preprocess;
        refused(pre(-1, f, f, f, f, 64, 64, 16, 16, pos, rot, 1, 1, 100, 0.01f, f, f, f, k, v, i32, 16, nullptr), "negative P");
        refused(pre(10, f, f, f, f, 0, 64, 16, 16, pos, rot, 1, 1, 100, 0.01f, f, f, f, k, v, i32, 16, nullptr), "zero width");
        refused(pre(10, f, f, f, f, 64, 64, 0, 16, pos, rot, 1, 1, 100, 0.01f, f, f, f, k, v, i32, 16, nullptr), "zero block");
        refused(pre(10, f, f, f, f, 64, 64, 16, 16, nullptr, rot, 1, 1, 100, 0.01f, f, f, f, k, v, i32, 16, nullptr), "null camera");
        refused(pre(10, f, f, f, f, 64, 64, 16, 16, pos, rot, 1, 1, 100, 0.01f, f, f, f, k, v, nullptr, 16, nullptr), "null curr_offset");
        refused(pre(10, nullptr, f, f, f, 64, 64, 16, 16, pos, rot, 1, 1, 100, 0.01f, f, f, f, k, v, i32, 16, nullptr), "null positions");
        refused(pre(10, f, f + 1, f, f, 64, 64, 16, 16, pos, rot, 1, 1, 100, 0.01f, f, f, f, k, v, i32, 16, nullptr), "misaligned shs");
        refused(pre(2147483647, f, f, f, f, 64, 64, 16, 16, pos, rot, 1, 1, 100, 0.01f, f, f, f, k, v, i32, 16, nullptr), "P near INT_MAX");
        expect(pre(0, nullptr, nullptr, nullptr, nullptr, 64, 64, 16, 16, pos, rot, 1, 1, 100, 0.01f, nullptr, nullptr, nullptr,
                   nullptr, nullptr, i32, 0, nullptr) == FGS_OK, "an empty scene is fine and launches nothing");
    }
    refused(fgs_preprocess_static((1 << 24) + 1, f, f, f, f, 64, 64, 16, 16, pos, rot, 1, 1, 100, 0.01f, f, f, f, k, v, i32, 16, nullptr),
            "more Gaussians than the built-in scan status holds");

    refused(fgs_sort_gaussian(-1, 64, 64, 16, 16, ws, 1 << 20, k, v, k, v, nullptr), "negative pair count");
    refused(fgs_sort_gaussian(1 << 30, 64, 64, 16, 16, ws, (size_t)1 << 40, k, v, k, v, nullptr), "pair count beyond FGS_MAX_RENDERED");
    refused(fgs_sort_gaussian(100, 64, 0, 16, 16, ws, 1 << 20, k, v, k, v, nullptr), "zero height");
    refused(fgs_sort_gaussian(100, 64, 64, 16, 16, nullptr, 1 << 20, k, v, k, v, nullptr), "null workspace");
    refused(fgs_sort_gaussian(100, 64, 64, 16, 16, ws + 4, (size_t)1 << 30, k, v, k, v, nullptr), "misaligned workspace");
    expect(fgs_sort_gaussian(100000, 64, 64, 16, 16, ws, 1000, k, v, k, v, nullptr) == FGS_E_WORKSPACE, "workspace too small");
    expect(fgs_sort_gaussian(0, 64, 64, 16, 16, nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr) == FGS_OK, "no pairs: nothing to do");

    refused(fgs_render_16x16(-1, 64, 64, f, f, f, k, v, i32, bg, u8, nullptr), "negative pair count in render");
    refused(fgs_render_16x16(5, 64, 64, nullptr, f, f, k, v, i32, bg, u8, nullptr), "null attributes in render");
    refused(fgs_render_32x16(0, 64, 64, f, f, f, k, v, i32, bg, nullptr, nullptr), "null image");
    refused(fgs_render_32x32(0, 0, 64, f, f, f, k, v, i32, bg, u8, nullptr), "zero width in render");
    refused(fgs_render_f32(8, 8, 0, 64, 64, f, f, f, k, v, i32, bg, u8, nullptr, nullptr), "unsupported tile");
    refused(fgs_render_ex(16, 16, 0, 64, 64, f, f, f, k, v, i32, bg, u8, nullptr, 64, nullptr), "unknown flags");
    refused(fgs_render_ex(16, 16, 0, 64, 64, f, f, f, k, v, i32, bg, u8, nullptr, FGS_BLEND_FP32 | FGS_BLEND_MATRIX_F16, nullptr),
            "both colour-sum modes at once");
    refused(fgs_blend_ex(16, 16, 64, 64, f, f, f, v, i32, bg, nullptr, nullptr, 0, nullptr), "no output in blend");
    refused(fgs_blend(16, 16, 64, 64, f, f + 1, f, v, i32, bg, u8, nullptr, nullptr), "misaligned rgb_depth");
    refused(fgs_tile_ranges(16, 16, -3, 64, 64, k, i32, nullptr), "negative pair count in tile_ranges");
    refused(fgs_tile_ranges(16, 16, 3, 64, 64, nullptr, i32, nullptr), "null keys in tile_ranges");
    expect(fgs_set_colour_sums(9) == -1, "unknown colour-sum mode");
    expect(fgs_set_colour_sums(FGS_COLOUR_SUMS_FP32) == FGS_COLOUR_SUMS_FP32, "the default colour-sum mode is fp32");
    expect(std::strcmp(fgs_blend_kernel_name(8, 8, 64, 64, 0), "") == 0, "no kernel name for an unsupported tile");
    expect(fgs_abi_version() == FGS_ABI_VERSION, "ABI version of header and library agree");
    {
        // the host-side poll for the mirrored pair count: finds what is there, says so when nothing comes
        int word = 4711, got = 0;
        expect(fgs_wait_count(&word, 1.0, &got) == FGS_OK && got == 4711, "a count that is there is returned");
        word = -2147483647 - 1;
        expect(fgs_wait_count(&word, 1.0, &got) == FGS_OK && got == word, "a negative count is a count");
        word = FGS_COUNT_PENDING;
        expect(fgs_wait_count(&word, 0.01, &got) == FGS_E_TIMEOUT && std::strlen(fgs_last_error()) > 0, "no count within the time given");
        refused(fgs_wait_count(nullptr, 1.0, &got), "null count word");
        refused(fgs_wait_count(&word, 1.0, nullptr), "null result");
        refused(fgs_preprocess_mirrored(16, f, f, f, f, 64, 64, 16, 16, pos, rot, 1, 1, 100, 0.01f, f, f, f, k, v, i32, 16, nullptr, nullptr),
                "null count mirror");
        refused(fgs_preprocess_mirrored(-1, f, f, f, f, 64, 64, 16, 16, pos, rot, 1, 1, 100, 0.01f, f, f, f, k, v, i32, 16, &word, nullptr),
                "negative P with a count mirror");
    }
}

void check_host_arithmetic()
{
    size_t prev = 0;
    for (int n : {0, 1, 63, 4096, 4097, 1 << 20, (1 << 27) + 3, FGS_MAX_RENDERED}) {
        const size_t s = fgs_get_sort_buffer_size(n);
        expect(s >= prev && (n == 0 || s >= (size_t)n * 12), "workspace sizes grow with the pair count");
        prev = s;
    }
    expect(fgs_get_sort_buffer_size(-1) == 0 && fgs_get_sort_buffer_size(1 << 30) == 0, "out-of-range counts have no workspace size");
    float view[16], proj[16];
    const float pos[3] = {3.f, -2.f, 7.f}, rot[9] = {0, 0, 1, 0, 1, 0, -1, 0, 0};
    fgs_camera_matrices(pos, rot, 7680, 4320, 3084.8f, 3084.8f, 100.f, 0.01f, view, proj);
    expect(view[15] == 1.0f && view[3] == 0.0f, "last row of the view matrix");
    expect(std::fabs(proj[3] - view[2]) < 1e-6f && std::fabs(proj[15] - view[14]) < 1e-5f, "w of a projected point is its view depth");
}

} // namespace

int main()
{
    check_ply();
    check_arguments();
    check_host_arithmetic();
    if (g_failures) {
        std::fprintf(stderr, "%d host check(s) failed\n", g_failures);
        return 1;
    }
    std::puts("host checks ok");
    return 0;
}

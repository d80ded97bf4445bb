// Reader of the binary little-endian .ply that 3DGS training writes, as FlashGS loadPly reads it
// (csrc/pybind.cpp:58-120 of the reference): after the text header, one record of 62 floats per
// vertex - position(3) normal(3) sh(48, planar: dc r,g,b then 15 r, 15 g, 15 b) opacity-logit(1)
// log-scale(3) quaternion(4, r x y z).
//
// Plain C++ with no dependency on torch, so that the parser of this untrusted input can also be
// built on its own with the address and undefined-behaviour sanitizers.
#pragma once

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <istream>
#include <stdexcept>
#include <string>

namespace fgs_ply {

constexpr int kPlyFloats = 62;
constexpr size_t kRecordBytes = kPlyFloats * sizeof(float);

// Reads the text header: the vertex count and the position of the first record.  The count is
// checked against what the file can hold *before* anybody allocates for it: a header may claim any
// number.  Error texts are the reference's where it has one (pybind.cpp:60-89).
inline int read_header(std::istream& file, uint64_t file_bytes)
{
    long long n = 0;             // stays 0 for a header without a vertex element, as in the reference
    bool header_done = false;
    std::string tok;
    while (file >> tok) {
        if (tok == "vertex") {
            if (!(file >> n) || n <= 0) throw std::runtime_error("Vertex number is not positive");
        } else if (tok == "end_header") {
            header_done = true;
            file.get();   // the newline that ends the header
            break;
        }
    }
    if (!header_done) throw std::runtime_error("Cannot find end of header");
    const std::streamoff at = file.tellg();
    if (at < 0 || (uint64_t)at > file_bytes) throw std::runtime_error("Cannot find end of header");
    const uint64_t room = (file_bytes - (uint64_t)at) / kRecordBytes;
    if ((uint64_t)n > room || n > 2147483647LL)
        throw std::runtime_error("Vertex number " + std::to_string(n) + " exceeds the " + std::to_string(room) +
                                 " records the file holds");
    return (int)n;
}

// Sigma from exp'd scales and a normalised quaternion, in the operation order of
// computeCov3D (pybind.cpp:22-56): M = S * R in GLM's column-major product, Sigma = M^T * M.
inline void cov3d_from(const float s[3], const float q[4], float out[6])
{
    const float r = q[0], x = q[1], y = q[2], z = q[3];
    // R[c][k]: GLM column c, element k (the nine constructor arguments fill columns)
    const float R[3][3] = {
        { 1.f - 2.f * (y * y + z * z), 2.f * (x * y - r * z), 2.f * (x * z + r * y) },
        { 2.f * (x * y + r * z), 1.f - 2.f * (x * x + z * z), 2.f * (y * z - r * x) },
        { 2.f * (x * z - r * y), 2.f * (y * z + r * x), 1.f - 2.f * (x * x + y * y) } };
    float M[3][3];   // M[c][k] = sum_j S[j][k] * R[c][j], S diagonal; the zero products are kept
    for (int c = 0; c < 3; c++)
        for (int k = 0; k < 3; k++) {
            float acc[3];
            for (int j = 0; j < 3; j++) acc[j] = (j == k ? s[k] : 0.0f) * R[c][j];
            M[c][k] = acc[0] + acc[1] + acc[2];
        }
    auto sigma = [&](int c, int k) {   // (M^T * M)[c][k] in GLM order: Mt[j][k] * M[c][j]
        return M[k][0] * M[c][0] + M[k][1] * M[c][1] + M[k][2] * M[c][2];
    };
    out[0] = sigma(0, 0); out[1] = sigma(0, 1); out[2] = sigma(0, 2);
    out[3] = sigma(1, 1); out[4] = sigma(1, 2); out[5] = sigma(2, 2);
}

// One record -> the four rows of the op surface's tensors: position[3], shs[48] interleaved per
// coefficient, opacity after the sigmoid, cov3d[6] = upper triangle of R S^2 R^T.
inline void convert_record(const float rec[kPlyFloats], float position[3], float shs[48], float* opacity, float cov3d[6])
{
    const float* sh = rec + 6;
    std::memcpy(position, rec, 3 * sizeof(float));
    shs[0] = sh[0]; shs[1] = sh[1]; shs[2] = sh[2];
    for (int j = 1; j < 16; j++) {           // planar rest coefficients -> interleaved RGB
        shs[3 * j + 0] = sh[3 + (j - 1)];
        shs[3 * j + 1] = sh[3 + 15 + (j - 1)];
        shs[3 * j + 2] = sh[3 + 30 + (j - 1)];
    }
    *opacity = 1.0f / (1.0f + std::exp(-rec[54]));
    const float s[3] = { std::exp(rec[55]), std::exp(rec[56]), std::exp(rec[57]) };
    // glm::normalize: v * (1 / sqrt(dot)), dot = (x*x + y*y) + (z*z + w*w)
    const float* q0 = rec + 58;
    const float inv = 1.0f / std::sqrt((q0[0] * q0[0] + q0[1] * q0[1]) + (q0[2] * q0[2] + q0[3] * q0[3]));
    const float q[4] = { q0[0] * inv, q0[1] * inv, q0[2] * inv, q0[3] * inv };
    cov3d_from(s, q, cov3d);
}

// Reads the n records that follow the header into caller-allocated arrays of n rows each.
inline void read_records(std::istream& file, int n, float* position, float* shs, float* opacity, float* cov3d)
{
    float rec[kPlyFloats];
    for (int i = 0; i < n; i++) {
        file.read(reinterpret_cast<char*>(rec), kRecordBytes);
        if (!file) throw std::runtime_error("Unexpected end of file in vertex data");
        convert_record(rec, position + 3 * (size_t)i, shs + 48 * (size_t)i, opacity + i, cov3d + 6 * (size_t)i);
    }
}

} // namespace fgs_ply

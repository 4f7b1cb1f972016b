// ply.hip - the on-disk format of a trained model either side of the training step: binary little-endian PLY with
// one float32 row per Gaussian (writer: src/core/splat_data.cpp:113-169, 402-418, 484-506; reader:
// src/loader/formats/ply.cpp:185-323, 446-476, 500-637).
//
// The reference assembles the rows on the CPU (transpose + flatten + cat of torch tensors, tinyply interleave) and
// scatters them back with TBB loops.  Here the row image is built / taken apart on the GPU: one kernel gathers the
// five parameter tensors into the interleaved [N, 14 + 3K] row image (SH coefficients channel-major, rotation
// normalised), one kernel scatters an arbitrary row layout back into the tensors; the host only moves whole
// buffers between pinned memory and the file.
#include <errno.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "gsx_common.h"

namespace gsx {

// row of the writer: x y z nx ny nz f_dc_0..2 f_rest_0..3(K-1)-1 opacity scale_0..2 rot_0..3
static inline uint32_t ply_row_floats(uint32_t K) { return 14u + 3u * K; }

__global__ void __launch_bounds__(256) ply_pack_rows_kernel(uint64_t total, uint32_t K, const float* __restrict__ means,
                                                             const float* __restrict__ shs,
                                                             const float* __restrict__ opacity_raw,
                                                             const float* __restrict__ scaling_raw,
                                                             const float* __restrict__ rotation_raw,
                                                             float* __restrict__ rows) {
    const uint32_t row_floats = 14u + 3u * K, B = K - 1u;
    for (uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x; idx < total; idx += (uint64_t)gridDim.x * 256u) {
        const uint64_t v = idx / row_floats;
        const uint32_t c = (uint32_t)(idx - v * row_floats);
        float out;
        if (c < 3u) {
            out = means[v * 3 + c];
        } else if (c < 6u) {
            out = 0.f; // normals (splat_data.cpp:489)
        } else if (c < 9u) {
            out = shs[v * K * 3 + (c - 6u)]; // sh0.transpose(1,2).flatten(1): one coefficient, channel order
        } else if (c < 9u + 3u * B) {
            const uint32_t j = c - 9u, channel = j / B, b = j - channel * B; // shN.transpose(1,2).flatten(1)
            out = shs[v * K * 3 + (1u + b) * 3u + channel];
        } else {
            const uint32_t t = c - (9u + 3u * B);
            if (t == 0u) {
                out = opacity_raw[v];
            } else if (t < 4u) {
                out = scaling_raw[v * 3 + (t - 1u)];
            } else {
                // F.normalize(rotation, dim=-1): x / max(|x|, 1e-12)  (splat_data.cpp:497-500)
                const float4 q = reinterpret_cast<const float4*>(rotation_raw)[v];
                const float n = gsx::sqrt(((q.x * q.x + q.y * q.y) + q.z * q.z) + q.w * q.w);
                const float d = n > 1e-12f ? n : 1e-12f;
                const float e = (t == 4u) ? q.x : (t == 5u) ? q.y : (t == 6u) ? q.z : q.w;
                out = e / d;
            }
        }
        rows[idx] = out;
    }
}

struct PlyLayoutDev {
    uint64_t vertex_count;
    uint32_t stride_floats;
    int32_t pos[3], opacity, scale[3], rot[4], dc_start, dc_count, rest_start, rest_count;
};

// One thread per element of the OUTPUT tensors (14 + 3K per Gaussian with K = 1 + shN coefficients), so the
// tensors are written coalesced; the rows are read through the cache.
__global__ void __launch_bounds__(256) ply_unpack_rows_kernel(const PlyLayoutDev L, uint32_t K,
                                                               const float* __restrict__ rows,
                                                               float* __restrict__ means, float* __restrict__ shs,
                                                               float* __restrict__ opacity_raw,
                                                               float* __restrict__ scaling_raw,
                                                               float* __restrict__ rotation_raw) {
    const uint32_t per = 11u + 3u * K; // 3 + 3K + 1 + 3 + 4
    const uint64_t total = L.vertex_count * per;
    const bool dc_ok = L.dc_count > 0 && L.dc_count % 3 == 0 && L.dc_start >= 0;       // ply.cpp:538
    const bool rest_ok = L.rest_count > 0 && L.rest_count % 3 == 0 && L.rest_start >= 0; // ply.cpp:548
    const uint32_t B0 = dc_ok ? (uint32_t)L.dc_count / 3u : 1u, Bn = K - B0;
    for (uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x; idx < total; idx += (uint64_t)gridDim.x * 256u) {
        const uint64_t v = idx / per;
        const uint32_t c = (uint32_t)(idx - v * per);
        const float* row = rows + v * L.stride_floats;
        if (c < 3u) {
            // ply.cpp:326-334: positions are extracted only when x is present
            means[v * 3 + c] = (L.pos[0] >= 0 && L.pos[c] >= 0) ? row[L.pos[c]] : 0.f;
        } else if (c < 3u + 3u * K) {
            const uint32_t e = c - 3u, k = e / 3u, channel = e - k * 3u;
            float val = 0.f;
            if (k < B0) {
                if (dc_ok)
                    val = row[L.dc_start + channel * B0 + k]; // ply.cpp:463-473: j = channel * B + b
            } else if (rest_ok) {
                val = row[L.rest_start + channel * Bn + (k - B0)];
            }
            shs[v * K * 3 + e] = val;
        } else {
            const uint32_t t = c - (3u + 3u * K);
            if (t == 0u) {
                opacity_raw[v] = L.opacity >= 0 ? row[L.opacity] : 0.f;
            } else if (t < 4u) {
                const int32_t o = L.scale[t - 1u];
                scaling_raw[v * 3 + (t - 1u)] = L.scale[0] >= 0 ? (o >= 0 ? row[o] : 0.f) : -5.0f; // ply.cpp:564-584
            } else {
                const int32_t o = L.rot[t - 4u];
                rotation_raw[v * 4 + (t - 4u)] =
                    L.rot[0] >= 0 ? (o >= 0 ? row[o] : 0.f) : (t == 4u ? 1.0f : 0.f); // ply.cpp:587-609
            }
        }
    }
}

static bool starts_with(const char* s, size_t len, const char* prefix) {
    const size_t n = strlen(prefix);
    return len >= n && strncmp(s, prefix, n) == 0;
}

// parse_header of ply.cpp:185-323.  Differences, both deliberate: a vertex property that is not `float` is an
// error (the reference skips the line without advancing the row stride and would misread every later property),
// and offsets are float indices, not byte offsets.
static int parse_header(const char* data, size_t size, gsx_ply_layout* out) {
    GSX_REQUIRE(data && out, GSX_ERR_INVALID_ARGUMENT, "ply_parse_header: null argument");
    GSX_REQUIRE(size >= 10, GSX_ERR_INVALID_ARGUMENT, "ply_parse_header: file too small to be valid PLY");
    bool crlf = false;
    if (strncmp(data, "ply\r\n", 5) == 0)
        crlf = true;
    else
        GSX_REQUIRE(strncmp(data, "ply\n", 4) == 0, GSX_ERR_INVALID_ARGUMENT,
                    "ply_parse_header: invalid PLY file - missing PLY header");
    gsx_ply_layout L;
    memset(&L, 0, sizeof(L));
    L.pos[0] = L.pos[1] = L.pos[2] = L.opacity = L.dc_start = L.rest_start = -1;
    L.scale[0] = L.scale[1] = L.scale[2] = L.rot[0] = L.rot[1] = L.rot[2] = L.rot[3] = -1;
    const char* ptr = data + (crlf ? 5 : 4);
    const char* end = data + size;
    bool binary = false, found_vertex = false, in_vertex = false;
    size_t lines = 0;
    while (ptr < end && lines < 10000) {
        const char* line = ptr;
        const char* line_end = nullptr;
        for (const char* p = ptr; p < end; ++p) {
            if (*p == '\n') {
                line_end = p, ptr = p + 1;
                break;
            }
            if (*p == '\r' && p + 1 < end && p[1] == '\n') {
                line_end = p, ptr = p + 2;
                break;
            }
        }
        if (!line_end)
            break;
        const size_t len = (size_t)(line_end - line);
        ++lines;
        if (len == 0 || line[0] == '#')
            continue;
        if (starts_with(line, len, "format binary_little_endian")) {
            binary = true;
        } else if (starts_with(line, len, "element vertex ")) {
            L.vertex_count = strtoull(line + 15, nullptr, 10);
            L.stride_floats = 0;
            found_vertex = in_vertex = true;
        } else if (starts_with(line, len, "element ")) {
            in_vertex = false; // rows of other elements follow the vertex rows and are not read
        } else if (starts_with(line, len, "property ") && in_vertex) {
            GSX_REQUIRE(starts_with(line, len, "property float ") || starts_with(line, len, "property float32 "),
                        GSX_ERR_UNSUPPORTED, "ply_parse_header: vertex property is not float32: %.*s", (int)len, line);
            const size_t skip = starts_with(line, len, "property float32 ") ? 17 : 15;
            const char* name = line + skip;
            size_t n = len - skip;
            while (n > 0 && (name[n - 1] == ' ' || name[n - 1] == '\t' || name[n - 1] == '\r'))
                --n;
            const int32_t at = (int32_t)L.stride_floats;
            if (n == 1) {
                if (*name == 'x')
                    L.pos[0] = at;
                else if (*name == 'y')
                    L.pos[1] = at;
                else if (*name == 'z')
                    L.pos[2] = at;
            } else if (n == 7 && strncmp(name, "opacity", 7) == 0) {
                L.opacity = at;
            } else if (n >= 5 && strncmp(name, "f_dc_", 5) == 0) {
                const int idx = atoi(name + 5);
                if (idx == 0)
                    L.dc_start = at;
                if (idx >= L.dc_count)
                    L.dc_count = idx + 1;
            } else if (n >= 7 && strncmp(name, "f_rest_", 7) == 0) {
                const int idx = atoi(name + 7);
                if (idx == 0)
                    L.rest_start = at;
                if (idx >= L.rest_count)
                    L.rest_count = idx + 1;
            } else if (n == 7 && strncmp(name, "scale_", 6) == 0) {
                const int idx = name[6] - '0';
                if (idx >= 0 && idx < 3)
                    L.scale[idx] = at;
            } else if (n == 5 && strncmp(name, "rot_", 4) == 0) {
                const int idx = name[4] - '0';
                if (idx >= 0 && idx < 4)
                    L.rot[idx] = at;
            }
            L.stride_floats += 1;
        } else if (starts_with(line, len, "end_header")) {
            GSX_REQUIRE(binary && found_vertex, GSX_ERR_UNSUPPORTED,
                        "ply_parse_header: only binary PLY with position supported");
            // the coefficient blocks are read as dc_count / rest_count consecutive floats (ply.cpp:463-466)
            GSX_REQUIRE(L.dc_start < 0 || (uint32_t)(L.dc_start + L.dc_count) <= L.stride_floats, GSX_ERR_INVALID_ARGUMENT,
                        "ply_parse_header: f_dc_* block leaves the vertex row");
            GSX_REQUIRE(L.rest_start < 0 || (uint32_t)(L.rest_start + L.rest_count) <= L.stride_floats,
                        GSX_ERR_INVALID_ARGUMENT, "ply_parse_header: f_rest_* block leaves the vertex row");
            L.data_offset = (uint64_t)(ptr - data);
            *out = L;
            return GSX_OK;
        }
    }
    GSX_REQUIRE(lines < 10000, GSX_ERR_INVALID_ARGUMENT, "ply_parse_header: header too large - exceeded 10000 lines");
    GSX_REQUIRE(false, GSX_ERR_INVALID_ARGUMENT, "ply_parse_header: no end_header found in PLY file");
    return GSX_ERR_INVALID_ARGUMENT;
}

static uint32_t layout_sh_coeffs(const gsx_ply_layout& L) {
    const uint32_t B0 = (L.dc_count > 0 && L.dc_count % 3 == 0 && L.dc_start >= 0) ? (uint32_t)L.dc_count / 3u : 1u;
    const uint32_t Bn = (L.rest_count > 0 && L.rest_count % 3 == 0 && L.rest_start >= 0) ? (uint32_t)L.rest_count / 3u
                                                                                        : 15u; // ply.cpp:554
    return B0 + Bn;
}

} // namespace gsx

extern "C" uint32_t gsx_ply_row_floats(uint32_t K) { return gsx::ply_row_floats(K); }

extern "C" int64_t gsx_ply_format_header(uint64_t N, uint32_t K, char* buf, size_t capacity) {
    // what tinyply's binary writer emits for one "vertex" element of float32 properties (splat_data.cpp:136-162)
    // with the attribute names of splat_data.cpp:402-418
    GSX_REQUIRE(K >= 1, GSX_ERR_INVALID_ARGUMENT, "ply_format_header: K must be >= 1");
    size_t len = 0;
    auto put = [&](const char* fmt, auto... a) {
        const int n = snprintf(buf && len < capacity ? buf + len : nullptr, buf && len < capacity ? capacity - len : 0,
                               fmt, a...);
        len += (size_t)n;
    };
    put("ply\nformat binary_little_endian 1.0\nelement vertex %llu\n", (unsigned long long)N);
    for (const char* s : {"x", "y", "z", "nx", "ny", "nz"})
        put("property float %s\n", s);
    for (uint32_t i = 0; i < 3; ++i)
        put("property float f_dc_%u\n", i);
    for (uint32_t i = 0; i < 3 * (K - 1); ++i)
        put("property float f_rest_%u\n", i);
    put("property float %s\n", "opacity");
    for (uint32_t i = 0; i < 3; ++i)
        put("property float scale_%u\n", i);
    for (uint32_t i = 0; i < 4; ++i)
        put("property float rot_%u\n", i);
    put("%s", "end_header\n");
    GSX_REQUIRE(!buf || len < capacity, GSX_ERR_WORKSPACE, "ply_format_header: buffer of %zu bytes, need %zu", capacity,
                len + 1);
    return (int64_t)len;
}

extern "C" int gsx_ply_parse_header(const char* data, size_t size, gsx_ply_layout* layout) {
    return gsx::parse_header(data, size, layout);
}

extern "C" uint32_t gsx_ply_layout_sh_coeffs(const gsx_ply_layout* layout) {
    return layout ? gsx::layout_sh_coeffs(*layout) : 0;
}

extern "C" int gsx_ply_pack_rows(uint64_t N, uint32_t K, const float* means, const float* shs, const float* opacity_raw,
                                 const float* scaling_raw, const float* rotation_raw, float* rows, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(means && shs && opacity_raw && scaling_raw && rotation_raw && rows, GSX_ERR_INVALID_ARGUMENT,
                "ply_pack_rows: null tensor");
    GSX_REQUIRE(K >= 1 && K <= 64, GSX_ERR_INVALID_ARGUMENT, "ply_pack_rows: K = %u", K);
    const uint64_t total = N * gsx::ply_row_floats(K);
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 20);
    hipLaunchKernelGGL(gsx::ply_pack_rows_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, total, K, means, shs,
                       opacity_raw, scaling_raw, rotation_raw, rows);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_ply_unpack_rows(const gsx_ply_layout* layout, const float* rows, float* means, float* shs,
                                   float* opacity_raw, float* scaling_raw, float* rotation_raw, void* stream) {
    GSX_REQUIRE(layout, GSX_ERR_INVALID_ARGUMENT, "ply_unpack_rows: null layout");
    if (layout->vertex_count == 0)
        return GSX_OK;
    GSX_REQUIRE(rows && means && shs && opacity_raw && scaling_raw && rotation_raw, GSX_ERR_INVALID_ARGUMENT,
                "ply_unpack_rows: null tensor");
    gsx::PlyLayoutDev L;
    L.vertex_count = layout->vertex_count, L.stride_floats = layout->stride_floats;
    const int32_t stride = (int32_t)layout->stride_floats;
    auto ok = [&](int32_t o) { return o >= -1 && o < stride; };
    bool fine = ok(layout->opacity) && ok(layout->dc_start) && ok(layout->rest_start);
    for (int i = 0; i < 3; ++i)
        L.pos[i] = layout->pos[i], L.scale[i] = layout->scale[i], fine = fine && ok(L.pos[i]) && ok(L.scale[i]);
    for (int i = 0; i < 4; ++i)
        L.rot[i] = layout->rot[i], fine = fine && ok(L.rot[i]);
    L.opacity = layout->opacity, L.dc_start = layout->dc_start, L.dc_count = layout->dc_count;
    L.rest_start = layout->rest_start, L.rest_count = layout->rest_count;
    fine = fine && (L.dc_start < 0 || (L.dc_count >= 0 && L.dc_start + L.dc_count <= stride)) &&
           (L.rest_start < 0 || (L.rest_count >= 0 && L.rest_start + L.rest_count <= stride));
    GSX_REQUIRE(fine, GSX_ERR_INVALID_ARGUMENT, "ply_unpack_rows: a property offset leaves the vertex row");
    const uint32_t K = gsx::layout_sh_coeffs(*layout);
    const uint64_t total = L.vertex_count * (11u + 3u * K);
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 20);
    hipLaunchKernelGGL(gsx::ply_unpack_rows_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, L, K, rows, means,
                       shs, opacity_raw, scaling_raw, rotation_raw);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

// ---- file side (host only) ----

extern "C" int gsx_ply_write_file(const char* path, uint64_t N, uint32_t K, const float* rows_host) {
    GSX_REQUIRE(path && (rows_host || N == 0), GSX_ERR_INVALID_ARGUMENT, "ply_write_file: null argument");
    char header[8192];
    const int64_t len = gsx_ply_format_header(N, K, header, sizeof(header));
    if (len < 0)
        return (int)len;
    FILE* f = fopen(path, "wb");
    GSX_REQUIRE(f, GSX_ERR_INVALID_ARGUMENT, "ply_write_file: cannot open %s: %s", path, strerror(errno));
    const size_t count = (size_t)N * gsx::ply_row_floats(K);
    const bool ok = fwrite(header, 1, (size_t)len, f) == (size_t)len && fwrite(rows_host, 4, count, f) == count;
    const bool closed = fclose(f) == 0;
    GSX_REQUIRE(ok && closed, GSX_ERR_INVALID_ARGUMENT, "ply_write_file: short write to %s", path);
    return GSX_OK;
}

extern "C" int gsx_ply_read_file_header(const char* path, gsx_ply_layout* layout) {
    GSX_REQUIRE(path && layout, GSX_ERR_INVALID_ARGUMENT, "ply_read_file_header: null argument");
    FILE* f = fopen(path, "rb");
    GSX_REQUIRE(f, GSX_ERR_INVALID_ARGUMENT, "PLY file does not exist: %s", path);
    // 10000 header lines at most: 1 MiB covers any header the parser accepts
    const size_t cap = 1u << 20;
    char* buf = (char*)malloc(cap);
    const size_t got = buf ? fread(buf, 1, cap, f) : 0;
    fseek(f, 0, SEEK_END);
    const long long file_size = ftello(f);
    fclose(f);
    int rc = buf ? gsx::parse_header(buf, got, layout) : GSX_ERR_INVALID_ARGUMENT;
    free(buf);
    if (rc != GSX_OK)
        return rc;
    const unsigned long long need = layout->data_offset + layout->vertex_count * layout->stride_floats * 4ull;
    GSX_REQUIRE((unsigned long long)file_size >= need, GSX_ERR_INVALID_ARGUMENT,
                "ply_read_file_header: %s holds %lld bytes, the header announces %llu", path, file_size, need);
    return GSX_OK;
}

extern "C" int gsx_ply_read_file_rows(const char* path, const gsx_ply_layout* layout, float* rows_host) {
    GSX_REQUIRE(path && layout && rows_host, GSX_ERR_INVALID_ARGUMENT, "ply_read_file_rows: null argument");
    FILE* f = fopen(path, "rb");
    GSX_REQUIRE(f, GSX_ERR_INVALID_ARGUMENT, "PLY file does not exist: %s", path);
    const size_t count = (size_t)layout->vertex_count * layout->stride_floats;
    const bool ok = fseeko(f, (off_t)layout->data_offset, SEEK_SET) == 0 && fread(rows_host, 4, count, f) == count;
    fclose(f);
    GSX_REQUIRE(ok, GSX_ERR_INVALID_ARGUMENT, "ply_read_file_rows: short read from %s", path);
    return GSX_OK;
}

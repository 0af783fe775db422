// lutgemm_pack: offline packer for BCQ weights.  Host only: no GPU is touched.
//
//   lutgemm_pack pack --k K --n N --q Q --groups G --bw bW.u32 --alpha alpha.f32
//                     [--qbias qbias.f32] [--f16] -o weight.lutw
//   lutgemm_pack info weight.lutw
//   lutgemm_pack unpack weight.lutw --bw bW.u32 --alpha alpha.f16 [--qbias qbias.f16]
//
// Raw input files are little-endian arrays in the reference's container layout
// (lutGEMM/include/nQWeight_fp16.h:29-31): bW uint32 [K/32][Q][N], alpha [G][Q][N] and q_bias
// [G][N] as float32 (or binary16 with --f16).  `unpack` writes alpha / q_bias as binary16, the
// precision the container holds.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/lutgemm_c.h"

namespace {

int usage()
{
    std::fprintf(stderr,
                 "usage:\n"
                 "  lutgemm_pack pack --k K --n N --q Q --groups G --bw FILE --alpha FILE [--qbias FILE] [--f16] -o OUT\n"
                 "  lutgemm_pack info FILE\n"
                 "  lutgemm_pack unpack FILE --bw OUT --alpha OUT [--qbias OUT]\n");
    return 2;
}

bool read_all(const std::string &path, size_t bytes, std::vector<uint8_t> *out)
{
    FILE *f = std::fopen(path.c_str(), "rb");
    if (!f) {
        std::fprintf(stderr, "lutgemm_pack: cannot open %s\n", path.c_str());
        return false;
    }
    out->resize(bytes);
    const size_t got = std::fread(out->data(), 1, bytes, f);
    const bool extra = std::fgetc(f) != EOF;
    std::fclose(f);
    if (got != bytes || extra) {
        std::fprintf(stderr, "lutgemm_pack: %s does not hold exactly %zu bytes\n", path.c_str(), bytes);
        return false;
    }
    return true;
}

bool write_all(const std::string &path, const void *data, size_t bytes)
{
    FILE *f = std::fopen(path.c_str(), "wb");
    if (!f || std::fwrite(data, 1, bytes, f) != bytes || std::fclose(f) != 0) {
        std::fprintf(stderr, "lutgemm_pack: cannot write %s\n", path.c_str());
        return false;
    }
    return true;
}

int fail_lib(int st)
{
    std::fprintf(stderr, "lutgemm_pack: %s: %s\n", lutgemm_status_string(st), lutgemm_last_error());
    return 1;
}

// binary16 arrays from a raw file of float32 (converted with the library's ingest rounding) or binary16
bool read_halves(const std::string &path, size_t count, bool f16, std::vector<uint16_t> *out)
{
    std::vector<uint8_t> raw;
    if (!read_all(path, count * (f16 ? 2 : 4), &raw)) return false;
    out->resize(count);
    if (f16) {
        std::memcpy(out->data(), raw.data(), count * 2);
        return true;
    }
    return lutgemm_float_to_half(reinterpret_cast<const float *>(raw.data()), out->data(), count) == LUTGEMM_OK;
}

}  // namespace

int main(int argc, char **argv)
{
    if (argc < 3) return usage();
    const std::string cmd = argv[1];
    std::string bw, alpha, qbias, out, file;
    long k = 0, n = 0, q = 0, groups = 1;
    bool f16 = false;
    for (int i = 2; i < argc; i++) {
        const std::string a = argv[i];
        auto value = [&](std::string *dst) {
            if (i + 1 >= argc) return false;
            *dst = argv[++i];
            return true;
        };
        std::string v;
        if (a == "--bw") { if (!value(&bw)) return usage(); }
        else if (a == "--alpha") { if (!value(&alpha)) return usage(); }
        else if (a == "--qbias") { if (!value(&qbias)) return usage(); }
        else if (a == "-o") { if (!value(&out)) return usage(); }
        else if (a == "--k") { if (!value(&v)) return usage(); k = std::atol(v.c_str()); }
        else if (a == "--n") { if (!value(&v)) return usage(); n = std::atol(v.c_str()); }
        else if (a == "--q") { if (!value(&v)) return usage(); q = std::atol(v.c_str()); }
        else if (a == "--groups") { if (!value(&v)) return usage(); groups = std::atol(v.c_str()); }
        else if (a == "--f16") f16 = true;
        else if (!a.empty() && a[0] != '-' && file.empty()) file = a;
        else return usage();
    }

    if (cmd == "pack") {
        if (bw.empty() || alpha.empty() || out.empty() || k <= 0 || n <= 0 || q <= 0 || groups <= 0) return usage();
        if (k % 32 != 0 || k > 0x7fffffff || n > 0x7fffffff || q > 8) {
            std::fprintf(stderr, "lutgemm_pack: need k %% 32 == 0 and 1 <= q <= 8\n");
            return 1;
        }
        std::vector<uint8_t> planes;
        std::vector<uint16_t> a16, z16;
        if (!read_all(bw, (size_t)(k / 32) * q * n * 4, &planes)) return 1;
        if (!read_halves(alpha, (size_t)groups * q * n, f16, &a16)) return 1;
        if (!qbias.empty() && !read_halves(qbias, (size_t)groups * n, f16, &z16)) return 1;
        const int st = lutgemm_pack_file(reinterpret_cast<const uint32_t *>(planes.data()), a16.data(),
                                         qbias.empty() ? nullptr : z16.data(), (int)k, (int)n, (int)q,
                                         (int)groups, out.c_str());
        if (st != LUTGEMM_OK) return fail_lib(st);
        std::printf("%s: k=%ld n=%ld q=%ld num_groups=%ld offset=%d\n", out.c_str(), k, n, q, groups,
                    qbias.empty() ? 0 : 1);
        return 0;
    }

    if (file.empty()) return usage();
    lutgemm_weight_info_t info;
    int st = lutgemm_unpack_file(file.c_str(), nullptr, nullptr, nullptr, &info);
    if (st != LUTGEMM_OK) return fail_lib(st);
    if (cmd == "info") {
        std::printf("k=%d n=%d q=%d num_groups=%d group_size=%d offset=%d packed_bytes=%zu\n", info.k, info.n,
                    info.q, info.num_groups, info.group_size, info.has_offset,
                    info.sign_bytes + info.scale_bytes + info.offset_bytes);
        return 0;
    }
    if (cmd == "unpack") {
        if (bw.empty() || alpha.empty() || (info.has_offset && qbias.empty())) return usage();
        std::vector<uint32_t> planes((size_t)(info.k / 32) * info.q * info.n);
        std::vector<uint16_t> a16((size_t)info.num_groups * info.q * info.n);
        std::vector<uint16_t> z16(info.has_offset ? (size_t)info.num_groups * info.n : 0);
        st = lutgemm_unpack_file(file.c_str(), planes.data(), a16.data(), info.has_offset ? z16.data() : nullptr,
                                 nullptr);
        if (st != LUTGEMM_OK) return fail_lib(st);
        if (!write_all(bw, planes.data(), planes.size() * 4) || !write_all(alpha, a16.data(), a16.size() * 2))
            return 1;
        if (info.has_offset && !write_all(qbias, z16.data(), z16.size() * 2)) return 1;
        return 0;
    }
    return usage();
}

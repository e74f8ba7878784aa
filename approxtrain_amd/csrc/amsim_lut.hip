// LUT handle: host-side loading (the counterpart of approx_mul_lut.h:15-46) and
// the device images the kernels read (the counterpart of the cudaMalloc +
// texture object of cuda/approx_mul_lut.cu:24-48).
#include "amsim_internal.h"
#include "amsim_bench.h"

#include <atomic>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <vector>

namespace amsim {

static thread_local std::string g_last_error;

void set_error(const std::string &msg) { g_last_error = msg; }

int fail(int status, const std::string &msg)
{
    g_last_error = msg;
    return status;
}

const std::string &last_error() { return g_last_error; }

int device_compute_units()
{
    constexpr int MAX_DEV = 64;
    static std::atomic<int> cus[MAX_DEV];  // 0 = not read yet
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV) {
        (void)hipGetLastError();
        return 256;
    }
    int n = cus[dev].load(std::memory_order_relaxed);
    if (n > 0) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return 256;
    }
    cus[dev].store(n, std::memory_order_relaxed);
    return n;
}

int check_lut_device(const Lut &lut)
{
    int dev = 0;
    AMSIM_HIP_CHECK(hipGetDevice(&dev));
    if (dev != lut.device)
        return fail(AMSIM_ERR_INVALID, "LUT handle was created on device " + std::to_string(lut.device) +
                                           ", the current device is " + std::to_string(dev));
    return AMSIM_OK;
}

// entries: one (carry, mantissa) pair per (ma, mb), mantissa in m bits
void lut_free(Lut &l);

static int build_images(int m, const std::vector<uint8_t> &carry, const std::vector<uint32_t> &mant, Lut *out)
{
    const size_t n = (size_t)1 << m, total = n * n;
    Lut l;
    l.m = m;
    l.entries = total;
    AMSIM_HIP_CHECK(hipGetDevice(&l.device));
    // device copy of a host vector; on failure everything uploaded so far is released
    auto upload = [&](auto **dst, const auto &host) -> int {
        const size_t bytes = host.size() * sizeof(host[0]);
        hipError_t e = hipMalloc(reinterpret_cast<void **>(dst), bytes);
        if (e == hipSuccess) e = hipMemcpy(*dst, host.data(), bytes, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            lut_free(l);
            return fail(AMSIM_ERR_HIP, std::string("LUT upload: ") + hipGetErrorString(e));
        }
        return AMSIM_OK;
    };
    int rc;
    {
        std::vector<uint32_t> l32(total);
        for (size_t i = 0; i < total; ++i) l32[i] = ((uint32_t)carry[i] << 23) | (mant[i] << (23 - m));
        if ((rc = upload(&l.lut32, l32)) != AMSIM_OK) return rc;
    }
    if (m <= 7) {
        // + one all-zero row of n entries after the table (selected by zero operands)
        const size_t padded = (total + n + 15) / 16 * 16;
        std::vector<uint8_t> ab(padded, 0), ba(padded, 0);
        for (size_t i = 0; i < n; ++i)
            for (size_t j = 0; j < n; ++j) {
                const uint8_t b = (uint8_t)((carry[i * n + j] << 7) | (mant[i * n + j] << (7 - m)));
                ab[i * n + j] = b;
                ba[j * n + i] = b;
            }
        if ((rc = upload(&l.img_ab, ab)) != AMSIM_OK) return rc;
        if ((rc = upload(&l.img_ba, ba)) != AMSIM_OK) return rc;
    } else {
        // + the all-zero row, + 4 KB: the row-staged GEMM copies whole KBs from a row's start
        std::vector<uint16_t> ab(total + n + 2048, 0), ba(total + n + 2048, 0);
        for (size_t i = 0; i < n; ++i)
            for (size_t j = 0; j < n; ++j) {
                const uint16_t b = (uint16_t)((carry[i * n + j] << 15) | (mant[i * n + j] << (15 - m)));
                ab[i * n + j] = b;
                ba[j * n + i] = b;
            }
        if ((rc = upload(&l.img16_ab, ab)) != AMSIM_OK) return rc;
        if ((rc = upload(&l.img16_ba, ba)) != AMSIM_OK) return rc;
    }
    if ((rc = probe_lds_d16_keeps(&l.d16_keeps)) != AMSIM_OK) {
        lut_free(l);
        return rc;
    }
    l.d16_keeps_probed = l.d16_keeps;
    *out = l;
    return AMSIM_OK;
}

int lut_from_entries(const void *entries, size_t n_bytes, int m, int entry_bytes, Lut *out)
{
    if (entries == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT entries");
    if (entry_bytes != 1 && entry_bytes != 4) return fail(AMSIM_ERR_LUT_FORMAT, "entry_bytes must be 1 or 4");
    if (m < 1 || (entry_bytes == 1 && m > 7) || m > 11)
        return fail(AMSIM_ERR_LUT_FORMAT, "mantissa width " + std::to_string(m) + " unsupported for " +
                                              std::to_string(entry_bytes) + "-byte entries");
    const size_t total = (size_t)1 << (2 * m);
    if (n_bytes < total * entry_bytes)
        return fail(AMSIM_ERR_LUT_FORMAT, "LUT holds " + std::to_string(n_bytes) + " bytes, needs " +
                                              std::to_string(total * entry_bytes));
    std::vector<uint8_t> carry(total);
    std::vector<uint32_t> mant(total);
    if (entry_bytes == 1) {
        // lut/lut_gen.cc:114-121: carry << 7 | mantissa (m bits, right-aligned)
        const uint8_t *e = static_cast<const uint8_t *>(entries);
        for (size_t i = 0; i < total; ++i) {
            carry[i] = e[i] >> 7;
            mant[i] = (e[i] & 0x7fu) & ((1u << m) - 1u);
        }
    } else {
        // lut/AMsimulator.inl:18-20: bit 31 = carry, bits 22..0 = mantissa in place
        const uint32_t *e = static_cast<const uint32_t *>(entries);
        for (size_t i = 0; i < total; ++i) {
            carry[i] = (uint8_t)(e[i] >> 31);
            mant[i] = (e[i] & 0x7fffffu) >> (23 - m);
        }
    }
    return build_images(m, carry, mant, out);
}

void lut_free(Lut &l)
{
    if (l.img_ab) (void)hipFree(l.img_ab);
    if (l.img_ba) (void)hipFree(l.img_ba);
    if (l.lut32) (void)hipFree(l.lut32);
    if (l.img16_ab) (void)hipFree(l.img16_ab);
    if (l.img16_ba) (void)hipFree(l.img16_ba);
    l = Lut{};
}

// approx_mul_lut.h:22-25: the width is the decimal number between the last
// '_' and the last '.' of the file name.
int parse_width_from_name(const std::string &path, int *m)
{
    const size_t us = path.find_last_of('_'), dot = path.find_last_of('.');
    if (us == std::string::npos || dot == std::string::npos || dot <= us + 1)
        return fail(AMSIM_ERR_LUT_FORMAT, "LUT file name '" + path + "' lacks the _<width>.<ext> suffix");
    const std::string w = path.substr(us + 1, dot - us - 1);
    for (char c : w)
        if (c < '0' || c > '9')
            return fail(AMSIM_ERR_LUT_FORMAT, "LUT file name '" + path + "': width '" + w + "' is not a number");
    if (w.size() > 3) return fail(AMSIM_ERR_LUT_FORMAT, "LUT file name '" + path + "': width out of range");
    *m = std::stoi(w);
    return AMSIM_OK;
}

}  // namespace amsim

using namespace amsim;

extern "C" {

const char *amsim_last_error(void) { return amsim::last_error().c_str(); }

const char *amsim_status_string(int status)
{
    switch (status) {
    case AMSIM_OK: return "ok";
    case AMSIM_ERR_INVALID: return "invalid argument";
    case AMSIM_ERR_IO: return "LUT file I/O error";
    case AMSIM_ERR_LUT_FORMAT: return "bad LUT format";
    case AMSIM_ERR_HIP: return "HIP runtime error";
    case AMSIM_ERR_WORKSPACE: return "workspace missing or too small";
    case AMSIM_ERR_UNSUPPORTED: return "unsupported";
    default: return "unknown status";
    }
}

int amsim_device_info(char *arch, size_t arch_len, int *compute_units)
{
    int dev = 0;
    AMSIM_HIP_CHECK(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    AMSIM_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
    if (arch && arch_len) {
        std::snprintf(arch, arch_len, "%s", prop.gcnArchName);
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    return AMSIM_OK;
}

int amsim_lut_create(const void *entries, size_t n_bytes, int mant_width, int entry_bytes, amsim_lut_t *out)
{
    if (out == nullptr) return fail(AMSIM_ERR_INVALID, "null output handle");
    *out = nullptr;
    Lut l;
    int rc = lut_from_entries(entries, n_bytes, mant_width, entry_bytes, &l);
    if (rc != AMSIM_OK) return rc;
    *out = new amsim_lut{l};
    return AMSIM_OK;
}

int amsim_lut_load_file(const char *path, amsim_lut_t *out)
{
    if (out == nullptr) return fail(AMSIM_ERR_INVALID, "null output handle");
    *out = nullptr;
    if (path == nullptr || *path == '\0') return fail(AMSIM_ERR_INVALID, "no mant lut file name given");
    int m = 0;
    int rc = parse_width_from_name(path, &m);
    if (rc != AMSIM_OK) return rc;
    if (m < 1 || m > 11)
        return fail(AMSIM_ERR_LUT_FORMAT, "LUT file mantissa width must be 1..11, got " + std::to_string(m));
    // one byte per entry up to width 7 (the reference's files); wider tables need more than
    // 7 mantissa bits per entry and are stored in the 4-byte layout
    const int entry_bytes = m <= 7 ? 1 : 4;
    std::ifstream file(path, std::ios::in | std::ios::binary);
    if (!file.is_open() || file.fail()) return fail(AMSIM_ERR_IO, std::string("lut file open failed: ") + path);
    const size_t total = ((size_t)1 << (2 * m)) * entry_bytes;
    std::vector<uint8_t> bytes(total);
    file.read(reinterpret_cast<char *>(bytes.data()), (std::streamsize)total);
    if ((size_t)file.gcount() != total)
        return fail(AMSIM_ERR_LUT_FORMAT, std::string("lut file too short: ") + path);
    return amsim_lut_create(bytes.data(), total, m, entry_bytes, out);
}

int amsim_lut_destroy(amsim_lut_t lut)
{
    if (lut == nullptr) return AMSIM_OK;
    lut_free(lut->l);
    delete lut;
    return AMSIM_OK;
}

int amsim_lut_mant_width(amsim_lut_t lut) { return lut ? lut->l.m : -1; }

int amsim_lut_set_engine(amsim_lut_t lut, int mode)
{
    if (lut == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT handle");
    if (mode < -1 || mode > AMSIM_ENGINE_DIRECT) return fail(AMSIM_ERR_INVALID, "engine mode must be -1 (process default) or an AMSIM_ENGINE_* value");
    lut->l.engine = mode;
    return AMSIM_OK;
}

int amsim_lut_set_split_k(amsim_lut_t lut, int mode)
{
    if (lut == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT handle");
    if (mode < -1 || mode > 1) return fail(AMSIM_ERR_INVALID, "split mode must be -1 (process default), 0 or 1");
    lut->l.split_k = mode;
    return AMSIM_OK;
}

int amsim_lut_force_gather_zeroing(amsim_lut_t lut, int on, int *probed)
{
    if (lut == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT handle");
    if (on != 0 && on != 1) return fail(AMSIM_ERR_INVALID, "on must be 0 or 1");
    lut->l.d16_keeps = on ? 1 : lut->l.d16_keeps_probed;
    if (probed) *probed = lut->l.d16_keeps_probed;
    return AMSIM_OK;
}

int amsim_lut_params(amsim_lut_t lut, uint32_t *mant_mask, int *a_shift, int *b_shift)
{
    if (lut == nullptr) return fail(AMSIM_ERR_INVALID, "null LUT handle");
    const int m = lut->l.m;
    if (mant_mask) *mant_mask = ((1u << m) - 1u) << (23 - m);
    if (a_shift) *a_shift = 23 - 2 * m;
    if (b_shift) *b_shift = 23 - m;
    return AMSIM_OK;
}

}  // extern "C"

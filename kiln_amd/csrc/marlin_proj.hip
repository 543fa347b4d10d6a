// Projection-level host glue: the C++ statement of the reference's
// crates/kiln-model/src/marlin_proj.rs (MarlinPackedProj, the three-phase pack,
// matmul_bf16, the environment switches) over the C ABI of the GEMM, plus the
// persisted artefact.  Host code only; the HIP runtime is used for memory and copies.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <memory>
#include <optional>
#include <string>
#include <thread>
#include <vector>

#include "kiln_marlin_proj.h"
#include "kiln_w4a16.h"

struct kiln_marlin_packed_proj {
    void *b_packed = nullptr;  // device, int32 [k/16, 2n]
    void *scales = nullptr;    // device, fp16 [k/g, n]
    int groupsize = 128;
    int64_t k = 0, n = 0;
    int dev = 0;
};

namespace kiln {
namespace proj {

namespace {

thread_local std::string g_last_error;

int fail(const std::string &msg) {
    g_last_error = msg;
    return KILN_PROJ_ERR;
}

bool env_truthy(const char *name) {
    const char *v = std::getenv(name);
    if (!v) return false;
    std::string s(v);
    const auto b = s.find_first_not_of(" \t\r\n"), e = s.find_last_not_of(" \t\r\n");
    if (b == std::string::npos) return false;
    s = s.substr(b, e - b + 1);
    for (char &c : s) c = (char)std::tolower((unsigned char)c);
    return s == "1" || s == "true" || s == "yes";
}

size_t num_groups(int64_t k, int groupsize) { return groupsize == -1 ? 1 : (size_t)(k / groupsize); }

// Sets the device for the current scope and restores the previous one.
struct DeviceScope {
    int prev = 0;
    bool ok;
    explicit DeviceScope(int dev) { ok = hipGetDevice(&prev) == hipSuccess && hipSetDevice(dev) == hipSuccess; }
    ~DeviceScope() { (void)hipSetDevice(prev); }
};

}  // namespace

// marlin_proj.rs:62-69
struct PackJobHost {
    std::vector<float> host_weight;  // [k, n] row-major
    int64_t k, n;
    int groupsize;
};

// marlin_proj.rs:73-80
struct PackedHost {
    std::vector<int32_t> b_packed_vec;
    std::vector<uint16_t> scales_vec;
    int64_t k, n;
    int groupsize;
};

bool shape_is_supported(int64_t k, int64_t n) { return k > 0 && n > 0 && k % 128 == 0 && n % 256 == 0; }

// Phase 1 (marlin_proj.rs:86-124): validate, download, widen bf16 to f32.  The
// reference casts on the device and copies f32; bf16 -> f32 is exact, so
// copying bf16 and widening on the host gives the same values at half the traffic.
// Returns KILN_PROJ_SKIPPED for an unsupported shape or a weight that is not on a GPU.
int prepare_pack_job(const void *weight_t, int64_t k, int64_t n, int groupsize, int dev,
                     std::optional<PackJobHost> &out) {
    out.reset();
    if (dev < 0) return KILN_PROJ_SKIPPED;
    if (!weight_t) return fail("marlin_proj: weight_t must be a 2D [k, n] tensor");
    if (!shape_is_supported(k, n)) return KILN_PROJ_SKIPPED;
    if (!(groupsize == -1 || groupsize == 128))
        return fail("marlin_proj: groupsize must be -1 or 128 (got " + std::to_string(groupsize) + ")");
    if (groupsize == 128 && k % 128 != 0)
        return fail("marlin_proj: k=" + std::to_string(k) + " not divisible by groupsize=128");
    DeviceScope scope(dev);
    if (!scope.ok) return fail("marlin_proj: download weight to host");
    std::vector<uint16_t> raw((size_t)k * n);
    if (hipMemcpy(raw.data(), weight_t, raw.size() * sizeof(uint16_t), hipMemcpyDeviceToHost) != hipSuccess)
        return fail("marlin_proj: download weight to host");
    PackJobHost job;
    job.k = k;
    job.n = n;
    job.groupsize = groupsize;
    job.host_weight.resize(raw.size());
    for (size_t i = 0; i < raw.size(); ++i) {
        const uint32_t bits = (uint32_t)raw[i] << 16;
        std::memcpy(&job.host_weight[i], &bits, sizeof(float));
    }
    out = std::move(job);
    return KILN_PROJ_OK;
}

// Phase 2 (marlin_proj.rs:130-144): pure CPU, safe on any thread.
PackedHost pack_host(const PackJobHost &job) {
    PackedHost p;
    p.k = job.k;
    p.n = job.n;
    p.groupsize = job.groupsize;
    p.b_packed_vec.resize((size_t)job.k * job.n / 8);
    p.scales_vec.resize(num_groups(job.k, job.groupsize) * (size_t)job.n);
    kiln_w4a16_quantize_and_pack(job.host_weight.data(), (int)job.k, (int)job.n, job.groupsize,
                                 p.b_packed_vec.data(), p.scales_vec.data(), nullptr);
    return p;
}

// Phase 3 (marlin_proj.rs:150-181).
int upload_packed(const PackedHost &packed, int dev, kiln_marlin_packed_proj_t **out) {
    *out = nullptr;
    DeviceScope scope(dev);
    if (!scope.ok) return fail("marlin_proj: upload b_packed to device");
    auto w = std::make_unique<kiln_marlin_packed_proj>();
    w->k = packed.k;
    w->n = packed.n;
    w->groupsize = packed.groupsize;
    w->dev = dev;
    const size_t b_bytes = packed.b_packed_vec.size() * sizeof(int32_t);
    const size_t s_bytes = packed.scales_vec.size() * sizeof(uint16_t);
    if (hipMalloc(&w->b_packed, b_bytes) != hipSuccess ||
        hipMemcpy(w->b_packed, packed.b_packed_vec.data(), b_bytes, hipMemcpyHostToDevice) != hipSuccess) {
        if (w->b_packed) (void)hipFree(w->b_packed);
        return fail("marlin_proj: upload b_packed to device");
    }
    if (hipMalloc(&w->scales, s_bytes) != hipSuccess ||
        hipMemcpy(w->scales, packed.scales_vec.data(), s_bytes, hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipFree(w->b_packed);
        if (w->scales) (void)hipFree(w->scales);
        return fail("marlin_proj: upload scales to device");
    }
    *out = w.release();
    return KILN_PROJ_OK;
}

// The three phases in one: the weight is quantised and packed where it lies, by two kernels on the
// device's default stream (same bits as the host quantiser; KILN_W4A16_HOST_PACK=1 keeps the host
// route of marlin_proj.rs:86-181).  Same validation, same results and messages as prepare_pack_job.
int pack_on_device(const void *weight_t, int64_t k, int64_t n, int groupsize, int dev,
                   kiln_marlin_packed_proj_t **out) {
    *out = nullptr;
    if (dev < 0) return KILN_PROJ_SKIPPED;
    if (!weight_t) return fail("marlin_proj: weight_t must be a 2D [k, n] tensor");
    if (!shape_is_supported(k, n)) return KILN_PROJ_SKIPPED;
    if (!(groupsize == -1 || groupsize == 128))
        return fail("marlin_proj: groupsize must be -1 or 128 (got " + std::to_string(groupsize) + ")");
    if (k > INT32_MAX || n > INT32_MAX) return fail("marlin_proj: weight too large");
    DeviceScope scope(dev);
    if (!scope.ok) return fail("marlin_proj: pack on device");
    auto w = std::make_unique<kiln_marlin_packed_proj>();
    w->k = k;
    w->n = n;
    w->groupsize = groupsize;
    w->dev = dev;
    const size_t b_bytes = (size_t)k * n / 8 * sizeof(int32_t);
    const size_t s_bytes = num_groups(k, groupsize) * (size_t)n * sizeof(uint16_t);
    if (hipMalloc(&w->b_packed, b_bytes) != hipSuccess) return fail("marlin_proj: allocate b_packed on device");
    if (hipMalloc(&w->scales, s_bytes) != hipSuccess) {
        (void)hipFree(w->b_packed);
        return fail("marlin_proj: allocate scales on device");
    }
    const int st = kiln_w4a16_quantize_and_pack_device(weight_t, (int)k, (int)n, groupsize, w->b_packed, w->scales, dev,
                                                       nullptr);
    if (st != KILN_W4A16_OK || hipStreamSynchronize(nullptr) != hipSuccess) {
        (void)hipFree(w->b_packed);
        (void)hipFree(w->scales);
        return fail(std::string("marlin_proj: pack on device: ") + kiln_w4a16_status_string((kiln_marlin_status_t)st));
    }
    *out = w.release();
    return KILN_PROJ_OK;
}

// marlin_proj.rs:198-207
int pack_from_bf16(const void *weight_t, int64_t k, int64_t n, int groupsize, int dev,
                   kiln_marlin_packed_proj_t **out) {
    *out = nullptr;
    if (!env_truthy("KILN_W4A16_HOST_PACK")) return pack_on_device(weight_t, k, n, groupsize, dev, out);
    std::optional<PackJobHost> job;
    const int st = prepare_pack_job(weight_t, k, n, groupsize, dev, job);
    if (st != KILN_PROJ_OK) return st;
    return upload_packed(pack_host(*job), dev, out);
}

// marlin_proj.rs:230-262: serial downloads, parallel pack, serial uploads.
int pack_from_bf16_batch(const void *const *weights_t, const int64_t *ks, const int64_t *ns, const int *groupsizes,
                         int count, int dev, kiln_marlin_packed_proj_t **outs) {
    for (int i = 0; i < count; ++i) outs[i] = nullptr;
    if (count <= 0) return KILN_PROJ_OK;
    if (!env_truthy("KILN_W4A16_HOST_PACK")) {  // nothing to overlap: every weight is packed where it lies
        for (int i = 0; i < count; ++i) {
            const int st = pack_on_device(weights_t[i], ks[i], ns[i], groupsizes[i], dev, &outs[i]);
            if (st == KILN_PROJ_ERR) {
                for (int j = 0; j < i; ++j) {
                    kiln_marlin_proj_free(outs[j]);
                    outs[j] = nullptr;
                }
                return st;
            }
        }
        return KILN_PROJ_OK;
    }
    std::vector<std::optional<PackJobHost>> jobs((size_t)count);
    for (int i = 0; i < count; ++i) {
        const int st = prepare_pack_job(weights_t[i], ks[i], ns[i], groupsizes[i], dev, jobs[i]);
        if (st == KILN_PROJ_ERR) return st;
    }
    std::vector<std::optional<PackedHost>> packed((size_t)count);
    if (env_truthy("KILN_DISABLE_PARALLEL_PACK")) {
        for (int i = 0; i < count; ++i)
            if (jobs[i]) packed[i] = pack_host(*jobs[i]);
    } else {
        // a small pool over the jobs; each job's quantiser is itself threaded over columns,
        // so a few jobs at a time keep the cores busy without oversubscribing them
        std::atomic<int> next{0};
        const unsigned hw = std::max(1u, std::thread::hardware_concurrency());
        const int workers = std::min<int>(count, (int)std::max(1u, hw / 4));
        std::vector<std::thread> pool;
        for (int t = 0; t < workers; ++t)
            pool.emplace_back([&] {
                for (int i = next.fetch_add(1); i < count; i = next.fetch_add(1))
                    if (jobs[i]) packed[i] = pack_host(*jobs[i]);
            });
        for (auto &th : pool) th.join();
    }
    for (int i = 0; i < count; ++i) {
        if (!packed[i]) continue;
        jobs[i].reset();  // free the f32 copy before the next upload
        const int st = upload_packed(*packed[i], dev, &outs[i]);
        if (st != KILN_PROJ_OK) {
            for (int j = 0; j < i; ++j) {
                kiln_marlin_proj_free(outs[j]);
                outs[j] = nullptr;
            }
            return st;
        }
    }
    return KILN_PROJ_OK;
}

int pack_from_gptq(const int32_t *qweight, const uint16_t *scales_f16, const int32_t *qzeros, int64_t k, int64_t n,
                   int groupsize, int dev, kiln_marlin_packed_proj_t **out) {
    *out = nullptr;
    if (dev < 0 || !shape_is_supported(k, n)) return KILN_PROJ_SKIPPED;
    if (!(groupsize == -1 || groupsize == 128))
        return fail("marlin_proj: groupsize must be -1 or 128 (got " + std::to_string(groupsize) + ")");
    if (!env_truthy("KILN_W4A16_HOST_PACK")) {
        // the checkpoint's tensors go to the device as they are and are rearranged there (same bits)
        if (!qweight || !scales_f16) return fail("marlin_proj: repack: null or inconsistent argument");
        if (k > INT32_MAX || n > INT32_MAX) return fail("marlin_proj: weight too large");
        DeviceScope scope(dev);
        if (!scope.ok) return fail("marlin_proj: upload b_packed to device");
        const size_t q_bytes = (size_t)k / 8 * n * sizeof(int32_t);
        const size_t s_bytes = num_groups(k, groupsize) * (size_t)n * sizeof(uint16_t);
        const size_t z_bytes = qzeros ? num_groups(k, groupsize) * (size_t)(n / 8) * sizeof(int32_t) : 0;
        void *raw = nullptr;  // qweight | scales | qzeros, each 256-byte aligned
        const size_t s_off = (q_bytes + 255) / 256 * 256, z_off = s_off + (s_bytes + 255) / 256 * 256;
        auto w = std::make_unique<kiln_marlin_packed_proj>();
        w->k = k;
        w->n = n;
        w->groupsize = groupsize;
        w->dev = dev;
        bool ok = hipMalloc(&raw, z_off + z_bytes + 256) == hipSuccess && hipMalloc(&w->b_packed, q_bytes) == hipSuccess &&
                  hipMalloc(&w->scales, s_bytes) == hipSuccess;
        ok = ok && hipMemcpy(raw, qweight, q_bytes, hipMemcpyHostToDevice) == hipSuccess &&
             hipMemcpy((char *)raw + s_off, scales_f16, s_bytes, hipMemcpyHostToDevice) == hipSuccess &&
             (!qzeros || hipMemcpy((char *)raw + z_off, qzeros, z_bytes, hipMemcpyHostToDevice) == hipSuccess);
        int st = KILN_W4A16_ERR_LAUNCH;
        if (ok) {
            st = kiln_w4a16_repack_gptq_device(raw, (char *)raw + s_off, qzeros ? (char *)raw + z_off : nullptr, (int)k, (int)n,
                                               groupsize, w->b_packed, w->scales, dev, nullptr);
            if (st == KILN_W4A16_OK && hipStreamSynchronize(nullptr) != hipSuccess) st = KILN_W4A16_ERR_LAUNCH;
        }
        if (raw) (void)hipFree(raw);
        if (!ok || st != KILN_W4A16_OK) {
            if (w->b_packed) (void)hipFree(w->b_packed);
            if (w->scales) (void)hipFree(w->scales);
            if (!ok) return fail("marlin_proj: upload b_packed to device");
            return fail(std::string("marlin_proj: repack: ") + kiln_w4a16_status_string((kiln_marlin_status_t)st));
        }
        *out = w.release();
        return KILN_PROJ_OK;
    }
    PackedHost p;
    p.k = k;
    p.n = n;
    p.groupsize = groupsize;
    p.b_packed_vec.resize((size_t)k * n / 8);
    p.scales_vec.resize(num_groups(k, groupsize) * (size_t)n);
    const int st = kiln_w4a16_repack_gptq(qweight, scales_f16, qzeros, (int)k, (int)n, groupsize,
                                          p.b_packed_vec.data(), p.scales_vec.data());
    if (st != KILN_W4A16_OK) return fail(std::string("marlin_proj: repack: ") + kiln_w4a16_status_string(st));
    return upload_packed(p, dev, out);
}

// marlin_proj.rs:285-319
int matmul_bf16(const kiln_marlin_packed_proj_t *w, const void *x, const int64_t *dims, int rank, void *y,
                void *workspace, size_t workspace_bytes, void *stream) {
    if (!w || !x || !y || !dims) return fail("marlin_proj: null argument");
    int64_t m, k;
    if (rank == 2) {
        m = dims[0];
        k = dims[1];
    } else if (rank == 3) {
        m = dims[0] * dims[1];  // [batch, seq, k] flattened to [batch * seq, k]
        k = dims[2];
    } else {
        return fail("marlin_proj: unsupported activation rank " + std::to_string(rank));
    }
    if (k != w->k)
        return fail("marlin_proj: x last-dim " + std::to_string(k) + " != packed weight k " + std::to_string(w->k));
    if (m < 0 || m > INT32_MAX) return fail("marlin_proj: kernel call: m out of range");
    if (workspace_bytes < kiln_w4a16_workspace_bytes((int)m, (int)w->n, (int)w->k))
        return fail("marlin_proj: workspace smaller than kiln_w4a16_workspace_bytes(m, n, k)");
    const int st = kiln_marlin_w4a16_gemm(x, w->b_packed, y, w->scales, (int)m, (int)w->n, (int)w->k, workspace,
                                          w->groupsize, w->dev, stream, -1, -1, -1, 16);
    if (st != KILN_W4A16_OK)
        return fail(std::string("marlin_proj: kernel call (") + (rank == 2 ? "2D" : "3D flat") +
                    "): kiln-marlin-gemm: " + kiln_w4a16_status_string(st));
    return KILN_PROJ_OK;
}

// ---- persisted artefact ----------------------------------------------------

namespace {

struct ArtifactHeader {
    char magic[8];
    uint32_t layout_version;
    int32_t groupsize;
    uint64_t k, n, b_bytes, s_bytes, checksum, reserved;
};
static_assert(sizeof(ArtifactHeader) == 64, "header is 64 bytes");
const char kMagic[8] = {'K', 'W', '4', 'A', '1', '6', 0, 0};

uint64_t fnv1a(uint64_t h, const void *data, size_t len) {
    const unsigned char *p = static_cast<const unsigned char *>(data);
    for (size_t i = 0; i < len; ++i) h = (h ^ p[i]) * 0x100000001B3ull;
    return h;
}
constexpr uint64_t kFnvBasis = 0xCBF29CE484222325ull;

struct File {
    std::FILE *f;
    explicit File(const char *path, const char *mode) : f(std::fopen(path, mode)) {}
    ~File() {
        if (f) std::fclose(f);
    }
};

int read_header(std::FILE *f, const char *path, ArtifactHeader &h) {
    if (std::fread(&h, sizeof(h), 1, f) != 1) return fail(std::string("marlin_proj: artefact too short: ") + path);
    if (std::memcmp(h.magic, kMagic, 8) != 0) return fail(std::string("marlin_proj: not a packed-weight artefact: ") + path);
    if ((int)h.layout_version != kiln_w4a16_layout_version())
        return fail("marlin_proj: artefact layout version " + std::to_string(h.layout_version) + " != library's " +
                    std::to_string(kiln_w4a16_layout_version()) + ": repack " + path);
    // k and n are bounded before they are multiplied: a crafted header must not wrap the products
    constexpr uint64_t kMaxDim = 1ull << 30;
    if (!(h.groupsize == -1 || h.groupsize == 128) || h.k > kMaxDim || h.n > kMaxDim ||
        !shape_is_supported((int64_t)h.k, (int64_t)h.n) ||
        h.b_bytes != h.k * h.n / 2 || h.s_bytes != num_groups((int64_t)h.k, h.groupsize) * h.n * 2)
        return fail(std::string("marlin_proj: inconsistent artefact header: ") + path);
    return KILN_PROJ_OK;
}

}  // namespace

int artifact_write(const char *path, const int32_t *b_packed, const uint16_t *scales, int64_t k, int64_t n,
                   int groupsize) {
    if (!path || !b_packed || !scales) return fail("marlin_proj: null argument");
    if (!shape_is_supported(k, n) || !(groupsize == -1 || groupsize == 128))
        return fail("marlin_proj: artefact shape must have k % 128 == 0, n % 256 == 0, groupsize -1 or 128");
    ArtifactHeader h{};
    std::memcpy(h.magic, kMagic, 8);
    h.layout_version = (uint32_t)kiln_w4a16_layout_version();
    h.groupsize = groupsize;
    h.k = (uint64_t)k;
    h.n = (uint64_t)n;
    h.b_bytes = h.k * h.n / 2;
    h.s_bytes = num_groups(k, groupsize) * h.n * 2;
    h.checksum = fnv1a(fnv1a(kFnvBasis, b_packed, h.b_bytes), scales, h.s_bytes);
    File file(path, "wb");
    if (!file.f) return fail(std::string("marlin_proj: cannot open for writing: ") + path);
    if (std::fwrite(&h, sizeof(h), 1, file.f) != 1 || std::fwrite(b_packed, 1, h.b_bytes, file.f) != h.b_bytes ||
        std::fwrite(scales, 1, h.s_bytes, file.f) != h.s_bytes)
        return fail(std::string("marlin_proj: short write: ") + path);
    return KILN_PROJ_OK;
}

int artifact_info(const char *path, int64_t *k, int64_t *n, int *groupsize, int *layout_version) {
    if (!path) return fail("marlin_proj: null argument");
    File file(path, "rb");
    if (!file.f) return fail(std::string("marlin_proj: cannot open: ") + path);
    ArtifactHeader h;
    const int st = read_header(file.f, path, h);
    if (st != KILN_PROJ_OK) return st;
    if (k) *k = (int64_t)h.k;
    if (n) *n = (int64_t)h.n;
    if (groupsize) *groupsize = h.groupsize;
    if (layout_version) *layout_version = (int)h.layout_version;
    return KILN_PROJ_OK;
}

int artifact_read(const char *path, int32_t *b_packed, uint16_t *scales) {
    if (!path || !b_packed || !scales) return fail("marlin_proj: null argument");
    File file(path, "rb");
    if (!file.f) return fail(std::string("marlin_proj: cannot open: ") + path);
    ArtifactHeader h;
    const int st = read_header(file.f, path, h);
    if (st != KILN_PROJ_OK) return st;
    if (std::fread(b_packed, 1, h.b_bytes, file.f) != h.b_bytes || std::fread(scales, 1, h.s_bytes, file.f) != h.s_bytes)
        return fail(std::string("marlin_proj: artefact body truncated: ") + path);
    if (fnv1a(fnv1a(kFnvBasis, b_packed, h.b_bytes), scales, h.s_bytes) != h.checksum)
        return fail(std::string("marlin_proj: artefact checksum mismatch: ") + path);
    return KILN_PROJ_OK;
}

int save(const kiln_marlin_packed_proj_t *w, const char *path) {
    if (!w || !path) return fail("marlin_proj: null argument");
    DeviceScope scope(w->dev);
    if (!scope.ok) return fail("marlin_proj: download packed weight");
    std::vector<int32_t> b((size_t)w->k * w->n / 8);
    std::vector<uint16_t> s(num_groups(w->k, w->groupsize) * (size_t)w->n);
    if (hipMemcpy(b.data(), w->b_packed, b.size() * sizeof(int32_t), hipMemcpyDeviceToHost) != hipSuccess ||
        hipMemcpy(s.data(), w->scales, s.size() * sizeof(uint16_t), hipMemcpyDeviceToHost) != hipSuccess)
        return fail("marlin_proj: download packed weight");
    return artifact_write(path, b.data(), s.data(), w->k, w->n, w->groupsize);
}

int load(const char *path, int dev, kiln_marlin_packed_proj_t **out) {
    *out = nullptr;
    int64_t k, n;
    int groupsize, version;
    int st = artifact_info(path, &k, &n, &groupsize, &version);
    if (st != KILN_PROJ_OK) return st;
    PackedHost p;
    p.k = k;
    p.n = n;
    p.groupsize = groupsize;
    try {  // no exception may cross the C boundary
        p.b_packed_vec.resize((size_t)k * n / 8);
        p.scales_vec.resize(num_groups(k, groupsize) * (size_t)n);
    } catch (const std::exception &) {
        return fail(std::string("marlin_proj: out of host memory reading ") + path);
    }
    st = artifact_read(path, p.b_packed_vec.data(), p.scales_vec.data());
    if (st != KILN_PROJ_OK) return st;
    return upload_packed(p, dev, out);
}

}  // namespace proj
}  // namespace kiln

extern "C" {

using namespace kiln::proj;

int kiln_marlin_proj_shape_is_supported(int64_t k, int64_t n) { return shape_is_supported(k, n) ? 1 : 0; }
int kiln_marlin_proj_env_enabled(void) { return env_truthy("KILN_W4A16") ? 1 : 0; }
int kiln_marlin_proj_parallel_pack_disabled(void) { return env_truthy("KILN_DISABLE_PARALLEL_PACK") ? 1 : 0; }
int kiln_marlin_proj_bf16_drop_disabled(void) { return env_truthy("KILN_DISABLE_MARLIN_BF16_DROP") ? 1 : 0; }

int kiln_marlin_proj_pack_from_bf16(const void *weight_t, int64_t k, int64_t n, int groupsize, int dev,
                                    kiln_marlin_packed_proj_t **out) {
    if (!out) return fail("marlin_proj: null argument");
    return pack_from_bf16(weight_t, k, n, groupsize, dev, out);
}

int kiln_marlin_proj_pack_from_bf16_batch(const void *const *weights_t, const int64_t *ks, const int64_t *ns,
                                          const int *groupsizes, int count, int dev,
                                          kiln_marlin_packed_proj_t **outs) {
    if (count > 0 && (!weights_t || !ks || !ns || !groupsizes || !outs)) return fail("marlin_proj: null argument");
    return pack_from_bf16_batch(weights_t, ks, ns, groupsizes, count, dev, outs);
}

int kiln_marlin_proj_pack_from_gptq(const int32_t *qweight, const uint16_t *scales_f16, const int32_t *qzeros,
                                    int64_t k, int64_t n, int groupsize, int dev,
                                    kiln_marlin_packed_proj_t **out) {
    if (!out || !qweight || !scales_f16) return fail("marlin_proj: null argument");
    return pack_from_gptq(qweight, scales_f16, qzeros, k, n, groupsize, dev, out);
}

int kiln_marlin_proj_matmul_bf16(const kiln_marlin_packed_proj_t *w, const void *x, const int64_t *dims, int rank,
                                 void *y, void *workspace, size_t workspace_bytes, void *stream) {
    return matmul_bf16(w, x, dims, rank, y, workspace, workspace_bytes, stream);
}

int64_t kiln_marlin_proj_k(const kiln_marlin_packed_proj_t *w) { return w ? w->k : 0; }
int64_t kiln_marlin_proj_n(const kiln_marlin_packed_proj_t *w) { return w ? w->n : 0; }
int kiln_marlin_proj_groupsize(const kiln_marlin_packed_proj_t *w) { return w ? w->groupsize : 0; }
const void *kiln_marlin_proj_b_packed(const kiln_marlin_packed_proj_t *w) { return w ? w->b_packed : nullptr; }
const void *kiln_marlin_proj_scales(const kiln_marlin_packed_proj_t *w) { return w ? w->scales : nullptr; }

void kiln_marlin_proj_free(kiln_marlin_packed_proj_t *w) {
    if (!w) return;
    int prev = 0;
    const bool have_prev = hipGetDevice(&prev) == hipSuccess;
    if (hipSetDevice(w->dev) == hipSuccess) {
        (void)hipFree(w->b_packed);
        (void)hipFree(w->scales);
    }
    if (have_prev) (void)hipSetDevice(prev);
    delete w;
}

const char *kiln_marlin_proj_last_error(void) { return g_last_error.c_str(); }

int kiln_w4a16_artifact_write(const char *path, const int32_t *b_packed, const uint16_t *scales, int64_t k, int64_t n,
                              int groupsize) {
    return artifact_write(path, b_packed, scales, k, n, groupsize);
}
int kiln_w4a16_artifact_info(const char *path, int64_t *k, int64_t *n, int *groupsize, int *layout_version) {
    return artifact_info(path, k, n, groupsize, layout_version);
}
int kiln_w4a16_artifact_read(const char *path, int32_t *b_packed, uint16_t *scales) {
    return artifact_read(path, b_packed, scales);
}
int kiln_marlin_proj_save(const kiln_marlin_packed_proj_t *w, const char *path) { return save(w, path); }
int kiln_marlin_proj_load(const char *path, int dev, kiln_marlin_packed_proj_t **out) {
    if (!out) return fail("marlin_proj: null argument");
    return load(path, dev, out);
}

}  // extern "C"

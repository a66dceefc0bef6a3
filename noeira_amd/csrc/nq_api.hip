// The C ABI of libnoeira_qlinear.so (include/noeira_qlinear.h): argument
// checking, the layer's storage, and dispatch to the kernels.  No C++
// exception crosses the boundary and nothing here aborts; every failure is a
// status code plus a sentence for nq_last_error().
#include <algorithm>
#include <cstring>
#include <new>
#include <string>

#include "nq_common.h"

namespace nq {

static thread_local std::string g_last_error;

int32_t fail(int32_t code, const std::string& msg) {
    g_last_error = msg;
    return code;
}

hipError_t set_max_lds_once(LdsAttrOnce& st, const void* kernel, size_t bytes) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const bool tracked = dev >= 0 && dev < 64;
    if (tracked && st.done[dev]) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e == hipSuccess && tracked) st.done[dev] = true;
    return e;
}

int32_t fail_hip(hipError_t e, const char* what) {
    g_last_error = std::string("HIP error ") + hipGetErrorName(e) + " (" + hipGetErrorString(e) + ") in " + what;
    return NQ_ERR_HIP;
}

namespace {

const char* fmt_name(int f) {
    switch (f) {
        case NQ_FMT_Q4_0: return "Q4_0";
        case NQ_FMT_W8_CHANNEL: return "W8_CHANNEL";
        case NQ_FMT_W4_GROUP: return "W4_GROUP";
        case NQ_FMT_FP8_E4M3: return "FP8_E4M3";
    }
    return "?";
}

std::string shape_tag(const nq_layer* L) {
    return "QLinear[" + std::to_string(L->in) + ", " + std::to_string(L->out) + "]";
}

int64_t logical_bytes(const nq_layer* L) {
    switch (L->format) {
        case NQ_FMT_Q4_0: return (int64_t)L->out * (L->in / Q4_GROUP) * Q4_BLOCK;
        case NQ_FMT_W4_GROUP: return (int64_t)L->out * (L->in / 2);
        default: return (int64_t)L->out * L->in;
    }
}

void free_device(nq_layer* L) {
    if (L->d_codes) (void)hipFree(L->d_codes);
    if (L->d_scales) (void)hipFree(L->d_scales);
    if (L->d_zps) (void)hipFree(L->d_zps);
    if (L->d_tiled) (void)hipFree(L->d_tiled);
    if (L->d_tile16) (void)hipFree(L->d_tile16);
    if (L->d_tile16_scales) (void)hipFree(L->d_tile16_scales);
    L->d_codes = nullptr, L->d_scales = nullptr, L->d_zps = nullptr, L->d_tiled = nullptr;
    L->d_tile16 = nullptr, L->d_tile16_scales = nullptr, L->tile_nj = 0, L->tiled_bytes = 0;
}

int32_t check_handle(nq_handle h, const char* what) {
    if (!h) return fail(NQ_ERR_INVALID, std::string(what) + ": null layer handle");
    return NQ_OK;
}

// the `_need_blocks` rule of noeira/nn/quant/qlinear.mojo:358-369
int32_t need_loaded(const nq_layer* L, const char* what) {
    if (!L->loaded)
        return fail(NQ_ERR_NOT_LOADED,
                    std::string("QLinear.") + what + ": no weights (set_weight or set_blocks first)");
    return NQ_OK;
}

int32_t need_blocks(const nq_layer* L, const char* what) {
    int32_t rc = need_loaded(L, what);
    if (rc) return rc;
    if (!L->has_host_blocks)
        return fail(NQ_ERR_NO_BLOCKS, std::string("QLinear.") + what +
                                          ": no blocks are kept (keep_only_repacked); only the forward is left");
    return NQ_OK;
}

int32_t bind_device(nq_layer* L) {
    int dev = 0;
    NQ_HIP(hipGetDevice(&dev));
    if (L->device >= 0 && L->device != dev && L->loaded)
        return fail(NQ_ERR_INVALID, "layer was loaded on device " + std::to_string(L->device) +
                                        " but the current device is " + std::to_string(dev));
    L->device = dev;
    hinv_dev_setup();  // (set-up of the entry point that allocates nothing: its scratch array's address on this device)
    return NQ_OK;
}

// upload the split Q4_0 layout from raw blocks that already sit on the device
int32_t adopt_q4_0_blocks(nq_layer* L, const uint8_t* raw_dev, hipStream_t s) {
    const int64_t nblocks = (int64_t)L->out * (L->in / Q4_GROUP);
    free_device(L);
    NQ_HIP(hipMalloc((void**)&L->d_codes, (size_t)nblocks * 16 + 16));
    NQ_HIP(hipMalloc(&L->d_scales, (size_t)nblocks * 2 + 16));
    int32_t rc = launch_q4_0_repack(raw_dev, L->d_codes, reinterpret_cast<uint16_t*>(L->d_scales), nblocks, s);
    if (rc) return rc;
    L->row_bytes = (int64_t)(L->in / Q4_GROUP) * 16;
    return build_tile_copy(L, s);
}

}  // namespace
}  // namespace nq

using namespace nq;

extern "C" {

int32_t nq_abi_version(void) { return NQ_ABI_VERSION; }

int64_t nq_last_error(char* buf, int64_t n) {
    const std::string& e = g_last_error;
    if (buf && n > 0) {
        size_t k = std::min((size_t)(n - 1), e.size());
        std::memcpy(buf, e.data(), k);
        buf[k] = 0;
    }
    return (int64_t)e.size();
}

int32_t nq_create(nq_handle* out, int32_t format, int32_t in_features, int32_t out_features, int32_t group,
                  int32_t flags) {
    if (!out) return fail(NQ_ERR_INVALID, "nq_create: null output handle");
    *out = nullptr;
    if (format < NQ_FMT_Q4_0 || format > NQ_FMT_FP8_E4M3)
        return fail(NQ_ERR_INVALID, "nq_create: unknown format " + std::to_string(format));
    if (in_features <= 0 || out_features <= 0)
        return fail(NQ_ERR_INVALID, "nq_create: IN and OUT must be positive");
    if (flags & ~(NQ_FLAG_NO_TILE_COPY | NQ_FLAG_PREFER_TILE)) return fail(NQ_ERR_INVALID, "nq_create: unknown flags");
    if (format == NQ_FMT_Q4_0) {
        // qlinear.mojo:243-245
        if (in_features % Q4_GROUP != 0)
            return fail(NQ_ERR_INVALID, "QLinear: IN must be a multiple of 32 (one Q4_0 group)");
        if (group != 0 && group != Q4_GROUP)
            return fail(NQ_ERR_INVALID, "nq_create: Q4_0 groups are 32 wide");
        group = Q4_GROUP;
    } else if (format == NQ_FMT_W4_GROUP) {
        if (group <= 0 || group % 32 != 0)
            return fail(NQ_ERR_INVALID, "nq_create: W4_GROUP needs a group width that is a multiple of 32");
        if (in_features % 32 != 0)
            return fail(NQ_ERR_INVALID, "nq_create: W4_GROUP needs IN to be a multiple of 32");
    } else {
        if (in_features % 16 != 0)
            return fail(NQ_ERR_INVALID, std::string("nq_create: ") + fmt_name(format) +
                                            " needs IN to be a multiple of 16");
        group = 0;
    }
    nq_layer* L = new (std::nothrow) nq_layer();
    if (!L) return fail(NQ_ERR_INVALID, "nq_create: out of host memory");
    L->format = format, L->in = in_features, L->out = out_features, L->group = group;
    L->groups = group ? (in_features + group - 1) / group : 0;
    L->no_tile_copy = (flags & NQ_FLAG_NO_TILE_COPY) != 0;
    L->prefer_tile = (flags & NQ_FLAG_PREFER_TILE) != 0;
    *out = L;
    return NQ_OK;
}

int32_t nq_destroy(nq_handle h) {
    if (!h) return NQ_OK;
    free_device(h);
    delete h;
    return NQ_OK;
}

int32_t nq_set_blocks(nq_handle h, const uint8_t* blocks_host, int64_t nbytes, void* stream) {
    int32_t rc = check_handle(h, "nq_set_blocks");
    if (rc) return rc;
    if (h->format != NQ_FMT_Q4_0)
        return fail(NQ_ERR_INVALID, "nq_set_blocks: the layer's format is not Q4_0");
    const int64_t want = logical_bytes(h);
    if (nbytes != want)  // qlinear.mojo:276-281
        return fail(NQ_ERR_SIZE, shape_tag(h) + ".set_blocks: " + std::to_string(nbytes) + " bytes, expected " +
                                     std::to_string(want));
    if (!blocks_host) return fail(NQ_ERR_INVALID, "nq_set_blocks: null blocks");
    hipStream_t s = (hipStream_t)stream;
    h->loaded = false;
    if ((rc = bind_device(h))) return rc;
    h->host_blocks.assign(blocks_host, blocks_host + nbytes);
    h->has_host_blocks = true;
    uint8_t* raw = nullptr;
    NQ_HIP(hipMalloc((void**)&raw, (size_t)nbytes + 16));
    hipError_t e = hipMemcpyAsync(raw, h->host_blocks.data(), (size_t)nbytes, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) {
        rc = adopt_q4_0_blocks(h, raw, s);
        if (rc == NQ_OK) e = hipStreamSynchronize(s);
    }
    (void)hipFree(raw);
    if (e != hipSuccess) return fail_hip(e, "nq_set_blocks upload");
    if (rc) return rc;
    h->loaded = true;
    return NQ_OK;
}

int32_t nq_set_weight_f32(nq_handle h, const float* w_host, int64_t n_values, void* stream) {
    int32_t rc = check_handle(h, "nq_set_weight_f32");
    if (rc) return rc;
    if (h->format != NQ_FMT_Q4_0)
        return fail(NQ_ERR_INVALID, "nq_set_weight_f32: the layer's format is not Q4_0");
    const int64_t want = (int64_t)h->in * h->out;
    if (n_values != want)  // q4_0.mojo:139-143
        return fail(NQ_ERR_SIZE, "quantize_rtn_q4_0: " + std::to_string(n_values) + " values for a [" +
                                     std::to_string(h->out) + ", " + std::to_string(h->in) + "] weight");
    if (!w_host) return fail(NQ_ERR_INVALID, "nq_set_weight_f32: null weight");
    hipStream_t s = (hipStream_t)stream;
    h->loaded = false;
    if ((rc = bind_device(h))) return rc;
    const int64_t nbytes = logical_bytes(h);
    float* wd = nullptr;
    uint8_t* raw = nullptr;
    NQ_HIP(hipMalloc((void**)&wd, (size_t)want * 4));
    hipError_t e = hipMalloc((void**)&raw, (size_t)nbytes + 16);
    if (e != hipSuccess) {
        (void)hipFree(wd);
        return fail_hip(e, "nq_set_weight_f32 alloc");
    }
    h->host_blocks.resize((size_t)nbytes);
    e = hipMemcpyAsync(wd, w_host, (size_t)want * 4, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) rc = launch_q4_0_rtn(wd, raw, h->out, h->in, s);
    if (e == hipSuccess && rc == NQ_OK)
        e = hipMemcpyAsync(h->host_blocks.data(), raw, (size_t)nbytes, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess && rc == NQ_OK) rc = adopt_q4_0_blocks(h, raw, s);
    if (e == hipSuccess && rc == NQ_OK) e = hipStreamSynchronize(s);
    (void)hipFree(wd);
    (void)hipFree(raw);
    if (e != hipSuccess) return fail_hip(e, "nq_set_weight_f32");
    if (rc) return rc;
    h->has_host_blocks = true;
    h->loaded = true;
    return NQ_OK;
}

int32_t nq_set_weight_i8(nq_handle h, const int8_t* w_host, const float* scales_host, void* stream) {
    int32_t rc = check_handle(h, "nq_set_weight_i8");
    if (rc) return rc;
    if (h->format != NQ_FMT_W8_CHANNEL)
        return fail(NQ_ERR_INVALID, "nq_set_weight_i8: the layer's format is not W8_CHANNEL");
    if (!w_host || !scales_host) return fail(NQ_ERR_INVALID, "nq_set_weight_i8: null weight or scales");
    hipStream_t s = (hipStream_t)stream;
    h->loaded = false;
    if ((rc = bind_device(h))) return rc;
    free_device(h);
    const size_t n = (size_t)h->in * h->out;
    std::vector<uint8_t> tiled;
    if (h->in <= 256 && h->out <= 256) {
        // the fused MLP's copy: one contiguous KiB per (16-row tile, 64-k step), in the int8 MFMA's operand order
        const int tiles = (h->out + 15) / 16, steps = (h->in + 63) / 64;
        tiled.assign((size_t)tiles * steps * 1024, 0);
        for (int j = 0; j < tiles; j++)
            for (int st = 0; st < steps; st++)
                for (int l = 0; l < 64; l++) {
                    const int row = 16 * j + (l & 15), k0 = 64 * st + 16 * (l >> 4);
                    if (row >= h->out) continue;
                    for (int b = 0; b < 16 && k0 + b < h->in; b++)
                        tiled[((size_t)j * steps + st) * 1024 + 16 * l + b] = (uint8_t)w_host[(size_t)row * h->in + k0 + b];
                }
    }
    h->host_blocks.assign(reinterpret_cast<const uint8_t*>(w_host), reinterpret_cast<const uint8_t*>(w_host) + n);
    h->has_host_blocks = true;
    h->row_bytes = h->in;
    hipError_t e = hipMalloc((void**)&h->d_codes, n + 16);
    if (e == hipSuccess) e = hipMalloc(&h->d_scales, (size_t)h->out * 4 + 16);
    if (e == hipSuccess && !tiled.empty()) e = hipMalloc((void**)&h->d_tiled, tiled.size());
    h->tiled_bytes = (int64_t)tiled.size();
    if (e == hipSuccess) e = hipMemcpyAsync(h->d_codes, w_host, n, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipMemcpyAsync(h->d_scales, scales_host, (size_t)h->out * 4, hipMemcpyHostToDevice, s);
    if (e == hipSuccess && !tiled.empty())
        e = hipMemcpyAsync(h->d_tiled, tiled.data(), tiled.size(), hipMemcpyHostToDevice, s);
    if (e == hipSuccess) rc = build_tile_copy(h, s);
    if (e == hipSuccess && rc == NQ_OK) e = hipStreamSynchronize(s);  // (tiled is read by the copy until here)
    if (e != hipSuccess || rc) {
        free_device(h);
        return e != hipSuccess ? fail_hip(e, "nq_set_weight_i8 upload") : rc;
    }
    h->loaded = true;
    return NQ_OK;
}

int32_t nq_set_weight_w4g(nq_handle h, const uint8_t* codes_host, const uint16_t* scales_f16_host,
                          const uint8_t* zps_host, void* stream) {
    int32_t rc = check_handle(h, "nq_set_weight_w4g");
    if (rc) return rc;
    if (h->format != NQ_FMT_W4_GROUP)
        return fail(NQ_ERR_INVALID, "nq_set_weight_w4g: the layer's format is not W4_GROUP");
    if (!codes_host || !scales_f16_host || !zps_host)
        return fail(NQ_ERR_INVALID, "nq_set_weight_w4g: null codes, scales or zero-points");
    hipStream_t s = (hipStream_t)stream;
    h->loaded = false;
    if ((rc = bind_device(h))) return rc;
    free_device(h);
    const size_t n = (size_t)h->out * (h->in / 2);
    const size_t ng = (size_t)h->out * h->groups;
    const size_t nz = (size_t)h->out * ((h->groups + 1) / 2);
    uint8_t* zp_packed = nullptr;
    h->host_blocks.assign(codes_host, codes_host + n);
    h->has_host_blocks = true;
    h->row_bytes = h->in / 2;
    hipError_t e = hipMalloc((void**)&h->d_codes, n + 16);
    if (e == hipSuccess) e = hipMalloc(&h->d_scales, ng * 2 + 16);
    if (e == hipSuccess) e = hipMalloc((void**)&h->d_zps, ng + 16);
    if (e == hipSuccess) e = hipMalloc((void**)&zp_packed, nz + 16);
    if (e == hipSuccess) e = hipMemcpyAsync(h->d_codes, codes_host, n, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipMemcpyAsync(h->d_scales, scales_f16_host, ng * 2, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipMemcpyAsync(zp_packed, zps_host, nz, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) rc = launch_w4g_unpack_zps(zp_packed, h->d_zps, h->out, h->groups, s);
    if (e == hipSuccess && rc == NQ_OK) rc = launch_w4g_repack(h->d_codes, (int64_t)h->out * (h->in / 32), s);
    if (e == hipSuccess && rc == NQ_OK) rc = build_tile_copy(h, s);
    if (e == hipSuccess && rc == NQ_OK) e = hipStreamSynchronize(s);
    (void)hipFree(zp_packed);
    if (e != hipSuccess || rc) {
        free_device(h);
        return e != hipSuccess ? fail_hip(e, "nq_set_weight_w4g upload") : rc;
    }
    h->loaded = true;
    return NQ_OK;
}

int32_t nq_set_weight_fp8(nq_handle h, const uint8_t* w_host, float scale, void* stream) {
    int32_t rc = check_handle(h, "nq_set_weight_fp8");
    if (rc) return rc;
    if (h->format != NQ_FMT_FP8_E4M3)
        return fail(NQ_ERR_INVALID, "nq_set_weight_fp8: the layer's format is not FP8_E4M3");
    if (!w_host) return fail(NQ_ERR_INVALID, "nq_set_weight_fp8: null weight");
    hipStream_t s = (hipStream_t)stream;
    h->loaded = false;
    if ((rc = bind_device(h))) return rc;
    free_device(h);
    const size_t n = (size_t)h->in * h->out;
    h->host_blocks.assign(w_host, w_host + n);
    h->has_host_blocks = true;
    hipError_t e = hipMalloc((void**)&h->d_codes, n + 16);
    if (e == hipSuccess) e = hipMemcpyAsync(h->d_codes, w_host, n, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) {
        free_device(h);
        return fail_hip(e, "nq_set_weight_fp8 upload");
    }
    h->scale = scale;
    h->row_bytes = h->in;
    h->loaded = true;
    return NQ_OK;
}

int64_t nq_blocks_bytes(nq_handle h) {
    if (!h) return 0;
    return logical_bytes(h);
}

int32_t nq_get_blocks(nq_handle h, uint8_t* out_host, int64_t nbytes) {
    int32_t rc = check_handle(h, "nq_get_blocks");
    if (rc) return rc;
    if ((rc = need_blocks(h, "blocks"))) return rc;
    if (nbytes != (int64_t)h->host_blocks.size())
        return fail(NQ_ERR_SIZE, shape_tag(h) + ".blocks: a buffer of " + std::to_string(nbytes) +
                                     " bytes, expected " + std::to_string(h->host_blocks.size()));
    if (!out_host) return fail(NQ_ERR_INVALID, "nq_get_blocks: null buffer");
    std::memcpy(out_host, h->host_blocks.data(), (size_t)nbytes);
    return NQ_OK;
}

int64_t nq_device_bytes(nq_handle h) {
    if (!h || !h->loaded) return 0;
    const int64_t rows = h->out;
    int64_t n = rows * h->row_bytes;
    switch (h->format) {
        case NQ_FMT_Q4_0: n += rows * (h->in / Q4_GROUP) * 2; break;
        case NQ_FMT_W4_GROUP: n += rows * h->groups * 3; break;  // fp16 scale + one byte of zero point per group
        case NQ_FMT_W8_CHANNEL: n += rows * 4; break;
        default: break;
    }
    if (h->d_tiled) n += h->tiled_bytes;
    if (h->d_tile16) {
        const int64_t tiles = (rows + 15) / 16 * h->tile_nj;
        n += tiles * 1024;
        if (h->d_tile16_scales) n += tiles * 16 * (h->format == NQ_FMT_W4_GROUP ? 4 : 8);
    }
    return n;
}

int32_t nq_keep_only_repacked(nq_handle h) {
    int32_t rc = check_handle(h, "nq_keep_only_repacked");
    if (rc) return rc;
    if ((rc = need_loaded(h, "keep_only_repacked"))) return rc;
    std::vector<uint8_t>().swap(h->host_blocks);
    h->has_host_blocks = false;
    return NQ_OK;
}

namespace {

// a view of rows [r0, r1) of a loaded layer (no ownership; for per-part launches)
void row_view(const nq_layer* L, int r0, int r1, nq_layer* v) {
    v->format = L->format, v->in = L->in, v->out = r1 - r0, v->group = L->group, v->groups = L->groups;
    v->loaded = true, v->has_host_blocks = false, v->device = L->device;
    v->scale = L->scale, v->row_bytes = L->row_bytes;
    v->d_codes = L->d_codes + (int64_t)r0 * L->row_bytes;
    v->d_zps = L->d_zps ? L->d_zps + (int64_t)r0 * L->groups : nullptr;
    int64_t srow = 0;  // bytes of scale data per row
    switch (L->format) {
        case NQ_FMT_Q4_0: srow = (int64_t)(L->in / Q4_GROUP) * 2; break;
        case NQ_FMT_W4_GROUP: srow = (int64_t)L->groups * 2; break;
        case NQ_FMT_W8_CHANNEL: srow = 4; break;
        default: srow = 0;
    }
    v->d_scales = L->d_scales ? reinterpret_cast<uint8_t*>(L->d_scales) + r0 * srow : nullptr;
    // the tile-ordered copy is in units of 16 rows: a part that starts on one has its own view of it
    v->prefer_tile = L->prefer_tile, v->no_tile_copy = L->no_tile_copy;
    if (L->d_tile16 && r0 % 16 == 0) {
        const int64_t t0 = (int64_t)(r0 / 16) * L->tile_nj;
        v->d_tile16 = L->d_tile16 + t0 * 1024;
        if (L->d_tile16_scales)
            v->d_tile16_scales = reinterpret_cast<uint8_t*>(L->d_tile16_scales) + t0 * 16 * (L->format == NQ_FMT_W4_GROUP ? 4 : 8);
        v->tile_nj = L->tile_nj;
    }
}

int32_t dispatch(const ForwardArgs& a) {
    if (a.L->glu) {
        // gate | up pairs meet in the epilogue of the kernels whose result layout keeps a pair in one wavefront
        if (a.M == 1 && gemv_m1_applicable(a)) return launch_gemv_m1(a);
        if (gemm_tile_mt_applicable(a)) return launch_gemm_tile_mt(a);
        if (a.M >= 2 && gemm_a16_applicable(a)) return launch_gemm_a16(a);
        return fail(NQ_ERR_UNSUPPORTED, "nq_forward: no SwiGLU kernel for this shape (IN = " + std::to_string(a.L->in) +
                                            ", M = " + std::to_string(a.M) + "): run gate | up with nq_forward_fused "
                                            "and apply SwiGLU separately");
    }
    if (a.x_dtype == NQ_DT_I8) {
        if (tile8_i8_applicable(a)) return launch_tile8_i8(a);
        if (gemm8_applicable(a)) return launch_gemm8(a);
        return launch_gemv_i8(a);
    }
    if (gemv_fp8_applicable(a)) return launch_gemv_fp8(a);
    if (gemm8_applicable(a)) return launch_gemm8(a);
    if (gemv_tile_rows_applicable(a)) return launch_gemv_tile_rows(a);
    if (gemv_tile8_rows_applicable(a)) return launch_gemv_tile8_rows(a);
    if (gemm_tile_mt_applicable(a)) return launch_gemm_tile_mt(a);
    if (gemm_a16_applicable(a)) return launch_gemm_a16(a);
    if (gemv_tile_applicable(a)) return launch_gemv_tile(a);
    if (gemv_split8_applicable(a)) return launch_gemv_split8(a);
    if (gemv_row4_applicable(a)) return launch_gemv_row4(a);
    if (gemv_row8_applicable(a)) return launch_gemv_row8(a);
    if (gemv_m1_applicable(a)) return launch_gemv_m1(a);
    return launch_gemv(a);
}

// the kernels that place rows through the part table themselves (one launch for all parts)
bool places_parts(const ForwardArgs& a) {
    if (a.x_dtype == NQ_DT_I8) return false;
    if (gemv_fp8_applicable(a) || gemm8_applicable(a)) return false;
    if (gemm_tile_mt_splits_parts(a)) return false;  // wide and narrow parts: each on the kernel of its own layer
    // (the same between the medium-M and the many-rows kernel, where neither tile kernel takes the call)
    if (!gemv_tile_rows_applicable(a) && !gemv_tile8_rows_applicable(a) && !gemm_tile_mt_applicable(a) && gemm_a16_splits_parts(a)) return false;
    return gemv_tile_rows_applicable(a) || gemv_tile8_rows_applicable(a) || gemm_tile_mt_applicable(a) || gemm_a16_applicable(a) || gemv_tile_applicable(a) || gemv_split8_applicable(a) || gemv_row4_applicable(a) || gemv_row8_applicable(a) || gemv_m1_applicable(a);
}

// argument checks shared by nq_forward and nq_forward_fused, then the launch(es)
// (lora: an adapter to fold into the launch, or null; folded only where the M-tile kernel is the one that runs the
// base call anyway - `*folded` says whether it was)
struct LoraArgs {
    const float* a;
    const float* b;
    int32_t r;
    float s;
    // a gate | up layer's second adapter (the up projection's; a / b / s are then the gate's), or null
    const float* a2 = nullptr;
    const float* b2 = nullptr;
    float s2 = 0.0f;
};
int32_t forward_impl(nq_handle h, const void* x, int32_t x_dtype, const float* x_scale, const SegTable& seg,
                     int32_t y_dtype, int32_t M, const void* bias, int32_t bias_dtype, int32_t epilogue,
                     void* stream, const LoraArgs* lora = nullptr, bool* folded = nullptr, bool fold_or_fail = false) {
    if (((uintptr_t)x & 15)) return fail(NQ_ERR_INVALID, "nq_forward: x must be 16-byte aligned and y 4-byte aligned");
    for (int t = 0; t < seg.nseg; t++)
        if (!seg.y[t] || ((uintptr_t)seg.y[t] & 3))
            return fail(NQ_ERR_INVALID, "nq_forward: x must be 16-byte aligned and y 4-byte aligned");
    if (epilogue != NQ_EPI_NONE && epilogue != NQ_EPI_RELU && epilogue != NQ_EPI_SWIGLU)
        return fail(NQ_ERR_INVALID, "nq_forward: unknown epilogue " + std::to_string(epilogue));
    if (h->glu != (epilogue == NQ_EPI_SWIGLU))
        return fail(NQ_ERR_INVALID, h->glu ? "nq_forward: a layer made by nq_fuse_glu runs with NQ_EPI_SWIGLU only"
                                           : "nq_forward: NQ_EPI_SWIGLU needs a layer made by nq_fuse_glu");
    if (h->glu && (bias || (x_dtype != NQ_DT_F32 && x_dtype != NQ_DT_BF16) || seg.nseg != 1))
        return fail(NQ_ERR_INVALID, "nq_forward: a SwiGLU layer takes fp32 or bf16 activations, no bias, one output");
    if (bias && bias_dtype != NQ_DT_F32 && bias_dtype != NQ_DT_BF16)
        return fail(NQ_ERR_INVALID, "nq_forward: bias must be fp32 or bf16");
    if (x_dtype == NQ_DT_I8) {
        if (h->format != NQ_FMT_W8_CHANNEL)
            return fail(NQ_ERR_INVALID, "nq_forward: int8 activations need a W8_CHANNEL layer");
        if (y_dtype == NQ_DT_I32) {
            if (bias || epilogue != NQ_EPI_NONE)
                return fail(NQ_ERR_INVALID, "nq_forward: raw int32 accumulators take no bias or epilogue");
        } else {
            if (y_dtype != NQ_DT_F32 && y_dtype != NQ_DT_BF16)
                return fail(NQ_ERR_INVALID, "nq_forward: y must be fp32, bf16 or int32");
            if (!x_scale) return fail(NQ_ERR_INVALID, "nq_forward: int8 activations need per-row scales");
        }
    } else {
        if (y_dtype != NQ_DT_F32 && y_dtype != NQ_DT_BF16)
            return fail(NQ_ERR_INVALID, "nq_forward: y must be fp32 or bf16");
        if (x_dtype == NQ_DT_FP8_E4M3) {
            if (h->format != NQ_FMT_FP8_E4M3)
                return fail(NQ_ERR_INVALID, "nq_forward: fp8 activations need an FP8_E4M3 layer");
            if (!x_scale) return fail(NQ_ERR_INVALID, "nq_forward: fp8 activations need a scale");
        } else if (x_dtype != NQ_DT_F32 && x_dtype != NQ_DT_BF16) {
            return fail(NQ_ERR_INVALID, "nq_forward: unknown x dtype " + std::to_string(x_dtype));
        }
    }
    ForwardArgs a{h, x, x_dtype, x_scale, seg.y[0], y_dtype, M, bias, bias_dtype, epilogue, (hipStream_t)stream, seg};
    if (lora && seg.nseg == 1 && lora->r <= 16 && !h->glu && epilogue == NQ_EPI_NONE && x_dtype != NQ_DT_I8 &&
        !gemv_fp8_applicable(a) && !gemm8_applicable(a) && !gemv_tile_rows_applicable(a) && gemm_tile_mt_applicable(a) && gemm_tile_mt_lora_foldable(a)) {
        a.lora_a = lora->a, a.lora_b = lora->b, a.lora_r = lora->r, a.lora_s = lora->s;
        *folded = true;
        return launch_gemm_tile_mt(a);
    }
    if (lora && lora->a2) {
        // a gate | up layer: both adapters' shares enter the accumulators ahead of the SwiGLU epilogue, in the M-tile
        // kernel only (nothing can add them afterwards: the layer's only output is the activation's)
        if (h->glu && lora->r <= 16 && gemm_tile_mt_takes_shape(a) && gemm_tile_mt_lora_foldable(a)) {
            a.lora_a = lora->a, a.lora_b = lora->b, a.lora_r = lora->r, a.lora_s = lora->s;
            a.lora_a2 = lora->a2, a.lora_b2 = lora->b2, a.lora_s2 = lora->s2;
            *folded = true;
            return launch_gemm_tile_mt(a);
        }
        return fail(NQ_ERR_UNSUPPORTED, "nq_forward_fused_lora: for this layer and M no kernel adds adapters ahead of SwiGLU; "
                                        "fuse gate and up with nq_fuse_rows and pass glu_out");
    }
    // (decided before anything is launched: a caller whose y cannot take a second, adding launch gets its answer
    // with y untouched)
    if (lora && fold_or_fail)
        return fail(NQ_ERR_UNSUPPORTED, "nq_forward_lora: for this layer and M the adapter is a second launch that adds "
                                        "into an fp32 y; ask for fp32 output");
    if (seg.nseg == 1 || places_parts(a)) return dispatch(a);
    // one launch per part, each on a view of its rows
    const int bias_es = bias_dtype == NQ_DT_F32 ? 4 : 2;
    int r0 = 0;
    for (int t = 0; t < seg.nseg; t++) {
        nq_layer view;
        row_view(h, r0, seg.end[t], &view);
        ForwardArgs v = a;
        v.L = &view, v.y = seg.y[t];
        v.bias = bias ? reinterpret_cast<const uint8_t*>(bias) + (int64_t)r0 * bias_es : nullptr;
        v.seg.nseg = 1, v.seg.end[0] = view.out, v.seg.y[0] = seg.y[t];
        const int32_t rc = dispatch(v);
        if (rc) return rc;
        r0 = seg.end[t];
    }
    return NQ_OK;
}

}  // namespace

int32_t nq_forward(nq_handle h, const void* x, int32_t x_dtype, const float* x_scale, void* y, int32_t y_dtype,
                   int32_t M, const void* bias, int32_t bias_dtype, int32_t epilogue, void* stream) {
    int32_t rc = check_handle(h, "nq_forward");
    if (rc) return rc;
    if ((rc = need_loaded(h, "forward"))) return rc;
    if (M < 0) return fail(NQ_ERR_INVALID, "nq_forward: M must be >= 0");
    if (M == 0) return NQ_OK;
    if (!x || !y) return fail(NQ_ERR_INVALID, "nq_forward: null x or y");
    SegTable seg{};
    seg.nseg = 1, seg.end[0] = h->out, seg.y[0] = y;
    return forward_impl(h, x, x_dtype, x_scale, seg, y_dtype, M, bias, bias_dtype, epilogue, stream);
}

int32_t nq_fuse_rows(nq_handle* out, const nq_handle* layers, int32_t n, void* stream) {
    if (!out) return fail(NQ_ERR_INVALID, "nq_fuse_rows: null output handle");
    *out = nullptr;
    if (!layers || n < 1 || n > 4) return fail(NQ_ERR_INVALID, "nq_fuse_rows: between 1 and 4 layers can be fused");
    int64_t rows = 0;
    for (int i = 0; i < n; i++) {
        int32_t rc = check_handle(layers[i], "nq_fuse_rows");
        if (rc) return rc;
        if ((rc = need_loaded(layers[i], "fuse_rows"))) return rc;
        const nq_layer* a = layers[0];
        const nq_layer* b = layers[i];
        if (b->format != a->format || b->in != a->in || b->group != a->group || b->device != a->device)
            return fail(NQ_ERR_INVALID, "nq_fuse_rows: the layers must share format, IN, group width and device");
        if (a->format == NQ_FMT_FP8_E4M3 && b->scale != a->scale)
            return fail(NQ_ERR_INVALID, "nq_fuse_rows: FP8_E4M3 layers must share their per-tensor scale");
        if (!b->seg_end.empty() || b->glu) return fail(NQ_ERR_INVALID, "nq_fuse_rows: a fused layer cannot be fused again");
        rows += b->out;
    }
    if (rows > INT32_MAX) return fail(NQ_ERR_INVALID, "nq_fuse_rows: too many rows");
    const nq_layer* a = layers[0];
    nq_layer* F = new (std::nothrow) nq_layer();
    if (!F) return fail(NQ_ERR_INVALID, "nq_fuse_rows: out of host memory");
    F->format = a->format, F->in = a->in, F->out = (int32_t)rows, F->group = a->group, F->groups = a->groups;
    F->scale = a->scale, F->row_bytes = a->row_bytes, F->device = a->device;
    F->no_tile_copy = a->no_tile_copy, F->prefer_tile = a->prefer_tile;
    int32_t rc = bind_device(F);
    if (rc) {
        delete F;
        return rc;
    }
    int64_t scale_row = 0;
    switch (a->format) {
        case NQ_FMT_Q4_0: scale_row = (int64_t)(a->in / Q4_GROUP) * 2; break;
        case NQ_FMT_W4_GROUP: scale_row = (int64_t)a->groups * 2; break;
        case NQ_FMT_W8_CHANNEL: scale_row = 4; break;
        default: scale_row = 0;
    }
    hipStream_t s = (hipStream_t)stream;
    hipError_t e = hipMalloc((void**)&F->d_codes, (size_t)(rows * F->row_bytes) + 128);
    if (e == hipSuccess && scale_row) e = hipMalloc(&F->d_scales, (size_t)(rows * scale_row) + 128);
    if (e == hipSuccess && a->d_zps) e = hipMalloc((void**)&F->d_zps, (size_t)(rows * F->groups) + 128);
    int64_t r0 = 0;
    bool all_blocks = true;
    for (int i = 0; i < n && e == hipSuccess; i++) {
        const nq_layer* b = layers[i];
        e = hipMemcpyAsync(F->d_codes + r0 * F->row_bytes, b->d_codes, (size_t)(b->out * F->row_bytes),
                           hipMemcpyDeviceToDevice, s);
        if (e == hipSuccess && scale_row)
            e = hipMemcpyAsync(reinterpret_cast<uint8_t*>(F->d_scales) + r0 * scale_row, b->d_scales,
                               (size_t)(b->out * scale_row), hipMemcpyDeviceToDevice, s);
        if (e == hipSuccess && a->d_zps)
            e = hipMemcpyAsync(F->d_zps + r0 * F->groups, b->d_zps, (size_t)((int64_t)b->out * F->groups),
                               hipMemcpyDeviceToDevice, s);
        r0 += b->out;
        F->seg_end.push_back((int32_t)r0);
        all_blocks = all_blocks && b->has_host_blocks;
    }
    if (e == hipSuccess) rc = build_tile_copy(F, s);
    if (e == hipSuccess && rc == NQ_OK) e = hipStreamSynchronize(s);
    if (e != hipSuccess || rc) {
        free_device(F);
        delete F;
        return e != hipSuccess ? fail_hip(e, "nq_fuse_rows") : rc;
    }
    // the logical bytes are row-major over OUT in every format, so the fused layer's are the
    // concatenation (W4_GROUP's logical form is three arrays: not kept)
    if (all_blocks && a->format != NQ_FMT_W4_GROUP) {
        for (int i = 0; i < n; i++)
            F->host_blocks.insert(F->host_blocks.end(), layers[i]->host_blocks.begin(), layers[i]->host_blocks.end());
        F->has_host_blocks = true;
    }
    F->loaded = true;
    *out = F;
    return NQ_OK;
}

int32_t nq_fuse_glu(nq_handle* out, nq_handle gate, nq_handle up, void* stream) {
    if (!out) return fail(NQ_ERR_INVALID, "nq_fuse_glu: null output handle");
    *out = nullptr;
    nq_handle both[2] = {gate, up};
    for (int i = 0; i < 2; i++) {
        int32_t rc = check_handle(both[i], "nq_fuse_glu");
        if (rc) return rc;
        if ((rc = need_loaded(both[i], "fuse_glu"))) return rc;
        if (!both[i]->seg_end.empty() || both[i]->glu)
            return fail(NQ_ERR_INVALID, "nq_fuse_glu: a fused layer cannot be fused again");
    }
    const nq_layer* a = gate;
    const nq_layer* b = up;
    if (a->format == NQ_FMT_FP8_E4M3)
        return fail(NQ_ERR_UNSUPPORTED, "nq_fuse_glu: Q4_0, W4_GROUP and W8_CHANNEL layers only");
    if (b->format != a->format || b->in != a->in || b->out != a->out || b->group != a->group || b->device != a->device)
        return fail(NQ_ERR_INVALID, "nq_fuse_glu: gate and up must share format, IN, OUT, group width and device");
    if ((int64_t)a->out * 2 > INT32_MAX) return fail(NQ_ERR_INVALID, "nq_fuse_glu: too many rows");
    nq_layer* F = new (std::nothrow) nq_layer();
    if (!F) return fail(NQ_ERR_INVALID, "nq_fuse_glu: out of host memory");
    F->format = a->format, F->in = a->in, F->out = 2 * a->out, F->group = a->group, F->groups = a->groups;
    F->scale = a->scale, F->row_bytes = a->row_bytes, F->device = a->device;
    F->no_tile_copy = a->no_tile_copy, F->prefer_tile = a->prefer_tile;
    F->glu = true;  // (of the tile kernels only the M-tile one carries the SwiGLU epilogue: the others check `glu`)
    int32_t rc = bind_device(F);
    if (rc) {
        delete F;
        return rc;
    }
    int64_t scale_row = 0;
    switch (a->format) {
        case NQ_FMT_Q4_0: scale_row = (int64_t)(a->in / Q4_GROUP) * 2; break;
        case NQ_FMT_W4_GROUP: scale_row = (int64_t)a->groups * 2; break;
        default: scale_row = 4;  // W8_CHANNEL
    }
    const int64_t rows = F->out, H = a->out;
    hipStream_t s = (hipStream_t)stream;
    hipError_t e = hipMalloc((void**)&F->d_codes, (size_t)(rows * F->row_bytes) + 128);
    if (e == hipSuccess) e = hipMalloc(&F->d_scales, (size_t)(rows * scale_row) + 128);
    if (e == hipSuccess && a->d_zps) e = hipMalloc((void**)&F->d_zps, (size_t)(rows * F->groups) + 128);
    // row 2 n <- gate row n, row 2 n + 1 <- up row n: strided device copies, one per array and source
    for (int i = 0; i < 2 && e == hipSuccess; i++) {
        const nq_layer* src = both[i];
        e = hipMemcpy2DAsync(F->d_codes + i * F->row_bytes, (size_t)(2 * F->row_bytes), src->d_codes, (size_t)F->row_bytes,
                             (size_t)F->row_bytes, (size_t)H, hipMemcpyDeviceToDevice, s);
        if (e == hipSuccess)
            e = hipMemcpy2DAsync(reinterpret_cast<uint8_t*>(F->d_scales) + i * scale_row, (size_t)(2 * scale_row),
                                 src->d_scales, (size_t)scale_row, (size_t)scale_row, (size_t)H, hipMemcpyDeviceToDevice, s);
        if (e == hipSuccess && a->d_zps)
            e = hipMemcpy2DAsync(F->d_zps + i * F->groups, (size_t)(2 * F->groups), src->d_zps, (size_t)F->groups,
                                 (size_t)F->groups, (size_t)H, hipMemcpyDeviceToDevice, s);
    }
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e == hipSuccess) rc = build_tile_copy(F, s);
    if (e == hipSuccess && rc == NQ_OK) e = hipStreamSynchronize(s);
    if (e != hipSuccess || rc != NQ_OK) {
        free_device(F);
        delete F;
        return e != hipSuccess ? fail_hip(e, "nq_fuse_glu") : rc;
    }
    F->loaded = true;
    *out = F;
    return NQ_OK;
}

int32_t nq_fused_parts(nq_handle h) {
    if (!h) return 0;
    return h->seg_end.empty() ? 1 : (int32_t)h->seg_end.size();
}

int32_t nq_forward_fused(nq_handle h, const void* x, int32_t x_dtype, const float* x_scale, void* const* ys,
                         int32_t n_ys, int32_t y_dtype, int32_t M, const void* bias, int32_t bias_dtype,
                         int32_t epilogue, void* stream) {
    int32_t rc = check_handle(h, "nq_forward_fused");
    if (rc) return rc;
    if ((rc = need_loaded(h, "forward"))) return rc;
    const int parts = nq_fused_parts(h);
    if (n_ys != parts)
        return fail(NQ_ERR_INVALID, "nq_forward_fused: " + std::to_string(n_ys) + " outputs for a layer of " +
                                        std::to_string(parts) + " fused parts");
    if (M < 0) return fail(NQ_ERR_INVALID, "nq_forward: M must be >= 0");
    if (M == 0) return NQ_OK;
    if (!x || !ys) return fail(NQ_ERR_INVALID, "nq_forward: null x or y");
    SegTable seg{};
    seg.nseg = parts;
    for (int t = 0; t < parts; t++) {
        seg.end[t] = h->seg_end.empty() ? h->out : h->seg_end[t];
        seg.y[t] = ys[t];
        if (!ys[t]) return fail(NQ_ERR_INVALID, "nq_forward: null x or y");
    }
    return forward_impl(h, x, x_dtype, x_scale, seg, y_dtype, M, bias, bias_dtype, epilogue, stream);
}

int32_t nq_dequantize(nq_handle h, float* out_dev, int64_t n_values, void* stream) {
    int32_t rc = check_handle(h, "nq_dequantize");
    if (rc) return rc;
    if ((rc = need_loaded(h, "dequantized"))) return rc;
    if (!out_dev && n_values == 0) {  // into the workspace the caller shared
        if (!h->workspace) return fail(NQ_ERR_INVALID, "nq_dequantize: no output and no workspace (nq_set_workspace)");
        return launch_dequantize(h, h->workspace, (hipStream_t)stream);
    }
    if (n_values < (int64_t)h->in * h->out)  // qlinear.mojo:334-338
        return fail(NQ_ERR_SIZE, "QLinear.share_scratch: " + std::to_string(n_values) + " values for a [" +
                                     std::to_string(h->out) + ", " + std::to_string(h->in) + "] weight");
    if (!out_dev || ((uintptr_t)out_dev & 15))
        return fail(NQ_ERR_INVALID, "nq_dequantize: the output must be a 16-byte aligned device buffer");
    return launch_dequantize(h, out_dev, (hipStream_t)stream);
}

int64_t nq_workspace_bytes(nq_handle h, int32_t M) {
    (void)M;  // (no forward of this library dequantizes to memory: the scratch is nq_dequantize's alone)
    if (!h) return 0;
    return (int64_t)h->in * h->out * 4;
}

int32_t nq_set_workspace(nq_handle h, void* dev, int64_t nbytes) {
    int32_t rc = check_handle(h, "nq_set_workspace");
    if (rc) return rc;
    if (!dev && nbytes == 0) {
        h->workspace = nullptr, h->workspace_bytes = 0;
        return NQ_OK;
    }
    if (nbytes < nq_workspace_bytes(h, 0))  // qlinear.mojo:334-338
        return fail(NQ_ERR_SIZE, "QLinear.share_scratch: " + std::to_string(nbytes < 0 ? 0 : nbytes / 4) + " values for a [" +
                                     std::to_string(h->out) + ", " + std::to_string(h->in) + "] weight");
    if (!dev || ((uintptr_t)dev & 15))
        return fail(NQ_ERR_INVALID, "nq_set_workspace: the workspace must be a 16-byte aligned device buffer");
    h->workspace = reinterpret_cast<float*>(dev), h->workspace_bytes = nbytes;
    return NQ_OK;
}

int32_t nq_grad_input(nq_handle h, const float* gy, float* gx, int32_t M, void* stream) {
    int32_t rc = check_handle(h, "nq_grad_input");
    if (rc) return rc;
    if ((rc = need_blocks(h, "vjp"))) return rc;
    if (h->format != NQ_FMT_Q4_0) return fail(NQ_ERR_UNSUPPORTED, "nq_grad_input: Q4_0 layers only");
    if (M < 0) return fail(NQ_ERR_INVALID, "nq_grad_input: M must be >= 0");
    if (M == 0) return NQ_OK;
    if (!gy || !gx) return fail(NQ_ERR_INVALID, "nq_grad_input: null gy or gx");
    return launch_grad_input_q4_0(h, gy, gx, M, (hipStream_t)stream);
}

int32_t nq_forward_lora(nq_handle h, const void* x, int32_t x_dtype, void* y, int32_t y_dtype, int32_t M,
                        const void* bias, int32_t bias_dtype, const float* lora_a, const float* lora_b, int32_t r_pad,
                        float scale, void* stream) {
    int32_t rc = check_handle(h, "nq_forward_lora");
    if (rc) return rc;
    if ((rc = need_loaded(h, "forward"))) return rc;
    if (M < 0) return fail(NQ_ERR_INVALID, "nq_forward_lora: M must be >= 0");
    if (M == 0) return NQ_OK;
    if (!x || !y || !lora_a || !lora_b) return fail(NQ_ERR_INVALID, "nq_forward_lora: null pointer");
    if (r_pad <= 0) return fail(NQ_ERR_INVALID, "nq_forward_lora: R_PAD must be positive");
    if (x_dtype != NQ_DT_F32 && x_dtype != NQ_DT_BF16)
        return fail(NQ_ERR_INVALID, "nq_forward_lora: x must be fp32 or bf16");
    SegTable seg{};
    seg.nseg = 1, seg.end[0] = h->out, seg.y[0] = y;
    const LoraArgs lora{lora_a, lora_b, r_pad, scale};
    bool folded = false;
    rc = forward_impl(h, x, x_dtype, nullptr, seg, y_dtype, M, bias, bias_dtype, NQ_EPI_NONE, stream, &lora, &folded,
                      /*fold_or_fail=*/y_dtype != NQ_DT_F32);
    if (rc || folded) return rc;
    // the base call ran on another kernel: the adapter as a launch of its own, into the fp32 output
    return nq_lora_forward_add(lora_a, lora_b, h->in, h->out, r_pad, scale, x, x_dtype, reinterpret_cast<float*>(y), M,
                               stream);
}

int32_t nq_forward_fused_lora(nq_handle h, const void* x, int32_t x_dtype, float* const* ys, int32_t n_ys, int32_t M,
                              const void* bias, int32_t bias_dtype, const nq_lora_part* adapters, void* glu_out,
                              int32_t glu_dtype, void* stream) {
    int32_t rc = check_handle(h, "nq_forward_fused_lora");
    if (rc) return rc;
    if ((rc = need_loaded(h, "forward"))) return rc;
    const int parts = nq_fused_parts(h);
    if (h->glu) {
        // a gate | up layer (nq_fuse_glu): adapters[0] is the gate projection's, adapters[1] the up projection's; the
        // only output is glu_out [M, OUT / 2] (ys is not read)
        if (M < 0) return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: M must be >= 0");
        if (M == 0) return NQ_OK;
        if (!x || !adapters || !glu_out) return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: null pointer");
        if (bias) return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: a SwiGLU pair takes no bias");
        if (glu_dtype != NQ_DT_F32 && glu_dtype != NQ_DT_BF16)
            return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: glu_out must be fp32 or bf16");
        const nq_lora_part &g = adapters[0], &u = adapters[1];
        for (const nq_lora_part* ad : {&g, &u})
            if ((ad->a == nullptr) != (ad->b == nullptr) || (ad->a && ad->r_pad <= 0))
                return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: an adapter is (a, b, r_pad > 0) or all null");
        SegTable seg{};
        seg.nseg = 1, seg.end[0] = h->out, seg.y[0] = glu_out;
        if (!g.a && !u.a) return forward_impl(h, x, x_dtype, nullptr, seg, glu_dtype, M, nullptr, NQ_DT_F32, NQ_EPI_SWIGLU, stream);
        if (!g.a || !u.a || g.r_pad != u.r_pad)
            return fail(NQ_ERR_UNSUPPORTED, "nq_forward_fused_lora: a layer made by nq_fuse_glu takes adapters on both projections, "
                                            "of one padded rank; otherwise fuse gate and up with nq_fuse_rows and pass glu_out");
        LoraArgs lora{g.a, g.b, g.r_pad, g.scale};
        lora.a2 = u.a, lora.b2 = u.b, lora.s2 = u.scale;
        bool folded = false;
        return forward_impl(h, x, x_dtype, nullptr, seg, glu_dtype, M, nullptr, NQ_DT_F32, NQ_EPI_SWIGLU, stream, &lora, &folded, true);
    }
    if (n_ys != parts)
        return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: " + std::to_string(n_ys) + " outputs for a layer of " +
                                        std::to_string(parts) + " fused parts");
    if (M < 0) return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: M must be >= 0");
    if (M == 0) return NQ_OK;
    if (!x || !ys || !adapters) return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: null pointer");
    if (x_dtype != NQ_DT_F32 && x_dtype != NQ_DT_BF16)
        return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: x must be fp32 or bf16");
    SegTable seg{};
    seg.nseg = parts;
    LoraPartArgs lp[4];
    int r0 = 0;
    for (int t = 0; t < parts; t++) {
        seg.end[t] = h->seg_end.empty() ? h->out : h->seg_end[t];
        seg.y[t] = ys[t];
        if (!ys[t]) return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: null output");
        const nq_lora_part& ad = adapters[t];
        if ((ad.a == nullptr) != (ad.b == nullptr) || (ad.a && ad.r_pad <= 0))
            return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: an adapter is (a, b, r_pad > 0) or all null");
        const int width = seg.end[t] - r0;
        if ((int64_t)M * h->in >= ((int64_t)1 << 32) || (int64_t)M * width >= ((int64_t)1 << 32))
            return fail(NQ_ERR_UNSUPPORTED, "nq_forward_fused_lora: M * IN and M * OUT must stay below 2^32");
        lp[t] = LoraPartArgs{ad.a, ad.b, ys[t], width, ad.r_pad, ad.scale};
        r0 = seg.end[t];
    }
    if (glu_out) {
        if (parts != 2 || lp[0].out != lp[1].out)
            return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: glu_out needs a layer of two parts of equal width (gate, up)");
        if (glu_dtype != NQ_DT_F32 && glu_dtype != NQ_DT_BF16)
            return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: glu_out must be fp32 or bf16");
        if (bias) return fail(NQ_ERR_INVALID, "nq_forward_fused_lora: a SwiGLU pair takes no bias");
    }
    rc = forward_impl(h, x, x_dtype, nullptr, seg, NQ_DT_F32, M, bias, bias_dtype, NQ_EPI_NONE, stream);
    if (rc) return rc;
    return launch_lora_multi(x, x_dtype, M, h->in, parts, lp, glu_out, glu_dtype, (hipStream_t)stream);
}

int32_t nq_lora_forward_add(const float* a, const float* b, int32_t in_features, int32_t out_features, int32_t r_pad,
                            float scale, const void* x, int32_t x_dtype, float* y, int32_t T, void* stream) {
    if (in_features <= 0 || out_features <= 0 || r_pad <= 0)
        return fail(NQ_ERR_INVALID, "LoRAAdapter.forward_add: IN, OUT and R_PAD must be positive");
    if (x_dtype != NQ_DT_F32 && x_dtype != NQ_DT_BF16)
        return fail(NQ_ERR_INVALID, "LoRAAdapter.forward_add: x must be fp32 or bf16");
    if (T < 0) return fail(NQ_ERR_INVALID, "LoRAAdapter.forward_add: T must be >= 0");
    if (T == 0) return NQ_OK;
    if (!a || !b || !x || !y) return fail(NQ_ERR_INVALID, "LoRAAdapter.forward_add: null pointer");
    if ((int64_t)T * in_features >= ((int64_t)1 << 32) || (int64_t)T * out_features >= ((int64_t)1 << 32))
        return fail(NQ_ERR_UNSUPPORTED, "LoRAAdapter.forward_add: T * IN and T * OUT must stay below 2^32 (the kernel "
                                        "addresses x and y with 32-bit element offsets)");
    return launch_lora_add(x, x_dtype, a, b, y, T, in_features, out_features, r_pad, scale, (hipStream_t)stream);
}

// ---- GPTQ (load time) ------------------------------------------------------------------------
struct nq_hessian_s {
    uint32_t magic = 0x4E514853u;  // "NQHS"
    int32_t n = 0;
    int64_t rows = 0;
    int device = -1;
    double* d_h = nullptr;
    hipStream_t last_stream = nullptr;  // the stream of the last nq_hessian_add: a reader on another stream waits for it
    bool pending = false;
};

// a call that reads H on `s` after nq_hessian_add enqueued on another stream waits for that stream first
static hipError_t hessian_order(nq_hessian h, hipStream_t s) {
    if (!h->pending || h->last_stream == s) return hipSuccess;
    const hipError_t e = hipStreamSynchronize(h->last_stream);
    if (e == hipSuccess) h->pending = false;
    return e;
}

static int32_t check_hessian(nq_hessian h, const char* what) {
    if (!h || h->magic != 0x4E514853u) return fail(NQ_ERR_INVALID, std::string(what) + ": not a Hessian handle");
    int dev = 0;
    NQ_HIP(hipGetDevice(&dev));
    if (dev != h->device)
        return fail(NQ_ERR_INVALID, std::string(what) + ": the Hessian lives on device " + std::to_string(h->device) +
                                        " but the current device is " + std::to_string(dev));
    return NQ_OK;
}

int32_t nq_hessian_create(nq_hessian* out, int32_t n) {
    if (!out) return fail(NQ_ERR_INVALID, "nq_hessian_create: null output handle");
    *out = nullptr;
    if (n <= 0) return fail(NQ_ERR_INVALID, "nq_hessian_create: n must be positive");
    nq_hessian h = new (std::nothrow) nq_hessian_s();
    if (!h) return fail(NQ_ERR_HIP, "nq_hessian_create: out of host memory");
    h->n = n;
    hipError_t e = hipGetDevice(&h->device);
    if (e == hipSuccess) hinv_dev_setup();
    if (e == hipSuccess) e = hipMalloc((void**)&h->d_h, (size_t)n * n * 8);
    if (e == hipSuccess) e = hipMemset(h->d_h, 0, (size_t)n * n * 8);
    if (e != hipSuccess) {
        (void)hipFree(h->d_h);
        delete h;
        return fail_hip(e, "nq_hessian_create");
    }
    *out = h;
    return NQ_OK;
}

int32_t nq_hessian_destroy(nq_hessian h) {
    if (!h) return NQ_OK;
    if (h->magic != 0x4E514853u) return fail(NQ_ERR_INVALID, "nq_hessian_destroy: not a Hessian handle");
    (void)hipFree(h->d_h);
    h->magic = 0;
    delete h;
    return NQ_OK;
}

int32_t nq_hessian_add(nq_hessian h, const void* x, int32_t x_dtype, int32_t rows, void* stream) {
    int32_t rc = check_hessian(h, "HessianAccumulator.add");
    if (rc) return rc;
    if (x_dtype != NQ_DT_F32 && x_dtype != NQ_DT_BF16)
        return fail(NQ_ERR_INVALID, "HessianAccumulator.add: the slab must be fp32 or bf16");
    if (rows < 0) return fail(NQ_ERR_INVALID, "HessianAccumulator.add: rows must be >= 0");
    if (rows == 0) return NQ_OK;
    if (!x) return fail(NQ_ERR_INVALID, "HessianAccumulator.add: null slab");
    NQ_HIP(hessian_order(h, (hipStream_t)stream));  // (adds on two streams: the second waits for the first)
    rc = launch_hessian_add(h->d_h, h->n, x, x_dtype, rows, (hipStream_t)stream);
    if (rc == NQ_OK) h->rows += rows, h->last_stream = (hipStream_t)stream, h->pending = true;
    return rc;
}

int64_t nq_hessian_rows(nq_hessian h) { return (h && h->magic == 0x4E514853u) ? h->rows : -1; }

int32_t nq_hessian_get(nq_hessian h, double* out_host, int64_t count) {
    int32_t rc = check_hessian(h, "nq_hessian_get");
    if (rc) return rc;
    if (!out_host || count != (int64_t)h->n * h->n)
        return fail(NQ_ERR_SIZE, "nq_hessian_get: the buffer must hold n * n = " +
                                     std::to_string((int64_t)h->n * h->n) + " values");
    NQ_HIP(hipDeviceSynchronize());
    h->pending = false;
    NQ_HIP(hipMemcpy(out_host, h->d_h, (size_t)count * 8, hipMemcpyDeviceToHost));
    return NQ_OK;
}

int32_t nq_hessian_set(nq_hessian h, const double* h_host, int64_t count, int64_t rows) {
    int32_t rc = check_hessian(h, "nq_hessian_set");
    if (rc) return rc;
    if (!h_host || count != (int64_t)h->n * h->n)
        return fail(NQ_ERR_SIZE, "nq_hessian_set: expected n * n = " + std::to_string((int64_t)h->n * h->n) +
                                     " values");
    NQ_HIP(hipDeviceSynchronize());
    h->pending = false;
    NQ_HIP(hipMemcpy(h->d_h, h_host, (size_t)count * 8, hipMemcpyHostToDevice));
    h->rows = rows;
    return NQ_OK;
}

int32_t nq_hinv_upper_f64(const double* h_host, int32_t n, double* u_host, void* stream) {
    if (!h_host || !u_host || n <= 0) return fail(NQ_ERR_INVALID, "hinv_upper_f64: null matrix or n <= 0");
    hipStream_t s = (hipStream_t)stream;
    const size_t bytes = (size_t)n * n * 8;
    double *hd = nullptr, *ud = nullptr;
    int* status = nullptr;
    hipError_t e = hipMalloc((void**)&hd, bytes);
    if (e == hipSuccess) e = hipMalloc((void**)&ud, bytes);
    if (e == hipSuccess) e = hipMalloc((void**)&status, 4);
    const int big = 0x7FFFFFFF;
    int pivot = big;
    int32_t rc = NQ_OK;
    if (e == hipSuccess) e = hipMemcpyAsync(hd, h_host, bytes, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipMemcpyAsync(status, &big, 4, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) rc = launch_hinv_upper_f64(hd, n, ud, status, s);
    if (e == hipSuccess && rc == NQ_OK) e = hipMemcpyAsync(u_host, ud, bytes, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess && rc == NQ_OK) e = hipMemcpyAsync(&pivot, status, 4, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess && rc == NQ_OK) e = hipStreamSynchronize(s);
    (void)hipFree(hd), (void)hipFree(ud), (void)hipFree(status);
    if (e != hipSuccess) return fail_hip(e, "hinv_upper_f64");
    if (rc) return rc;
    if (pivot != big)  // the factorization runs on the index-reversed matrix
        return fail(NQ_ERR_INVALID, "cholesky_f64: not positive definite (pivot " + std::to_string(pivot) + ")");
    return NQ_OK;
}

int32_t nq_hinv_upper_f64_dev(const double* h_dev, int32_t n, double* u_dev, int32_t* pivot_dev, void* stream) {
    if (!h_dev || !u_dev || !pivot_dev || n <= 0)
        return fail(NQ_ERR_INVALID, "hinv_upper_f64_dev: null matrix, null pivot or n <= 0");
    if (n > hinv_dev_max_n())
        return fail(NQ_ERR_SIZE, "hinv_upper_f64_dev: n = " + std::to_string(n) + " exceeds the " +
                                     std::to_string(hinv_dev_max_n()) + " the library's fixed scratch holds "
                                     "(nq_hinv_upper_f64 takes any n)");
    if (((uintptr_t)h_dev & 7) || ((uintptr_t)u_dev & 7) || ((uintptr_t)pivot_dev & 3))
        return fail(NQ_ERR_INVALID, "hinv_upper_f64_dev: misaligned pointer");
    return run_hinv_upper_f64_dev(h_dev, n, u_dev, pivot_dev, (hipStream_t)stream);
}

int32_t nq_set_weight_gptq(nq_handle h, const float* w_host, int64_t n_values, nq_hessian hess, double damp_frac,
                           int64_t* dead_out, double* damp_out, void* stream) {
    int32_t rc = check_handle(h, "nq_set_weight_gptq");
    if (rc) return rc;
    if (h->format != NQ_FMT_Q4_0) return fail(NQ_ERR_INVALID, "nq_set_weight_gptq: the layer's format is not Q4_0");
    if ((rc = check_hessian(hess, "gptq_q4_0"))) return rc;
    const int64_t want = (int64_t)h->in * h->out;
    if (n_values < want || hess->n != h->in)  // gptq.mojo:80-83
        return fail(NQ_ERR_SIZE, "gptq_q4_0: w or h is smaller than [n, k] / [k, k] (w holds " +
                                     std::to_string(n_values) + " values, h is " + std::to_string(hess->n) + " x " +
                                     std::to_string(hess->n) + ", the layer is [" + std::to_string(h->out) + ", " +
                                     std::to_string(h->in) + "])");
    if (!w_host) return fail(NQ_ERR_INVALID, "nq_set_weight_gptq: null weight");
    if (!(damp_frac >= 0)) return fail(NQ_ERR_INVALID, "nq_set_weight_gptq: damp_frac must be >= 0");
    hipStream_t s = (hipStream_t)stream;
    h->loaded = false;
    if ((rc = bind_device(h))) return rc;
    const int64_t nbytes = logical_bytes(h);
    const size_t hbytes = (size_t)h->in * h->in * 8;
    float* wd = nullptr;
    uint8_t* raw = nullptr;
    double* hd = nullptr;
    hipError_t e = hessian_order(hess, s);
    if (e == hipSuccess) e = hipMalloc((void**)&wd, (size_t)want * 4);
    if (e == hipSuccess) e = hipMalloc((void**)&raw, (size_t)nbytes + 16);
    if (e == hipSuccess) e = hipMalloc((void**)&hd, hbytes);
    double stats[2] = {0, 0};
    if (e == hipSuccess) e = hipMemcpyAsync(wd, w_host, (size_t)want * 4, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipMemcpyAsync(hd, hess->d_h, hbytes, hipMemcpyDeviceToDevice, s);  // gptq consumes its copy
    if (e == hipSuccess) rc = run_gptq_q4_0(wd, h->out, h->in, hd, damp_frac, raw, stats, s);
    if (e == hipSuccess && rc == NQ_OK) {
        h->host_blocks.resize((size_t)nbytes);
        e = hipMemcpyAsync(h->host_blocks.data(), raw, (size_t)nbytes, hipMemcpyDeviceToHost, s);
    }
    if (e == hipSuccess && rc == NQ_OK) rc = adopt_q4_0_blocks(h, raw, s);
    if (e == hipSuccess && rc == NQ_OK) e = hipStreamSynchronize(s);
    (void)hipFree(wd), (void)hipFree(raw), (void)hipFree(hd);
    if (e != hipSuccess) return fail_hip(e, "nq_set_weight_gptq");
    if (rc) return rc;
    if (dead_out) *dead_out = (int64_t)stats[0];
    if (damp_out) *damp_out = stats[1];
    h->has_host_blocks = true;
    h->loaded = true;
    return NQ_OK;
}

int32_t nq_q4_0_objective(nq_handle h, const float* w_host, int64_t n_values, nq_hessian hess, double* out,
                          void* stream) {
    int32_t rc = check_handle(h, "nq_q4_0_objective");
    if (rc) return rc;
    if ((rc = need_loaded(h, "q4_0_objective"))) return rc;
    if (h->format != NQ_FMT_Q4_0) return fail(NQ_ERR_INVALID, "nq_q4_0_objective: the layer's format is not Q4_0");
    if ((rc = check_hessian(hess, "q4_0_objective"))) return rc;
    const int64_t want = (int64_t)h->in * h->out;
    if (n_values < want || hess->n != h->in || !w_host || !out)
        return fail(NQ_ERR_SIZE, "q4_0_objective: w must hold [OUT, IN] values and h be [IN, IN]");
    hipStream_t s = (hipStream_t)stream;
    float *wd = nullptr, *deq = nullptr;
    hipError_t e = hessian_order(hess, s);
    if (e == hipSuccess) e = hipMalloc((void**)&wd, (size_t)want * 4);
    if (e == hipSuccess) e = hipMalloc((void**)&deq, (size_t)want * 4);
    if (e == hipSuccess) e = hipMemcpyAsync(wd, w_host, (size_t)want * 4, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) rc = launch_dequantize(h, deq, s);
    if (e == hipSuccess && rc == NQ_OK) rc = run_q4_0_objective(wd, deq, h->out, h->in, hess->d_h, out, s);
    (void)hipFree(wd), (void)hipFree(deq);
    if (e != hipSuccess) return fail_hip(e, "nq_q4_0_objective");
    return rc;
}

int32_t nq_diag_mfma_rate(int32_t kind, const void* operands, int64_t operand_bytes, int32_t iters, int32_t workgroups,
                          int64_t* stamps, void* stream) {
    if (kind < 0 || kind > 3)
        return fail(NQ_ERR_INVALID, "nq_diag_mfma_rate: kind must be 0 / 1 (fp8 / int8, 32 x 32) or 2 / 3 (fp8 / int8, 16 x 16)");
    if (!operands || operand_bytes < 4096 || ((uintptr_t)operands & 3))
        return fail(NQ_ERR_INVALID, "nq_diag_mfma_rate: at least 4096 bytes of 4-byte aligned operands are needed");
    if (iters <= 0 || workgroups <= 0 || !stamps)
        return fail(NQ_ERR_INVALID, "nq_diag_mfma_rate: iters and workgroups must be positive, stamps not null");
    // (the kernel's sink is never written: its condition cannot hold; stamps doubles as its address)
    return launch_mfma_rate(kind, reinterpret_cast<const int*>(operands), (int)std::min<int64_t>(operand_bytes / 4, 1 << 24),
                            iters, workgroups, stamps, reinterpret_cast<float*>(stamps), (hipStream_t)stream);
}

int32_t nq_diag_stream_read(const void* src, int64_t nbytes, void* stream) {
    if (!src || nbytes < 1024 || ((uintptr_t)src & 15))
        return fail(NQ_ERR_INVALID, "nq_diag_stream_read: at least 1 KiB at a 16-byte aligned device address is needed");
    return launch_stream_read(src, nbytes / 1024, (hipStream_t)stream);
}

int32_t nq_diag_gemm8_timeline(nq_handle h, const void* x, int32_t x_dtype, const float* x_scale, void* y,
                               int32_t y_dtype, int32_t M, uint64_t* stamps, int64_t max_tiles, void* stream) {
    int32_t rc = check_handle(h, "nq_diag_gemm8_timeline");
    if (rc) return rc;
    if (!stamps || M < 64 || (x_dtype != NQ_DT_I8 && x_dtype != NQ_DT_FP8_E4M3))
        return fail(NQ_ERR_INVALID, "nq_diag_gemm8_timeline: 8-bit activations, M >= 64 and a stamp buffer are needed");
    const int64_t tiles = (int64_t)((M + 255) / 256) * ((h->out + 255) / 256);
    if (tiles > max_tiles) return fail(NQ_ERR_INVALID, "nq_diag_gemm8_timeline: the stamp buffer is smaller than the tile count");
    if ((rc = need_loaded(h, "forward"))) return rc;
    if (!x || !y || !x_scale || (y_dtype != NQ_DT_F32 && y_dtype != NQ_DT_BF16 && !(y_dtype == NQ_DT_I32 && x_dtype == NQ_DT_I8)))
        return fail(NQ_ERR_INVALID, "nq_diag_gemm8_timeline: x, its scale(s) and an fp32 or bf16 y (int8: or raw int32) are needed");
    SegTable seg{};
    seg.nseg = 1, seg.end[0] = h->out, seg.y[0] = y;
    ForwardArgs a{h, x, x_dtype, x_scale, y, y_dtype, M, nullptr, NQ_DT_F32, NQ_EPI_NONE, (hipStream_t)stream, seg};
    if (!gemm8_applicable(a))
        return fail(NQ_ERR_UNSUPPORTED, "nq_diag_gemm8_timeline: the large-tile GEMM does not take this layer (format, IN % 128)");
    a.diag_stamps = reinterpret_cast<unsigned long long*>(stamps);
    rc = launch_gemm8(a);
    if (rc) return rc;
    NQ_HIP(hipStreamSynchronize((hipStream_t)stream));
    return NQ_OK;
}

int32_t nq_diag_forward_gemm8(nq_handle h, const void* x, int32_t x_dtype, const float* x_scale, void* y, int32_t y_dtype,
                              int32_t M, const void* bias, int32_t bias_dtype, int32_t epilogue, int32_t tile, void* stream) {
    int32_t rc = check_handle(h, "nq_diag_forward_gemm8");
    if (rc) return rc;
    if ((rc = need_loaded(h, "forward"))) return rc;
    if (tile != 128 && tile != 256 && tile != 2564 && tile != 2568 && tile != 1282)
        return fail(NQ_ERR_INVALID, "nq_diag_forward_gemm8: tile is 128, 256, 2564 / 2568 (256 with four / eight wavefronts) or 1282 (128 x 256)");
    if (!x || !y || !x_scale || ((uintptr_t)x & 15) || ((uintptr_t)y & 3) || (x_dtype != NQ_DT_I8 && x_dtype != NQ_DT_FP8_E4M3) ||
        (y_dtype != NQ_DT_F32 && y_dtype != NQ_DT_BF16 && !(y_dtype == NQ_DT_I32 && x_dtype == NQ_DT_I8 && !bias && epilogue == NQ_EPI_NONE)) ||
        (epilogue != NQ_EPI_NONE && epilogue != NQ_EPI_RELU) || (bias && bias_dtype != NQ_DT_F32 && bias_dtype != NQ_DT_BF16))
        return fail(NQ_ERR_INVALID, "nq_diag_forward_gemm8: nq_forward's arguments for 8-bit activations are needed");
    SegTable seg{};
    seg.nseg = 1, seg.end[0] = h->out, seg.y[0] = y;
    ForwardArgs a{h, x, x_dtype, x_scale, y, y_dtype, M, bias, bias_dtype, epilogue, (hipStream_t)stream, seg};
    if (h->glu || !h->seg_end.empty() || !gemm8_applicable(a))
        return fail(NQ_ERR_UNSUPPORTED, "nq_diag_forward_gemm8: the 8-bit GEMM does not take this call (format, M >= 64, IN % 128)");
    if (tile > 256) a.diag_gemm8_waves = tile == 1282 ? 12 : tile % 10;
    if (tile == 128) a.diag_gemm8_waves = 16;
    return launch_gemm8(a);
}

int32_t nq_diag_forward_a16(nq_handle h, const void* x, int32_t x_dtype, void* y, int32_t y_dtype, int32_t M,
                            int32_t mw, int32_t nw, void* stream) {
    int32_t rc = check_handle(h, "nq_diag_forward_a16");
    if (rc) return rc;
    if ((rc = need_loaded(h, "forward"))) return rc;
    if ((mw != 1 && mw != 2) || (nw != 1 && nw != 2 && nw != 4) || (mw == 2 && nw == 1) ||
        (mw == 2 && nw == 4 && x_dtype == NQ_DT_F32))
        return fail(NQ_ERR_INVALID, "nq_diag_forward_a16: shapes are 1 x 1, 1 x 2, 1 x 4, 2 x 2, 2 x 4 (2 x 4 with bf16 activations only)");
    if (!x || !y || ((uintptr_t)x & 15) || ((uintptr_t)y & 3) || (y_dtype != NQ_DT_F32 && y_dtype != NQ_DT_BF16))
        return fail(NQ_ERR_INVALID, "nq_diag_forward_a16: x (16-byte aligned) and an fp32 or bf16 y (4-byte aligned) are needed");
    SegTable seg{};
    seg.nseg = 1, seg.end[0] = h->out, seg.y[0] = y;
    ForwardArgs a{h, x, x_dtype, nullptr, y, y_dtype, M, nullptr, NQ_DT_F32, NQ_EPI_NONE, (hipStream_t)stream, seg};
    if (h->glu || !h->seg_end.empty() || !gemm_a16_applicable(a))
        return fail(NQ_ERR_UNSUPPORTED, "nq_diag_forward_a16: the 16-row tile kernel does not take this call (fp32 / bf16 "
                                        "activations, M >= 2, an ordinary layer)");
    a.diag_a16_shape = mw << 4 | nw;
    return launch_gemm_a16(a);
}

int32_t nq_quantize_rows_i8(const void* x, int32_t x_dtype, int8_t* q, float* scales, int32_t M, int32_t K,
                            void* stream) {
    if (M < 0 || K <= 0 || K % 4 != 0)
        return fail(NQ_ERR_INVALID, "nq_quantize_rows_i8: M >= 0 and K a positive multiple of 4 are required");
    if (x_dtype != NQ_DT_F32 && x_dtype != NQ_DT_BF16)
        return fail(NQ_ERR_INVALID, "nq_quantize_rows_i8: x must be fp32 or bf16");
    if (M == 0) return NQ_OK;
    if (!x || !q || !scales) return fail(NQ_ERR_INVALID, "nq_quantize_rows_i8: null pointer");
    if (((uintptr_t)x & 15) || ((uintptr_t)q & 3))
        return fail(NQ_ERR_INVALID, "nq_quantize_rows_i8: x must be 16-byte and q 4-byte aligned");
    return launch_quantize_rows_i8(x, x_dtype, q, scales, M, K, (hipStream_t)stream);
}

int32_t nq_cast_pad_bf16(const float* src, uint16_t* dst, int32_t rows, int32_t cols, int32_t cols_pad,
                         void* stream) {
    if (rows < 0 || cols < 0 || cols_pad < cols)
        return fail(NQ_ERR_INVALID, "nq_cast_pad_bf16: need rows >= 0 and cols_pad >= cols >= 0");
    if (rows && cols_pad && (!src || !dst)) return fail(NQ_ERR_INVALID, "nq_cast_pad_bf16: null pointer");
    return launch_cast_pad_bf16(src, dst, rows, cols, cols_pad, (hipStream_t)stream);
}

int32_t nq_slice_cast_f32(const uint16_t* src, float* dst, int32_t rows, int32_t cols, int32_t cols_pad,
                          void* stream) {
    if (rows < 0 || cols < 0 || cols_pad < cols)
        return fail(NQ_ERR_INVALID, "nq_slice_cast_f32: need rows >= 0 and cols_pad >= cols >= 0");
    if (rows && cols && (!src || !dst)) return fail(NQ_ERR_INVALID, "nq_slice_cast_f32: null pointer");
    return launch_slice_cast_f32(src, dst, rows, cols, cols_pad, (hipStream_t)stream);
}

int32_t nq_mlp3_w8a8_forward(nq_handle l1, nq_handle l2, nq_handle l3, const float* x, float* y, int32_t M,
                             const float* b1, const float* b2, const float* b3, int32_t final_epilogue,
                             void* stream) {
    nq_handle ls[3] = {l1, l2, l3};
    for (int i = 0; i < 3; i++) {
        int32_t rc = check_handle(ls[i], "nq_mlp3_w8a8_forward");
        if (rc) return rc;
        if ((rc = need_loaded(ls[i], "forward"))) return rc;
        if (ls[i]->format != NQ_FMT_W8_CHANNEL)
            return fail(NQ_ERR_INVALID, "nq_mlp3_w8a8_forward: every layer must be W8_CHANNEL");
        if (ls[i]->in <= 256 && ls[i]->out <= 256 && !ls[i]->d_tiled)
            return fail(NQ_ERR_INVALID, "nq_mlp3_w8a8_forward: layer " + std::to_string(i + 1) +
                                            " was not loaded with nq_set_weight_i8 (a row-fused layer cannot be used here)");
        if (ls[i]->in > 256 || ls[i]->out > 256)
            return fail(NQ_ERR_UNSUPPORTED, "nq_mlp3_w8a8_forward: layer " + std::to_string(i + 1) + " is [" +
                                                std::to_string(ls[i]->in) + " -> " + std::to_string(ls[i]->out) +
                                                "]; the fused kernel holds at most 256 features per token");
    }
    if (l1->out != l2->in || l2->out != l3->in)
        return fail(NQ_ERR_INVALID, "nq_mlp3_w8a8_forward: the layers do not chain (" + std::to_string(l1->in) + " -> " +
                                        std::to_string(l1->out) + ", " + std::to_string(l2->in) + " -> " +
                                        std::to_string(l2->out) + ", " + std::to_string(l3->in) + " -> " +
                                        std::to_string(l3->out) + ")");
    if (final_epilogue != NQ_EPI_NONE && final_epilogue != NQ_EPI_RELU)
        return fail(NQ_ERR_INVALID, "nq_mlp3_w8a8_forward: unknown epilogue " + std::to_string(final_epilogue));
    if (M < 0) return fail(NQ_ERR_INVALID, "nq_mlp3_w8a8_forward: M must be >= 0");
    if (M == 0) return NQ_OK;
    if (!x || !y) return fail(NQ_ERR_INVALID, "nq_mlp3_w8a8_forward: null x or y");
    if ((uintptr_t)x & 15) return fail(NQ_ERR_INVALID, "nq_mlp3_w8a8_forward: x must be 16-byte aligned");
    return launch_mlp3_w8a8(l1, l2, l3, x, y, M, b1, b2, b3, final_epilogue, (hipStream_t)stream);
}

}  // extern "C"

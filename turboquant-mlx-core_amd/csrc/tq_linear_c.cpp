// C-ABI of the TQ8 linear path (declared in include/turboquant_c/tq_linear.h).
// Host-side logic only: argument checks, mode inference exactly as the reference
// does it (src/dequantizer.cpp:72-75,118-133,674-675), decode-table construction,
// device buffer ownership and kernel dispatch.  Nothing here computes on the CPU:
// a missing GPU or a failed HIP call is reported as an error.
#include "turboquant_c/tq_linear.h"
#include "turboquant_c/tq_mlp.h"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "tq_device.h"
#include "tq_gemv_common.h"
#include "tq_prefill_common.h"

namespace {
thread_local std::string g_last_error;
}

namespace tq {
void set_error(const std::string& msg) { g_last_error = msg; }

bool hip_ok(hipError_t e, const char* what) {
    if (e == hipSuccess) return true;
    set_error(std::string(what) + ": " + hipGetErrorString(e));
    return false;
}
}  // namespace tq

namespace {
using tq::set_error;
using tq::hip_ok;

int device_cu_count() {
    static std::atomic<int> cached{0};          // any host thread may be the first to ask
    int cus = cached.load(std::memory_order_relaxed);
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            cus = prop.multiProcessorCount;
        if (cus <= 0) cus = 256;
        cached.store(cus, std::memory_order_relaxed);
    }
    return cus;
}

size_t dtype_size(int dt) { return dt == TQ_DTYPE_F32 ? 4 : 2; }
bool dtype_valid(int dt) { return dt == TQ_DTYPE_F32 || dt == TQ_DTYPE_F16 || dt == TQ_DTYPE_BF16; }

}  // namespace

struct tq_linear_s {
    tq::LayerView view{};
    uint8_t* d_primary = nullptr;
    uint8_t* d_residual = nullptr;
    uint8_t* d_combined = nullptr;
    float* d_norms = nullptr;
    float* d_tables = nullptr;
    // 5-bit primary with a residual of at most 3 bits (or none): the fused kernels run it as a
    // shared-rotation layer over a one-byte-per-weight plane (r << 5 | p) and its 256-entry table.
    float* d_tables_fwd = nullptr;
    tq::LayerView fwd_view{};
    bool has_fwd_view = false;
    // 5-bit primary that keeps its two planes (own residual rotation, or a 4-bit residual): each plane by
    // itself is a layer the tuned kernels take, plane_view[0] the byte plane as a one-byte-per-weight
    // layer with the table cP[min(b, nP - 1)], plane_view[1] the residual nibbles as a primary-only layer
    // with the residual codebook and the residual's rotation; the layer is their sum (two or more rows).
    tq::LayerView plane_view[2]{};
    bool has_plane_views = false;
    float* d_tables_plane[2] = {nullptr, nullptr};
    // fp32 [batch, out] partial results of the two planes.
    void* d_sum = nullptr; size_t sum_bytes = 0;
    int primary_cols = 0;
    int residual_cols = 0;
    // Staging for the *_host entry points, grown on demand.
    void* d_stage_x = nullptr; size_t stage_x_bytes = 0;
    void* d_stage_y = nullptr; size_t stage_y_bytes = 0;
    // Rotated-activation workspace of the prefill path, grown on demand.
    void* d_work = nullptr; size_t work_bytes = 0;
    // Per-chunk partial products of the small-batch path.
    void* d_partial = nullptr; size_t partial_bytes = 0;
    // Rotated activation row (both rotations) of the batch-1 path, layers wider than 16384 columns only.
    float* d_xrot = nullptr;
    // Workspaces that were outgrown: a captured graph may still hold their addresses, so they live as long
    // as the handle does (each growth at least doubles the size: their sum stays below the current one).
    std::vector<void*> retired;

    ~tq_linear_s() {
        if (d_primary) (void)hipFree(d_primary);
        if (d_residual) (void)hipFree(d_residual);
        if (d_combined) (void)hipFree(d_combined);
        if (d_norms) (void)hipFree(d_norms);
        if (d_tables) (void)hipFree(d_tables);
        if (d_tables_fwd) (void)hipFree(d_tables_fwd);
        if (d_stage_x) (void)hipFree(d_stage_x);
        if (d_stage_y) (void)hipFree(d_stage_y);
        if (d_work) (void)hipFree(d_work);
        if (d_partial) (void)hipFree(d_partial);
        if (d_xrot) (void)hipFree(d_xrot);
        if (d_tables_plane[0]) (void)hipFree(d_tables_plane[0]);
        if (d_tables_plane[1]) (void)hipFree(d_tables_plane[1]);
        if (d_sum) (void)hipFree(d_sum);
        for (void* p : retired) (void)hipFree(p);
    }
};

// Workspace of the matrix-core paths for callers that cannot allocate (tq_linear_forward_static):
// rotated activations (tile images, or the fp16 rows of the whole-row kernel for 2..12 rows) followed by the per-chunk
// partial products of the small-batch kernels.  One copy per GPU, held until the process ends; every call on a GPU shares it, so calls
// that overlap on one GPU race.  Nothing in it has to start at zero: the kernels write every element
// they later read (rows past the batch are computed from whatever is there and never stored).
static __device__ __align__(256) unsigned char scratch[TQ_STATIC_SCRATCH_BYTES];

namespace {

// Device address of `scratch` on the current device (the array's name is only a host-side stand-in).
void* static_scratch_ptr() {
    static std::mutex mu;
    static void* ptrs[64] = {};
    int dev = 0;
    if (!hip_ok(hipGetDevice(&dev), "hipGetDevice")) return nullptr;
    if (dev < 0 || dev >= 64) { set_error("tq_linear_forward_static: device index out of range"); return nullptr; }
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void* p = nullptr;
        if (!hip_ok(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return nullptr;
        ptrs[dev] = p;
    }
    return ptrs[dev];
}

}  // namespace

namespace {

// Decode tables as 256 floats.
//   shared 4-bit : lut[(r << 4) | p] = cP[p] + cR[r], zero where p >= n_primary
//                  (src/dequantizer.cpp:144-150, 669-688)
//   other 4-bit  : [0..15] primary, [16..31] residual, index clamped to the last
//                  centroid (src/dequantizer.cpp:94,103,229)
//   5-bit primary: [0..31] primary, [32..47] residual, clamped likewise
void build_tables(int mode, const float* cbp, int np, const float* cbr, int nr, float* t) {
    std::memset(t, 0, 256 * sizeof(float));
    if (mode == tq::kSharedLut) {
        // (the reference's loop as written: the index wraps at 8 bits, so entries p >= 16 of an oversized
        // primary codebook land on ((r | 1) << 4) | (p & 15) and later writes win)
        for (int r = 0; r < 16; ++r)
            for (int p = 0; p < np; ++p)
                t[(uint8_t)((r << 4) | p)] = cbp[p] + cbr[r < nr ? r : nr - 1];
        return;
    }
    const bool five = mode >= tq::kShared5;
    const int pn = five ? 32 : 16;
    for (int i = 0; i < pn; ++i) t[i] = cbp[i < np ? i : np - 1];
    for (int i = 0; i < 16; ++i) t[pn + i] = cbr[i < nr ? i : nr - 1];
}

// Grows a workspace of a handle.  A buffer that a captured graph may still reference is never
// replaced while the stream is being captured: growth during capture is an error.
// Grows *buf to at least `need` bytes.  Refused while `stream` is being captured (an allocation cannot be
// captured).  With `retired`, an outgrown buffer is kept until the handle is freed instead of being freed
// here, and the new one is at least twice as large.
bool ensure_stage(void** buf, size_t* have, size_t need, hipStream_t stream = nullptr,
                  std::vector<void*>* retired = nullptr) {
    if (*have >= need) return true;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (stream && hipStreamIsCapturing(stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone) {
        set_error("workspace too small while the stream is being captured: call tq_linear_reserve first");
        return false;
    }
    void* fresh = nullptr;
    const size_t want = (retired && *buf && need < 2 * *have) ? 2 * *have : need;
    if (!hip_ok(hipMalloc(&fresh, want), "hipMalloc(staging)")) return false;
    if (*buf) {
        if (retired) retired->push_back(*buf);
        else (void)hipFree(*buf);
    }
    *buf = fresh;
    *have = want;
    return true;
}

tq_linear_t create_impl(int in_features, int out_features,
                        const uint8_t* pp, int primary_cols,
                        const uint8_t* pr, int residual_cols,
                        const float* norms, const uint32_t* seeds,
                        const float* cbp, int np, const float* cbr, int nr,
                        uint32_t block_size, bool from_device) {
    if (!pp || !pr || !norms || !seeds || !cbp || !cbr) { set_error("tq_linear_create: NULL argument"); return nullptr; }
    if (in_features <= 0 || out_features <= 0 || np <= 0 || nr <= 0 || np > 32 || nr > 16) {
        set_error("tq_linear_create: bad dimensions"); return nullptr;
    }
    // Shape inference as the reference does it (src/dequantizer.cpp:72-75).
    const bool five = (primary_cols == residual_cols * 2);
    const int in_inferred = five ? primary_cols : primary_cols * 2;
    if (in_inferred != in_features || residual_cols * 2 != in_features) {
        set_error("tq_linear_create: packed shapes do not match in_features"); return nullptr;
    }
    if (block_size == 0 || in_features % (int)block_size != 0) {
        set_error("tq_linear_create: in_features must be divisible by block_size"); return nullptr;
    }
    if (!tq::layout_valid(in_features, block_size)) {
        set_error("tq_linear_create: unsupported shape (need an even in_features and a power-of-two block_size "
                  "in [1, 2048])");
        return nullptr;
    }

    // tq_linear_forward_static must not do runtime work on its first call (a caller may be capturing its
    // stream): the address of the static workspace on this device is looked up here, once.
    if (!static_scratch_ptr()) return nullptr;
    tq_linear_s* h = new (std::nothrow) tq_linear_s();
    if (!h) { set_error("tq_linear_create: out of host memory"); return nullptr; }
    const size_t pbytes = (size_t)out_features * primary_cols;
    const size_t rbytes = (size_t)out_features * residual_cols;
    const hipMemcpyKind kind = from_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice;
    bool ok = hip_ok(hipMalloc((void**)&h->d_primary, pbytes), "hipMalloc(packed_primary)") &&
              hip_ok(hipMalloc((void**)&h->d_residual, rbytes), "hipMalloc(packed_residual)") &&
              hip_ok(hipMalloc((void**)&h->d_norms, (size_t)out_features * sizeof(float)), "hipMalloc(norms)") &&
              hip_ok(hipMalloc((void**)&h->d_tables, 256 * sizeof(float)), "hipMalloc(tables)") &&
              hip_ok(hipMemcpy(h->d_primary, pp, pbytes, kind), "copy packed_primary") &&
              hip_ok(hipMemcpy(h->d_residual, pr, rbytes, kind), "copy packed_residual") &&
              hip_ok(hipMemcpy(h->d_norms, norms, (size_t)out_features * sizeof(float), kind), "copy norms");
    if (!ok) { delete h; return nullptr; }

    // Residual presence: any non-zero byte (src/dequantizer.cpp:118-128).
    bool has_residual = false;
    if (from_device) {
        int* d_flag = nullptr; int flag = 0;
        ok = hip_ok(hipMalloc((void**)&d_flag, sizeof(int)), "hipMalloc(flag)") &&
             hip_ok(hipMemset(d_flag, 0, sizeof(int)), "hipMemset(flag)") &&
             hip_ok(tq::launch_any_nonzero(h->d_residual, rbytes, d_flag, nullptr), "any_nonzero") &&
             hip_ok(hipMemcpy(&flag, d_flag, sizeof(int), hipMemcpyDeviceToHost), "copy flag");
        if (d_flag) (void)hipFree(d_flag);
        if (!ok) { delete h; return nullptr; }
        has_residual = flag != 0;
    } else {
        for (size_t i = 0; i < rbytes; ++i) if (pr[i] != 0) { has_residual = true; break; }
    }
    const bool shared = (seeds[1] == 0 && has_residual);          // src/dequantizer.cpp:133
    int mode;
    if (!has_residual) mode = five ? tq::kPrimaryOnly5 : tq::kPrimaryOnly;
    else if (shared)   mode = five ? tq::kShared5 : tq::kSharedLut;
    else               mode = five ? tq::kDual5 : tq::kDual;

    float tables[256];
    build_tables(mode, cbp, np, cbr, nr, tables);
    if (!hip_ok(hipMemcpy(h->d_tables, tables, sizeof(tables), hipMemcpyHostToDevice), "copy tables")) {
        delete h; return nullptr;
    }

    if (mode == tq::kSharedLut) {
        // The shared-rotation kernels stream one byte per weight; interleave the planes once and drop them.
        const size_t cbytes = (size_t)out_features * in_features;
        ok = hip_ok(hipMalloc((void**)&h->d_combined, cbytes), "hipMalloc(packed_combined)") &&
             hip_ok(tq::launch_combine_planes(h->d_primary, h->d_residual, h->d_combined, pbytes, nullptr), "combine_planes") &&
             hip_ok(hipDeviceSynchronize(), "combine_planes sync");
        if (!ok) { delete h; return nullptr; }
        (void)hipFree(h->d_primary); h->d_primary = nullptr;
        (void)hipFree(h->d_residual); h->d_residual = nullptr;
    }

    // (a primary-only layer never reads its residual codebook, whatever its length)
    const bool fused5 = (mode == tq::kShared5 && nr <= 8) || mode == tq::kPrimaryOnly5;
    if (fused5) {
        const size_t cbytes = (size_t)out_features * in_features;
        float lut[256];
        std::memset(lut, 0, sizeof(lut));
        for (int r = 0; r < 8; ++r)
            for (int p5 = 0; p5 < 32; ++p5) {
                const float c = cbp[p5 < np ? p5 : np - 1];
                lut[(r << 5) | p5] = mode == tq::kShared5 ? c + cbr[r < nr ? r : nr - 1] : c;   // src/dequantizer.cpp:186-212
            }
        ok = hip_ok(hipMalloc((void**)&h->d_combined, cbytes), "hipMalloc(packed_combined)") &&
             hip_ok(hipMalloc((void**)&h->d_tables_fwd, sizeof(lut)), "hipMalloc(tables)") &&
             hip_ok(hipMemcpy(h->d_tables_fwd, lut, sizeof(lut), hipMemcpyHostToDevice), "copy tables") &&
             hip_ok(tq::launch_combine_planes5(h->d_primary, h->d_residual, h->d_combined, rbytes, np < 32 ? np : 32, nr,
                                               nullptr), "combine_planes5") &&
             hip_ok(hipDeviceSynchronize(), "combine_planes5 sync");
        if (!ok) { delete h; return nullptr; }
        (void)hipFree(h->d_primary); h->d_primary = nullptr;
        (void)hipFree(h->d_residual); h->d_residual = nullptr;
    }

    h->primary_cols = primary_cols;
    h->residual_cols = residual_cols;
    tq::LayerView& v = h->view;
    v.packed_primary = h->d_primary;
    v.packed_residual = h->d_residual;
    v.packed_combined = h->d_combined;
    v.norms = h->d_norms;
    v.tables = h->d_tables;
    v.out_features = out_features;
    v.in_features = in_features;
    v.block_size = block_size;
    v.seed_primary = seeds[0];
    v.seed_residual = seeds[1];
    v.mode = mode;
    v.inv_scale = 1.0f / std::sqrt(static_cast<float>(in_features));      // src/dequantizer.cpp:76
    v.inv_sqrt_bs = 1.0f / std::sqrt(static_cast<float>(block_size));     // src/rotation.cpp:333
    // Scratch row for the rotated activations of one batch row (both rotations): rows wider than 16384
    // columns and the generic kernels rotate in a kernel of their own.  Allocated here so that a forward
    // call never allocates on the batch-1 path.
    if (!hip_ok(hipMalloc((void**)&h->d_xrot, (size_t)2 * in_features * sizeof(float)), "hipMalloc(rotated row)")) {
        delete h; return nullptr;
    }
    v.xrot_work = h->d_xrot;
    {
        float big = 0.0f;
        for (int i = 0; i < np; ++i) big = std::fmax(big, std::fabs(cbp[i]));
        for (int i = 0; i < nr; ++i) big = std::fmax(big, std::fabs(cbr[i]));
        v.fp16_centroids_ok = (big < 30000.0f) ? 1 : 0;      // NaN compares false
    }
    if (fused5) {
        h->fwd_view = v;
        h->fwd_view.mode = tq::kSharedLut;
        h->fwd_view.tables = h->d_tables_fwd;
        h->has_fwd_view = true;
    } else if (mode >= tq::kShared5 && tq::lanes_supported(in_features, block_size)) {
        float ta[256], tb[256];
        std::memset(tb, 0, sizeof(tb));
        for (int b = 0; b < 256; ++b) ta[b] = cbp[b < np ? b : np - 1];          // index clamp of src/dequantizer.cpp:94
        for (int i = 0; i < 16; ++i) tb[i] = cbr[i < nr ? i : nr - 1];            // :103
        ok = hip_ok(hipMalloc((void**)&h->d_tables_plane[0], sizeof(ta)), "hipMalloc(tables)") &&
             hip_ok(hipMalloc((void**)&h->d_tables_plane[1], sizeof(tb)), "hipMalloc(tables)") &&
             hip_ok(hipMemcpy(h->d_tables_plane[0], ta, sizeof(ta), hipMemcpyHostToDevice), "copy tables") &&
             hip_ok(hipMemcpy(h->d_tables_plane[1], tb, sizeof(tb), hipMemcpyHostToDevice), "copy tables");
        if (!ok) { delete h; return nullptr; }
        tq::LayerView& a = h->plane_view[0];
        a = v;
        a.mode = tq::kSharedLut;
        a.packed_combined = h->d_primary;
        a.packed_primary = nullptr;
        a.packed_residual = nullptr;
        a.tables = h->d_tables_plane[0];
        a.seed_residual = 0;
        tq::LayerView& b = h->plane_view[1];
        b = v;
        b.mode = tq::kPrimaryOnly;
        b.packed_primary = h->d_residual;
        b.packed_residual = nullptr;
        b.packed_combined = nullptr;
        b.tables = h->d_tables_plane[1];
        b.seed_primary = mode == tq::kDual5 ? seeds[1] : seeds[0];
        b.seed_residual = 0;
        h->has_plane_views = true;
    }
    return h;
}

}  // namespace

namespace {

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

}  // namespace

// Shared by tq_linear_forward, tq_linear_forward_static and the MLP block.  gate: optional fp32
// [batch, out]; the batch-1..15 kernel then stores silu(gate) * y.  static_ws: the workspaces of the
// matrix-core paths come from there (TQ_STATIC_SCRATCH_BYTES) instead of the handle's own buffers,
// and nothing is allocated.  Returns 0 on success.
// One layer view through the tuned kernels (or the generic ones where they do not take its shape).
// static_ws / static_cap: the caller's share of the static array, or NULL: the handle's own workspaces.
int forward_view(tq_linear_s* h, const tq::LayerView& V, bool generic_only, const void* x_dev, int x_dtype, int batch,
                 void* y_dev, int y_dtype, hipStream_t stream, const float* gate, void* static_ws, size_t static_cap) {
    const bool lanes = !generic_only && tq::lanes_supported(V.in_features, V.block_size);
    // (the gated store is a feature of the one-row kernels; 16..32 rows: the small-batch kernel where it takes the layer)
    // (two to twelve rows: whole weight rows per stream, 4 x 4 x 4 matrix blocks; a
    // workspace only where the rows are rotated by a kernel of their own)
    if (lanes && !gate && tq::gemv_few_supported(V, batch, device_cu_count())) {
        const size_t need = tq::gemv_few_workspace_bytes(V, batch);
        void* few_ws = nullptr;
        if (need && static_ws) {
            if (need > static_cap) { set_error("tq_linear_forward_static: the workspace of this call does not fit the static array"); return 1; }
            few_ws = static_ws;
        } else if (need) {
            if (!ensure_stage(&h->d_work, &h->work_bytes, need, stream, &h->retired)) return 1;
            few_ws = h->d_work;
        }
        return hip_ok(tq::launch_gemv_few(V, x_dev, x_dtype, batch, y_dev, y_dtype, few_ws, device_cu_count(), stream),
                      "tq_gemv_few launch") ? 0 : 1;
    }
    const bool skinny = lanes && !gate && tq::skinny_supported(V, x_dtype, batch);
    const bool prefill = lanes && !skinny && !gate && tq::prefill_supported(V, x_dtype, batch);
    if (!prefill && !skinny && (generic_only || !tq::shape_supported(V.in_features, V.block_size))) {
        if (!tq::generic_supported(V)) { set_error("tq_linear_forward: unsupported layer shape"); return 1; }
        return hip_ok(tq::launch_gemv_generic(V, x_dev, x_dtype, batch, y_dev, y_dtype, device_cu_count(), stream, gate),
                      "tq_gemv_generic launch") ? 0 : 1;
    }
    void* work = nullptr;
    float* partial = nullptr;
    tq::PrefillPlan plan{};
    // (more than 256 rows and enough output tiles: 512-row activation panels, tq_prefill_panel.hip)
    const bool panel = prefill && tq::prefill_panel_supported(V, batch, device_cu_count(), static_ws ? static_cap : ~(size_t)0);
    if (prefill && !panel) plan = tq::prefill_plan(V, batch, device_cu_count(), static_ws ? static_cap : ~(size_t)0);
    if (prefill || skinny) {
        const size_t work_need = panel ? tq::prefill_panel_workspace_bytes(V, batch, device_cu_count(), static_ws ? static_cap : ~(size_t)0)
                                       : prefill ? plan.total_bytes : tq::skinny_workspace_bytes(V, batch);
        const size_t partial_need = skinny ? tq::skinny_partial_bytes(V, batch) : 0;
        if (static_ws) {
            if (align256(work_need) + partial_need > static_cap) {
                set_error("tq_linear_forward_static: this layer and batch need a workspace of " +
                          std::to_string(align256(work_need) + partial_need + ((size_t)TQ_STATIC_SCRATCH_BYTES - static_cap)) +
                          " bytes, more than the static " + std::to_string((size_t)TQ_STATIC_SCRATCH_BYTES)); return 1;
            }
            work = static_ws;
            partial = reinterpret_cast<float*>(static_cast<unsigned char*>(static_ws) + align256(work_need));
        } else {
            // The first call with a larger batch allocates (not capturable in a graph); tq_linear_reserve
            // sizes the workspaces ahead of time.
            if (!ensure_stage(&h->d_work, &h->work_bytes, work_need, stream, &h->retired)) return 1;
            if (skinny && !ensure_stage(&h->d_partial, &h->partial_bytes, partial_need, stream, &h->retired)) return 1;
            work = h->d_work;
            partial = static_cast<float*>(h->d_partial);
        }
    }
    if (panel)
        return hip_ok(tq::launch_prefill_panel(V, x_dev, x_dtype, batch, y_dev, y_dtype, work,
                                               tq::prefill_panel_workspace_bytes(V, batch, device_cu_count(), static_ws ? static_cap : ~(size_t)0),
                                               device_cu_count(), stream),
                      "tq_prefill_panel launch") ? 0 : 1;
    if (prefill) {
        // Dense contraction: rotate once, dequantise tiles to fp16 in LDS, MFMA.
        return hip_ok(tq::launch_prefill(V, x_dev, x_dtype, batch, y_dev, y_dtype, work, plan, stream),
                      "tq_prefill launch") ? 0 : 1;
    }
    if (skinny) {
        // 2..32 rows: batch rows on the matrix cores, fp16 weights and rotated activations.
        return hip_ok(tq::launch_skinny(V, x_dev, x_dtype, batch, y_dev, y_dtype, work, partial, device_cu_count(), stream),
                      "tq_skinny launch") ? 0 : 1;
    }
    return hip_ok(tq::launch_gemv(V, x_dev, x_dtype, batch, y_dev, y_dtype, device_cu_count(), stream, gate),
                  "tq_gemv launch") ? 0 : 1;
}

// Bytes of fp32 partial results a two-plane 5-bit layer needs for `batch` rows written as y_dtype.
size_t plane_sum_bytes(const tq_linear_s* h, int batch, int y_dtype) {
    return align256((size_t)batch * h->view.out_features * sizeof(float)) * (y_dtype == tq::kF32 ? 1 : 2);
}

int forward_impl(tq_linear_s* h, const void* x_dev, int x_dtype, int batch, void* y_dev, int y_dtype,
                 hipStream_t stream, const float* gate, void* static_ws = nullptr) {
    // 5-bit primaries with their own residual rotation or a 4-bit residual keep their two planes.  One
    // row runs on the generic kernels (both planes in one pass); two or more rows run each plane through
    // the tuned kernels as a layer of its own and add the two results: y = P x~p + R x~r, the same sum the
    // reference's kernel forms per element (metal/turboquant_dequant_mm.metal:240-248, 277-292).
    const bool two_plane5 = h->view.mode >= tq::kShared5 && !h->has_fwd_view;
    const size_t cap = (size_t)TQ_STATIC_SCRATCH_BYTES;
    if (two_plane5 && batch >= 2 && !gate && h->has_plane_views) {
        const size_t one = align256((size_t)batch * h->view.out_features * sizeof(float));
        const size_t need = plane_sum_bytes(h, batch, y_dtype);
        unsigned char* sums = nullptr;
        void* sub_ws = nullptr;
        size_t sub_cap = 0;
        if (static_ws) {
            if (need >= cap) {
                set_error("tq_linear_forward_static: this layer and batch need a workspace of more than the static " +
                          std::to_string(cap) + " bytes"); return 1;
            }
            sums = static_cast<unsigned char*>(static_ws);
            sub_ws = sums + need;
            sub_cap = cap - need;
        } else {
            if (!ensure_stage(&h->d_sum, &h->sum_bytes, need, stream, &h->retired)) return 1;
            sums = static_cast<unsigned char*>(h->d_sum);
        }
        float* const t1 = reinterpret_cast<float*>(sums);
        float* const t0 = y_dtype == tq::kF32 ? static_cast<float*>(y_dev) : reinterpret_cast<float*>(sums + one);
        if (forward_view(h, h->plane_view[0], false, x_dev, x_dtype, batch, t0, tq::kF32, stream, nullptr, sub_ws, sub_cap) != 0) return 1;
        if (forward_view(h, h->plane_view[1], false, x_dev, x_dtype, batch, t1, tq::kF32, stream, nullptr, sub_ws, sub_cap) != 0) return 1;
        return hip_ok(tq::launch_add(t0, t1, y_dev, y_dtype, (size_t)batch * h->view.out_features, stream), "tq_add launch") ? 0 : 1;
    }
    const tq::LayerView& V = h->has_fwd_view ? h->fwd_view : h->view;
    return forward_view(h, V, two_plane5, x_dev, x_dtype, batch, y_dev, y_dtype, stream, gate, static_ws, static_ws ? cap : 0);
}

extern "C" {

const char* tq_last_error(void) { return g_last_error.c_str(); }

tq_linear_t tq_linear_create(int in_features, int out_features,
                             const uint8_t* packed_primary_host, int primary_cols,
                             const uint8_t* packed_residual_host, int residual_cols,
                             const float* norms_host, const uint32_t* seeds_host,
                             const float* cb_primary_host, int n_primary,
                             const float* cb_residual_host, int n_residual,
                             uint32_t block_size) {
    try {
        return create_impl(in_features, out_features, packed_primary_host, primary_cols,
                           packed_residual_host, residual_cols, norms_host, seeds_host,
                           cb_primary_host, n_primary, cb_residual_host, n_residual, block_size, false);
    } catch (...) { set_error("tq_linear_create: exception"); return nullptr; }
}

tq_linear_t tq_linear_create_from_device(int in_features, int out_features,
                             const uint8_t* packed_primary_dev, int primary_cols,
                             const uint8_t* packed_residual_dev, int residual_cols,
                             const float* norms_dev, const uint32_t* seeds_host,
                             const float* cb_primary_host, int n_primary,
                             const float* cb_residual_host, int n_residual,
                             uint32_t block_size) {
    try {
        return create_impl(in_features, out_features, packed_primary_dev, primary_cols,
                           packed_residual_dev, residual_cols, norms_dev, seeds_host,
                           cb_primary_host, n_primary, cb_residual_host, n_residual, block_size, true);
    } catch (...) { set_error("tq_linear_create_from_device: exception"); return nullptr; }
}

int tq_linear_in_features(tq_linear_t h) { return h ? h->view.in_features : 0; }
int tq_linear_out_features(tq_linear_t h) { return h ? h->view.out_features : 0; }
int tq_linear_mode(tq_linear_t h) { return h ? h->view.mode : 0; }

int tq_linear_forward(tq_linear_t h, const void* x_dev, int x_dtype, int batch,
                      void* y_dev, int y_dtype, void* stream) {
    try {
        if (!h || !x_dev || !y_dev) { set_error("tq_linear_forward: NULL argument"); return 1; }
        if (batch <= 0 || !dtype_valid(x_dtype) || !dtype_valid(y_dtype)) {
            set_error("tq_linear_forward: bad batch or dtype"); return 1;
        }
        return forward_impl(h, x_dev, x_dtype, batch, y_dev, y_dtype, static_cast<hipStream_t>(stream), nullptr);
    } catch (...) { set_error("tq_linear_forward: exception"); return 1; }
}

namespace {
// Workspace of the whole-row kernel (2..12 rows) for every batch up to max_batch, thrice: the first layer of a group holds
// the rotated rows of all its layers.
size_t few_reserve_bytes(const tq::LayerView& V, int max_batch) {
    size_t need = 0;
    for (int b = 2; b <= max_batch && b <= 12; ++b) need = std::max(need, 3 * tq::gemv_few_workspace_bytes(V, b));
    return need;
}
}  // namespace

int tq_linear_reserve(tq_linear_t h, int max_batch) {
    try {
        if (!h || max_batch <= 0) { set_error("tq_linear_reserve: bad argument"); return 1; }
        if (max_batch < 2) return 0;                       // one row uses no workspace
        if (h->has_plane_views) {                          // two planes, each a layer of its own, plus their fp32 results
            size_t work = 0, part = 0;
            for (int k = 0; k < 2; ++k) {
                const tq::LayerView& P = h->plane_view[k];
                const int rows = max_batch < tq::kSkinnyMaxRows ? max_batch : tq::kSkinnyMaxRows;
                const bool sk = tq::skinny_supported(P, tq::kBF16, rows);        // (layers the small-batch kernels never take need none of it)
                const size_t small = sk ? tq::skinny_workspace_bytes(P, rows) : 0;
                const size_t big = max_batch >= 16 ? tq::prefill_reserve_bytes(P, max_batch, device_cu_count()) : 0;
                work = std::max(work, std::max(small, big));
                work = std::max(work, few_reserve_bytes(P, max_batch));
                if (sk) part = std::max(part, tq::skinny_partial_bytes(P, rows));
            }
            if (!ensure_stage(&h->d_work, &h->work_bytes, work, nullptr, &h->retired)) return 1;
            if (!ensure_stage(&h->d_partial, &h->partial_bytes, part, nullptr, &h->retired)) return 1;
            if (!ensure_stage(&h->d_sum, &h->sum_bytes, plane_sum_bytes(h, max_batch, tq::kBF16), nullptr, &h->retired)) return 1;
            return 0;
        }
        const tq::LayerView& V = h->has_fwd_view ? h->fwd_view : h->view;
        const int rows = max_batch < tq::kSkinnyMaxRows ? max_batch : tq::kSkinnyMaxRows;
        // (a layer the small-batch kernels never take needs neither their tile images nor their partial products)
        const bool sk = tq::lanes_supported(V.in_features, V.block_size) && tq::skinny_supported(V, tq::kBF16, rows);
        const size_t small = sk ? tq::skinny_workspace_bytes(V, rows) : 0;
        const bool pf = tq::lanes_supported(V.in_features, V.block_size) && max_batch >= 16 && tq::prefill_supported(V, tq::kBF16, max_batch);
        const size_t big = pf ? tq::prefill_reserve_bytes(V, max_batch, device_cu_count()) : 0;
        const size_t few = few_reserve_bytes(V, max_batch);
        const size_t work = std::max(few, std::max(small, big));
        if (work && !ensure_stage(&h->d_work, &h->work_bytes, work, nullptr, &h->retired)) return 1;
        if (sk && !ensure_stage(&h->d_partial, &h->partial_bytes, tq::skinny_partial_bytes(V, rows), nullptr, &h->retired)) return 1;
        return 0;
    } catch (...) { set_error("tq_linear_reserve: exception"); return 1; }
}

int tq_linear_forward_static(tq_linear_t h, const void* x_dev, int x_dtype, int batch,
                             void* y_dev, int y_dtype, void* stream) {
    try {
        if (!h || !x_dev || !y_dev) { set_error("tq_linear_forward_static: NULL argument"); return 1; }
        if (batch <= 0 || !dtype_valid(x_dtype) || !dtype_valid(y_dtype)) {
            set_error("tq_linear_forward_static: bad batch or dtype"); return 1;
        }
        void* ws = static_scratch_ptr();
        if (!ws) return 1;
        return forward_impl(h, x_dev, x_dtype, batch, y_dev, y_dtype, static_cast<hipStream_t>(stream), nullptr, ws);
    } catch (...) { set_error("tq_linear_forward_static: exception"); return 1; }
}

int tq_linear_forward_group(const tq_linear_t* hs, int n, const void* x_dev, int x_dtype, int batch,
                            void* const* y_devs, int y_dtype, void* stream) {
    try {
        if (!hs || !x_dev || !y_devs || n < 1 || n > 3) { set_error("tq_linear_forward_group: bad arguments (1 to 3 layers)"); return 1; }
        if (batch <= 0 || !dtype_valid(x_dtype) || !dtype_valid(y_dtype)) { set_error("tq_linear_forward_group: bad batch or dtype"); return 1; }
        tq::LayerView views[3];
        bool plain = true;
        for (int j = 0; j < n; ++j) {
            if (!hs[j] || !y_devs[j]) { set_error("tq_linear_forward_group: NULL layer or output"); return 1; }
            if (hs[j]->view.mode >= tq::kShared5 && !hs[j]->has_fwd_view) plain = false;
            views[j] = hs[j]->has_fwd_view ? hs[j]->fwd_view : hs[j]->view;
            if (views[j].in_features != views[0].in_features) {
                set_error("tq_linear_forward_group: the layers must have the same in_features"); return 1;
            }
        }
        hipStream_t st = static_cast<hipStream_t>(stream);
        if (plain && batch == 1 && tq::gemv_wide_group_supported(views, n, device_cu_count())) {
            tq::GemvArgs as[3] = {};
            for (int j = 0; j < n; ++j) {
                as[j].L = views[j];
                as[j].x = x_dev; as[j].y = y_devs[j];
                as[j].x_dtype = x_dtype; as[j].y_dtype = y_dtype;
                as[j].out_scale = views[j].inv_scale * views[j].inv_sqrt_bs;
                as[j].gate = nullptr;
            }
            return hip_ok(tq::launch_gemv_wide_group(as, n, device_cu_count(), st), "tq_gemv group launch") ? 0 : 1;
        }
        if (plain && tq::gemv_few_group_supported(views, n, batch, device_cu_count())) {
            // (rows that a kernel of its own rotates: one part of the first layer's workspace per layer; allocated on
            // the first such call, not capturable in a graph, as in tq_linear_forward)
            const size_t need = n * tq::gemv_few_workspace_bytes(views[0], batch);
            if (need && !ensure_stage(&hs[0]->d_work, &hs[0]->work_bytes, need, st, &hs[0]->retired)) return 1;
            return hip_ok(tq::launch_gemv_few_group(views, n, x_dev, x_dtype, batch, y_devs, y_dtype,
                                                    need ? hs[0]->d_work : nullptr, device_cu_count(), st),
                          "tq_gemv_few group launch") ? 0 : 1;
        }
        // (a layer that a call of its own would send to the kernel above keeps it: the group is then run layer by layer)
        bool any_few = false;
        for (int j = 0; j < n; ++j) any_few = any_few || tq::gemv_few_supported(views[j], batch, device_cu_count());
        if (plain && !any_few && tq::skinny_group_supported(views, n, x_dtype, batch, device_cu_count())) {
            // 2..32 rows on the matrix cores; the per-chunk partial products are per layer and allocated
            // on the first such call (not capturable in a graph), as in tq_linear_forward.
            float* partials[3] = {nullptr, nullptr, nullptr};
            for (int j = 0; j < n; ++j) {
                if (!ensure_stage(&hs[j]->d_partial, &hs[j]->partial_bytes, tq::skinny_partial_bytes(views[j], batch), st, &hs[j]->retired)) return 1;
                partials[j] = static_cast<float*>(hs[j]->d_partial);
            }
            return hip_ok(tq::launch_skinny_group(views, n, x_dev, x_dtype, batch, y_devs, y_dtype, partials,
                                                  device_cu_count(), st), "tq_skinny group launch") ? 0 : 1;
        }
        for (int j = 0; j < n; ++j)
            if (forward_impl(hs[j], x_dev, x_dtype, batch, y_devs[j], y_dtype, st, nullptr) != 0) return 1;
        return 0;
    } catch (...) { set_error("tq_linear_forward_group: exception"); return 1; }
}

int tq_linear_forward_host(tq_linear_t h, const void* x_host, int x_dtype, int batch,
                           void* y_host, int y_dtype) {
    try {
        if (!h || !x_host || !y_host) { set_error("tq_linear_forward_host: NULL argument"); return 1; }
        if (batch <= 0 || !dtype_valid(x_dtype) || !dtype_valid(y_dtype)) {
            set_error("tq_linear_forward_host: bad batch or dtype"); return 1;
        }
        const size_t xb = (size_t)batch * h->view.in_features * dtype_size(x_dtype);
        const size_t yb = (size_t)batch * h->view.out_features * dtype_size(y_dtype);
        if (!ensure_stage(&h->d_stage_x, &h->stage_x_bytes, xb)) return 1;
        if (!ensure_stage(&h->d_stage_y, &h->stage_y_bytes, yb)) return 1;
        if (!hip_ok(hipMemcpy(h->d_stage_x, x_host, xb, hipMemcpyHostToDevice), "copy x")) return 1;
        if (tq_linear_forward(h, h->d_stage_x, x_dtype, batch, h->d_stage_y, y_dtype, nullptr) != 0) return 1;
        if (!hip_ok(hipMemcpy(y_host, h->d_stage_y, yb, hipMemcpyDeviceToHost), "copy y")) return 1;
        return 0;
    } catch (...) { set_error("tq_linear_forward_host: exception"); return 1; }
}

int tq_linear_dequantize_as(tq_linear_t h, void* w_dev, int w_dtype, void* stream) {
    try {
        if (!h || !w_dev) { set_error("tq_linear_dequantize: NULL argument"); return 1; }
        if (w_dtype < tq::kF32 || w_dtype > tq::kBF16) { set_error("tq_linear_dequantize: bad dtype"); return 1; }
        if (!tq::lanes_supported(h->view.in_features, h->view.block_size))     // blocks of 1 to 16 columns
            return hip_ok(tq::launch_dequant_small(h->view, w_dev, w_dtype, static_cast<hipStream_t>(stream)),
                          "tq_dequant launch") ? 0 : 1;
        return hip_ok(tq::launch_dequant(h->view, w_dev, w_dtype, static_cast<hipStream_t>(stream)),
                      "tq_dequant launch") ? 0 : 1;
    } catch (...) { set_error("tq_linear_dequantize: exception"); return 1; }
}

int tq_linear_dequantize(tq_linear_t h, float* w_dev, void* stream) {
    return tq_linear_dequantize_as(h, w_dev, tq::kF32, stream);
}

int tq_linear_dequantize_as_host(tq_linear_t h, void* w_host, int w_dtype) {
    try {
        if (!h || !w_host) { set_error("tq_linear_dequantize_host: NULL argument"); return 1; }
        const size_t bytes = (size_t)h->view.out_features * h->view.in_features * (w_dtype == tq::kF32 ? 4 : 2);
        void* d = nullptr;
        if (!hip_ok(hipMalloc(&d, bytes), "hipMalloc(weight)")) return 1;
        bool ok = tq_linear_dequantize_as(h, d, w_dtype, nullptr) == 0 &&
                  hip_ok(hipMemcpy(w_host, d, bytes, hipMemcpyDeviceToHost), "copy weight");
        (void)hipFree(d);
        return ok ? 0 : 1;
    } catch (...) { set_error("tq_linear_dequantize_host: exception"); return 1; }
}

int tq_linear_dequantize_host(tq_linear_t h, float* w_host) {
    return tq_linear_dequantize_as_host(h, w_host, tq::kF32);
}

void tq_linear_free(tq_linear_t h) {
    if (!h) return;
    delete h;
}

int tq_wht_rotate(const float* in_dev, float* out_dev, int rows, int cols,
                  uint32_t seed, uint32_t block_size, int inverse, void* stream) {
    try {
        if (!in_dev || !out_dev || rows <= 0 || cols <= 0) { set_error("tq_wht_rotate: bad argument"); return 1; }
        if (block_size == 0 || cols % (int)block_size != 0) {
            set_error("tq_wht_rotate: in_features must be divisible by block_size"); return 1;
        }
        if (block_size > 2048 || (block_size & (block_size - 1))) {
            set_error("tq_wht_rotate: block_size must be a power of two of at most 2048"); return 1;
        }
        const float inv_sqrt_bs = 1.0f / std::sqrt(static_cast<float>(block_size));
        if (block_size < 2 || cols % tq::kChunk != 0) {
            if (block_size > 16) { set_error("tq_wht_rotate: unsupported shape"); return 1; }   // cannot happen: bs divides cols
            return hip_ok(tq::launch_wht_small(in_dev, out_dev, rows, cols, seed, block_size, inv_sqrt_bs, inverse,
                                               static_cast<hipStream_t>(stream)), "tq_wht launch") ? 0 : 1;
        }
        return hip_ok(tq::launch_wht(in_dev, out_dev, rows, cols, seed, block_size, inv_sqrt_bs, inverse,
                                     static_cast<hipStream_t>(stream)), "tq_wht launch") ? 0 : 1;
    } catch (...) { set_error("tq_wht_rotate: exception"); return 1; }
}

int tq_wht_rotate_host(const float* in_host, float* out_host, int rows, int cols,
                       uint32_t seed, uint32_t block_size, int inverse) {
    try {
        if (!in_host || !out_host || rows <= 0 || cols <= 0) { set_error("tq_wht_rotate_host: bad argument"); return 1; }
        const size_t bytes = (size_t)rows * cols * sizeof(float);
        float* d = nullptr;
        if (!hip_ok(hipMalloc((void**)&d, bytes), "hipMalloc(matrix)")) return 1;
        bool ok = hip_ok(hipMemcpy(d, in_host, bytes, hipMemcpyHostToDevice), "copy in") &&
                  tq_wht_rotate(d, d, rows, cols, seed, block_size, inverse, nullptr) == 0 &&
                  hip_ok(hipMemcpy(out_host, d, bytes, hipMemcpyDeviceToHost), "copy out");
        (void)hipFree(d);
        return ok ? 0 : 1;
    } catch (...) { set_error("tq_wht_rotate_host: exception"); return 1; }
}

// ---------------------------------------------------------------------------
// Gated MLP block: y = down( silu(gate(x)) * up(x) ), fp32 between the linears.
// ---------------------------------------------------------------------------
struct tq_mlp_s {
    tq_linear_t gate, up, down;
    int max_batch;
    float* d_gate = nullptr;    // [max_batch, intermediate] fp32
    float* d_up = nullptr;      // [max_batch, intermediate] fp32 (batched path only)
    void* d_act = nullptr;      // [max_batch, intermediate] fp32
    ~tq_mlp_s() {
        if (d_gate) (void)hipFree(d_gate);
        if (d_up) (void)hipFree(d_up);
        if (d_act) (void)hipFree(d_act);
    }
};

tq_mlp_t tq_mlp_create(tq_linear_t gate, tq_linear_t up, tq_linear_t down, int max_batch) {
    try {
        if (!gate || !up || !down) { set_error("tq_mlp_create: NULL layer"); return nullptr; }
        if (max_batch <= 0) { set_error("tq_mlp_create: max_batch must be positive"); return nullptr; }
        const int hidden = gate->view.in_features, inter = gate->view.out_features;
        if (up->view.in_features != hidden || up->view.out_features != inter || down->view.in_features != inter) {
            set_error("tq_mlp_create: layer shapes do not form gate/up [I, H], down [O, I]"); return nullptr;
        }
        tq_mlp_s* m = new (std::nothrow) tq_mlp_s{gate, up, down, max_batch};
        if (!m) { set_error("tq_mlp_create: out of host memory"); return nullptr; }
        const size_t n = (size_t)max_batch * inter;
        bool ok = hip_ok(hipMalloc((void**)&m->d_gate, n * sizeof(float)), "hipMalloc(gate)") &&
                  hip_ok(hipMalloc((void**)&m->d_up, n * sizeof(float)), "hipMalloc(up)") &&
                  hip_ok(hipMalloc(&m->d_act, n * sizeof(float)), "hipMalloc(act)");
        // The batched path of the three layers needs rotated-activation workspaces: size them now so
        // that tq_mlp_forward never allocates.
        for (tq_linear_t l : {gate, up, down})
            if (ok) ok = tq_linear_reserve(l, max_batch) == 0;
        if (!ok) { delete m; return nullptr; }
        return m;
    } catch (...) { set_error("tq_mlp_create: exception"); return nullptr; }
}

int tq_mlp_forward(tq_mlp_t m, const void* x_dev, int x_dtype, int batch, void* y_dev, int y_dtype, void* stream) {
    try {
        if (!m || !x_dev || !y_dev) { set_error("tq_mlp_forward: NULL argument"); return 1; }
        if (batch <= 0 || batch > m->max_batch || !dtype_valid(x_dtype) || !dtype_valid(y_dtype)) {
            set_error("tq_mlp_forward: bad batch (larger than max_batch?) or dtype"); return 1;
        }
        hipStream_t st = static_cast<hipStream_t>(stream);
        const size_t n = (size_t)batch * m->gate->view.out_features;
        if (batch == 1 && !m->gate->has_fwd_view && !m->up->has_fwd_view && !m->down->has_fwd_view &&
            m->gate->view.mode < tq::kShared5 && m->up->view.mode < tq::kShared5 && m->down->view.mode < tq::kShared5) {
            // One row, gate and up of equal width and mode, an intermediate row wider than 16384 columns:
            // gate and up share a launch, and silu(gate) * up is formed by the kernel that rotates the
            // row for the down projection: three launches and one kernel start less than below.
            const tq::LayerView pair[2] = {m->gate->view, m->up->view};
            if (tq::gemv_wide_group_supported(pair, 2, device_cu_count()) && tq::gemv_x_gate_supported(m->down->view)) {
                tq::GemvArgs as[2] = {};
                float* outs[2] = {m->d_gate, m->d_up};
                for (int j = 0; j < 2; ++j) {
                    as[j].L = pair[j];
                    as[j].x = x_dev; as[j].y = outs[j];
                    as[j].x_dtype = x_dtype; as[j].y_dtype = tq::kF32;
                    as[j].out_scale = pair[j].inv_scale * pair[j].inv_sqrt_bs;
                }
                if (!hip_ok(tq::launch_gemv_wide_group(as, 2, device_cu_count(), st), "tq_gemv group launch")) return 1;
                return hip_ok(tq::launch_gemv(m->down->view, m->d_up, tq::kF32, 1, y_dev, y_dtype, device_cu_count(), st,
                                              nullptr, m->d_gate), "tq_gemv launch") ? 0 : 1;
            }
        }
        if (batch == 1) {
            // decode: three launches, the SiLU gate folded into the store of the up projection
            if (forward_impl(m->gate, x_dev, x_dtype, batch, m->d_gate, tq::kF32, st, nullptr) != 0) return 1;
            if (forward_impl(m->up, x_dev, x_dtype, batch, m->d_act, tq::kF32, st, m->d_gate) != 0) return 1;
            return forward_impl(m->down, m->d_act, tq::kF32, batch, y_dev, y_dtype, st, nullptr);
        }
        // two or more rows: matrix-core paths for all three layers (small-batch or prefill kernel), one
        // elementwise kernel; the activation is handed to the down projection as fp32
        const tq::LayerView both[2] = {m->gate->has_fwd_view ? m->gate->fwd_view : m->gate->view,
                                       m->up->has_fwd_view ? m->up->fwd_view : m->up->view};
        const bool plain = !(m->gate->view.mode >= tq::kShared5 && !m->gate->has_fwd_view) &&
                           !(m->up->view.mode >= tq::kShared5 && !m->up->has_fwd_view);
        const bool any_few = tq::gemv_few_supported(both[0], batch, device_cu_count()) ||
                             tq::gemv_few_supported(both[1], batch, device_cu_count());
        if (plain && tq::gemv_few_group_supported(both, 2, batch, device_cu_count())) {
            // two to four rows: gate and up share one launch of the kernel that reads whole rows
            void* outs[2] = {m->d_gate, m->d_up};
            const size_t need = 2 * tq::gemv_few_workspace_bytes(both[0], batch);      // (sized by tq_mlp_create)
            if (need && !ensure_stage(&m->gate->d_work, &m->gate->work_bytes, need, st, &m->gate->retired)) return 1;
            if (!hip_ok(tq::launch_gemv_few_group(both, 2, x_dev, x_dtype, batch, outs, tq::kF32,
                                                  need ? m->gate->d_work : nullptr, device_cu_count(), st),
                        "tq_gemv_few group launch")) return 1;
        } else if (plain && !any_few && tq::skinny_group_supported(both, 2, x_dtype, batch, device_cu_count())) {
            // gate and up share the small-batch kernel and its reduction (workspaces sized by tq_mlp_create)
            void* outs[2] = {m->d_gate, m->d_up};
            float* partials[2] = {static_cast<float*>(m->gate->d_partial), static_cast<float*>(m->up->d_partial)};
            if (!hip_ok(tq::launch_skinny_group(both, 2, x_dev, x_dtype, batch, outs, tq::kF32, partials,
                                                device_cu_count(), st), "tq_skinny group launch")) return 1;
        } else {
            if (forward_impl(m->gate, x_dev, x_dtype, batch, m->d_gate, tq::kF32, st, nullptr) != 0) return 1;
            if (forward_impl(m->up, x_dev, x_dtype, batch, m->d_up, tq::kF32, st, nullptr) != 0) return 1;
        }
        const int act_dtype = tq::kF32;
        if (!hip_ok(tq::launch_silu_mul(m->d_gate, m->d_up, m->d_act, act_dtype, n, st), "silu_mul launch")) return 1;
        return forward_impl(m->down, m->d_act, act_dtype, batch, y_dev, y_dtype, st, nullptr);
    } catch (...) { set_error("tq_mlp_forward: exception"); return 1; }
}

void tq_mlp_free(tq_mlp_t m) {
    if (!m) return;
    delete m;
}

}  // extern "C"

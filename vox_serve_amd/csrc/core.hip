// Core of libvoxhip that every engine needs: the error channel, the per-GPU context and hipGraph capture.
#include <stdarg.h>
#include <string.h>

#include <vector>

#include "vox_internal.h"

static thread_local char g_err[512] = "";

int vox_fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" {

int vox_abi_version(void) { return VOX_ABI_VERSION; }
const char* vox_last_error(void) { return g_err; }

int vox_ctx_create(int device, vox_ctx** out) {
    if (!out) return vox_fail(VOX_ERR_INVALID, "ctx_create: out is NULL");
    int n = 0;
    VOX_HIP(hipGetDeviceCount(&n));
    if (device < 0 || device >= n) return vox_fail(VOX_ERR_INVALID, "ctx_create: device %d of %d", device, n);
    VOX_HIP(hipSetDevice(device));
    hipDeviceProp_t p;
    VOX_HIP(hipGetDeviceProperties(&p, device));
    vox_ctx* c = new vox_ctx();
    c->device = device;
    c->n_cu = p.multiProcessorCount;
    c->lds_bytes = (int64_t)p.maxSharedMemoryPerMultiProcessor;
    c->hbm_bytes = (int64_t)p.totalGlobalMem;
    c->samp_ws = nullptr;
    if (hipMalloc(&c->samp_ws, SAMP_WS_BYTES) != hipSuccess || hipMemset(c->samp_ws, 0, SAMP_WS_BYTES) != hipSuccess) {
        delete c;
        return vox_fail(VOX_ERR_NOMEM, "ctx_create: sampler scratch");
    }
    *out = c;
    return VOX_OK;
}
void vox_ctx_destroy(vox_ctx* ctx) {
    if (!ctx) return;
    (void)hipFree(ctx->samp_ws);
    delete ctx;
}
int vox_ctx_set_exact_rows(vox_ctx* ctx, int rows) {
    if (!ctx || rows < 1 || rows > 8) return vox_fail(VOX_ERR_INVALID, "ctx_set_exact_rows: rows must be 1..8");
    ctx->exact_rows = rows;
    return VOX_OK;
}
int vox_ctx_props(vox_ctx* ctx, int64_t out[3]) {
    if (!ctx || !out) return vox_fail(VOX_ERR_INVALID, "ctx_props: NULL");
    out[0] = ctx->n_cu; out[1] = ctx->lds_bytes; out[2] = ctx->hbm_bytes;
    return VOX_OK;
}

int vox_graph_begin(vox_ctx* ctx, void* stream) {
    (void)ctx;
    VOX_HIP(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
    return VOX_OK;
}
int vox_graph_end(vox_ctx* ctx, void* stream, vox_graph** out) {
    (void)ctx;
    hipGraph_t g = nullptr;
    VOX_HIP(hipStreamEndCapture((hipStream_t)stream, &g));
#ifdef VOX_DEV_KNOBS
    if (getenv("VOX_GRAPH_INFO")) {     // (dev knob: node / edge counts and node types of the captured graph)
        size_t nn = 0, ne = 0;
        (void)hipGraphGetNodes(g, nullptr, &nn); (void)hipGraphGetEdges(g, nullptr, nullptr, &ne);
        std::vector<hipGraphNode_t> nodes(nn);
        (void)hipGraphGetNodes(g, nodes.data(), &nn);
        int types[16] = {0};
        for (auto n : nodes) { hipGraphNodeType t; if (hipGraphNodeGetType(n, &t) == hipSuccess && (int)t < 16) types[(int)t]++; }
        fprintf(stderr, "[vox graph] %zu nodes, %zu edges; types:", nn, ne);
        for (int t = 0; t < 16; ++t) if (types[t]) fprintf(stderr, " %d:%d", t, types[t]);
        fprintf(stderr, "\n");
        if (const char* dot = getenv("VOX_GRAPH_DOT")) (void)hipGraphDebugDotPrint(g, dot, 0);
    }
#endif
    hipGraphExec_t e = nullptr;
    hipError_t err = hipGraphInstantiate(&e, g, nullptr, nullptr, 0);
    if (err != hipSuccess) {
        (void)hipGraphDestroy(g);
        return vox_fail(VOX_ERR_HIP, "hipGraphInstantiate: %s", hipGetErrorString(err));
    }
    vox_graph* vg = new vox_graph();
    vg->graph = g;
    vg->exec = e;
    *out = vg;
    return VOX_OK;
}
int vox_graph_launch(vox_graph* g, void* stream) {
    if (!g) return vox_fail(VOX_ERR_INVALID, "graph_launch: NULL");
    VOX_HIP(hipGraphLaunch(g->exec, (hipStream_t)stream));
    return VOX_OK;
}
void vox_graph_destroy(vox_graph* g) {
    if (!g) return;
    (void)hipGraphExecDestroy(g->exec);
    (void)hipGraphDestroy(g->graph);
    delete g;
}

}  // extern "C"

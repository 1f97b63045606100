// cblas_sgemm / cblas_dgemm as the reference declares them itself (rl_tools/devices/cpu_openblas.h:9-27), forwarded to
// a CBLAS that exists in this image but cannot be linked by name: scipy's bundled OpenBLAS exports the same
// functions with a `scipy_` prefix; MKL's libmkl_rt.so exports them un-prefixed. The provider is picked at the first call
// from $RLT_CBLAS_LIB (a path) or the built-in search list, and pinned to one thread, which the reference's OpenBLAS
// device requires (devices/cpu_openblas.h:31-47).
#include <dlfcn.h>
#include <glob.h>
#include <cstdio>
#include <cstdlib>
#include <cstring>

extern "C" {
typedef void (*sgemm_fn)(int, int, int, int, int, int, float, const float*, int, const float*, int, float, float*, int);
typedef void (*dgemm_fn)(int, int, int, int, int, int, double, const double*, int, const double*, int, double, double*, int);

static sgemm_fn g_sgemm = nullptr;
static dgemm_fn g_dgemm = nullptr;
static char g_name[512] = "";

static bool try_load(const char* path) {
    void* h = dlopen(path, RTLD_NOW | RTLD_LOCAL);
    if (!h) return false;
    void* s = dlsym(h, "cblas_sgemm"); if (!s) s = dlsym(h, "scipy_cblas_sgemm");
    void* d = dlsym(h, "cblas_dgemm"); if (!d) d = dlsym(h, "scipy_cblas_dgemm");
    if (!s || !d || s == (void*)&g_sgemm) return false;
    typedef void (*set_threads_fn)(int);
    const char* setters[] = {"openblas_set_num_threads", "scipy_openblas_set_num_threads", "MKL_Set_Num_Threads"};
    for (const char* n : setters) if (void* st = dlsym(h, n)) { ((set_threads_fn)st)(1); break; }
    g_sgemm = (sgemm_fn)s; g_dgemm = (dgemm_fn)d;
    std::snprintf(g_name, sizeof g_name, "%s", path);
    return true;
}
static void resolve() {
    if (g_sgemm) return;
    if (const char* env = std::getenv("RLT_CBLAS_LIB")) if (try_load(env)) return;
    const char* patterns[] = {
        "/usr/local/lib/python3*/dist-packages/scipy.libs/libscipy_openblas-*.so",
        "/usr/lib/x86_64-linux-gnu/libopenblas.so*",
        "/opt/conda/lib/libmkl_rt.so",
    };
    for (const char* p : patterns) {
        glob_t g; std::memset(&g, 0, sizeof g);
        if (glob(p, 0, nullptr, &g) == 0) for (size_t i = 0; i < g.gl_pathc; i++) if (try_load(g.gl_pathv[i])) { globfree(&g); return; }
        globfree(&g);
    }
    std::fprintf(stderr, "rlt_ref: no CBLAS provider found (set RLT_CBLAS_LIB)\n");
    std::abort();
}
const char* rlt_ref_cblas_name(void) { resolve(); return g_name; }

void cblas_sgemm(int order, int ta, int tb, int m, int n, int k, float alpha, const float* a, int lda, const float* b, int ldb, float beta, float* c, int ldc) {
    resolve(); g_sgemm(order, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
}
void cblas_dgemm(int order, int ta, int tb, int m, int n, int k, double alpha, const double* a, int lda, const double* b, int ldb, double beta, double* c, int ldc) {
    resolve(); g_dgemm(order, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
}
}

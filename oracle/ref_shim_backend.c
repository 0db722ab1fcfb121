/* TEST INFRASTRUCTURE ONLY -- never linked into, loaded by, or timed as the product.
 *
 * Lets the reference's own engine code (decoder_run, local_step_device: src/graph.c) drive the
 * gfx950 library through the reference's own `struct mynah_backend`, the way a maintainer's
 * `#if defined(MYNAH_ENABLE_HIP)` block in src/backend.c would: the same assignments, field by
 * field, as the CUDA branch at src/backend.c:442-465.  The reference source is NOT copied: the
 * include below resolves through -I<reference>/src (oracle/Makefile) and takes the place of
 * compiling src/backend.c by itself, so this translation unit sees the struct's definition
 * (src/backend.c:26-70), which no header exports.
 *
 * The library is found at run time with dlopen, so the compiled reference still loads where no
 * GPU runtime is installed.  The C-ABI header is included for its prototypes: every assignment
 * below is then checked by the compiler against the function-pointer type of the reference's
 * field (built with -Werror=incompatible-pointer-types).
 */
#include "backend.c"

#include <dlfcn.h>

#include "mynah_hip.h"

/* dlsym through a pointer of the header's own prototype type: `backend->field = p` fails to
 * compile when the header and the reference's struct disagree. */
#define REF_BIND(field, symbol)                                                    \
    do {                                                                           \
        __typeof__(&symbol) p_ = (__typeof__(&symbol))dlsym(handle, #symbol);      \
        if (p_ == NULL) {                                                          \
            if (error != NULL && error_capacity > 0)                               \
                snprintf(error, error_capacity, "missing symbol %s", #symbol);     \
            free(backend);                                                         \
            return NULL;                                                           \
        }                                                                          \
        backend->field = p_;                                                       \
    } while (0)

/* What mynah_backend_open(MYNAH_TTS_DEVICE_HIP, ...) would do (src/backend.c:367-475).  The
 * device value 3 is the enum member the integration adds after CUDA (src/mynah_tts.h:11-15). */
mynah_backend *ref_backend_open_hip(const char *library_path, char *error, size_t error_capacity) {
    void *handle = dlopen(library_path, RTLD_NOW | RTLD_GLOBAL);
    if (handle == NULL) {
        if (error != NULL && error_capacity > 0) snprintf(error, error_capacity, "dlopen: %s", dlerror());
        return NULL;
    }
    mynah_backend *backend = (mynah_backend *)calloc(1, sizeof(*backend));
    if (backend == NULL) return NULL;
    backend->device = (mynah_tts_device)3;
    backend->name = "hip";
    __typeof__(&mynah_backend_hip_open) open_fn =
        (__typeof__(&mynah_backend_hip_open))dlsym(handle, "mynah_backend_hip_open");
    if (open_fn == NULL) {
        if (error != NULL && error_capacity > 0) snprintf(error, error_capacity, "missing symbol mynah_backend_hip_open");
        free(backend);
        return NULL;
    }
    if (open_fn(&backend->state, &backend->matmul, &backend->sgemm, &backend->close, &backend->self_test,
                error, error_capacity) != 0) {
        free(backend);
        return NULL;
    }
    REF_BIND(upload, mynah_hip_upload);
    REF_BIND(download, mynah_hip_download);
    REF_BIND(sync, mynah_hip_sync);
    REF_BIND(batch_begin, mynah_hip_batch_begin);
    REF_BIND(gelu_dev, mynah_hip_gelu_dev);
    REF_BIND(layer_norm_dev, mynah_hip_layer_norm_dev);
    REF_BIND(residual_add_dev, mynah_hip_residual_add_dev);
    REF_BIND(matmul_dev, mynah_hip_matmul_dev);
    REF_BIND(sgemm_dev, mynah_hip_sgemm_dev);
    REF_BIND(dev_alloc, mynah_hip_dev_alloc);
    REF_BIND(dev_free, mynah_hip_dev_free);
    REF_BIND(h2d, mynah_hip_h2d);
    REF_BIND(d2h, mynah_hip_d2h);
    REF_BIND(copy_dev, mynah_hip_copy_dev);
    REF_BIND(scale_dev, mynah_hip_scale_dev);
    REF_BIND(clip_dev, mynah_hip_clip_dev);
    REF_BIND(argmax_dev, mynah_hip_argmax_dev);
    REF_BIND(matvec_dev, mynah_hip_matvec_dev);
    REF_BIND(gelu_inplace, mynah_hip_gelu_inplace);
    REF_BIND(residual_inplace, mynah_hip_residual_inplace);
    REF_BIND(layer_norm_inplace, mynah_hip_layer_norm_inplace);
    REF_BIND(matmul_to_dev, mynah_hip_matmul_to_dev);
    REF_BIND(matmul_d2d, mynah_hip_matmul_d2d);
    REF_BIND(self_attention_dev, mynah_hip_self_attention_dev);
    REF_BIND(cross_attention_dev, mynah_hip_cross_attention_dev);
    REF_BIND(conv1d, mynah_hip_conv1d);
    REF_BIND(conv_transpose_dev, mynah_hip_conv_transpose_dev);
    REF_BIND(snake_dev, mynah_hip_snake_dev);
    REF_BIND(im2col, mynah_hip_im2col);
    REF_BIND(gelu_host, mynah_hip_gelu_host);
    REF_BIND(gelu_host_f64, mynah_hip_gelu_host_f64);
    REF_BIND(matmul_graph, mynah_hip_matmul_graph);
    if (error != NULL && error_capacity > 0) error[0] = '\0';
    return backend;
}

/* The backend's opaque state, for the one library call the tests make beside the engine
 * (choosing the weight storage type of a backend that is already open). */
void *ref_backend_state(const mynah_backend *backend) { return backend != NULL ? backend->state : NULL; }

int ref_backend_self_test(const mynah_backend *backend, char *error, size_t error_capacity) {
    if (backend == NULL || backend->self_test == NULL) return -1;
    return backend->self_test(backend->state, error, error_capacity);
}

// Text-encoder prefill on the matrix cores (placeholder translation unit: filled in below).
#include "kernels.h"

struct mynah_hip_encoder { int unused; };

using namespace mynah;

extern "C" int mynah_hip_encoder_create(void *, const mynah_hip_encoder_desc *, mynah_hip_encoder **out, char *error, size_t capacity) {
    if (out != nullptr) *out = nullptr;
    set_error(error, capacity, "encoder prefill is not available in this build");
    return -1;
}
extern "C" void mynah_hip_encoder_destroy(void *, mynah_hip_encoder *) {}
extern "C" int mynah_hip_encoder_prefill(void *, mynah_hip_encoder *, const int32_t *, size_t, uint16_t *, float *, char *error, size_t capacity) {
    set_error(error, capacity, "encoder prefill is not available in this build");
    return -1;
}

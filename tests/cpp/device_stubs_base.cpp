// Host stand-ins for the device half of the C ABI, for a CPU-only build of the host layer
// (host/*.cpp + include/et/*.h) under AddressSanitizer / UndefinedBehaviorSanitizer:
// "device" buffers are calloc'ed host memory, copies are memcpy, fills really fill, streams,
// graphs and events are opaque tokens.  The compute entry points are generated next to this
// file by tests/test_host_sanitized.py as functions that return ET_OK and touch nothing.
// No header of the library is included on purpose: the generated stand-ins are declared
// without parameters, which C linkage allows and the ABI header would contradict.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

extern "C" {

static thread_local char g_err[512];
const char *et_last_error(void) { return g_err; }
void et_set_last_error(const char *m) { snprintf(g_err, sizeof g_err, "%s", m ? m : ""); }
const char *et_status_string(int) { return "stand-in"; }

int et_malloc(void **p, size_t n) {
    *p = calloc(n ? n : 16, 1);
    return *p ? 0 : -3;
}
int et_free(void *p) {
    free(p);
    return 0;
}
int et_memcpy_h2d(void *d, const void *s, size_t n) {
    if (n) memcpy(d, s, n);
    return 0;
}
int et_memcpy_d2h(void *d, const void *s, size_t n) {
    if (n) memcpy(d, s, n);
    return 0;
}
int et_memcpy_d2d(void *d, const void *s, size_t n, void *) {
    if (n) memmove(d, s, n);
    return 0;
}
int et_memcpy_auto(void *d, const void *s, size_t n) {
    if (n) memmove(d, s, n);
    return 0;
}
int et_memset(void *d, int b, size_t n, void *) {
    if (n) memset(d, b, n);
    return 0;
}
int et_fill_f16(uint16_t *d, size_t n, uint16_t v, void *) {
    for (size_t i = 0; i < n; i++) d[i] = v;
    return 0;
}
int et_fill_i32(int32_t *d, size_t n, int32_t v, void *) {
    for (size_t i = 0; i < n; i++) d[i] = v;
    return 0;
}
int et_stream_create(void **s) {
    *s = reinterpret_cast<void *>(0x10);
    return 0;
}
int et_graph_end_capture(void *, void **g) {
    *g = reinterpret_cast<void *>(0x20);
    return 0;
}
int et_event_create(void **e) {
    *e = reinterpret_cast<void *>(0x30);
    return 0;
}
int et_event_elapsed_ms(float *ms, void *, void *) {
    *ms = 1.0f;
    return 0;
}
int et_device_info(char *name, int cap, int *cu, int *lds) {
    if (name && cap > 0) snprintf(name, (size_t)cap, "stand-in");
    if (cu) *cu = 256;
    if (lds) *lds = 160 * 1024;
    return 0;
}
int et_linear_bsr16_fused_ln_supported(int, int, int) { return 0; }

}  // extern "C"

// Host-side exercise of the C ABI for a sanitised CPU build (AddressSanitizer + UndefinedBehaviorSanitizer on
// the host pass; no device code is compiled or run).  It walks the parts of the library that run before any
// kernel is launched: status strings, the thread-local error text (including messages longer than its buffer),
// the support predicates, every entry point's argument checks, and the launch-geometry arithmetic
// (make_row_plan) over a sweep of shapes including 64-bit row counts.  With no GPU in the machine a call whose
// arguments pass the checks stops at the device query and returns TT_NORM_EHIP; when a GPU is present those
// calls are skipped, because their pointers are made up.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/teletron_norm.h"
#include "../../include/teletron_probe.h"
#include "../../teletron_amd/csrc/norm_host.h"

// The host objects register their (absent) device code at load time; nothing here launches a kernel.
extern "C" void **__hipRegisterFatBinary(const void *) {
    static void *handle = nullptr;
    return &handle;
}
extern "C" void __hipRegisterFunction(void **, const void *, char *, const char *, unsigned, void *, void *, void *,
                                      void *, int *) {}
extern "C" void __hipRegisterVar(void **, void *, char *, const char *, int, size_t, int, int) {}
extern "C" void __hipUnregisterFatBinary(void **) {}

static int g_failures = 0;
#define EXPECT(cond)                                                                  \
    do {                                                                              \
        if (!(cond)) {                                                                \
            fprintf(stderr, "%s:%d: EXPECT(%s) failed; last error: %s\n", __FILE__, __LINE__, #cond, \
                    tt_norm_last_error());                                            \
            ++g_failures;                                                             \
        }                                                                             \
    } while (0)

static void *fake(uintptr_t a) { return reinterpret_cast<void *>(a); }

static void status_strings() {
    for (int s = -3; s < 12; ++s) {
        const char *t = tt_norm_status_string(s);
        EXPECT(t != nullptr && strlen(t) > 1);
    }
    EXPECT(strcmp(tt_norm_status_string(TT_NORM_OK), "ok") == 0);
    EXPECT(tt_norm_abi_version() == TT_NORM_ABI_VERSION);
    EXPECT(tt_probe_abi_version() == TT_PROBE_ABI_VERSION);
    // a message far longer than the error buffer must be cut, not overflow it
    char longname[2048];
    memset(longname, 'x', sizeof(longname) - 1);
    longname[sizeof(longname) - 1] = 0;
    EXPECT(ttn::fail(TT_NORM_EINVAL, "%s: %s", longname, longname) == TT_NORM_EINVAL);
    EXPECT(strlen(tt_norm_last_error()) < 600);
}

static void predicates() {
    const int dts[] = {TT_NORM_BF16, TT_NORM_F32, TT_NORM_F16, 3, -1, 1 << 30};
    const int64_t cols[] = {INT64_MIN, -8, 0, 1, 4, 8, 12, 128, 3064, 3072, 3080, 4096, 8192, 8200, 1 << 20,
                            INT64_MAX};
    for (int dt : dts)
        for (int64_t c : cols) {
            const int s = tt_norm_supported(c, dt), t = tt_norm_tuned(c, dt), w = tt_norm_wide_forms_supported(c, dt);
            EXPECT((s == 0 || s == 1) && (t == 0 || t == 1) && (w == 0 || w == 1));
            EXPECT(!t || s);   // tuned shapes are supported shapes
            EXPECT(!w || s);   // the wide forms exist for supported shapes only
        }
    EXPECT(tt_norm_wide_forms_supported(3072, TT_NORM_F32) == 1 && tt_norm_wide_forms_supported(1540, TT_NORM_F32) == 1);
    EXPECT(tt_norm_wide_forms_supported(4100, TT_NORM_F32) == 0 && tt_norm_wide_forms_supported(3076, TT_NORM_BF16) == 0);
}

static void row_plans() {
    const int64_t rows[] = {0, 1, 2, 3, 4, 5, 15, 16, 17, 1023, 1024, 1025, 29700, 118800, 712800, (int64_t)1 << 31,
                            ((int64_t)1 << 40) + 3, INT64_MAX / 64};
    const int64_t batches[] = {1, 2, 3, 4, 255, 256, 257, 700, 100000};
    const int rpws[] = {1, 2, 4, 8, 24, 48};
    const int per_cu[] = {1, 2, 3, 6, 16, 1 << 20};
    const int cus[] = {1, 8, 104, 256, 304};
    for (int64_t r : rows)
        for (int64_t b : batches)
            for (int w : rpws)
                for (int pc : per_cu)
                    for (int cu : cus) {
                        const ttn::RowPlan p = ttn::make_row_plan(b, r, w, pc, cu);
                        EXPECT(p.blocks_per_sample >= 1);
                        EXPECT(p.blocks == b * p.blocks_per_sample);
                        EXPECT(p.rows_per_wave == w);
                        const int64_t per_block = (int64_t)ttn::kRowWaves * w;
                        const int64_t needed = r / per_block + (r % per_block != 0);
                        EXPECT(p.blocks_per_sample <= (needed > 1 ? needed : 1));   // no workgroup without rows
                    }
}

static void argument_checks(bool have_gpu) {
    void *a = fake(0x10000), *b = fake(0x20000), *c = fake(0x30000), *d = fake(0x40000), *odd = fake(0x10008);
    float *f = reinterpret_cast<float *>(fake(0x50000));
    // null pointers, negative sizes, unsupported widths, misaligned pointers: all decided on the host
    EXPECT(tt_rmsnorm_forward(nullptr, f, b, c, 4, 3072, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_EINVAL);
    EXPECT(tt_rmsnorm_forward(a, f, b, c, -1, 3072, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_EINVAL);
    EXPECT(tt_rmsnorm_forward(a, f, b, c, 4, 1004, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_EUNSUPPORTED);
    EXPECT(tt_rmsnorm_forward(a, f, b, c, 4, 3072, 1e-6, 9, nullptr) == TT_NORM_EUNSUPPORTED);
    EXPECT(tt_rmsnorm_forward(odd, f, b, c, 4, 3072, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_EALIGN);
    EXPECT(tt_rmsnorm_forward(a, nullptr, b, c, 4, 3072, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_EINVAL);
    EXPECT(tt_rmsnorm_forward(nullptr, nullptr, nullptr, nullptr, 0, 3072, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_OK);
    EXPECT(tt_rmsnorm_backward(a, nullptr, b, c, d, f, 4, 3072, TT_NORM_BF16, nullptr, 0, nullptr) == TT_NORM_EINVAL);
    EXPECT(tt_rmsnorm_backward_from_out(a, b, b, c, d, f, 4, 256, TT_NORM_BF16, nullptr, 0, nullptr) == TT_NORM_EUNSUPPORTED);
    EXPECT(tt_adaln_forward(a, f, f, b, c, d, 0, 4, 3072, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_EINVAL);
    EXPECT(tt_adaln_forward(a, nullptr, f, b, c, d, 1, 4, 3072, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_EINVAL);
    EXPECT(tt_adaln_forward_xnorm(a, b, f, b, c, d, 1, 4, 1536, 1e-6, TT_NORM_F16, nullptr) == TT_NORM_EUNSUPPORTED);
    EXPECT(tt_adaln_backward(a, nullptr, b, c, d, a, f, f, 1, 4, 3072, TT_NORM_BF16, nullptr, 0, nullptr) == TT_NORM_EINVAL);
    EXPECT(tt_adaln_backward_from_xnorm(a, b, c, d, a, b, f, 1, 4, 640, TT_NORM_BF16, nullptr, 0, nullptr) ==
           TT_NORM_EUNSUPPORTED);
    // sequence-first: batch * cols * element size above 256 MiB is refused
    EXPECT(tt_adaln_forward_seq_first(a, f, f, b, c, d, 40000, 4, 8192, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_EINVAL);
    // strided views: negative sizes, strides that are not multiples of 16 bytes, row strides above 256 MiB
    EXPECT(tt_rmsnorm_forward_strided(a, f, b, c, 1, -2, 3, 0, 0, 128, 128, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_EINVAL);
    EXPECT(tt_rmsnorm_forward_strided(a, f, b, c, 1, 2, 3, 0, 0, 132, 128, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_EALIGN);
    EXPECT(tt_rmsnorm_forward_strided(a, f, b, c, 1, 2, 3, 0, 0, -128, 128, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_EALIGN);
    EXPECT(tt_rmsnorm_forward_strided(a, f, b, c, 1, 2, 3, 0, 0, (int64_t)1 << 28, 128, 1e-6, TT_NORM_BF16, nullptr) ==
           TT_NORM_EINVAL);
    EXPECT(tt_rmsnorm_backward_strided(a, b, c, d, a, f, 1, 2, 3, 0, 384, 9216, 0, 4, 9216, 128, TT_NORM_BF16, nullptr, 0,
                                       nullptr) == TT_NORM_EALIGN);
    EXPECT(tt_norm_copy_rows_strided(a, b, 1, 1, 64, 0, 0, 388, 128, TT_NORM_BF16, nullptr) == TT_NORM_EALIGN);
    EXPECT(tt_norm_copy_rows_strided(a, b, 1, 1, 64, 0, 0, 384, 100, TT_NORM_BF16, nullptr) == TT_NORM_EUNSUPPORTED);
    EXPECT(tt_norm_copy_rows_strided(a, b, 0, 1, 64, 0, 0, 384, 128, TT_NORM_BF16, nullptr) == TT_NORM_OK);
    // rotary form: head dimension 128 only, table length within the token count
    EXPECT(tt_rmsnorm_rope_forward_strided(a, f, b, c, f, f, 4, 1, 2, 3, 0, 0, 128, 128, 1e-6, TT_NORM_BF16, nullptr) ==
           TT_NORM_EINVAL);
    EXPECT(tt_rmsnorm_rope_forward_strided(a, f, b, c, f, f, 2, 1, 2, 3, 0, 0, 64, 64, 1e-6, TT_NORM_BF16, nullptr) ==
           TT_NORM_EUNSUPPORTED);
    // gated / residual forms on rows that are not whole 16-byte pieces, or wider than 1024 of them
    EXPECT(tt_gated_residual_adaln_forward(a, b, f, f, a, b, c, d, a, 1, 4, 3076, 1e-6, TT_NORM_BF16, nullptr) ==
           TT_NORM_EUNSUPPORTED);
    EXPECT(tt_adaln_backward_residual(a, b, c, d, a, b, c, f, f, 1, 4, 4100, TT_NORM_F32, nullptr, 0, nullptr) ==
           TT_NORM_EUNSUPPORTED);
    EXPECT(tt_gated_residual_adaln_backward_workspace_bytes(1, 4, 8200, TT_NORM_BF16) == 0);
    // the entry point with static scratch: a shape that cannot fit is refused before anything else happens
    EXPECT(tt_adaln_backward_static(a, b, c, d, a, b, f, f, -1, 4, 3072, TT_NORM_BF16, nullptr) == TT_NORM_EINVAL);
    // the event hook: both or neither
    EXPECT(tt_norm_profile_next_row_kernel(a, nullptr) == TT_NORM_EINVAL);
    EXPECT(tt_norm_profile_next_row_kernel(nullptr, nullptr) == TT_NORM_OK);
    // workspace queries with nonsense
    EXPECT(tt_rmsnorm_backward_workspace_bytes(-5, 3072, TT_NORM_BF16) == 0);
    EXPECT(tt_rmsnorm_backward_workspace_bytes(5, 3071, TT_NORM_BF16) == 0);
    EXPECT(tt_adaln_backward_workspace_bytes(0, 5, 3072, TT_NORM_BF16) == 0);
    // the probe library's checks
    EXPECT(tt_probe_stream_copy(nullptr, a, 32, nullptr) == 1);
    EXPECT(tt_probe_stream_copy(a, b, 24, nullptr) == 1);
    EXPECT(tt_probe_stream_copy(odd, b, 32, nullptr) == 3);
    EXPECT(tt_probe_stream_copy(a, b, 0, nullptr) == 0);
    EXPECT(tt_probe_stream(a, 4096, b, 4096, c, 4096, 4096, 3, 1, 1, 0, 0, nullptr) == 1);
    EXPECT(tt_probe_stream(a, 4096, b, 4096, c, 4096, 4096, 2, 1, 3, 0, 0, nullptr) == 2);
    EXPECT(tt_probe_stream(a, 4096, b, 4096, c, 4096, 4100, 2, 1, 1, 0, 0, nullptr) == 1);
    EXPECT(strlen(tt_probe_last_error()) > 0);
    if (!have_gpu) {
        // arguments that pass every check: the call stops at the device query
        EXPECT(tt_rmsnorm_forward(a, f, b, c, 4, 3072, 1e-6, TT_NORM_BF16, nullptr) == TT_NORM_EHIP);
        EXPECT(tt_adaln_forward(a, f, f, b, c, d, 2, 4, 1000, 1e-6, TT_NORM_F16, nullptr) == TT_NORM_EHIP);
        EXPECT(tt_rmsnorm_backward_workspace_bytes(5, 3072, TT_NORM_BF16) == 0);
        EXPECT(tt_adaln_backward_static(a, b, c, d, a, b, f, f, 1, 4, 3072, TT_NORM_BF16, nullptr) != TT_NORM_OK);
    }
}

int main() {
    int n = 0;
    const bool have_gpu = hipGetDeviceCount(&n) == hipSuccess && n > 0;
    (void)hipGetLastError();
    status_strings();
    predicates();
    row_plans();
    argument_checks(have_gpu);
    if (g_failures) {
        fprintf(stderr, "%d expectation(s) failed\n", g_failures);
        return 1;
    }
    printf("host sanitize driver ok (gpu present: %d)\n", (int)have_gpu);
    return 0;
}

/* TEST INFRASTRUCTURE: hardware half<->float conversions (x86 F16C), used to pin
 * the oracle's software conversions.  The `half` crate the reference uses
 * (Q/reference/q4_k.rs:351-353, Q/quantize.rs:201) defines the same IEEE binary16
 * round-to-nearest-even semantics. */
#include <immintrin.h>
#include <stddef.h>
#include <stdint.h>

void oxq_f16c_to_f32(const uint16_t *h, float *out, size_t n) {
    for (size_t i = 0; i < n; i++) {
        out[i] = _cvtsh_ss(h[i]);
    }
}

void oxq_f16c_from_f32(const float *f, uint16_t *out, size_t n) {
    for (size_t i = 0; i < n; i++) {
        out[i] = _cvtss_sh(f[i], _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
    }
}

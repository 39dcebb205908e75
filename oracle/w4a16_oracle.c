/* TEST INFRASTRUCTURE ONLY - scalar C restatement of the reference's CPU loops,
 * compiled with gcc so that the exact sequential semantics can be evaluated at
 * full problem sizes.  Never linked into the product library.
 *
 * Follows (PE = programming_examples):
 *   oracle_matvec_loop   PE/matrix_vector_multiplication/int4_awq/matvec_int4_packed.py:272-287
 *   oracle_dequant_awq   PE/llms/llama32_1b_int4/awq_repacker.py:41-82 (unpack + dequant)
 *
 * Checked in tests/test_oracle_reference.py against the Python restatement
 * (oracle/reference.py, oracle/awq.py) and closed forms.
 */
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu)) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* D[r] = bf16( sequential float32 sum over k of (nib - z) * s * b[k] ), where each
 * term is evaluated in double and the running sum is rounded to float32 after
 * every addition (NumPy: float32 array element += float64 scalar). */
void oracle_matvec_loop(const uint8_t *a_q, const uint16_t *a_s, const uint8_t *a_z,
                        const uint16_t *b, int M, int K, int gs, uint16_t *out) {
    int n_groups = K / gs;
    (void)n_groups;
    for (int r = 0; r < M; ++r) {
        float d = 0.0f;
        for (int kk = 0; kk < K; ++kk) {
            uint8_t byte = a_q[(size_t)r * (K / 2) + kk / 2];
            int nib = (kk % 2 == 0) ? (byte & 0x0F) : ((byte >> 4) & 0x0F);
            int g = kk / gs;
            double term = (double)(nib - (int)a_z[(size_t)g * M + r]) *
                          (double)bf16_to_f32(a_s[(size_t)g * M + r]) * (double)bf16_to_f32(b[kk]);
            d = (float)((double)d + term);
        }
        out[r] = f32_to_bf16(d);
    }
}

/* natural column j of an 8-column block sits at bit position 4 * perm[j] */
static const int awq_unpack_perm[8] = {0, 4, 1, 5, 2, 6, 3, 7};

void oracle_dequant_awq(const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                        int K, int N, int gs, uint16_t *out) {
    int nb = N / 8;
    for (int k = 0; k < K; ++k) {
        int g = k / gs;
        for (int n = 0; n < N; ++n) {
            uint32_t w = (uint32_t)qweight[(size_t)k * nb + n / 8];
            uint32_t zw = (uint32_t)qzeros[(size_t)g * nb + n / 8];
            int sh = 4 * awq_unpack_perm[n % 8];
            int q = (int)((w >> sh) & 0xF);
            int z = (int)((zw >> sh) & 0xF);
            float v = (float)(q - z) * bf16_to_f32(scales[(size_t)g * N + n]);
            out[(size_t)k * N + n] = f32_to_bf16(v);
        }
    }
}

/*
 * Driver around the reference's vendored ggml C quantizers (TEST INFRASTRUCTURE).
 * Linked against third_party/llama.cpp-fork/ggml/src/ggml-quants.c compiled where it lies in the reference tree;
 * no reference source is copied here. Usage: ggml_quant_ref <q8_0|q4_0> <in.f32> <out.bin>
 * in.f32 = n*32 little-endian floats; out.bin = n ggml blocks (q8_0: 34 B = f16 d + 32 int8; q4_0: 18 B).
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* prototypes of ggml-quants.h:17-28 restated with opaque block pointers */
void quantize_row_q8_0_ref(const float *x, void *y, int64_t k);
void quantize_row_q4_0_ref(const float *x, void *y, int64_t k);
void dequantize_row_q8_0(const void *x, float *y, int64_t k);
void dequantize_row_q4_0(const void *x, float *y, int64_t k);

int main(int argc, char **argv) {
    if (argc != 4) { fprintf(stderr, "usage: %s <q8_0|q4_0|dq8_0|dq4_0> in out\n", argv[0]); return 2; }
    FILE *f = fopen(argv[2], "rb");
    if (!f) { perror(argv[2]); return 2; }
    fseek(f, 0, SEEK_END);
    const long bytes = ftell(f);
    fseek(f, 0, SEEK_SET);
    void *in = malloc((size_t) bytes + 64);
    if (fread(in, 1, (size_t) bytes, f) != (size_t) bytes) { perror("read"); return 2; }
    fclose(f);
    void *out = NULL;
    size_t out_bytes = 0;
    if (!strcmp(argv[1], "q8_0") || !strcmp(argv[1], "q4_0")) {
        const int64_t n = bytes / 4 / 32 * 32;
        const size_t bb = argv[1][1] == '8' ? 34 : 18;
        out_bytes = (size_t) (n / 32) * bb;
        out = calloc(out_bytes + 64, 1);
        if (argv[1][1] == '8') quantize_row_q8_0_ref((const float *) in, out, n);
        else quantize_row_q4_0_ref((const float *) in, out, n);
    } else {
        const size_t bb = argv[1][2] == '8' ? 34 : 18;
        const int64_t n = (int64_t) (bytes / bb) * 32;
        out_bytes = (size_t) n * 4;
        out = calloc(out_bytes + 64, 1);
        if (argv[1][2] == '8') dequantize_row_q8_0(in, (float *) out, n);
        else dequantize_row_q4_0(in, (float *) out, n);
    }
    f = fopen(argv[3], "wb");
    if (!f) { perror(argv[3]); return 2; }
    fwrite(out, 1, out_bytes, f);
    fclose(f);
    return 0;
}

// TEST INFRASTRUCTURE. Command-line front end of the oracle's dequantiser with the argument contract of the
// reference's tools/dqcpu.c:7 and tools/dqtest.c:16: <ggml type> <K> <rows> <raw blocks in> <float32 out>.
// Exit codes follow the reference: 2 usage, 3 unsupported type, 1 I/O.
#include "qw_oracle.h"
#include <stdio.h>
#include <stdlib.h>

int main(int argc, char **argv) {
    if (argc != 6) { fprintf(stderr, "usage: %s <type> <K> <rows> <in> <out>\n", argv[0]); return 2; }
    const int type = atoi(argv[1]), K = atoi(argv[2]), rows = atoi(argv[3]);
    if (!qwo_dq_ok(type)) { fprintf(stderr, "unsupported type %d\n", type); return 3; }
    if (rows <= 0 || K <= 0 || K % qwo_block_values(type)) { fprintf(stderr, "bad shape\n"); return 2; }
    FILE *f = fopen(argv[4], "rb");
    if (!f) return 1;
    const size_t rb = qwo_row_bytes(type, K), n = rb * (size_t)rows;
    unsigned char *in = malloc(n);
    float *out = malloc(sizeof(float) * (size_t)K * (size_t)rows);
    if (fread(in, 1, n, f) != n) { fprintf(stderr, "short input\n"); return 1; }
    fclose(f);
    for (int r = 0; r < rows; r++) qwo_dq_row(type, in + (size_t)r * rb, out + (size_t)r * K, K);
    f = fopen(argv[5], "wb");
    if (!f) return 1;
    fwrite(out, sizeof(float), (size_t)K * (size_t)rows, f);
    fclose(f);
    return 0;
}

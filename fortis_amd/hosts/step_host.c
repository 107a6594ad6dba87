/* A plain C host for a generated step file: it knows the entry points only by name, as a Fortran host
 * does through bind(c) (benchmarks/toy/bench_fortis.f90:5-11, bench_dev.f90:4-11), and links against
 * step_tables.o + weights.o + libfortis_rt.so.
 *
 *   step_host <mode> <in.bin> <out.bin> <in_bytes> <out_bytes> [calls] [rows]
 *     call     mlp_forward(in, out)                                   (whole-array / boundary verdict)
 *     dev      mlp_upload(in); mlp_forward_dev() x calls; mlp_download(out)
 *     slice    mlp_forward_batched(in, out)                           (batched verdict, slice form)
 *     packed   fortis_pack(row, col) x rows; mlp_forward_batched(); fortis_unpack(row, col) x rows
 * Prints `checksum: <sum of the output read as float>` and the microseconds per call. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

void mlp_forward(void* in, void* out);
void mlp_upload(void* in);
void mlp_forward_dev(void);
void mlp_download(void* out);
void mlp_forward_batched(void* in, void* out);
void fortis_pack(void* row, int col);
void fortis_unpack(void* row, int col);

int main(int argc, char** argv)
{
    if (argc < 6) { fprintf(stderr, "usage: step_host call|dev|slice|packed in.bin out.bin in_bytes out_bytes [calls] [rows]\n"); return 2; }
    const char* mode = argv[1];
    const long nin = atol(argv[4]), nout = atol(argv[5]);
    const int calls = argc > 6 ? atoi(argv[6]) : 1;
    const long rows = argc > 7 ? atol(argv[7]) : 1;
    char* in = malloc(nin);
    char* out = calloc(nout, 1);
    FILE* f = fopen(argv[2], "rb");
    if (!in || !out || !f || fread(in, 1, nin, f) != (size_t)nin) { fprintf(stderr, "step_host: cannot read %ld bytes of %s\n", nin, argv[2]); return 1; }
    fclose(f);
    struct timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    if (!strcmp(mode, "call")) {
        for (int c = 0; c < calls; c++) mlp_forward(in, out);
    } else if (!strcmp(mode, "dev")) {
        mlp_upload(in);
        for (int c = 0; c < calls; c++) mlp_forward_dev();
        mlp_download(out);
    } else if (!strcmp(mode, "slice")) {
        for (int c = 0; c < calls; c++) mlp_forward_batched(in, out);
    } else if (!strcmp(mode, "packed")) {
        const long rin = nin / rows, rout = nout / rows;
        for (int c = 0; c < calls; c++) {
            for (long r = 0; r < rows; r++) fortis_pack(in + r * rin, (int)r);
            mlp_forward_batched(0, 0);
            for (long r = 0; r < rows; r++) fortis_unpack(out + r * rout, (int)r);
        }
    } else { fprintf(stderr, "step_host: unknown mode %s\n", mode); return 2; }
    clock_gettime(CLOCK_MONOTONIC, &t1);
    f = fopen(argv[3], "wb");
    if (!f || fwrite(out, 1, nout, f) != (size_t)nout) { fprintf(stderr, "step_host: cannot write %s\n", argv[3]); return 1; }
    fclose(f);
    double sum = 0;
    for (long i = 0; i < nout / 4; i++) sum += ((float*)out)[i];
    printf("checksum: %.6f\nper-call us: %.2f\n", sum, ((t1.tv_sec - t0.tv_sec) * 1e9 + (t1.tv_nsec - t0.tv_nsec)) / 1e3 / calls);
    return 0;
}

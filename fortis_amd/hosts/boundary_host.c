/* A host with a boundary verdict: its own double-precision column-major arrays go to mlp_forward, and the
 * normalisation vectors are program-scope arrays of the host that the step file names as host globals
 * (fortis.host boundary.pre / boundary.post; benchmarks/cam host, driver/fortis_emit2d.py:20-52).  The vectors
 * are filled at run time, before the first call and after every load-time constructor has run.
 *
 *   boundary_host <in.bin> <vectors.bin> <out.bin>     NI x NIN doubles in, NIN x 3 + NOUT doubles of vectors */
#include <stdio.h>
#include <stdlib.h>
#ifndef NI
#error "compile with -DNI= -DNIN= -DNOUT="
#endif
double cam_mean[NIN], cam_max[NIN], cam_min[NIN], cam_oscale[NOUT];
void mlp_forward(void* in, void* out);

int main(int argc, char** argv)
{
    if (argc < 4) return 2;
    double* in = malloc(sizeof(double) * NI * NIN);
    double* out = calloc(NI * NOUT, sizeof(double));
    FILE* f = fopen(argv[1], "rb");
    if (!f || fread(in, sizeof(double), NI * NIN, f) != NI * NIN) return 1;
    fclose(f);
    f = fopen(argv[2], "rb");
    if (!f || fread(cam_mean, sizeof(double), NIN, f) != NIN || fread(cam_max, sizeof(double), NIN, f) != NIN ||
        fread(cam_min, sizeof(double), NIN, f) != NIN || fread(cam_oscale, sizeof(double), NOUT, f) != NOUT) return 1;
    fclose(f);
    mlp_forward(in, out);
    mlp_forward(in, out);
    f = fopen(argv[3], "wb");
    if (!f || fwrite(out, sizeof(double), NI * NOUT, f) != NI * NOUT) return 1;
    fclose(f);
    printf("boundary host ok\n");
    return 0;
}

/* A caller of the MD entry written in plain C99 against include/staf.h only -- what a molecular-dynamics code that
 * links libstaf_hip.so does each step (the reference's caller is lammps/USER-STAF/pair_staf.cpp:181-240).
 *
 *   md_step <model_dir> <pos_file> <box_file> <type_counts_file> [precision 0|1] [steps]
 *
 * pos_file: 3N numbers (x y z per atom, species-sorted), box_file: Lx xy xz Ly yz Lz, type_counts_file: atoms per
 * species.  Prints the energy, the root mean square force component and the virial of every step as
 *   step <i> rc <code> E <e> rmsF <r> virial <xx> <yy> <zz> <xy> <xz> <yz>
 * and exits with the last return code of staf_compute (negated), or 100 on a usage / file error.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#include "staf.h"

static double* read_numbers(const char* path, int* n) {
  FILE* f = fopen(path, "r");
  int cap = 1024, cnt = 0;
  double* v;
  double x;
  if (!f) return NULL;
  v = (double*)malloc((size_t)cap * sizeof(double));
  while (v && fscanf(f, "%lf", &x) == 1) {
    if (cnt == cap) {
      double* w;
      cap *= 2;
      w = (double*)realloc(v, (size_t)cap * sizeof(double));
      if (!w) { free(v); v = NULL; break; }
      v = w;
    }
    v[cnt++] = x;
  }
  fclose(f);
  *n = cnt;
  return v;
}

int main(int argc, char** argv) {
  int npos = 0, nbox = 0, ncnt = 0, natoms = 0, steps = 1, i, k, s, rc = 0;
  double *pos, *box, *cnt, *force, e = 0.0, virial[6];
  int* type;
  StafOptions opt;
  StafModel* model;
  if (argc < 5) {
    fprintf(stderr, "usage: %s model_dir pos_file box_file type_counts_file [precision] [steps]\n", argv[0]);
    return 100;
  }
  pos = read_numbers(argv[2], &npos);
  box = read_numbers(argv[3], &nbox);
  cnt = read_numbers(argv[4], &ncnt);
  if (!pos || !box || !cnt || npos % 3 || nbox != 6 || ncnt < 1) {
    fprintf(stderr, "md_step: cannot read the configuration\n");
    return 100;
  }
  for (k = 0; k < ncnt; k++) natoms += (int)cnt[k];
  if (natoms * 3 != npos) {
    fprintf(stderr, "md_step: %d coordinates for %d atoms\n", npos, natoms);
    return 100;
  }
  type = (int*)malloc((size_t)natoms * sizeof(int));
  force = (double*)malloc((size_t)npos * sizeof(double));
  if (!type || !force) return 100;
  for (k = 0, i = 0; k < ncnt; k++)
    for (s = 0; s < (int)cnt[k]; s++) type[i++] = k;

  staf_options_default(&opt);
  opt.precision = argc > 5 ? atoi(argv[5]) : 0;
  if (argc > 6) steps = atoi(argv[6]);
  model = staf_load(argv[1], &opt);
  if (!model) {
    fprintf(stderr, "md_step: staf_load failed\n");
    return 100;
  }
  for (s = 0; s < steps; s++) {
    double ss = 0.0;
    rc = staf_compute(model, natoms, 0, pos, box, type, NULL, NULL, 0, &e, force, virial);
    for (i = 0; i < npos; i++) ss += force[i] * force[i];
    printf("step %d rc %d E %.17g rmsF %.17g virial %.17g %.17g %.17g %.17g %.17g %.17g\n", s, rc, e,
           sqrt(ss / npos), virial[0], virial[1], virial[2], virial[3], virial[4], virial[5]);
    if (rc) break;
    /* a rigid shift of all atoms leaves energy and forces unchanged: the next step runs on moved coordinates */
    for (i = 0; i < npos; i++) pos[i] += 0.25;
  }
  staf_free(model);
  free(pos); free(box); free(cnt); free(type); free(force);
  return rc ? -rc : 0;
}

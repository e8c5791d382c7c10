// TEST INFRASTRUCTURE ONLY.  Thin extern "C" driver around the reference's own legacy CPU
// neighbour list (STAF/src/descriptor_builder/cell_list.cu.cc: getList, fullUpdateList,
// calculateInteractionMapWithCutoffDistanceOrdered), compiled from the reference sources where
// they lie (see Makefile target _ref).  It is a second witness for the oracle's neighbour
// list; the reference records this list as identical to its GPU list (test/A3_PREP.md:90-94).
// Built for double (-DSTAF_REAL_DOUBLE) and float separately.
#include <stdio.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include "vector.h"
#include "interaction_map.h"
#include "cell_list.h"

extern "C" int ref_neighbor_list(int N, const real* frac /*[N,3]*/, const real* box6, real cutoff, int nr,
                                 int* with /*[N,nr]*/, real* dist2 /*[N,nr]*/, int* howmany /*[N]*/) {
  vector* pos = (vector*)malloc(sizeof(vector) * N);
  for (int i = 0; i < N; i++) { pos[i].x = frac[3 * i]; pos[i].y = frac[3 * i + 1]; pos[i].z = frac[3 * i + 2]; }
  interactionmap* ime = createInteractionMap(N, nr);
  resetInteractionMap(ime);
  listcell* l = getList(box6, cutoff, N);
  fullUpdateList(l, pos, N, box6, cutoff);
  calculateInteractionMapWithCutoffDistanceOrdered(l, ime, pos, box6, cutoff);
  int mx = 0;
  for (int i = 0; i < N; i++) {
    howmany[i] = ime->howmany[i];
    if (howmany[i] > mx) mx = howmany[i];
    for (int k = 0; k < nr; k++) {
      with[i * nr + k] = k < howmany[i] ? ime->with[i][k] : 0;
      dist2[i * nr + k] = k < howmany[i] ? ime->rij2[i][k] : 0;
    }
  }
  free(pos);
  return mx;
}

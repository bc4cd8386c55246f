/*
 * Integration shim for building the reference's toolkits (toolkits/main.cpp) in an image whose
 * reference tree has an empty third_party/METIS submodule.  TOOLKIT BUILD ONLY: it is on the include
 * path of oracle/build_toolkits.sh and of nothing else, pins nothing, and is never used for the
 * reference-built checkers under oracle/_ref/ that tests compare the oracle with.
 *
 * core/MetisPartition.hpp (included through core/ntsSampler.hpp:25) names the METIS types, a few option
 * indices and two partitioning calls; the only call site (core/ntsSampler.hpp, batch_type METIS) is not
 * reached by any configuration this repository runs.  The calls below report that METIS is absent and
 * return METIS_ERROR, which the reference treats as a failed partitioning.
 */
#ifndef NTS_TOOLKIT_SHIM_METIS_H
#define NTS_TOOLKIT_SHIM_METIS_H

#include <stdint.h>
#include <stdio.h>

typedef int64_t idx_t; /* IDXTYPEWIDTH=64, as the reference's CMakeLists.txt:107-113 sets it */
typedef float real_t;  /* REALTYPEWIDTH=32 */

#define METIS_API(type) type
#define METIS_NOPTIONS 40

typedef enum { METIS_OK = 1, METIS_ERROR_INPUT = -2, METIS_ERROR_MEMORY = -3, METIS_ERROR = -4 } rstatus_et;
typedef enum {
  METIS_OPTION_PTYPE,
  METIS_OPTION_OBJTYPE,
  METIS_OPTION_CTYPE,
  METIS_OPTION_IPTYPE,
  METIS_OPTION_RTYPE,
  METIS_OPTION_DBGLVL,
  METIS_OPTION_NIPARTS,
  METIS_OPTION_NITER,
  METIS_OPTION_NCUTS,
  METIS_OPTION_SEED,
  METIS_OPTION_ONDISK,
  METIS_OPTION_MINCONN,
  METIS_OPTION_CONTIG,
  METIS_OPTION_COMPRESS,
  METIS_OPTION_CCORDER,
  METIS_OPTION_PFACTOR,
  METIS_OPTION_NSEPS,
  METIS_OPTION_UFACTOR,
  METIS_OPTION_NUMBERING,
  METIS_OPTION_DROPEDGES,
  METIS_OPTION_NO2HOP,
  METIS_OPTION_TWOHOP,
  METIS_OPTION_FAST
} moptions_et;
typedef enum { METIS_OBJTYPE_CUT, METIS_OBJTYPE_VOL, METIS_OBJTYPE_NODE } mobjtype_et;

static inline int METIS_SetDefaultOptions(idx_t *options) {
  for (int i = 0; i < METIS_NOPTIONS; ++i) options[i] = -1;
  return METIS_OK;
}
static inline int nts_shim_metis_absent(const char *what) {
  fprintf(stderr, "%s: METIS is not part of this build (empty third_party/METIS submodule)\n", what);
  return METIS_ERROR;
}
static inline int METIS_PartGraphKway(idx_t *, idx_t *, idx_t *, idx_t *, idx_t *, idx_t *, idx_t *, idx_t *, real_t *,
                                      real_t *, idx_t *, idx_t *, idx_t *) {
  return nts_shim_metis_absent("METIS_PartGraphKway");
}
static inline int METIS_PartGraphRecursive(idx_t *, idx_t *, idx_t *, idx_t *, idx_t *, idx_t *, idx_t *, idx_t *,
                                           real_t *, real_t *, idx_t *, idx_t *, idx_t *) {
  return nts_shim_metis_absent("METIS_PartGraphRecursive");
}

#endif

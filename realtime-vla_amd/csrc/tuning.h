// The only place where a build of the library looks at its environment.  The shipped library is compiled without
// RTVLA_TUNING: both hooks are then empty inline functions and the library reads no environment variable.  A variant build
// (build.py -DRTVLA_TUNING -o other.so) lets a sweep force the block tile and split-K factor the cost model would pick:
//   RTVLA_FORCE_TILE=<GemmTile>  RTVLA_FORCE_SPLIT=<n>  RTVLA_FORCE_FOR=<substring of the launch name>  RTVLA_PRINT_TILES=1
// and set how many action-expert layers of the first flow step follow the prefix pass per graph-branch edge: RTVLA_FORK_GROUP=<n>
#pragma once
#ifdef RTVLA_TUNING
#include <cstdio>
#include <cstdlib>
#include <cstring>
inline bool tuning_forced_tile(const char* what, bool splittable, int* tile, int* nsplit) {
    const char* only_for = getenv("RTVLA_FORCE_FOR");
    const char* e = (only_for && !strstr(what, only_for)) ? nullptr : getenv("RTVLA_FORCE_TILE");
    if (!e) return false;
    *tile = atoi(e); *nsplit = 1;
    if (const char* s = getenv("RTVLA_FORCE_SPLIT")) if (splittable) *nsplit = atoi(s);
    return true;
}
inline void tuning_report_tile(const char* what, int M, int N, int stages, int bm, int bn, int nsplit, double model_us) {
    if (getenv("RTVLA_PRINT_TILES"))
        fprintf(stderr, "rtvla tile choice: %-18s M=%d N=%d stages=%d -> %dx%d split %d (model %.1f us)\n", what, M, N, stages, bm, bn, nsplit, model_us);
}
inline int tuning_fork_group(int dflt) { const char* e = getenv("RTVLA_FORK_GROUP"); return e && atoi(e) > 0 ? atoi(e) : dflt; }
#else
inline int tuning_fork_group(int dflt) { return dflt; }
inline bool tuning_forced_tile(const char*, bool, int*, int*) { return false; }
inline void tuning_report_tile(const char*, int, int, int, int, int, int, double) {}
#endif

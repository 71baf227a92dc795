// The variants of one kind; compiled once per kind with -DSWEEP_KIND=0..6 so that the kinds build side by side.
#include "sweep.h"

#ifndef SWEEP_KIND
#error "compile with -DSWEEP_KIND=0..6"
#endif

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)

template <int LAUX, int SAUX, int U>
static void add_threads(std::vector<Variant> &v) {
    v.push_back({SWEEP_KIND, LAUX, SAUX, U, 256, &go<SWEEP_KIND, LAUX, SAUX, U, 256>});
    v.push_back({SWEEP_KIND, LAUX, SAUX, U, 512, &go<SWEEP_KIND, LAUX, SAUX, U, 512>});
    v.push_back({SWEEP_KIND, LAUX, SAUX, U, 1024, &go<SWEEP_KIND, LAUX, SAUX, U, 1024>});
}
template <int LAUX, int SAUX>
static void add_tiles(std::vector<Variant> &v) {
    if (SWEEP_KIND != R4W1W && SWEEP_KIND != R1W4W) add_threads<LAUX, SAUX, 2>(v);  // the wide byte side needs four vectors
    add_threads<LAUX, SAUX, 4>(v);
    add_threads<LAUX, SAUX, 8>(v);
    add_threads<LAUX, SAUX, 12>(v);
    add_threads<LAUX, SAUX, 16>(v);
}
template <int LAUX>
static void add_store_policies(std::vector<Variant> &v) {
    add_tiles<LAUX, 0>(v);
    if (SWEEP_KIND == R4) return;  // nothing is stored
    add_tiles<LAUX, 1>(v);
    add_tiles<LAUX, 2>(v);
    add_tiles<LAUX, 16>(v);
    add_tiles<LAUX, 17>(v);
    add_tiles<LAUX, 19>(v);
}

void CAT(register_kind_, SWEEP_KIND)(std::vector<Variant> &v) {
    add_store_policies<0>(v);
    if (SWEEP_KIND != W4) add_store_policies<2>(v);  // W4 loads nothing
}

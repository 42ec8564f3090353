// Tuning switches of the kernels and of the launch policy (FLEX_TUNE_* macros given with -D).
//
// A library built with any of them is a measurement variant, not a product library: the generator has to
// be told (it writes them into flexspmv_signature() under "tuning", where loaders look), and this header
// checks that what the compiler sees is what the generator was told.  Three switches change results or
// drop a safety check and need FLEX_TUNE_ALLOW_WRONG_RESULTS beside them.
#pragma once

#if defined(FLEX_TUNE_ABLATE_STORES) || defined(FLEX_TUNE_UNSAFE_BIG_TILE) || defined(FLEX_TUNE_FORCE_MERGE)
#ifndef FLEX_TUNE_ALLOW_WRONG_RESULTS
#error "FLEX_TUNE_ABLATE_STORES / FLEX_TUNE_UNSAFE_BIG_TILE / FLEX_TUNE_FORCE_MERGE give wrong results or drop a safety check: define FLEX_TUNE_ALLOW_WRONG_RESULTS as well to build such an ablation"
#endif
#endif

#if defined(FLEX_TUNE_ABLATE_STORES) || defined(FLEX_TUNE_ALLOW_WRONG_RESULTS) || defined(FLEX_TUNE_BISECTION_ONLY) ||   \
    defined(FLEX_TUNE_FORCE_MERGE) || defined(FLEX_TUNE_INBLOCK_MAX_TILES) || defined(FLEX_TUNE_LDS_DIRECT_ALL) ||        \
    defined(FLEX_TUNE_NOMINAL) || defined(FLEX_TUNE_NO_LDS_DIRECT) || defined(FLEX_TUNE_NO_ROW_CAP) ||                    \
    defined(FLEX_TUNE_NO_ROW_GROUP) || defined(FLEX_TUNE_NT_LOADS) || defined(FLEX_TUNE_PERSISTENT) ||                    \
    defined(FLEX_TUNE_PLAIN_STORES) || defined(FLEX_TUNE_ROW_BRANCH) || defined(FLEX_TUNE_ROW_PATH_ANY_SHAPE) ||          \
    defined(FLEX_TUNE_ROW_PATH_MAX_LEN) || defined(FLEX_TUNE_SEARCH_BLOCK) || defined(FLEX_TUNE_SEARCH_GROUP) ||          \
    defined(FLEX_TUNE_SEPARATE_OUT_BYTES) || defined(FLEX_TUNE_SINGLE_FIXUP_MAX_TILES) || defined(FLEX_TUNE_SNAP_BYTES) || \
    defined(FLEX_TUNE_STAGE_WORDS) || defined(FLEX_TUNE_THREAD_SEARCH) || defined(FLEX_TUNE_UNSAFE_BIG_TILE) ||           \
    defined(FLEX_TUNE_XCD_RUN_SHIFT) || defined(FLEX_TUNE_PARTIAL_PER_WAVE) || defined(FLEX_TUNE_TICKET_SUM) ||       \
    defined(FLEX_TUNE_GATHER_POLICY) || defined(FLEX_TUNE_NO_ROUND_BALANCE)
#define FLEX_TUNING_ACTIVE 1
#else
#define FLEX_TUNING_ACTIVE 0
#endif

// The generated translation unit defines FLEX_TUNING_DECLARED (0 or 1: whether the generator was given
// switches) before it includes the kernels.
#ifdef FLEX_TUNING_DECLARED
static_assert(FLEX_TUNING_DECLARED == FLEX_TUNING_ACTIVE,
              "FLEX_TUNE_* switches on the compiler's command line must be the ones the generator was given "
              "(flexspmv_amd.build.compile_graph(..., extra_flags=[...]) passes them to both)");
#endif

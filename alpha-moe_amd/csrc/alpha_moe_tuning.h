/*
 * Internal hook of libalpha_moe_hip.so for experiments and tests; not part of the operator's C ABI
 * (include/alpha_moe_hip.h) and free to change between versions.
 *
 * alpha_moe_set_tunable installs (set != 0) or clears (set == 0) a tuning override.  `name` is one of
 * ALPHA_MOE_PATH (1 direct, 2 stream, 3 tile, 4 wide), ALPHA_MOE_STRICT_QUEUE, ALPHA_MOE_KBPI, ALPHA_MOE_TPI,
 * ALPHA_MOE_LAG, ALPHA_MOE_GRID, ALPHA_MOE_TILE_GPS, ALPHA_MOE_TILE_LAG, ALPHA_MOE_TILE_GRID, ALPHA_MOE_TILE_NT,
 * ALPHA_MOE_WIDE_PP (wide kernel: 1 = up/gate loop with the wavefronts of a SIMD half a step apart, 0 = in step;
 * unset = by routed rows per expert; same bits either way).
 * The environment variables of the same names are read once, when the library is first used; no launch reads the
 * environment.  Not thread-safe against concurrent launches.  Results stay within the parity bar whatever is set.
 * Returns ALPHA_MOE_ERR_SHAPE for an unknown name.
 */
#ifndef ALPHA_MOE_TUNING_H
#define ALPHA_MOE_TUNING_H
#ifdef __cplusplus
extern "C" {
#endif
int alpha_moe_set_tunable(const char *name, int value, int set);
#ifdef __cplusplus
}
#endif
#endif

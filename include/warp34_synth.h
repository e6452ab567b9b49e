/* Deterministic synthetic inputs for the benchmarks and tests of the paged KV path.
 *
 * Not part of the reference's ABI (it has no counterpart there): the benchmark configurations
 * prescribe inputs that two machines can generate bit for bit without a random-number library:
 * a SplitMix64 stream -> Box-Muller in double precision -> round-to-nearest-even to bf16, 3 of
 * 256 channels per kv head scaled x20 ("1 % outlier channels"), and seeded Fisher-Yates
 * permutations for page orders.  Element i of a stream depends on (seed, i) only, so the
 * generators fill large tensors with several host threads and can start at any row.
 */
#ifndef WARP34_SYNTH_H
#define WARP34_SYNTH_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* dst[0 .. n) = elements first .. first + n of the N(0,1) stream of `seed`, as bf16 bits.
 * `first` must be even (values come in Box-Muller pairs). */
void warp34_synth_normal_bf16(uint16_t* dst, size_t first, size_t n, uint64_t seed);

/* K or V rows [rows][kv_heads][head_dim] as bf16 bits, rows first_row .. first_row + rows of the
 * tensor of `seed`: N(0,1), with n_outliers channels per kv head (the first entries of a seeded
 * permutation of the channels) multiplied by 20 before rounding. */
void warp34_synth_kv_rows_bf16(uint16_t* dst, size_t first_row, size_t rows, int kv_heads, int head_dim,
                               uint64_t seed, int n_outliers);

/* dst = seeded Fisher-Yates permutation of 0 .. n-1 */
void warp34_synth_permutation(int32_t* dst, int n, uint64_t seed);

/* dst[i] = lo + (draw i of the stream of `seed`) mod (hi - lo + 1), for lo <= hi */
void warp34_synth_uniform_i32(int32_t* dst, int n, int32_t lo, int32_t hi, uint64_t seed);

#ifdef __cplusplus
}
#endif
#endif /* WARP34_SYNTH_H */

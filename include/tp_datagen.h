/*
 * tp_datagen.h -- seeded synthetic payloads for the benchmark configurations
 * (uniform bytes, N(0, sigma) in fp32 / bf16 / fp16, log-uniform tensor sizes).
 * Counter-based (splitmix64 finaliser over seed + index), so any slice can be
 * generated independently and identically on every machine. The reference has
 * no generator of its own beyond the benchmark fill pattern
 * (tensorpipe/benchmark/benchmark_pipe.cc:144-151), restated here as
 * tpdg_bench_pattern.
 */
#ifndef TP_DATAGEN_H_
#define TP_DATAGEN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* i-th 64-bit word of stream `seed`. */
uint64_t tpdg_u64(uint64_t seed, uint64_t i);

/* n uniform random bytes: byte j is byte (j % 8), little-endian, of word j / 8. */
void tpdg_fill_u8(uint64_t seed, uint8_t* out, uint64_t n);

/* Box-Muller in double precision: pair p uses words 2p and 2p+1 and yields
 * elements 2p (cosine branch) and 2p+1 (sine branch), scaled by sigma, then
 * rounded to the storage type (round to nearest even). */
void tpdg_fill_normal_f32(uint64_t seed, double sigma, float* out, uint64_t n);
void tpdg_fill_normal_bf16(uint64_t seed, double sigma, uint16_t* out, uint64_t n);
void tpdg_fill_normal_f16(uint64_t seed, double sigma, uint16_t* out, uint64_t n);

/* n sizes, log-uniform in [lo, hi], rounded to an even number of bytes. */
void tpdg_loguniform_sizes(uint64_t seed, uint64_t lo, uint64_t hi, uint64_t* out, uint32_t n);

void tpdg_bench_pattern(uint8_t* out, uint64_t n);

/* FNV-1a 64 over a byte range (cheap digest for fixtures and live checks). */
uint64_t tpdg_fnv1a64(const uint8_t* data, uint64_t n);

#ifdef __cplusplus
}
#endif
#endif /* TP_DATAGEN_H_ */

/* ojas_data.h -- C ABI of the data step in front of the training path: the token bin reader and
 * the seeded epoch sampler that turn a token file into (x, y) batches.
 *
 * Replaces, for callers of the training step, `ojas_data::TokenBin`
 * (ojas-data/src/tokens.rs:38-330) and `ojas_data::BatchSampler`
 * (ojas-data/src/sampler.rs:117-319). Same streams bit for bit: the window order is the 4-round
 * Feistel permutation keyed by SplitMix64 that `permutation_is_pinned`
 * (ojas-data/tests/sampler.rs:231-254) holds fixed.
 *
 * Host code only (no device work): a sampler produces either whole batches on the host
 * (`odata_sampler_next_batch`) or just the window starts (`odata_sampler_next_starts`), which
 * `omx_token_windows` (ojas_mi355x.h) turns into a batch on the device from a bin that is resident
 * in HBM.
 *
 * Every function returns 0 on success and ODATA_ERROR otherwise (the reference's single
 * `DataError`, ojas-data/src/error.rs); `odata_last_error` returns the message of the calling
 * thread's last failure.
 */
#ifndef OJAS_DATA_H
#define OJAS_DATA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ODATA_OK 0
#define ODATA_ERROR 1

/* BinLayout (tokens.rs:49-60). */
#define ODATA_HEADERLESS 0
#define ODATA_FINEWEB 1
/* TokenWidth (tokens.rs:22-35); ODATA_WIDTH_ANY is `BinLayout::FineWeb(None)`. */
#define ODATA_WIDTH_ANY 0
#define ODATA_WIDTH_U16 2
#define ODATA_WIDTH_U32 4

typedef struct odata_bin odata_bin;
typedef struct odata_sampler odata_sampler;

/* Copies the calling thread's last error message (NUL-terminated, truncated to cap) and
 * returns its full length. */
size_t odata_last_error(char* buf, size_t cap);

/* TokenBin::open (tokens.rs:104-207). Headerless: `width` must be U16 or U32 and the file length a
 * multiple of it. FineWeb: 256 little-endian i32 header words (magic 20240520 + version 1 = u16
 * tokens, magic 20240801 + version 7 or 1 = u32 tokens, word 2 = token count, file length must
 * match exactly); `width` ANY takes what the magic names, otherwise it must agree. */
int32_t odata_bin_open(const char* path, int32_t layout, int32_t width, odata_bin** out);
void odata_bin_close(odata_bin* bin);
/* TokenBin::len / bytes_per_token (tokens.rs:209-223). */
uint64_t odata_bin_len(const odata_bin* bin);
int32_t odata_bin_bytes_per_token(const odata_bin* bin);
/* TokenBin::read_into_u32 (tokens.rs:245-308): tokens [index, index + n) widened to u32; a window
 * past the end is an error, n = 0 reads nothing. */
int32_t odata_bin_read_u32(const odata_bin* bin, uint64_t index, uint32_t* dst, uint64_t n);
/* TokenBin::read_into (tokens.rs:231-243): the same into u16; a u32 token above 65535 is an error
 * naming the token and its index. */
int32_t odata_bin_read_u16(const odata_bin* bin, uint64_t index, uint16_t* dst, uint64_t n);
/* The raw little-endian token bytes [index, index + n), for uploading a bin to the device. */
int32_t odata_bin_read_raw(const odata_bin* bin, uint64_t index, void* dst, uint64_t n);

/* BatchSampler::resume (sampler.rs:159-214); (epoch, ordinal) = DataCursor{shard, token_index},
 * (0, 0) for BatchSampler::new. The bin must outlive the sampler. */
int32_t odata_sampler_new(const odata_bin* bin, uint64_t seq_len, uint64_t batch, uint64_t seed, uint64_t epoch,
                          uint64_t ordinal, odata_sampler** out);
void odata_sampler_free(odata_sampler* s);
/* The same sampler over a bin of `n_tokens` tokens that is not held by this library (resident on
 * the device): only `odata_sampler_next_starts` and `odata_sampler_window_start` work on it. */
int32_t odata_sampler_new_detached(uint64_t n_tokens, uint64_t seq_len, uint64_t batch, uint64_t seed, uint64_t epoch,
                                   uint64_t ordinal, odata_sampler** out);
/* BatchSampler::windows_per_epoch / cursor (sampler.rs:216-227). */
uint64_t odata_sampler_windows_per_epoch(const odata_sampler* s);
void odata_sampler_cursor(const odata_sampler* s, uint64_t* epoch, uint64_t* ordinal);
/* BatchSampler::window_start (sampler.rs:229-239): first token of window `ordinal` of `epoch`. */
int32_t odata_sampler_window_start(const odata_sampler* s, uint64_t epoch, uint64_t ordinal, uint64_t* start);
/* BatchSampler::next_batch (sampler.rs:241-283): the next `batch` windows, x = tokens
 * [start, start + T), y = [start + 1, start + T + 1), both [batch, seq_len] u32; the cursor moves
 * only on success. */
int32_t odata_sampler_next_batch(odata_sampler* s, uint32_t* x, uint32_t* y);
/* The window starts of the next batch (`batch` values) and the same cursor movement, without
 * reading tokens. */
int32_t odata_sampler_next_starts(odata_sampler* s, uint64_t* starts);

/* SamplerRngState::encode / decode (sampler.rs:70-110): 16 bytes, u32 LE version 1, u32 LE
 * generator 1 (4-round Feistel over SplitMix64), u64 LE seed; any other length, version or
 * generator is refused. */
void odata_rng_state_encode(uint64_t seed, uint8_t out[16]);
int32_t odata_rng_state_decode(const uint8_t* bytes, uint64_t n, uint64_t* seed);

#ifdef __cplusplus
}
#endif
#endif

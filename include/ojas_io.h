/* ojas_io.h -- C ABI of the wire formats on either side of the training path: safetensors files
 * (weights in, weights and optimizer state out) and the checkpoint-v1 state file.
 *
 * Replaces, for callers of the training step, `ojas_io::SafeTensors` / `write_safetensors`
 * (ojas-io/src/safetensors.rs:340-700, 1224-1260; header rules :1616-1800) and
 * `ojas_io::{write,read}_checkpoint` (ojas-io/src/checkpoint.rs:18-330; layout
 * docs/checkpoint-v1.md, types ojas-core/src/checkpoint.rs:11-115). Files written here are read by
 * the reference and the other way round. Host code only.
 *
 * Every function returns 0 on success and OIO_ERROR otherwise (the reference's `IoError`);
 * `oio_last_error` returns the message of the calling thread's last failure.
 */
#ifndef OJAS_IO_H
#define OJAS_IO_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OIO_OK 0
#define OIO_ERROR 1
/* MAX_HEADER_BYTES (safetensors.rs:26) and MAX_CHECKPOINT_BYTES (checkpoint.rs:42). */
#define OIO_MAX_HEADER_BYTES 100000000ull
#define OIO_MAX_CHECKPOINT_BYTES (1ull << 30)

size_t oio_last_error(char* buf, size_t cap);

/* ---- safetensors ---- */
typedef struct oio_safetensors oio_safetensors;

/* SafeTensors::open (safetensors.rs:408-500): 8-byte little-endian header length (1..=100 MB, inside
 * the file), a UTF-8 JSON object of at most three levels whose keys are tensor names (not empty,
 * not repeated) mapping to exactly {dtype, shape, data_offsets} with non-negative integer entries,
 * plus an optional "__metadata__" object of strings. The tensors must tile the data buffer: each
 * range has the byte length its shape and dtype give, and the sorted ranges leave no gap, overlap
 * or tail (check_tiling, :1762-1800). The payload is read on demand, not at open. */
int32_t oio_st_open(const char* path, oio_safetensors** out);
void oio_st_close(oio_safetensors* s);
/* Tensor names in ascending byte order (the reference's BTreeMap order). */
uint64_t oio_st_count(const oio_safetensors* s);
const char* oio_st_name(const oio_safetensors* s, uint64_t index);
/* TensorInfo (safetensors.rs:195-220): dtype tag ("F32", "BF16", "F16", "I64", "U16", "U8", "I8",
 * "BOOL", "I16", "I32", "U32", "F64", "U64", "F8_E4M3", ...), rank, up to shape_cap extents, and the
 * byte length. */
int32_t oio_st_info(const oio_safetensors* s, const char* name, const char** dtype, uint32_t* rank, uint64_t* shape,
                    uint32_t shape_cap, uint64_t* nbytes);
/* SafeTensors::read_into (safetensors.rs:528-598): n bytes of the tensor from byte `offset`. */
int32_t oio_st_read(const oio_safetensors* s, const char* name, uint64_t offset, void* dst, uint64_t n);
/* read_f32 / read_f32_widened (safetensors.rs:620-647): F32 as is, BF16 and F16 widened exactly;
 * any other dtype is an error. numel must be the tensor's element count. */
int32_t oio_st_read_f32(const oio_safetensors* s, const char* name, float* dst, uint64_t numel);
uint64_t oio_st_metadata_count(const oio_safetensors* s);
const char* oio_st_metadata_key(const oio_safetensors* s, uint64_t index);
/* Null when the key is absent. */
const char* oio_st_metadata(const oio_safetensors* s, const char* key);

typedef struct {
  const char* name;
  const char* dtype; /* a tag oio_st_info returns */
  uint32_t rank;
  const uint64_t* shape;
  const void* data;
  uint64_t nbytes; /* must equal the shape's element count times the dtype's size */
} oio_tensor_out;
/* write_safetensors (safetensors.rs:1224-1260): tensors in the order given (names not empty, not
 * repeated), header padded with spaces to a multiple of 8 bytes, written to a temporary file in
 * the same directory and renamed over `path`. */
int32_t oio_st_write(const char* path, const oio_tensor_out* tensors, uint64_t count, const char* const* meta_keys,
                     const char* const* meta_values, uint64_t meta_count);

/* ---- checkpoint v1 (docs/checkpoint-v1.md) ---- */
/* NamedBlob (ojas-core/src/checkpoint.rs:69-80): dtype_tag 0 = F32, 1 = Bf16, 2 = F16, 3 = U32;
 * element 0 of the tensor is at `byte_offset` inside the payload, and
 * byte_offset + numel * size <= payload_len. */
typedef struct {
  const char* name;
  uint32_t dtype_tag;
  uint32_t rank;
  const uint64_t* shape;
  uint64_t byte_offset;
  const void* payload;
  uint64_t payload_len;
} oio_blob;
/* CheckpointV1 (ojas-core/src/checkpoint.rs:104-115). sections: weights, optimizer.muon_momentum,
 * optimizer.adamw_first_moment, optimizer.adamw_second_moment, in file order. */
typedef struct {
  const void* config;
  uint64_t config_len;
  uint8_t tokenizer_hash[32];
  uint8_t git_sha[20];
  uint64_t step;
  uint64_t cursor_shard, cursor_token_index;
  const void* rng_state;
  uint64_t rng_state_len;
  const oio_blob* sections[4];
  uint64_t counts[4];
} oio_checkpoint;
typedef struct oio_ckpt oio_ckpt;

/* checkpoint_file_len / write_checkpoint (checkpoint.rs:18-40): "OJAS0001", u32 1, then the body in
 * the order of the struct; every section is u64 byte length, u64 record count, records. Names must
 * not repeat inside a section; files above 1 GiB are refused. Written through a temporary file and
 * a rename. */
int32_t oio_ckpt_file_len(const oio_checkpoint* c, uint64_t* len);
int32_t oio_ckpt_write(const char* path, const oio_checkpoint* c);
/* read_checkpoint (checkpoint.rs:55-84, 187-330): refuses a wrong magic or version, a truncated or
 * oversized file, record counts and ranks their section cannot hold, a byte window past its
 * payload, and trailing bytes. `view` is filled with pointers into the handle, valid until
 * oio_ckpt_free. */
int32_t oio_ckpt_read(const char* path, oio_ckpt** out, oio_checkpoint* view);
void oio_ckpt_free(oio_ckpt* c);

#ifdef __cplusplus
}
#endif
#endif

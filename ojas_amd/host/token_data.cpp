// Token bin reader and seeded epoch sampler behind include/ojas_data.h.
//
// Follows ojas-data/src/tokens.rs (TokenBin) and ojas-data/src/sampler.rs (BatchSampler): windows
// of seq_len + 1 tokens at multiples of seq_len, visited once per epoch in the order of a 4-round
// Feistel permutation over the smallest even number of bits covering the window count,
// cycle-walked into range; round function and round keys are SplitMix64 (ojas-kernels/src/rng.rs).
#include "ojas_data.h"

#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cinttypes>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <string>
#include <vector>

namespace {

thread_local std::string g_error;

int32_t fail(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_error = buf;
  return ODATA_ERROR;
}

// SplitMix64 (ojas-kernels/src/rng.rs): the state is the seed; each draw adds the golden gamma.
struct SplitMix64 {
  uint64_t state;
  explicit SplitMix64(uint64_t seed) : state(seed) {}
  uint64_t next() {
    state += 0x9E3779B97F4A7C15ull;
    uint64_t z = state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
  }
};

constexpr int kRounds = 4;                             // sampler.rs:36
constexpr uint64_t kEpochStep = 0xD1B54A32D192ED03ull;  // sampler.rs:41
constexpr uint64_t kFinewebHeaderBytes = 256 * 4;      // tokens.rs:18
constexpr int32_t kFinewebMagic = 20240520, kFinewebVersion = 1;
constexpr int32_t kFinewebU32Magic = 20240801, kFinewebU32Version = 7;

bool read_exact_at(int fd, void* dst, uint64_t n, uint64_t offset) {
  char* p = static_cast<char*>(dst);
  while (n > 0) {
    const ssize_t got = pread(fd, p, n, static_cast<off_t>(offset));
    if (got < 0) {
      if (errno == EINTR) continue;
      return false;
    }
    if (got == 0) {
      errno = 0;  // short file
      return false;
    }
    p += got;
    offset += static_cast<uint64_t>(got);
    n -= static_cast<uint64_t>(got);
  }
  return true;
}

int32_t le_i32(const unsigned char* h, int word) {
  const unsigned char* p = h + 4 * word;
  return static_cast<int32_t>(static_cast<uint32_t>(p[0]) | static_cast<uint32_t>(p[1]) << 8 |
                              static_cast<uint32_t>(p[2]) << 16 | static_cast<uint32_t>(p[3]) << 24);
}

}  // namespace

struct odata_bin {
  int fd = -1;
  uint64_t data_offset = 0;
  uint64_t len_tokens = 0;
  int32_t width = ODATA_WIDTH_U16;  // bytes per token
};

struct odata_sampler {
  const odata_bin* bin = nullptr;  // null for a detached sampler
  uint64_t seq_len = 0, batch = 0, seed = 0;
  uint64_t windows = 0;
  uint32_t half_bits = 1;
  uint64_t epoch = 0, ordinal = 0;
  std::vector<uint32_t> row;

  void round_keys(uint64_t e, uint64_t keys[kRounds]) const {
    // CounterRng::new(seed) then set_state(seed ^ epoch * EPOCH_STEP) (sampler.rs:298-306).
    SplitMix64 rng(seed ^ (e * kEpochStep));
    for (int i = 0; i < kRounds; ++i) keys[i] = rng.next();
  }
  uint64_t feistel(uint64_t v, const uint64_t keys[kRounds]) const {
    const uint32_t h = half_bits;
    const uint64_t mask = (1ull << h) - 1;
    uint64_t left = (v >> h) & mask, right = v & mask;
    for (int i = 0; i < kRounds; ++i) {
      const uint64_t f = SplitMix64(right ^ keys[i]).next() & mask;
      const uint64_t next = left ^ f;
      left = right;
      right = next;
    }
    return (left << h) | right;
  }
  uint64_t permute(uint64_t e, uint64_t ord) const {
    uint64_t keys[kRounds];
    round_keys(e, keys);
    uint64_t v = ord;
    // Cycle walk: the network permutes 0..2^(2h) and ord lies on its own cycle, so this ends.
    do v = feistel(v, keys);
    while (v >= windows);
    return v;
  }
};

namespace {

int32_t open_fineweb(odata_bin& bin, uint64_t len) {
  if (len < kFinewebHeaderBytes) return fail("truncated FineWeb header, %" PRIu64 " bytes", len);
  unsigned char header[kFinewebHeaderBytes];
  if (!read_exact_at(bin.fd, header, kFinewebHeaderBytes, 0)) return fail("header: %s", strerror(errno));
  const int32_t magic = le_i32(header, 0), version = le_i32(header, 1), count = le_i32(header, 2);
  uint64_t bpt;
  if (magic == kFinewebMagic) {
    if (version != kFinewebVersion) return fail("version %d != %d", version, kFinewebVersion);
    bpt = 2;
  } else if (magic == kFinewebU32Magic) {
    if (version != kFinewebU32Version && version != 1) return fail("version %d != %d", version, kFinewebU32Version);
    bpt = 4;
  } else {
    return fail("magic %d != %d", magic, kFinewebMagic);
  }
  if (count < 0) return fail("token count %d is negative", count);
  const uint64_t expect = kFinewebHeaderBytes + static_cast<uint64_t>(count) * bpt;  // count < 2^31: no overflow
  if (len != expect) return fail("size mismatch, expected %" PRIu64 " bytes, got %" PRIu64, expect, len);
  bin.data_offset = kFinewebHeaderBytes;
  bin.len_tokens = static_cast<uint64_t>(count);
  bin.width = static_cast<int32_t>(bpt);
  return ODATA_OK;
}

// TokenBin::read_window's range checks (tokens.rs:266-287); returns the byte offset.
int32_t window_bytes(const odata_bin* bin, uint64_t index, uint64_t n, uint64_t* byte_off, uint64_t* nbytes) {
  if (!bin) return fail("token bin is null");
  const uint64_t end = index + n;
  if (end < index) return fail("token index overflows");
  if (end > bin->len_tokens)
    return fail("token window [%" PRIu64 ", %" PRIu64 ") past length %" PRIu64, index, end, bin->len_tokens);
  const uint64_t bpt = static_cast<uint64_t>(bin->width);
  *byte_off = index * bpt + bin->data_offset;  // end <= len_tokens, whose bytes fit the file length
  *nbytes = n * bpt;
  return ODATA_OK;
}

int32_t sampler_init(odata_sampler& s, uint64_t n_tokens, uint64_t seq_len, uint64_t batch, uint64_t seed,
                     uint64_t epoch, uint64_t ordinal) {
  if (seq_len == 0 || batch == 0)
    return fail("sampler: seq_len %" PRIu64 " and batch %" PRIu64 " must be non-zero", seq_len, batch);
  if (seq_len == UINT64_MAX) return fail("sampler: seq_len + 1 overflows");
  const uint64_t need = seq_len + 1;
  if (n_tokens < need)
    return fail("sampler: a window needs %" PRIu64 " tokens, the bin has %" PRIu64, need, n_tokens);
  unsigned __int128 cells = static_cast<unsigned __int128>(batch) * seq_len + seq_len;
  if (cells > static_cast<unsigned __int128>(SIZE_MAX) / 8) return fail("sampler: batch * seq_len overflows");
  const uint64_t windows = (n_tokens - 1) / seq_len;
  if (ordinal >= windows)
    return fail("sampler: cursor window %" PRIu64 " is past the %" PRIu64 " windows of an epoch", ordinal, windows);
  // bits = u64::BITS - (windows - 1).leading_zeros(); half = max(ceil(bits / 2), 1)
  uint32_t bits = 0;
  for (uint64_t v = windows - 1; v; v >>= 1) ++bits;
  uint32_t half = (bits + 1) / 2;
  if (half < 1) half = 1;
  s.seq_len = seq_len;
  s.batch = batch;
  s.seed = seed;
  s.windows = windows;
  s.half_bits = half;
  s.epoch = epoch;
  s.ordinal = ordinal;
  return ODATA_OK;
}

// The next batch's starts and the cursor after them; the sampler itself is not changed.
int32_t plan_batch(const odata_sampler* s, uint64_t* starts, uint64_t* epoch_after, uint64_t* ordinal_after) {
  uint64_t epoch = s->epoch, ordinal = s->ordinal;
  for (uint64_t i = 0; i < s->batch; ++i) {
    starts[i] = s->permute(epoch, ordinal) * s->seq_len;
    if (++ordinal == s->windows) {
      ordinal = 0;
      if (epoch == UINT64_MAX) return fail("sampler: epoch counter overflows");
      ++epoch;
    }
  }
  *epoch_after = epoch;
  *ordinal_after = ordinal;
  return ODATA_OK;
}

}  // namespace

extern "C" {

size_t odata_last_error(char* buf, size_t cap) {
  if (buf && cap) {
    const size_t n = g_error.size() < cap - 1 ? g_error.size() : cap - 1;
    memcpy(buf, g_error.data(), n);
    buf[n] = 0;
  }
  return g_error.size();
}

int32_t odata_bin_open(const char* path, int32_t layout, int32_t width, odata_bin** out) {
  if (!path || !out) return fail("token bin: null argument");
  *out = nullptr;
  if (layout != ODATA_HEADERLESS && layout != ODATA_FINEWEB) return fail("%s: unknown layout %d", path, layout);
  if (width != ODATA_WIDTH_ANY && width != ODATA_WIDTH_U16 && width != ODATA_WIDTH_U32)
    return fail("%s: unknown token width %d", path, width);
  if (layout == ODATA_HEADERLESS && width == ODATA_WIDTH_ANY) return fail("%s: a headerless bin needs a token width", path);
  struct stat st;
  if (stat(path, &st) != 0) return fail("%s: %s", path, strerror(errno));
  if (!S_ISREG(st.st_mode)) return fail("%s: not a regular file", path);
  odata_bin* bin = new (std::nothrow) odata_bin;
  if (!bin) return fail("%s: allocation refused", path);
  bin->fd = open(path, O_RDONLY | O_CLOEXEC);
  if (bin->fd < 0) {
    const int e = errno;
    delete bin;
    return fail("%s: %s", path, strerror(e));
  }
  const uint64_t len = static_cast<uint64_t>(st.st_size);
  int32_t rc = ODATA_OK;
  if (layout == ODATA_HEADERLESS) {
    const uint64_t bpt = static_cast<uint64_t>(width);
    if (len % bpt != 0) {
      rc = fail("truncated token bin, %" PRIu64 " bytes is not a multiple of %" PRIu64, len, bpt);
    } else {
      bin->data_offset = 0;
      bin->len_tokens = len / bpt;
      bin->width = width;
    }
  } else {
    rc = open_fineweb(*bin, len);
    if (rc == ODATA_OK && width != ODATA_WIDTH_ANY && width != bin->width)
      rc = fail("expected %s FineWeb bin, found %s", width == ODATA_WIDTH_U16 ? "u16" : "u32",
                bin->width == ODATA_WIDTH_U16 ? "U16" : "U32");
  }
  if (rc != ODATA_OK) {
    const std::string inner = g_error;
    close(bin->fd);
    delete bin;
    return fail("%s: %s", path, inner.c_str());
  }
  *out = bin;
  return ODATA_OK;
}

void odata_bin_close(odata_bin* bin) {
  if (!bin) return;
  if (bin->fd >= 0) close(bin->fd);
  delete bin;
}

uint64_t odata_bin_len(const odata_bin* bin) { return bin ? bin->len_tokens : 0; }
int32_t odata_bin_bytes_per_token(const odata_bin* bin) { return bin ? bin->width : 0; }

int32_t odata_bin_read_raw(const odata_bin* bin, uint64_t index, void* dst, uint64_t n) {
  uint64_t off = 0, nbytes = 0;
  if (window_bytes(bin, index, n, &off, &nbytes) != ODATA_OK) return ODATA_ERROR;
  if (n == 0) return ODATA_OK;
  if (!dst) return fail("token read: null destination");
  if (!read_exact_at(bin->fd, dst, nbytes, off)) return fail("token read: %s", errno ? strerror(errno) : "short file");
  return ODATA_OK;
}

int32_t odata_bin_read_u32(const odata_bin* bin, uint64_t index, uint32_t* dst, uint64_t n) {
  uint64_t off = 0, nbytes = 0;
  if (window_bytes(bin, index, n, &off, &nbytes) != ODATA_OK) return ODATA_ERROR;
  if (n == 0) return ODATA_OK;
  if (!dst) return fail("token read: null destination");
  if (bin->width == ODATA_WIDTH_U32) {
    if (!read_exact_at(bin->fd, dst, nbytes, off)) return fail("token read: %s", errno ? strerror(errno) : "short file");
    return ODATA_OK;  // little-endian host: the bytes are the values
  }
  // u16 tokens are read into the upper half of the destination and widened in place, front to back.
  unsigned char* narrow = reinterpret_cast<unsigned char*>(dst) + 2 * n;
  if (!read_exact_at(bin->fd, narrow, nbytes, off)) return fail("token read: %s", errno ? strerror(errno) : "short file");
  for (uint64_t i = 0; i < n; ++i) {
    uint16_t v;
    memcpy(&v, narrow + 2 * i, 2);
    const uint32_t wide = v;
    memcpy(reinterpret_cast<unsigned char*>(dst) + 4 * i, &wide, 4);
  }
  return ODATA_OK;
}

int32_t odata_bin_read_u16(const odata_bin* bin, uint64_t index, uint16_t* dst, uint64_t n) {
  uint64_t off = 0, nbytes = 0;
  if (window_bytes(bin, index, n, &off, &nbytes) != ODATA_OK) return ODATA_ERROR;
  if (n == 0) return ODATA_OK;
  if (!dst) return fail("token read: null destination");
  if (bin->width == ODATA_WIDTH_U16) {
    if (!read_exact_at(bin->fd, dst, nbytes, off)) return fail("token read: %s", errno ? strerror(errno) : "short file");
    return ODATA_OK;
  }
  std::vector<uint32_t> wide;
  try {
    wide.resize(n);
  } catch (const std::bad_alloc&) {
    return fail("allocation of %" PRIu64 " bytes refused", nbytes);
  }
  if (!read_exact_at(bin->fd, wide.data(), nbytes, off)) return fail("token read: %s", errno ? strerror(errno) : "short file");
  for (uint64_t i = 0; i < n; ++i) {
    if (wide[i] > 65535u)
      return fail("token %u at index %" PRIu64 " exceeds u16::MAX (65535)", wide[i], index + i);
    dst[i] = static_cast<uint16_t>(wide[i]);
  }
  return ODATA_OK;
}

int32_t odata_sampler_new(const odata_bin* bin, uint64_t seq_len, uint64_t batch, uint64_t seed, uint64_t epoch,
                          uint64_t ordinal, odata_sampler** out) {
  if (!bin || !out) return fail("sampler: null argument");
  *out = nullptr;
  odata_sampler* s = new (std::nothrow) odata_sampler;
  if (!s) return fail("sampler: allocation refused");
  if (sampler_init(*s, bin->len_tokens, seq_len, batch, seed, epoch, ordinal) != ODATA_OK) {
    delete s;
    return ODATA_ERROR;
  }
  s->bin = bin;
  try {
    s->row.resize(seq_len + 1);
  } catch (const std::bad_alloc&) {
    delete s;
    return fail("sampler: allocation of the row buffer refused");
  }
  *out = s;
  return ODATA_OK;
}

int32_t odata_sampler_new_detached(uint64_t n_tokens, uint64_t seq_len, uint64_t batch, uint64_t seed, uint64_t epoch,
                                   uint64_t ordinal, odata_sampler** out) {
  if (!out) return fail("sampler: null argument");
  *out = nullptr;
  odata_sampler* s = new (std::nothrow) odata_sampler;
  if (!s) return fail("sampler: allocation refused");
  if (sampler_init(*s, n_tokens, seq_len, batch, seed, epoch, ordinal) != ODATA_OK) {
    delete s;
    return ODATA_ERROR;
  }
  *out = s;
  return ODATA_OK;
}

void odata_sampler_free(odata_sampler* s) { delete s; }

uint64_t odata_sampler_windows_per_epoch(const odata_sampler* s) { return s ? s->windows : 0; }

void odata_sampler_cursor(const odata_sampler* s, uint64_t* epoch, uint64_t* ordinal) {
  if (epoch) *epoch = s ? s->epoch : 0;
  if (ordinal) *ordinal = s ? s->ordinal : 0;
}

int32_t odata_sampler_window_start(const odata_sampler* s, uint64_t epoch, uint64_t ordinal, uint64_t* start) {
  if (!s || !start) return fail("sampler: null argument");
  if (ordinal >= s->windows) return fail("sampler: window %" PRIu64 " past %" PRIu64 " per epoch", ordinal, s->windows);
  *start = s->permute(epoch, ordinal) * s->seq_len;
  return ODATA_OK;
}

int32_t odata_sampler_next_starts(odata_sampler* s, uint64_t* starts) {
  if (!s || !starts) return fail("sampler: null argument");
  uint64_t epoch = 0, ordinal = 0;
  if (plan_batch(s, starts, &epoch, &ordinal) != ODATA_OK) return ODATA_ERROR;
  s->epoch = epoch;
  s->ordinal = ordinal;
  return ODATA_OK;
}

int32_t odata_sampler_next_batch(odata_sampler* s, uint32_t* x, uint32_t* y) {
  if (!s || !x || !y) return fail("sampler: null argument");
  if (!s->bin) return fail("sampler: this sampler holds no token bin; take the starts instead");
  std::vector<uint64_t> starts;
  try {
    starts.resize(s->batch);
  } catch (const std::bad_alloc&) {
    return fail("sampler: allocation of the batch refused");
  }
  uint64_t epoch = 0, ordinal = 0;
  if (plan_batch(s, starts.data(), &epoch, &ordinal) != ODATA_OK) return ODATA_ERROR;
  const uint64_t t = s->seq_len;
  for (uint64_t b = 0; b < s->batch; ++b) {
    if (odata_bin_read_u32(s->bin, starts[b], s->row.data(), t + 1) != ODATA_OK) return ODATA_ERROR;
    memcpy(x + b * t, s->row.data(), t * sizeof(uint32_t));
    memcpy(y + b * t, s->row.data() + 1, t * sizeof(uint32_t));
  }
  s->epoch = epoch;
  s->ordinal = ordinal;
  return ODATA_OK;
}

void odata_rng_state_encode(uint64_t seed, uint8_t out[16]) {
  const uint32_t version = 1, generator = 1;
  for (int i = 0; i < 4; ++i) out[i] = static_cast<uint8_t>(version >> (8 * i));
  for (int i = 0; i < 4; ++i) out[4 + i] = static_cast<uint8_t>(generator >> (8 * i));
  for (int i = 0; i < 8; ++i) out[8 + i] = static_cast<uint8_t>(seed >> (8 * i));
}

int32_t odata_rng_state_decode(const uint8_t* bytes, uint64_t n, uint64_t* seed) {
  if (!seed || (!bytes && n)) return fail("rng_state: null argument");
  if (n != 16) return fail("rng_state: %" PRIu64 " bytes, the v1 layout is 16", n);
  auto word = [&](int at) {
    return static_cast<uint32_t>(bytes[at]) | static_cast<uint32_t>(bytes[at + 1]) << 8 |
           static_cast<uint32_t>(bytes[at + 2]) << 16 | static_cast<uint32_t>(bytes[at + 3]) << 24;
  };
  if (word(0) != 1) return fail("rng_state: version %u, expected 1", word(0));
  if (word(4) != 1) return fail("rng_state: generator %u, this sampler is 1", word(4));
  uint64_t v = 0;
  for (int i = 0; i < 8; ++i) v |= static_cast<uint64_t>(bytes[8 + i]) << (8 * i);
  *seed = v;
  return ODATA_OK;
}

}  // extern "C"

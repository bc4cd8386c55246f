// Host-side readers of the reference's on-disk dataset formats: the binary edge list
// (dep/gemini/type.hpp:99-106, core/graph.hpp:1050-1061), the text feature / label / mask files
// (core/ntsDataloador.hpp:264-395) and the comma-separated feature variant (:397-437), plus a plain
// binary table format for features that does not need parsing at all.  No device work happens
// here; callers hand in host buffers (pinned ones when the data is uploaded or zero-copied next).
#include <errno.h>
#include <fcntl.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <string>
#include <thread>
#include <vector>

#include "common.hpp"

namespace nts {
namespace {

// Read-only mapping of a whole file.
struct MappedFile {
  const unsigned char *data = nullptr;
  size_t size = 0;
  int fd = -1;
  ~MappedFile() {
    if (data && size) munmap(const_cast<unsigned char *>(data), size);
    if (fd >= 0) close(fd);
  }
  int open_path(const char *path, const char *who) {
    if (!path) return fail(NTS_ERR_INVALID, (std::string(who) + ": null path").c_str());
    fd = open(path, O_RDONLY);
    if (fd < 0) return fail(NTS_ERR_INVALID, (std::string(who) + ": cannot open " + path + ": " + strerror(errno)).c_str());
    struct stat st;
    if (fstat(fd, &st) != 0) return fail(NTS_ERR_INVALID, (std::string(who) + ": cannot stat " + path).c_str());
    size = static_cast<size_t>(st.st_size);
    if (size == 0) return NTS_OK;
    void *p = mmap(nullptr, size, PROT_READ, MAP_PRIVATE, fd, 0);
    if (p == MAP_FAILED) {
      size = 0;
      return fail(NTS_ERR_NOMEM, (std::string(who) + ": cannot map " + path).c_str());
    }
    data = static_cast<const unsigned char *>(p);
    madvise(p, size, MADV_SEQUENTIAL);
    return NTS_OK;
  }
};

// The characters `std::istream >>` skips between tokens in the "C" locale.
inline bool is_space(unsigned char c) { return c == ' ' || (c >= '\t' && c <= '\r'); }

int clamp_threads(int threads, size_t bytes) {
  int t = threads > 0 ? threads : static_cast<int>(std::thread::hardware_concurrency());
  if (t < 1) t = 1;
  if (t > 64) t = 64;
  const size_t by_size = bytes / (1u << 16) + 1;  // no point in threads for tiny files
  if (static_cast<size_t>(t) > by_size) t = static_cast<int>(by_size);
  return t;
}

// First byte position >= pos that starts a token (a non-space byte preceded by a space or the file start).
size_t next_token_start(const unsigned char *d, size_t n, size_t pos) {
  if (pos >= n) return n;
  if (pos > 0 && !is_space(d[pos - 1]))
    while (pos < n && !is_space(d[pos])) ++pos;  // inside a token that began earlier: skip its rest
  while (pos < n && is_space(d[pos])) ++pos;
  return pos;
}

template <typename Fn>
void for_each_token(const unsigned char *d, size_t begin, size_t end, size_t n, Fn &&fn) {
  // Tokens whose first byte lies in [begin, end); begin is a token start or `end`.
  size_t p = begin;
  while (p < end) {
    size_t q = p;
    while (q < n && !is_space(d[q])) ++q;
    fn(p, q);
    p = q;
    while (p < n && is_space(d[p])) ++p;
  }
}

bool parse_u64(const unsigned char *b, const unsigned char *e, uint64_t *out) {
  if (b == e) return false;
  if (*b == '+') ++b;
  if (b == e || e - b > 19) return false;
  uint64_t v = 0;
  for (; b < e; ++b) {
    if (*b < '0' || *b > '9') return false;
    v = v * 10 + (*b - '0');
  }
  *out = v;
  return true;
}

bool parse_i64(const unsigned char *b, const unsigned char *e, int64_t *out) {
  bool neg = false;
  if (b < e && *b == '-') {
    neg = true;
    ++b;
  }
  uint64_t v;
  if (!parse_u64(b, e, &v)) return false;
  *out = neg ? -static_cast<int64_t>(v) : static_cast<int64_t>(v);
  return true;
}

const float kPow10f[11] = {1e0f, 1e1f, 1e2f, 1e3f, 1e4f, 1e5f, 1e6f, 1e7f, 1e8f, 1e9f, 1e10f};

// Decimal text -> nearest float, the value `std::istream >> float` (strtof) produces.  Plain
// "[-]ddd.ddd" tokens with fewer than 2^24 as their digit string and at most 10 fraction digits are
// one exact integer divided by one exact power of ten: a single correctly rounded float division.
// Everything else goes through strtof on a bounded copy.
bool parse_f32(const unsigned char *b, const unsigned char *e, float *out) {
  const unsigned char *p = b;
  bool neg = false;
  if (p < e && (*p == '-' || *p == '+')) {
    neg = *p == '-';
    ++p;
  }
  uint32_t mant = 0;
  int digits = 0, frac = 0;
  bool dot = false, simple = true;
  for (const unsigned char *q = p; q < e && simple; ++q) {
    const unsigned char c = *q;
    if (c >= '0' && c <= '9') {
      mant = mant * 10 + (c - '0');
      if (mant >= (1u << 24)) simple = false;  // also keeps mant far from overflowing
      ++digits;
      if (dot) ++frac;
    } else if (c == '.' && !dot) {
      dot = true;
    } else {
      simple = false;
    }
  }
  if (simple && digits > 0 && frac <= 10) {
    const float v = static_cast<float>(mant) / kPow10f[frac];
    *out = neg ? -v : v;
    return true;
  }
  // General case.  Only the characters of a decimal floating literal are accepted (no "nan", "inf"
  // or hexadecimal forms, which the stream extraction rejects as well).
  char buf[128];
  const size_t len = static_cast<size_t>(e - b);
  if (len == 0 || len >= sizeof(buf)) return false;
  for (size_t i = 0; i < len; ++i) {
    const unsigned char c = b[i];
    if (!((c >= '0' && c <= '9') || c == '+' || c == '-' || c == '.' || c == 'e' || c == 'E')) return false;
    buf[i] = static_cast<char>(c);
  }
  buf[len] = 0;
  char *endp = nullptr;
  const float v = strtof(buf, &endp);
  if (endp != buf + len) return false;
  *out = v;
  return true;
}

int mask_code(const unsigned char *b, const unsigned char *e) {
  const size_t n = static_cast<size_t>(e - b);
  if (n == 5 && memcmp(b, "train", 5) == 0) return 0;
  if ((n == 4 && memcmp(b, "eval", 4) == 0) || (n == 3 && memcmp(b, "val", 3) == 0)) return 1;
  if (n == 4 && memcmp(b, "test", 4) == 0) return 2;
  return 3;
}

template <typename Fn>
void run_threads(int threads, Fn &&fn) {
  if (threads <= 1) {
    fn(0);
    return;
  }
  std::vector<std::thread> pool;
  pool.reserve(threads);
  for (int t = 0; t < threads; ++t) pool.emplace_back([&fn, t] { fn(t); });
  for (auto &th : pool) th.join();
}

struct TableHeader {  // 32 bytes, little endian
  char magic[8];      // "NTSTABLE"
  uint64_t rows;
  uint64_t cols;
  uint32_t elem_bytes;
  uint32_t reserved;
};
const char kMagic[8] = {'N', 'T', 'S', 'T', 'A', 'B', 'L', 'E'};

}  // namespace
}  // namespace nts

using namespace nts;

extern "C" {

int nts_edge_file_count(const char *path, uint64_t *edges) {
  NTS_TRACE_RANGE("nts_edge_file_count");
  if (!path || !edges) return fail(NTS_ERR_INVALID, "nts_edge_file_count: null argument");
  struct stat st;
  if (stat(path, &st) != 0) return fail(NTS_ERR_INVALID, (std::string("nts_edge_file_count: cannot stat ") + path).c_str());
  *edges = static_cast<uint64_t>(st.st_size) / 8;  // trailing bytes short of a record are ignored
  return NTS_OK;
}

int nts_edge_file_read(const char *path, uint32_t *pairs, uint64_t first, uint64_t n, uint32_t *max_id) {
  NTS_TRACE_RANGE("nts_edge_file_read");
  if (!path || (!pairs && n)) return fail(NTS_ERR_INVALID, "nts_edge_file_read: null argument");
  const int fd = open(path, O_RDONLY);
  if (fd < 0) return fail(NTS_ERR_INVALID, (std::string("nts_edge_file_read: cannot open ") + path).c_str());
  unsigned char *dst = reinterpret_cast<unsigned char *>(pairs);
  uint64_t done = 0;
  const uint64_t bytes = n * 8;
  while (done < bytes) {
    const size_t want = static_cast<size_t>(bytes - done < (1ull << 30) ? bytes - done : (1ull << 30));
    const ssize_t got = pread(fd, dst + done, want, static_cast<off_t>(first * 8 + done));
    if (got < 0 && errno == EINTR) continue;
    if (got <= 0) {
      close(fd);
      return fail(NTS_ERR_INVALID, "nts_edge_file_read: file shorter than the requested edge range");
    }
    done += static_cast<uint64_t>(got);
  }
  close(fd);
  if (max_id) {
    const int threads = clamp_threads(0, static_cast<size_t>(bytes));
    std::vector<uint32_t> part(threads, 0);
    run_threads(threads, [&](int t) {
      const uint64_t lo = 2 * n * t / threads, hi = 2 * n * (t + 1) / threads;
      uint32_t m = 0;
      for (uint64_t i = lo; i < hi; ++i) m = pairs[i] > m ? pairs[i] : m;
      part[t] = m;
    });
    uint32_t m = 0;
    for (uint32_t v : part) m = v > m ? v : m;
    *max_id = m;
  }
  return NTS_OK;
}

// Feature file: records of 1 + F tokens "id f0 .. fF-1".  Fills table rows by id and `ids` with the
// id of every record in file order.
static int feature_text_read(const char *path, float *table, std::vector<uint32_t> &ids_out, uint32_t V, uint32_t F,
                             int threads) {
  if (!table || F == 0) return fail(NTS_ERR_INVALID, "nts_read_feature_label_mask (features): null table or F is 0");
  MappedFile f;
  if (int rc = f.open_path(path, "nts_read_feature_label_mask")) return rc;
  const unsigned char *d = f.data;
  const size_t n = f.size;
  const int T = clamp_threads(threads, n);
  std::vector<size_t> cut(T + 1);
  for (int t = 0; t <= T; ++t) cut[t] = next_token_start(d, n, n / T * t + (t == T ? n % T : 0));
  cut[T] = n;
  // Pass 1: tokens per slice, so that every slice knows the index of its first token and with it
  // the record and field of each of its tokens, whatever the line structure of the file is.
  std::vector<uint64_t> count(T + 1, 0);
  run_threads(T, [&](int t) {
    uint64_t c = 0;
    for_each_token(d, cut[t], cut[t + 1], n, [&](size_t, size_t) { ++c; });
    count[t + 1] = c;
  });
  for (int t = 0; t < T; ++t) count[t + 1] += count[t];
  const uint64_t per = static_cast<uint64_t>(F) + 1;
  const uint64_t tokens = count[T];
  if (tokens % per != 0) return fail(NTS_ERR_INVALID, "nts_read_feature_label_mask (features): the last record is incomplete");
  const uint64_t records = tokens / per;
  // Pass 2: the id token of every record.
  ids_out.assign(records, 0);
  uint32_t *ids = ids_out.data();
  std::atomic<int> bad{0};
  run_threads(T, [&](int t) {
    uint64_t k = count[t];
    for_each_token(d, cut[t], cut[t + 1], n, [&](size_t b, size_t e) {
      if (k % per == 0) {
        uint64_t id;
        if (!parse_u64(d + b, d + e, &id) || id > 0xFFFFFFFFull) bad.store(1);
        else ids[k / per] = static_cast<uint32_t>(id);
      }
      ++k;
    });
  });
  if (bad.load()) return fail(NTS_ERR_INVALID, "nts_read_feature_label_mask (features): a vertex id is not an unsigned 32-bit integer");
  // Pass 3: the values, placed by the record's id; records of ids outside [0, V) are skipped as the
  // reference skips vertices outside its partition.
  run_threads(T, [&](int t) {
    uint64_t k = count[t];
    for_each_token(d, cut[t], cut[t + 1], n, [&](size_t b, size_t e) {
      const uint64_t j = k % per;
      if (j != 0) {
        const uint32_t id = ids[k / per];
        if (id < V) {
          float v;
          if (!parse_f32(d + b, d + e, &v)) bad.store(1);
          else table[static_cast<size_t>(id) * F + (j - 1)] = v;
        }
      }
      ++k;
    });
  });
  if (bad.load()) return fail(NTS_ERR_INVALID, "nts_read_feature_label_mask (features): a feature value is not a decimal number");
  return NTS_OK;
}

int nts_feature_csv_read(const char *path, float *table, uint32_t V, uint32_t F, int threads) {
  NTS_TRACE_RANGE("nts_feature_csv_read");
  if (!table || F == 0) return fail(NTS_ERR_INVALID, "nts_feature_csv_read: null table or F is 0");
  MappedFile f;
  if (int rc = f.open_path(path, "nts_feature_csv_read")) return rc;
  const unsigned char *d = f.data;
  const size_t n = f.size;
  const int T = clamp_threads(threads, n);
  // Slices begin after a newline; line k of the file is vertex k.
  std::vector<size_t> cut(T + 1);
  for (int t = 0; t <= T; ++t) {
    size_t p = n / T * t;
    if (t == T) p = n;
    if (p > 0 && p < n) {
      while (p < n && d[p - 1] != '\n') ++p;
    }
    cut[t] = p;
  }
  std::vector<uint64_t> lines(T + 1, 0);
  run_threads(T, [&](int t) {
    uint64_t c = 0;
    for (size_t p = cut[t]; p < cut[t + 1]; ++p) c += d[p] == '\n';
    if (t == T - 1 && n > 0 && d[n - 1] != '\n' && cut[t] < n) ++c;  // last line without a newline
    lines[t + 1] = c;
  });
  for (int t = 0; t < T; ++t) lines[t + 1] += lines[t];
  if (lines[T] < V) return fail(NTS_ERR_INVALID, "nts_feature_csv_read: fewer lines than vertices");
  std::atomic<int> bad{0};
  run_threads(T, [&](int t) {
    uint64_t row = lines[t];
    size_t p = cut[t];
    while (p < cut[t + 1] && row < V) {
      size_t eol = p;
      while (eol < n && d[eol] != '\n') ++eol;
      uint32_t col = 0;
      size_t q = p;
      // Fields as `getline(ss, field, ',')` yields them: empty fields between commas count (and
      // read as 0), an empty field after the last comma does not.
      while (q < eol) {
        size_t r = q;
        while (r < eol && d[r] != ',') ++r;
        if (col >= F) {
          ++col;
          break;
        }
        // std::atof: strtod on the field (leading blanks skipped, trailing text ignored), narrowed to float.
        char buf[128];
        size_t len = r - q;
        if (len >= sizeof(buf)) len = sizeof(buf) - 1;
        memcpy(buf, d + q, len);
        buf[len] = 0;
        table[static_cast<size_t>(row) * F + col] = static_cast<float>(strtod(buf, nullptr));
        ++col;
        q = r + 1;
      }
      if (col != F) bad.store(1);
      ++row;
      p = eol + 1;
    }
  });
  if (bad.load()) return fail(NTS_ERR_INVALID, "nts_feature_csv_read: a line does not hold exactly F fields");
  return NTS_OK;
}

// Label file: records "id label" (classes <= 1) or "id count idx_1 .. idx_count".  record_ids == NULL
// places a record by its own id, otherwise the k-th record goes to record_ids[k].
static int label_text_read(const char *path, int64_t *labels, const uint32_t *record_ids, uint64_t n_records,
                           uint32_t V, uint32_t classes) {
  if (!labels) return fail(NTS_ERR_INVALID, "nts_read_feature_label_mask (labels): null labels");
  MappedFile f;
  if (int rc = f.open_path(path, "nts_read_feature_label_mask")) return rc;
  const unsigned char *d = f.data;
  const size_t n = f.size;
  size_t p = next_token_start(d, n, 0);
  auto next = [&](size_t *b, size_t *e) {
    if (p >= n) return false;
    *b = p;
    while (p < n && !is_space(d[p])) ++p;
    *e = p;
    while (p < n && is_space(d[p])) ++p;
    return true;
  };
  const uint32_t width = classes > 1 ? classes : 1;
  uint64_t rec = 0;
  size_t b, e;
  while (next(&b, &e)) {
    uint64_t file_id;
    const bool id_ok = parse_u64(d + b, d + e, &file_id);
    // Placement: by the label file's own id (global table), or by the id of the feature file's
    // record at the same position (local table; the label file's id column is then only skipped).
    uint64_t id;
    if (record_ids) {
      if (rec >= n_records) break;
      id = record_ids[rec];
    } else {
      if (!id_ok) break;  // `while (input_lbl >> id)` ends at the first token that is no integer
      id = file_id;
    }
    ++rec;
    const bool keep = id < V;
    if (classes > 1) {
      int64_t sz;
      if (!next(&b, &e) || !parse_i64(d + b, d + e, &sz)) return fail(NTS_ERR_INVALID, "nts_read_feature_label_mask (labels): missing label count");
      for (int64_t i = 0; i < sz; ++i) {
        int64_t idx;
        if (!next(&b, &e) || !parse_i64(d + b, d + e, &idx)) return fail(NTS_ERR_INVALID, "nts_read_feature_label_mask (labels): missing class index");
        if (idx < 0 || idx >= static_cast<int64_t>(classes)) return fail(NTS_ERR_INVALID, "nts_read_feature_label_mask (labels): class index out of range");
        if (keep) labels[id * width + static_cast<uint64_t>(idx)] = 1;
      }
    } else {
      int64_t v;
      if (!next(&b, &e) || !parse_i64(d + b, d + e, &v)) return fail(NTS_ERR_INVALID, "nts_read_feature_label_mask (labels): missing label");
      if (keep) labels[id] = v;
    }
  }
  return NTS_OK;
}

static int mask_text_read(const char *path, int32_t *mask, const uint32_t *record_ids, uint64_t n_records,
                          uint32_t V) {
  if (!mask) return fail(NTS_ERR_INVALID, "nts_read_feature_label_mask (masks): null mask");
  MappedFile f;
  if (int rc = f.open_path(path, "nts_read_feature_label_mask")) return rc;
  const unsigned char *d = f.data;
  const size_t n = f.size;
  size_t p = next_token_start(d, n, 0);
  auto next = [&](size_t *b, size_t *e) {
    if (p >= n) return false;
    *b = p;
    while (p < n && !is_space(d[p])) ++p;
    *e = p;
    while (p < n && is_space(d[p])) ++p;
    return true;
  };
  uint64_t rec = 0;
  size_t b, e;
  while (next(&b, &e)) {
    uint64_t file_id;
    const bool id_ok = parse_u64(d + b, d + e, &file_id);
    uint64_t id;
    if (record_ids) {
      if (rec >= n_records) break;
      id = record_ids[rec];
    } else {
      if (!id_ok) break;
      id = file_id;
    }
    ++rec;
    if (!next(&b, &e)) return fail(NTS_ERR_INVALID, "nts_read_feature_label_mask (masks): missing mask word");
    if (id < V) mask[id] = mask_code(d + b, d + e);
  }
  return NTS_OK;
}

int nts_read_feature_label_mask(const char *path_f, const char *path_l, const char *path_m, uint32_t V, uint32_t F,
                                uint32_t classes, float *local_feature, int64_t *local_label, int32_t *local_mask,
                                int64_t *global_label, int32_t *global_mask, int threads) {
  NTS_TRACE_RANGE("nts_read_feature_label_mask");
  std::vector<uint32_t> ids;
  if (int rc = feature_text_read(path_f, local_feature, ids, V, F, threads)) return rc;
  if (local_label)
    if (int rc = label_text_read(path_l, local_label, ids.data(), ids.size(), V, classes)) return rc;
  if (local_mask)
    if (int rc = mask_text_read(path_m, local_mask, ids.data(), ids.size(), V)) return rc;
  if (global_label)
    if (int rc = label_text_read(path_l, global_label, nullptr, 0, V, classes)) return rc;
  if (global_mask)
    if (int rc = mask_text_read(path_m, global_mask, nullptr, 0, V)) return rc;
  return NTS_OK;
}

int nts_int_list_text_read(const char *path, int64_t *out, uint64_t capacity, uint64_t *count) {
  NTS_TRACE_RANGE("nts_int_list_text_read");
  if (!count) return fail(NTS_ERR_INVALID, "nts_int_list_text_read: null count");
  MappedFile f;
  if (int rc = f.open_path(path, "nts_int_list_text_read")) return rc;
  const unsigned char *d = f.data;
  const size_t n = f.size;
  uint64_t k = 0;
  bool stop = false;
  for_each_token(d, next_token_start(d, n, 0), n, n, [&](size_t b, size_t e) {
    int64_t v;
    if (stop || !parse_i64(d + b, d + e, &v)) {  // extraction ends at the first token that is no integer
      stop = true;
      return;
    }
    if (out && k < capacity) out[k] = v;
    ++k;
  });
  *count = k;
  return NTS_OK;
}

int nts_table_bin_write(const char *path, const void *data, uint64_t rows, uint64_t cols, uint32_t elem_bytes) {
  NTS_TRACE_RANGE("nts_table_bin_write");
  if (!path || (!data && rows * cols)) return fail(NTS_ERR_INVALID, "nts_table_bin_write: null argument");
  const int fd = open(path, O_WRONLY | O_CREAT | O_TRUNC, 0644);
  if (fd < 0) return fail(NTS_ERR_INVALID, (std::string("nts_table_bin_write: cannot create ") + path).c_str());
  TableHeader h;
  memcpy(h.magic, kMagic, 8);
  h.rows = rows;
  h.cols = cols;
  h.elem_bytes = elem_bytes;
  h.reserved = 0;
  bool ok = write(fd, &h, sizeof(h)) == static_cast<ssize_t>(sizeof(h));
  const unsigned char *src = static_cast<const unsigned char *>(data);
  uint64_t left = rows * cols * elem_bytes;
  while (ok && left) {
    const size_t want = static_cast<size_t>(left < (1ull << 30) ? left : (1ull << 30));
    const ssize_t got = write(fd, src, want);
    if (got < 0 && errno == EINTR) continue;
    if (got <= 0) ok = false;
    else {
      src += got;
      left -= static_cast<uint64_t>(got);
    }
  }
  ok = close(fd) == 0 && ok;
  return ok ? NTS_OK : fail(NTS_ERR_INVALID, "nts_table_bin_write: write failed");
}

int nts_feature_text_write(const char *path, const float *table, const uint32_t *ids, uint32_t V, uint32_t F,
                           int decimals, int threads) {
  NTS_TRACE_RANGE("nts_feature_text_write");
  if (!path || (!table && static_cast<uint64_t>(V) * F)) return fail(NTS_ERR_INVALID, "nts_feature_text_write: null argument");
  if (decimals < 0 || decimals > 9) return fail(NTS_ERR_INVALID, "nts_feature_text_write: decimals outside 0..9");
  const int T = clamp_threads(threads, static_cast<size_t>(V) * F * 4);
  // Each thread formats a contiguous block of records into its own buffer; the buffers are then
  // written in order.
  std::vector<std::string> parts(T);
  const uint32_t per = (V + T - 1) / T;
  run_threads(T, [&](int t) {
    const uint32_t r0 = std::min<uint64_t>(V, static_cast<uint64_t>(t) * per), r1 = std::min<uint64_t>(V, r0 + per);
    std::string &out = parts[t];
    out.reserve(static_cast<size_t>(r1 - r0) * (12 + static_cast<size_t>(F) * (decimals + 6)));
    char buf[64];
    for (uint32_t r = r0; r < r1; ++r) {
      out.append(buf, static_cast<size_t>(snprintf(buf, sizeof buf, "%u", ids ? ids[r] : r)));
      const float *row = table + static_cast<size_t>(r) * F;
      for (uint32_t c = 0; c < F; ++c)
        out.append(buf, static_cast<size_t>(snprintf(buf, sizeof buf, " %.*f", decimals, static_cast<double>(row[c]))));
      out.push_back('\n');
    }
  });
  FILE *f = fopen(path, "wb");
  if (!f) return fail(NTS_ERR_INVALID, (std::string("nts_feature_text_write: cannot create ") + path).c_str());
  bool ok = true;
  for (const std::string &part : parts) ok = ok && fwrite(part.data(), 1, part.size(), f) == part.size();
  ok = fclose(f) == 0 && ok;
  return ok ? NTS_OK : fail(NTS_ERR_INVALID, "nts_feature_text_write: write failed");
}

int nts_table_bin_info(const char *path, uint64_t *rows, uint64_t *cols, uint32_t *elem_bytes) {
  NTS_TRACE_RANGE("nts_table_bin_info");
  if (!path) return fail(NTS_ERR_INVALID, "nts_table_bin_info: null path");
  const int fd = open(path, O_RDONLY);
  if (fd < 0) return fail(NTS_ERR_INVALID, (std::string("nts_table_bin_info: cannot open ") + path).c_str());
  TableHeader h;
  const ssize_t got = pread(fd, &h, sizeof(h), 0);
  struct stat st;
  const bool stat_ok = fstat(fd, &st) == 0;
  close(fd);
  if (got != static_cast<ssize_t>(sizeof(h)) || memcmp(h.magic, kMagic, 8) != 0)
    return fail(NTS_ERR_INVALID, "nts_table_bin_info: not a table file");
  if (!stat_ok || static_cast<uint64_t>(st.st_size) < sizeof(h) + h.rows * h.cols * h.elem_bytes)
    return fail(NTS_ERR_INVALID, "nts_table_bin_info: file shorter than its header says");
  if (rows) *rows = h.rows;
  if (cols) *cols = h.cols;
  if (elem_bytes) *elem_bytes = h.elem_bytes;
  return NTS_OK;
}

int nts_table_bin_read(const char *path, void *out, uint64_t row_begin, uint64_t rows) {
  NTS_TRACE_RANGE("nts_table_bin_read");
  uint64_t R, C;
  uint32_t eb;
  if (int rc = nts_table_bin_info(path, &R, &C, &eb)) return rc;
  if (row_begin > R || rows > R - row_begin) return fail(NTS_ERR_INVALID, "nts_table_bin_read: row range outside the table");
  if (!out && rows * C) return fail(NTS_ERR_INVALID, "nts_table_bin_read: null out");
  const int fd = open(path, O_RDONLY);
  if (fd < 0) return fail(NTS_ERR_INVALID, "nts_table_bin_read: cannot open file");
  unsigned char *dst = static_cast<unsigned char *>(out);
  const uint64_t bytes = rows * C * eb;
  const uint64_t base = sizeof(TableHeader) + row_begin * C * eb;
  uint64_t done = 0;
  while (done < bytes) {
    const size_t want = static_cast<size_t>(bytes - done < (1ull << 30) ? bytes - done : (1ull << 30));
    const ssize_t got = pread(fd, dst + done, want, static_cast<off_t>(base + done));
    if (got < 0 && errno == EINTR) continue;
    if (got <= 0) {
      close(fd);
      return fail(NTS_ERR_INVALID, "nts_table_bin_read: short read");
    }
    done += static_cast<uint64_t>(got);
  }
  close(fd);
  return NTS_OK;
}

}  // extern "C"

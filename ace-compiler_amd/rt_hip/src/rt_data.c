/* rt_data.c -- the weight side-file of a compiled model and the plaintexts made from it.
 *
 * File layout (fhe-cmplr/include/fhe/core/rt_data_def.h:62-84, rt_data_writer.h:34-107): a 136-byte header
 * at offset 0, entries from offset 4096 on, each padded to 2^_ent_align bytes, and a lookup table of
 * 32-byte records at _lut_ofst.  Message files (float or double entries) are read whole at Prepare_context,
 * as Pt_mgr_init does (rtlib/ant/porting/pt_mgr.c:35-99); Pt_from_msg encodes `len` values of entry `index`
 * (pt_mgr.c:188-243).  A file of pre-encoded plaintexts (DE_PLAINTEXT) holds, per entry, a PLAINTEXT_BUFFER
 * (fhe-cmplr/include/fhe/core/rt_encode_api.h:20-27): magic, version, size, then the host image of a PLAINTEXT
 * with a null `_data` followed by its words; such files can be far larger than host memory, so their entries
 * are read one at a time, on demand, and uploaded (Pt_get, pt_mgr.c:117-177).
 *
 * RT_HIP_DATA_FILE names the file when the path compiled into the program does not exist here.
 * RT_HIP_SYNTHETIC_WEIGHTS=<amplitude> replaces a missing file by reproducible pseudo-random values in
 * (-amplitude, amplitude): for timing a model whose weights are not at hand, never for its accuracy.
 */
#include <math.h>
#include <time.h>

#include "rt_internal.h"

#define DATA_PAGE 4096
typedef struct {
  char            magic[8];
  uint32_t        rt_ver;
  uint16_t        flag;
  uint8_t         ent_type, ent_align;
  uint64_t        ent_count, lut_ofst;
  struct timespec ctime;
  char            model[48], uuid[40];
} DATA_HDR;
typedef struct {
  char     name[16];
  uint32_t index, size;
  uint64_t scale : 8, level : 8, ofst : 48;
} LUT_ENTRY;
_Static_assert(sizeof(DATA_HDR) == 136 && sizeof(LUT_ENTRY) == 32, "side-file records");

static struct {
  bool       open, synthetic;
  double     amplitude;
  /* synthetic entries are made once and kept, as a file's entries are: [index] -> values from 0 on */
  double** syn;
  size_t*  syn_len;
  size_t   syn_count;
  DATA_HDR   hdr;
  LUT_ENTRY* lut;
  char*      buf; /* the bytes between the first page and the lookup table */
  uint64_t   size;
  FILE*       file; /* a file of pre-encoded plaintexts stays open */
  PLAINTEXT** pt;   /* [ent_count]: the entries uploaded so far */
} Data;

/* Encoded weight plaintexts kept in HBM.  A program encodes the same entries for every input it is run on (the
 * reference avoids that only with files of pre-encoded plaintexts); with a few hundred GB of HBM the encoded
 * polynomial of each (entry, range, scale degree, level) is kept after its first use and copied from then on.
 * RT_HIP_PLAINTEXT_CACHE_GB bounds the space (default 96; 0 switches it off). */
typedef struct {
  uint64_t k1, k2; /* (index, scale, level), (offset, length); k1 == 0 marks a free cell (level is never 0) */
  int64_t* dev;
} PT_CELL;
static struct {
  PT_CELL*  cell;
  size_t    cap, count, words, limit_words;
  int64_t** slab; /* the polynomials live in 1 GiB slabs: one device allocation per 100-odd plaintexts */
  size_t    n_slabs, slab_left;
} Cache;
#define PT_SLAB_WORDS ((size_t)1 << 27)

static int64_t* cache_room(size_t words) {
  if (words > PT_SLAB_WORDS) return NULL;
  if (Cache.slab_left < words) {
    Cache.slab                  = (int64_t**)realloc(Cache.slab, (Cache.n_slabs + 1) * sizeof(int64_t*));
    Cache.slab[Cache.n_slabs++] = Rt_dev_alloc_raw(PT_SLAB_WORDS);
    Cache.slab_left             = PT_SLAB_WORDS;
  }
  int64_t* p = Cache.slab[Cache.n_slabs - 1] + (PT_SLAB_WORDS - Cache.slab_left);
  Cache.slab_left -= words;
  return p;
}

/* room for `count` polynomials of `words` words one after the other (a batch is encoded straight into it) */
static int64_t* cache_room_run(size_t words, size_t count) {
  if (words * count > PT_SLAB_WORDS) return NULL;
  if (Cache.slab_left < words * count) Cache.slab_left = 0; /* the rest of the slab stays unused */
  int64_t* first = cache_room(words);
  for (size_t i = 1; first && i < count; ++i) (void)cache_room(words);
  return first;
}

static PT_CELL* cache_find(uint64_t k1, uint64_t k2) {
  if (!Cache.cap) return NULL;
  uint64_t h = (k1 * 0x9E3779B97F4A7C15ull) ^ (k2 * 0xC2B2AE3D27D4EB4Full);
  for (size_t i = (size_t)(h >> 20) & (Cache.cap - 1);; i = (i + 1) & (Cache.cap - 1)) {
    PT_CELL* c = &Cache.cell[i];
    if (c->k1 == 0 || (c->k1 == k1 && c->k2 == k2)) return c;
  }
}
static void cache_grow(void) {
  PT_CELL* old     = Cache.cell;
  size_t   old_cap = Cache.cap;
  Cache.cap        = old_cap ? 2 * old_cap : 4096;
  Cache.cell       = (PT_CELL*)calloc(Cache.cap, sizeof(PT_CELL));
  for (size_t i = 0; i < old_cap; ++i)
    if (old[i].k1) *cache_find(old[i].k1, old[i].k2) = old[i];
  free(old);
}
static void cache_clear(void) {
  for (size_t i = 0; i < Cache.n_slabs; ++i) Rt_dev_free(Cache.slab[i]);
  free(Cache.slab);
  free(Cache.cell);
  memset(&Cache, 0, sizeof(Cache));
}

static void flight_land(void);
bool Pt_mgr_init(const char* fname) {
  const char* gb    = getenv("RT_HIP_PLAINTEXT_CACHE_GB");
  cache_clear();
  Cache.limit_words = (size_t)((gb ? atof(gb) : 96.0) * (double)(1ull << 27));
  const char* over = getenv("RT_HIP_DATA_FILE");
  const char* syn  = getenv("RT_HIP_SYNTHETIC_WEIGHTS");
  if (over && *over) fname = over;
  memset(&Data, 0, sizeof(Data));
  FILE* f = fname ? fopen(fname, "rb") : NULL;
  if (!f) {
    if (syn && atof(syn) > 0) {
      Data.open = Data.synthetic = true;
      Data.amplitude             = atof(syn);
      fprintf(stderr, "rt_hip: %s not found: synthetic weights of amplitude %g\n", fname ? fname : "(no file)", Data.amplitude);
      return true;
    }
    Rt_fatal(__FILE__, __LINE__, "failed to open rt data file %s (RT_HIP_DATA_FILE overrides the compiled-in path)",
             fname ? fname : "(null)");
  }
  FMT_ASSERT(fread(&Data.hdr, sizeof(DATA_HDR), 1, f) == 1, "failed to read rt data file header");
  FMT_ASSERT(memcmp(Data.hdr.magic, "!ANTFHE\0", 8) == 0, "%s is not an rt data file", fname);
  FMT_ASSERT(Data.hdr.ent_type == DE_MSG_F32 || Data.hdr.ent_type == DE_MSG_F64 || Data.hdr.ent_type == DE_PLAINTEXT,
             "unknown entry type %u in rt data file", (unsigned)Data.hdr.ent_type);
  FMT_ASSERT(Data.hdr.lut_ofst >= DATA_PAGE, "lookup table inside the first page");
  Data.lut = (LUT_ENTRY*)malloc((Data.hdr.ent_count ? Data.hdr.ent_count : 1) * sizeof(LUT_ENTRY));
  FMT_ASSERT(fseek(f, (long)Data.hdr.lut_ofst, SEEK_SET) == 0 &&
                 fread(Data.lut, sizeof(LUT_ENTRY), Data.hdr.ent_count, f) == Data.hdr.ent_count,
             "failed to read rt data file lookup table");
  Data.size = Data.hdr.lut_ofst - DATA_PAGE;
  if (Data.hdr.ent_type == DE_PLAINTEXT) {
    Data.file = f;
    Data.pt   = (PLAINTEXT**)calloc(Data.hdr.ent_count ? Data.hdr.ent_count : 1, sizeof(PLAINTEXT*));
    Data.open = true;
    return true;
  }
  Data.buf  = (char*)malloc(Data.size ? Data.size : 1);
  FMT_ASSERT(fseek(f, DATA_PAGE, SEEK_SET) == 0 && fread(Data.buf, 1, Data.size, f) == Data.size,
             "failed to fill data from file");
  fclose(f);
  Data.open = true;
  return true;
}

void Pt_mgr_fini(void) {
  flight_land();
  cache_clear();
  if (Data.pt)
    for (uint64_t i = 0; i < Data.hdr.ent_count; ++i)
      if (Data.pt[i]) Pt_free((uint32_t)i);
  free(Data.pt);
  if (Data.file) fclose(Data.file);
  for (size_t i = 0; i < Data.syn_count; ++i) free(Data.syn[i]);
  free(Data.syn);
  free(Data.syn_len);
  free(Data.lut);
  free(Data.buf);
  memset(&Data, 0, sizeof(Data));
}

static const double* synthetic_entry(uint32_t index, size_t upto);
static void          Pt_encode_entry(void* pt, uint32_t index, size_t ofst, size_t len, uint32_t scale, uint32_t level);

/* entry `index` from value `first` on, `len` values, as doubles */
static double* entry_values(uint32_t index, size_t first, size_t len) {
  FMT_ASSERT(Data.open, "the program has no rt data file (Get_rt_data_info)");
  double* v = (double*)malloc((len ? len : 1) * sizeof(double));
  if (Data.synthetic) {
    memcpy(v, synthetic_entry(index, first + len) + first, len * sizeof(double));
    return v;
  }
  size_t width = Data.hdr.ent_type == DE_MSG_F32 ? sizeof(float) : sizeof(double);
  FMT_ASSERT(index < Data.hdr.ent_count, "index out of entry range");
  const LUT_ENTRY* e = &Data.lut[index];
  FMT_ASSERT(e->size >= (first + len) * width, "entry size too small");
  FMT_ASSERT(e->ofst >= DATA_PAGE && e->ofst - DATA_PAGE + (first + len) * width <= Data.size, "entry offset too large");
  const char* p = Data.buf + (e->ofst - DATA_PAGE) + first * width;
  for (size_t i = 0; i < len; ++i) {
    if (width == sizeof(float)) {
      float x;
      memcpy(&x, p + i * width, width);
      v[i] = (double)x;
    } else {
      memcpy(&v[i], p + i * width, width);
    }
  }
  return v;
}

/* the entry's values where they lie (floats or doubles of the file, possibly unaligned: only ever copied) */
/* room in the table of synthetic entries for the indices below `count` (one thread at a time) */
static void synthetic_reserve(size_t count) {
  if (count <= Data.syn_count) return;
  size_t n     = count + 64;
  Data.syn     = (double**)realloc(Data.syn, n * sizeof(double*));
  Data.syn_len = (size_t*)realloc(Data.syn_len, n * sizeof(size_t));
  for (size_t i = Data.syn_count; i < n; ++i) {
    Data.syn[i]     = NULL;
    Data.syn_len[i] = 0;
  }
  Data.syn_count = n;
}
/* the values of one entry up to `upto`; entries are independent of each other */
static void synthetic_fill(uint32_t index, size_t upto) {
  if (Data.syn_len[index] >= upto) return;
  Data.syn[index] = (double*)realloc(Data.syn[index], upto * sizeof(double));
  for (size_t i = Data.syn_len[index]; i < upto; ++i) {
    uint64_t z = ((uint64_t)index << 32 | (uint64_t)i) + 0x9E3779B97F4A7C15ull;
    z          = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z          = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    Data.syn[index][i] = Data.amplitude * ((double)(int64_t)(z >> 11) / (double)(1ull << 52) - 1.0);
  }
  Data.syn_len[index] = upto;
}
static const double* synthetic_entry(uint32_t index, size_t upto) {
  synthetic_reserve((size_t)index + 1);
  synthetic_fill(index, upto);
  return Data.syn[index];
}
/* The entries index .. index + count - 1 made by several host threads: a weight file's entries are there to be
 * copied, and the values that stand in for them (a hash per value, 100 million of them for ResNet-20) should not
 * cost a run more than reading the file would. */
static void synthetic_entries(uint32_t index, size_t count, size_t upto) {
  synthetic_reserve((size_t)index + count);
#pragma omp parallel for schedule(static, 1) num_threads(8) if (count > 1)
  for (size_t n = 0; n < count; ++n) synthetic_fill(index + (uint32_t)n, upto);
}

static const void* entry_bytes(uint32_t index, size_t first, size_t len, int* is_f32) {
  FMT_ASSERT(Data.open, "the program has no rt data file (Get_rt_data_info)");
  if (Data.synthetic) {
    *is_f32 = 0;
    return synthetic_entry(index, first + len) + first;
  }
  size_t width = Data.hdr.ent_type == DE_MSG_F32 ? sizeof(float) : sizeof(double);
  FMT_ASSERT(index < Data.hdr.ent_count, "index out of entry range");
  const LUT_ENTRY* e = &Data.lut[index];
  FMT_ASSERT(e->size >= (first + len) * width, "entry size too small");
  FMT_ASSERT(e->ofst >= DATA_PAGE && e->ofst - DATA_PAGE + (first + len) * width <= Data.size, "entry offset too large");
  *is_f32 = width == sizeof(float);
  return Data.buf + (e->ofst - DATA_PAGE) + first * width;
}

/* Programs ask for the entries of a tensor one after the other (index, index + 1, ... with the same range, scale
 * and level: the taps and channels of a convolution), each a handful of small launches on one polynomial.  On a
 * miss the entries that follow are therefore encoded along with the one asked for, in one set of launches
 * (ace_encode_real_batch: the same bits), straight into the kept plaintexts; a guess that the program does not
 * follow costs the encodes it does not use.  RT_HIP_PLAINTEXT_AHEAD sets how many (default 16, 1 = none). */
#define PT_AHEAD_MAX 64
static bool entry_has(uint32_t index, size_t first, size_t len) {
  if (Data.synthetic) return true;
  if (index >= Data.hdr.ent_count) return false;
  size_t           width = Data.hdr.ent_type == DE_MSG_F32 ? sizeof(float) : sizeof(double);
  const LUT_ENTRY* e     = &Data.lut[index];
  return e->size >= (first + len) * width && e->ofst >= DATA_PAGE && e->ofst - DATA_PAGE + (first + len) * width <= Data.size;
}
static uint64_t cache_key1(uint32_t index, uint32_t scale, uint32_t level) {
  return ((uint64_t)index << 32) | ((uint64_t)(scale & 0xFFFF) << 16) | (level ? level : Get_q_cnt());
}
static size_t ahead_count(void) {
  static size_t ahead;
  if (!ahead) {
    const char* env = getenv("RT_HIP_PLAINTEXT_AHEAD");
    ahead           = env ? (size_t)atoi(env) : 16;
    if (ahead < 1) ahead = 1;
    if (ahead > PT_AHEAD_MAX) ahead = PT_AHEAD_MAX;
  }
  return ahead;
}
/* Encodes the entries index, index + 1, ... (up to the first one kept already, at most `ahead_count()`, at least
 * `at_least`) in one set of launches on the current stream, straight into the kept plaintexts; returns how many. */
static size_t encode_run(uint32_t index, size_t ofst, size_t len, uint32_t scale, uint32_t level, size_t words,
                         size_t at_least, int64_t** first) {
  const size_t   ahead = ahead_count();
  const uint64_t k2    = ((uint64_t)ofst << 32) | (uint64_t)len;
  const void*    vals[PT_AHEAD_MAX];
  int            is_f32 = 0;
  size_t         n      = 0;
  while (4 * (Cache.count + ahead + 1) > 3 * Cache.cap) cache_grow();
  if (Data.synthetic && (uint64_t)index + ahead < (1ull << 32)) synthetic_entries(index, ahead, ofst + len);
  for (; n < ahead && (uint64_t)index + n < (1ull << 32); ++n) {
    uint32_t idx = index + (uint32_t)n;
    if (Cache.words + (n + 1) * words > Cache.limit_words || !entry_has(idx, ofst, len)) break;
    if (cache_find(cache_key1(idx, scale, level), k2)->k1) break; /* kept already: the run ends here */
    vals[n] = entry_bytes(idx, ofst, len, &is_f32);
  }
  if (n < at_least) return 0;
  int64_t* base = cache_room_run(words, n);
  if (!base) return 0;
  Rt_encode_real_batch(base, words, vals, is_f32, len, n, scale, level);
  for (size_t i = 0; i < n; ++i) {
    PT_CELL* c = cache_find(cache_key1(index + (uint32_t)i, scale, level), k2);
    c->k1      = cache_key1(index + (uint32_t)i, scale, level);
    c->k2      = k2;
    c->dev     = base + i * words;
    ++Cache.count;
    Cache.words += words;
  }
  if (first) *first = base;
  return n;
}

/* While the program works through one run of entries, the next run is encoded on the library's second stream
 * (ace_fork / ace_fork_switch): a polynomial's encoding is a dozen launches too small for the machine, like the
 * products that consume the one before it, and the two overlap.  One run is in flight at a time; the first request
 * for one of its entries makes the program's stream wait for it (ace_join) and sends off the run after it.  Only
 * while a single host thread uses the runtime (several threads fill the machine by themselves, and their streams
 * already share the hardware's queues); RT_HIP_PLAINTEXT_ASYNC=0 keeps every encoding on the program's stream. */
static struct {
  bool     active;
  ace_ctx* ctx; /* the context (of the one thread there was) whose second stream carries the run */
  uint32_t first, count, scale, level;
  uint64_t k2;
} Flight;
static bool async_encodes(void) {
  static int off = -1;
  if (off < 0) off = getenv("RT_HIP_PLAINTEXT_ASYNC") && atoi(getenv("RT_HIP_PLAINTEXT_ASYNC")) == 0;
  return !off && ahead_count() >= 2 && Rt_lane_count() == 1;
}
static void flight_land(void) {
  if (!Flight.active) return;
  if (Flight.ctx != RT_CTX) { /* another thread has come since: it cannot join that context's streams, it waits */
    ACE_OK(ace_sync_device(RT_CTX));
    return;
  }
  ACE_OK(ace_join(RT_CTX));
  Flight.active = false;
}
static void flight_start(uint32_t index, size_t ofst, size_t len, uint32_t scale, uint32_t level, size_t words) {
  if (Flight.active || !async_encodes()) return;
  ACE_OK(ace_fork(RT_CTX));
  size_t n = encode_run(index, ofst, len, scale, level, words, 1, NULL);
  ACE_OK(ace_fork_switch(RT_CTX));
  if (!n) {
    ACE_OK(ace_join(RT_CTX));
    return;
  }
  Flight.active = true;
  Flight.ctx    = RT_CTX;
  Flight.first = index, Flight.count = (uint32_t)n, Flight.scale = scale, Flight.level = level;
  Flight.k2 = ((uint64_t)ofst << 32) | (uint64_t)len;
}
/* before anything else uses the second stream, and before the kept plaintexts go away */
void Rt_plaintexts_settle(void) {
  Rt_shared_lock();
  flight_land();
  Rt_shared_unlock();
}

static bool encode_ahead(void* pt, uint32_t index, size_t ofst, size_t len, uint32_t scale, uint32_t level, size_t words) {
  if (ahead_count() < 2) return false;
  int64_t* base = NULL;
  size_t   n    = encode_run(index, ofst, len, scale, level, words, 2, &base);
  if (!n) return false;
  Rt_copy_words(Rt_plain_prepare((PLAIN)pt, scale, level), base, words);
  flight_start(index + (uint32_t)n, ofst, len, scale, level, words);
  return true;
}

/* The kept plaintexts and the synthetic entries are shared by the program's threads: one thread at a time looks
 * them up or adds to them, and a thread that has added polynomials waits for its stream before it lets go, because
 * the next thread copies them on a stream of its own. */
static void* from_msg_locked(void* pt, uint32_t index, size_t ofst, size_t len, uint32_t scale, uint32_t level, bool* added);
void* Pt_from_msg_ofst(void* pt, uint32_t index, size_t ofst, size_t len, uint32_t scale, uint32_t level) {
  bool added = false;
  Rt_shared_lock();
  from_msg_locked(pt, index, ofst, len, scale, level, &added);
  if (added) Rt_shared_publish();
  Rt_shared_unlock();
  return pt;
}
static void* from_msg_locked(void* pt, uint32_t index, size_t ofst, size_t len, uint32_t scale, uint32_t level, bool* added) {
  const size_t   words = (size_t)(level ? level : Get_q_cnt()) * Degree();
  const uint64_t k1    = cache_key1(index, scale, level);
  const uint64_t k2    = ((uint64_t)ofst << 32) | (uint64_t)len;
  PT_CELL*       cell  = NULL;
  if (Cache.limit_words && len > 1 && ofst < (1ull << 32) && len < (1ull << 32) && scale < 0x10000) {
    if (4 * (Cache.count + 1) > 3 * Cache.cap) cache_grow();
    cell = cache_find(k1, k2);
    if (cell->k1) { /* encoded before: the polynomial is copied */
      if (Flight.active && Flight.scale == scale && Flight.level == level && Flight.k2 == k2 && index >= Flight.first &&
          index - Flight.first < Flight.count) { /* ... once the run it belongs to has landed; the next run goes off */
        const uint32_t next = Flight.first + Flight.count;
        int64_t* const dev  = cell->dev;
        flight_land();
        flight_start(next, ofst, len, scale, level, words);
        *added = true;
        Rt_copy_words(Rt_plain_prepare((PLAIN)pt, scale, level), dev, words);
        return pt;
      }
      Rt_copy_words(Rt_plain_prepare((PLAIN)pt, scale, level), cell->dev, words);
      return pt;
    }
    if (Cache.words + words > Cache.limit_words) cell = NULL;
    if (cell && encode_ahead(pt, index, ofst, len, scale, level, words)) {
      *added = true;
      return pt;
    }
    if (cell) cell = cache_find(k1, k2); /* the table may have grown */
  }
  Pt_encode_entry(pt, index, ofst, len, scale, level);
  if (cell && (cell->dev = cache_room(words)) != NULL) {
    Rt_copy_words(cell->dev, ((PLAIN)pt)->_poly._data, words);
    cell->k1 = k1;
    cell->k2 = k2;
    ++Cache.count;
    Cache.words += words;
    *added = true;
  }
  return pt;
}
static void Pt_encode_entry(void* pt, uint32_t index, size_t ofst, size_t len, uint32_t scale, uint32_t level) {
  int         is_f32 = 0;
  const void* raw    = len > 1 ? entry_bytes(index, ofst, len, &is_f32) : NULL;
  if (raw) {
    Rt_encode_real((PLAIN)pt, raw, is_f32, len, scale, level);
    return;
  }
  double* v = entry_values(index, ofst, len);
  Encode_double((PLAIN)pt, v, len, scale, level);
  free(v);
}
void* Pt_from_msg(void* pt, uint32_t index, size_t len, uint32_t scale, uint32_t level) {
  return Pt_from_msg_ofst(pt, index, 0, len, scale, level);
}
void Pt_from_msg_ofst_validate(void* pt, float* buf, uint32_t index, size_t ofst, size_t len, uint32_t scale, uint32_t level) {
  Rt_shared_lock();
  double* v = entry_values(index, ofst, len);
  Rt_shared_unlock();
  for (size_t i = 0; i < len; ++i)
    FMT_ASSERT(fabs((double)buf[i] - v[i]) < 0.000001, "Pt_from_msg_validate failed. index=%u, i=%zu: %f != %f.", index, i,
               (double)buf[i], v[i]);
  Encode_double((PLAIN)pt, v, len, scale, level);
  free(v);
}
void Pt_from_msg_validate(void* pt, float* buf, uint32_t index, size_t len, uint32_t scale, uint32_t level) {
  Pt_from_msg_ofst_validate(pt, buf, index, 0, len, scale, level);
}
/* ---- files of pre-encoded plaintexts ------------------------------------------------------------------- */
static bool plaintext_file(void) { return Data.open && !Data.synthetic && Data.hdr.ent_type == DE_PLAINTEXT; }
static PLAINTEXT* load_plain_entry(uint32_t index) {
  FMT_ASSERT(plaintext_file(), "Pt_get: the program's rt data file does not hold pre-encoded plaintexts");
  FMT_ASSERT(index < Data.hdr.ent_count, "index out of entry range");
  if (Data.pt[index]) return Data.pt[index];
  const LUT_ENTRY* e = &Data.lut[index];
  FMT_ASSERT(e->ofst >= DATA_PAGE && e->ofst + e->size <= Data.hdr.lut_ofst, "entry offset too large");
  FMT_ASSERT(e->size >= 16 + sizeof(PLAINTEXT), "Plaintext buffer too small");
  char* raw = (char*)malloc(e->size);
  FMT_ASSERT(fseek(Data.file, (long)e->ofst, SEEK_SET) == 0 && fread(raw, 1, e->size, Data.file) == e->size,
             "failed to fill data from file");
  uint32_t version, size; /* Cast_buffer_to_plain (ckks/src/plain.c:262-292) */
  memcpy(&version, raw + 8, 4);
  memcpy(&size, raw + 12, 4);
  FMT_ASSERT(memcmp(raw, "ANTPLAIN", 8) == 0, "Plaintext buffer magic mismatch");
  FMT_ASSERT(version == RT_DATA_VERSION, "Plaintext buffer version mismatch");
  FMT_ASSERT((uint64_t)size + 16 <= e->size, "Plaintext buffer too small");
  PLAINTEXT* pt = (PLAINTEXT*)malloc(sizeof(PLAINTEXT));
  memcpy(pt, raw + 16, sizeof(PLAINTEXT));
  POLY poly = &pt->_poly;
  FMT_ASSERT(poly->_data == NULL, "Plaintext poly data is not NULL");
  size_t words = poly->_num_alloc_primes * (size_t)poly->_ring_degree;
  FMT_ASSERT(size == words * sizeof(int64_t) + sizeof(PLAINTEXT), "Plaintext size mismatch");
  FMT_ASSERT(poly->_ring_degree == Degree() && poly->_num_primes >= 1 && poly->_num_primes <= Get_q_cnt() &&
                 (poly->_num_primes_p == 0 || poly->_num_primes_p == Get_p_cnt()) &&
                 poly->_num_alloc_primes >= poly->_num_primes + poly->_num_primes_p,
             "plaintext %u does not fit this context (degree %u, %zu + %zu primes)", index, poly->_ring_degree,
             poly->_num_primes, poly->_num_primes_p);
  poly->_data = Rt_dev_alloc_raw(words);
  ACE_OK(ace_upload(RT_CTX, poly->_data, (const int64_t*)(raw + 16 + sizeof(PLAINTEXT)), words)); /* waits for the copy */
  free(raw);
  return Data.pt[index] = pt;
}
void* Pt_get(uint32_t index, size_t len, uint32_t scale, uint32_t level) {
  (void)len, (void)scale, (void)level; /* the entry carries its own shape, as in the reference */
  Rt_shared_lock(); /* the upload waits for the copy, so the entry is whole when the lock is released */
  PLAINTEXT* pt = load_plain_entry(index);
  Rt_shared_unlock();
  return pt;
}
void Pt_prefetch(uint32_t index) {
  Rt_shared_lock();
  if (plaintext_file() && index < Data.hdr.ent_count) (void)load_plain_entry(index);
  Rt_shared_unlock();
}
void Pt_free(uint32_t index) {
  Rt_shared_lock();
  FMT_ASSERT(plaintext_file() && index < Data.hdr.ent_count && Data.pt[index], "BLOCK_INFO state is not ready");
  Free_poly_data(&Data.pt[index]->_poly);
  free(Data.pt[index]);
  Data.pt[index] = NULL;
  Rt_shared_unlock();
}
void* Pt_get_validate(float* buf, uint32_t index, size_t len, uint32_t scale, uint32_t level) {
  (void)buf, (void)len, (void)scale, (void)level;
  Rt_fatal(__FILE__, __LINE__, "Pt_get_validate(%u): TODO: not implemented", index); /* pt_mgr.c:161-164 */
}
/* Free_data (pt_mgr.c:179-183): the polynomial of a plaintext made by Pt_from_msg; a plaintext of Pt_get
 * belongs to the manager and is left alone */
void Free_data(void* poly) {
  if (!plaintext_file()) Free_poly_data((POLY)poly);
}

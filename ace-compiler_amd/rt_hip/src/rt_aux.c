/* Host-side aids of the runtime that compiled programs can reach through rt_ant.h besides the polynomial and
 * ciphertext API: the plain-float models of the operators that the compiler's validation mode compares against
 * (rtlib/include/common/rt_validate.h, rtlib/common/src/rt_validate.c), the run-time switches
 * (include/common/rt_config.h, common/src/rt_config.c), the trace file (include/common/trace.h, common/src/trace.c),
 * the named ciphertext slots (include/common/io_api.h, common/src/io_lib.c) and the table of times per event
 * (include/common/rtlib_timing.h, common/linux/rtlib_timing.c).  Nothing here touches the GPU except the
 * synchronisation a time mark needs. */
#include <math.h>
#include <time.h>

#include "rt_internal.h"

/* ---- validation (rt_validate.c:15-263) ---------------------------------------------------------------------
 * The models work on NCHW tensors of doubles with float weights, accumulate in double in the reference's loop
 * order (so a run that matches the reference's bit for bit on finite data), and return malloc'ed results. */
void Validate_impl(double* res, double* msg, uint32_t len, int32_t epsilon) {
  const double bound = pow(10, epsilon);
  uint32_t     bad   = len;
  for (uint32_t i = 0; i < len && bad == len; ++i)
    if (fabs(res[i] - msg[i]) > bound) bad = i;
  if (bad != len) { /* the mismatch with eight neighbours on either side, as the reference prints it */
    fprintf(stderr, "ERROR: validation failed at %d. %f != %f\n", bad, res[bad], msg[bad]);
    const uint32_t from = bad > 8 ? bad - 8 : 0, to = from + 16 < len ? from + 16 : len;
    fprintf(stderr, "idx: ");
    for (uint32_t j = from; j < to; ++j) fprintf(stderr, "%7d%c ", j, j == bad ? '*' : ' ');
    fprintf(stderr, "\nres: ");
    for (uint32_t j = from; j < to; ++j) fprintf(stderr, "%8.4f ", res[j]);
    fprintf(stderr, "\nstd: ");
    for (uint32_t j = from; j < to; ++j) fprintf(stderr, "%8.4f ", msg[j]);
    fprintf(stderr, "\n");
  }
  fprintf(stdout, "%s: internal validation %s.\n", bad != len ? "ERROR" : "INFO", bad != len ? "fail" : "pass");
  fflush(stdout);
}

void Validate_value_range(bool within_range) {
  if (!within_range) fprintf(stdout, "Please set a higher level or increase the difference between q0 and sf.\n");
  fprintf(stdout, "%s: internal value range validation %s.\n", within_range ? "INFO" : "ERROR",
          within_range ? "pass" : "fail");
  fflush(stdout);
}

void Validate(CIPHER ciph, double* msg, uint32_t len, int32_t epsilon) { /* rt_validate.h:49-55 */
  double* res = Get_msg(ciph);
  Validate_impl(res, msg, len, epsilon);
  free(res);
  Validate_value_range(Within_value_range(ciph, msg, len));
}

static double* new_doubles(size_t n) { return (double*)malloc(sizeof(double) * (n ? n : 1)); }

double* Add_impl(double* a, double* b, uint32_t len) {
  double* r = new_doubles(len);
  for (uint32_t i = 0; i < len; ++i) r[i] = a[i] + b[i];
  return r;
}
double* Mul_impl(double* a, double* b, uint32_t len) {
  double* r = new_doubles(len);
  for (uint32_t i = 0; i < len; ++i) r[i] = a[i] * b[i];
  return r;
}
/* res[i] = op[(i + step) mod len] for -len <= step <= len */
double* Rotate_impl(double* op, uint32_t len, int32_t step) {
  double* r = new_doubles(len);
  for (int64_t i = 0; i < (int64_t)len; ++i) {
    int64_t from = i + step;
    if (from < 0) from += len;
    else if (from >= (int64_t)len) from -= len;
    r[i] = op[from];
  }
  return r;
}
double* Relu_impl(double* op, uint32_t len) {
  double* r  = new_doubles(len);
  double  lo = op[0], hi = op[0];
  for (uint32_t i = 0; i < len; ++i) {
    if (op[i] > hi) hi = op[i];
    if (op[i] < lo) lo = op[i];
    r[i] = op[i] < 0 ? 0 : op[i];
  }
  fprintf(stderr, "INFO: relu value range [%.4f, %.4f].\n", lo, hi);
  return r;
}

/* a copy of the tensor with ph rows and pw columns of zeros on every side of each plane */
static double* padded(const double* t, int planes, int h, int w, int ph, int pw) {
  const int H = h + 2 * ph, W = w + 2 * pw;
  const size_t total = (size_t)planes * H * W;
  double*      r     = (double*)calloc(total ? total : 1, sizeof(double));
  for (int p = 0; p < planes; ++p)
    for (int y = 0; y < h; ++y)
      memcpy(r + ((size_t)p * H + y + ph) * W + pw, t + ((size_t)p * h + y) * w, sizeof(double) * w);
  return r;
}

double* Conv_impl(double* in, int n, int c, int h, int w, float* weight, int kn, int kc, int kh, int kw, float* bias,
                  int bw, int sh, int sw, int pn, int pc, int ph, int pw) {
  (void)pn, (void)pc;
  IS_TRUE(kc == c, "channel mismatch");
  IS_TRUE(kn == bw, "bias length mismatch");
  const bool pad = ph != 0 || pw != 0;
  if (pad) {
    in = padded(in, n * c, h, w, ph, pw);
    h += 2 * ph;
    w += 2 * pw;
  }
  const int oh = (h - kh) / sh + 1, ow = (w - kw) / sw + 1;
  double*   out = new_doubles((size_t)n * kn * oh * ow);
  for (int img = 0; img < n; ++img)
    for (int f = 0; f < kn; ++f)
      for (int oy = 0; oy < oh; ++oy)
        for (int ox = 0; ox < ow; ++ox) {
          double acc = 0;
          for (int ch = 0; ch < kc; ++ch)
            for (int ky = 0; ky < kh; ++ky) {
              const int y = oy * sh + ky;
              if (y >= h) continue;
              for (int kx = 0; kx < kw; ++kx) {
                const int x = ox * sw + kx;
                if (x >= w) continue;
                const double a = in[(((size_t)img * c + ch) * h + y) * w + x];
                const double b = weight[(((size_t)f * kc + ch) * kh + ky) * kw + kx];
                acc += a * b;
              }
            }
          out[(((size_t)img * kn + f) * oh + oy) * ow + ox] = acc + bias[f];
        }
  if (pad) free(in);
  return out;
}

double* Gemm_impl(double* in, int h, int w, float* weight, int wh, int ww, float* bias, int bw) {
  IS_TRUE(h == 1, "height not 1?");
  IS_TRUE(w == ww, "weight width mismatch");
  IS_TRUE(wh == bw, "bias width mismatch");
  double* out = new_doubles((size_t)h * wh);
  for (int row = 0; row < h; ++row)
    for (int j = 0; j < wh; ++j) {
      double acc = 0;
      for (int k = 0; k < ww; ++k) acc += in[(size_t)row * ww + k] * weight[(size_t)j * ww + k];
      out[(size_t)row * wh + j] = acc;
    }
  for (int j = 0; j < bw; ++j) out[j] += bias[j];
  return out;
}

/* The reference's pooling model steps the window by its own size (the stride arguments only set the output
 * shape) and walks the output with the roles of width and height exchanged; both only matter for shapes that are
 * not square or whose stride differs from the window, and are kept so that the two models agree everywhere. */
double* Average_pool_impl(double* in, int n, int c, int h, int w, int kh, int kw, int sh, int sw, int pn, int pc,
                          int ph, int pw) {
  (void)pn, (void)pc;
  const bool pad = ph != 0 || pw != 0;
  if (pad) {
    in = padded(in, n * c, h, w, ph, pw);
    h += 2 * ph;
    w += 2 * pw;
  }
  const int    oh = (h - kh) / sh + 1, ow = (w - kw) / sw + 1;
  const double scale = 1.0 / (double)(kh * kw);
  double*      out   = new_doubles((size_t)n * c * oh * ow);
  for (int p = 0; p < n * c; ++p)
    for (int a = 0; a < ow; ++a)
      for (int b = 0; b < oh; ++b) {
        double sum = 0.0;
        for (int ky = 0; ky < kh; ++ky)
          for (int kx = 0; kx < kw; ++kx) sum += in[((size_t)p * h + a * kh + ky) * w + b * kw + kx];
        out[((size_t)p * oh + a) * ow + b] = sum * scale;
      }
  if (pad) free(in);
  return out;
}

double* Global_average_pool_impl(double* in, int n, int c, int h, int w) {
  const size_t plane = (size_t)h * w;
  const double scale = 1.0 / (double)(h * w);
  double*      out   = new_doubles((size_t)n * c);
  for (size_t p = 0; p < (size_t)n * c; ++p) {
    double acc = 0;
    for (size_t j = 0; j < plane; ++j) acc += in[p * plane + j];
    out[p] = acc * scale;
  }
  return out;
}

/* ---- run-time switches (rt_config.c:16-56): defaults, overridden from the environment once ----------------- */
static int64_t Config[CONF_LAST];
static bool    Config_ready;
void           Init_rtlib_config(void) {
  static const struct {
    RTLIB_CONFIG_ID id;
    int64_t         dflt;
    const char*     env;
  } all[] = {{CONF_OP_FUSION_DECOMP_MODUP, 1, "OP_FUSION_DECOMP_MODUP"},
             {CONF_BTS_CLEAR_IMAG, 0, "RT_BTS_CLEAR_IMAG"},
             {CONF_FAST_DOT_PROD, 0, "FAST_DOT_PROD"}};
  for (size_t i = 0; i < sizeof(all) / sizeof(all[0]); ++i) {
    const char* v      = getenv(all[i].env);
    Config[all[i].id] = v ? (atoi(v) != 0) : all[i].dflt;
  }
  Config_ready = true;
}
int64_t Get_rtlib_config(RTLIB_CONFIG_ID id) {
  if (!Config_ready) Init_rtlib_config();
  return Config[id];
}
void Set_rtlib_config(RTLIB_CONFIG_ID id, int64_t value) {
  if (!Config_ready) Init_rtlib_config();
  Config[id] = value;
}

/* ---- trace file (trace.c:16-60): RTLIB_TRACE_FILE names it ("stdout", "stderr" or a path; default fhe_trace.t) */
static FILE* Trace_file;
static bool  Trace_on;
void         Set_trace_file(char* filename) {
  if (Trace_file && Trace_file != stdout && Trace_file != stderr) fclose(Trace_file);
  Trace_file = filename ? fopen(filename, "w") : NULL;
}
FILE* Get_trace_file(void) {
  if (Trace_file) return Trace_file;
  const char* name = getenv("RTLIB_TRACE_FILE");
  if (name && !strcmp(name, "stdout")) return Trace_file = stdout;
  if (name && !strcmp(name, "stderr")) return Trace_file = stderr;
  Trace_file = fopen(name ? name : "fhe_trace.t", "w");
  if (!Trace_file) Trace_file = stderr;
  return Trace_file;
}
void Close_trace_file(void) {
  if (Trace_file && Trace_file != stdout && Trace_file != stderr) {
    fclose(Trace_file);
    Trace_file = NULL;
  }
}
void Set_trace_on(bool v) { Trace_on = v; }
bool Is_trace_on(void) { return Trace_on; }

/* ---- named ciphertext slots (io_lib.c:25-118): pointers are kept, not copies; Get_input_data / Set_output_data
 * and the harness entry points work on the same store ------------------------------------------------------- */
void Io_init(void) {}
void Io_fini(void) {
  IO_SLOT** tab[2] = {&LANE.in, &LANE.out};
  size_t*   cnt[2] = {&LANE.n_in, &LANE.n_out};
  for (int k = 0; k < 2; ++k) {
    for (size_t i = 0; i < *cnt[k]; ++i) free((*tab[k])[i].name);
    free(*tab[k]);
    *tab[k] = NULL;
    *cnt[k] = 0;
  }
}
static void* slot_get(IO_SLOT* s, size_t n, const char* name, size_t idx) {
  IO_SLOT* f = Rt_find_slot(s, n, name, idx);
  FMT_ASSERT(f, "fail to find %s.", name);
  return f->ct;
}
void Io_set_input(const char* name, size_t idx, void* ct) {
  IO_SLOT* s = Rt_find_slot(LANE.in, LANE.n_in, name, idx);
  if (!s) s = Rt_add_slot(&LANE.in, &LANE.n_in, name, idx);
  s->ct = (CIPHERTEXT*)ct;
}
void* Io_get_input(const char* name, size_t idx) { return slot_get(LANE.in, LANE.n_in, name, idx); }
void  Io_set_output(const char* name, size_t idx, void* ct) {
  IO_SLOT* s = Rt_find_slot(LANE.out, LANE.n_out, name, idx);
  if (!s) s = Rt_add_slot(&LANE.out, &LANE.n_out, name, idx);
  s->ct = (CIPHERTEXT*)ct;
}
void* Io_get_output(const char* name, size_t idx) { return slot_get(LANE.out, LANE.n_out, name, idx); }

/* ---- time per event (rtlib_timing.c:18-126) -------------------------------------------------------------------
 * Events are numbered as the compiler numbers them: its core, NN and FHE lists (air/base/rt_timing.h:20,
 * nn/core/rt_timing.h:22-32, fhe/core/rt_timing.h:22-32) followed by the library's own
 * (include/common/rtlib_timing.h:45-102).  The table goes to the file RTLIB_TIMING_OUTPUT names ("stdout", "-",
 * "stderr" or a path); without that variable no mark records anything or waits.  The GPU works asynchronously, so
 * a recording mark first waits for the device: an event's time then covers its work. */
static const struct {
  const char* name;
  int         level;
} Rtm_events[] = {
#define X(NAME, LEVEL) {#NAME, LEVEL},
    RT_RTM_EVENTS(X)
#undef X
};
#define RTM_COUNT (sizeof(Rtm_events) / sizeof(Rtm_events[0]))
/* per thread, as in the reference's OpenMP build (include/common/rtlib_timing.h:123-126): the table that
 * Report_rtlib_timing prints is the calling thread's */
static __thread uint64_t       Rtm_nsec[RTM_COUNT], Rtm_sub_nsec[RTM_COUNT], Rtm_calls[RTM_COUNT];
__thread struct RTM_INFO_STACK Rtm_stack = {{{0, 0, 0, 0, 0}}, 0, RTLIB_TIMING_MAX_LEVEL};
static int            Rtm_enabled = -1;

static bool rtm_on(void) {
  if (Rtm_enabled < 0) Rtm_enabled = getenv("RTLIB_TIMING_OUTPUT") != NULL;
  return Rtm_enabled;
}
void Init_rtlib_timing(void) {
  memset(Rtm_nsec, 0, sizeof(Rtm_nsec));
  memset(Rtm_sub_nsec, 0, sizeof(Rtm_sub_nsec));
  memset(Rtm_calls, 0, sizeof(Rtm_calls));
  Rtm_stack._size = 0;
  Rtm_enabled     = -1;
}
void Append_rtlib_timing(uint32_t event, uint32_t id, uint64_t nsec, uint64_t sub_nsec) {
  (void)id;
  FMT_ASSERT(event < RTM_COUNT, "unknown timed event %u", event);
  Rtm_nsec[event] += nsec;
  Rtm_sub_nsec[event] += sub_nsec;
  Rtm_calls[event]++;
}
void Mark_rtm_start(uint32_t event, uint32_t id) {
  if (!rtm_on()) return;
  IS_TRUE(Rtm_stack._size < Rtm_stack._max_size, "FATAL: RTM stack overflow");
  if (G.root) (void)ace_sync(RT_CTX);
  struct RTM_INFO* info = &Rtm_stack._info[Rtm_stack._size++];
  struct timespec  ts;
  clock_gettime(CLOCK_REALTIME, &ts);
  *info = (struct RTM_INFO){event, id, (uint32_t)ts.tv_sec, (uint32_t)ts.tv_nsec, 0};
}
void Mark_rtm_end(uint32_t event, uint64_t id) {
  if (!rtm_on()) return;
  if (G.root) (void)ace_sync(RT_CTX);
  struct timespec ts;
  clock_gettime(CLOCK_REALTIME, &ts);
  IS_TRUE(Rtm_stack._size > 0, "FATAL: RTM stack underflow");
  struct RTM_INFO* info = &Rtm_stack._info[--Rtm_stack._size];
  IS_TRUE(info->_event == event && info->_id == id, "FATAL: RTM stack mismatch");
  const uint64_t nsec = (uint64_t)(((int64_t)(uint32_t)ts.tv_sec - (int64_t)info->_sec) * 1000000000 + ts.tv_nsec - info->_nsec);
  /* a nested NN operator or bootstrap is also charged to the event around it, which reports it apart */
  if (Rtm_stack._size > 1 && ((event >= RTM_NN && event <= RTM_NN_RELU) || event == RTM_FHE_BOOTSTRAP))
    Rtm_stack._info[Rtm_stack._size - 1]._sub_nsec += nsec;
  Append_rtlib_timing(event, (uint32_t)id, nsec, info->_sub_nsec);
}
/* One line per event that ran, indented by its level, in the order of the lists; a group's sub total (the time of
 * its members less what they report as nested) follows the group. */
void Report_rtlib_timing(void) {
  const char* fname = getenv("RTLIB_TIMING_OUTPUT");
  if (!fname) return;
  FILE* fp = !strcmp(fname, "stdout") || !strcmp(fname, "-") ? stdout : !strcmp(fname, "stderr") ? stderr : fopen(fname, "w");
  if (!fp) return;
  fprintf(fp, "%-24s\t%12s\t%12s\n", "RTLib functions", "Count", "Elapse");
  fprintf(fp, "%-24s\t%12s\t%12s\n", "--------------------", "--------", "--------");
  uint64_t sum[RTLIB_TIMING_MAX_LEVEL] = {0};
  size_t   head[RTLIB_TIMING_MAX_LEVEL] = {0};
  int      depth = 0;
  for (size_t i = 0; i <= RTM_COUNT; ++i) {
    const bool last  = i == RTM_COUNT;
    const bool group = !last && i + 1 < RTM_COUNT && Rtm_events[i].level < Rtm_events[i + 1].level;
    if (!last && !Rtm_calls[i] && !group) continue;
    const int level = last ? 0 : Rtm_events[i].level;
    for (; depth > level; --depth) {
      fprintf(fp, "%*s%-24s\t%12s\t%12.6f sec\n", depth - 1, "", Rtm_events[head[depth - 1]].name, "sub total",
              (double)sum[depth] * 1e-9);
      sum[depth] = 0;
    }
    if (last) break;
    sum[level] += Rtm_nsec[i] - Rtm_sub_nsec[i];
    head[level] = i;
    const double all = (double)Rtm_nsec[i] * 1e-9, sub = (double)Rtm_sub_nsec[i] * 1e-9;
    if (!Rtm_calls[i]) fprintf(fp, "%*s%-24s\t%12c\t%12c\n", level, "", Rtm_events[i].name, '-', '-');
    else if (sub > 0) fprintf(fp, "%*s%-24s\t%12lu\t%12.6f sec (%.6f - %.6f)\n", level, "", Rtm_events[i].name, (unsigned long)Rtm_calls[i], all - sub, all, sub);
    else fprintf(fp, "%*s%-24s\t%12lu\t%12.6f sec\n", level, "", Rtm_events[i].name, (unsigned long)Rtm_calls[i], all);
    depth = level;
  }
  if (fp != stdout && fp != stderr) fclose(fp);
}

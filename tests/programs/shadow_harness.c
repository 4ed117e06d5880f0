/* The plain-float run of a compiled model: the generated program, included unchanged over the stand-in runtime of
 * tests/programs/shadow/rt_ant/rt_ant.h, with the image and the pseudo-random weights model_harness.c gives the GPU
 * run (same seed, same amplitude).  Host only.
 *
 * usage: <model>_shadow <channels> <height> <width> <outputs to print> <seed> [images]
 * prints one "output: v0 v1 ..." line per image, as model_harness does. */
#include "rt_ant/rt_ant.h"

uint32_t Shadow_slots, Shadow_top_level;
double   Shadow_amplitude;
MODULUS  Shadow_moduli[128];

/* rotation tables, one per step, kept */
static struct { int32_t step; int64_t* order; } Orders[512];
static int N_orders;
int64_t* Auto_order(int32_t rot_idx) {
  for (int i = 0; i < N_orders; ++i)
    if (Orders[i].step == rot_idx) return Orders[i].order;
  if (N_orders == 512) abort();
  int64_t* o = (int64_t*)malloc(Shadow_slots * sizeof(int64_t));
  for (uint32_t i = 0; i < Shadow_slots; ++i) /* slot i of the result is slot i + step of the operand */
    o[i] = (int64_t)(((int64_t)i + rot_idx) % (int64_t)Shadow_slots + Shadow_slots) % Shadow_slots;
  Orders[N_orders].step  = rot_idx;
  Orders[N_orders].order = o;
  ++N_orders;
  return o;
}

static void Fill(PLAIN plain, const double* v, size_t len, uint32_t sc_degree, uint32_t level) {
  if (!plain->_poly._data) Alloc_poly_data(&plain->_poly, Shadow_slots, 1, 0);
  double* d = Sh(plain->_poly._data);
  if (len == 1) {
    for (uint32_t i = 0; i < Shadow_slots; ++i) d[i] = v[0]; /* a single value is a constant polynomial */
  } else {
    if (len > Shadow_slots) abort();
    memcpy(d, v, len * sizeof(double));
    memset(d + len, 0, (Shadow_slots - len) * sizeof(double));
  }
  plain->_level     = level ? level : Shadow_top_level;
  plain->_sc_degree = sc_degree;
}
void Encode_double(PLAIN plain, double* input, size_t len, uint32_t sc_degree, uint32_t level) {
  Fill(plain, input, len, sc_degree, level);
}
void Encode_float(PLAIN plain, float* input, size_t len, uint32_t sc_degree, uint32_t level) {
  double* v = (double*)malloc(len * sizeof(double));
  for (size_t i = 0; i < len; ++i) v[i] = (double)input[i];
  Fill(plain, v, len, sc_degree, level);
  free(v);
}
/* value i of weight entry `index` when the weight file is replaced by pseudo-random values of the given amplitude */
static double Synthetic(uint32_t index, size_t i) {
  uint64_t z = ((uint64_t)index << 32 | (uint64_t)i) + 0x9E3779B97F4A7C15ull;
  z          = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z          = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  return Shadow_amplitude * ((double)(int64_t)(z >> 11) / (double)(1ull << 52) - 1.0);
}
void* Pt_from_msg(void* pt, uint32_t index, size_t len, uint32_t scale, uint32_t level) {
  double* v = (double*)malloc(len * sizeof(double));
  for (size_t i = 0; i < len; ++i) v[i] = Synthetic(index, i);
  Fill((PLAIN)pt, v, len, scale, level);
  free(v);
  return pt;
}

static CIPHERTEXT Input, Output;
CIPHERTEXT Get_input_data(const char* name, size_t idx) {
  (void)name, (void)idx;
  CIPHERTEXT c;
  memset(&c, 0, sizeof(c));
  Copy_ciph(&c, &Input);
  return c;
}
void Set_output_data(const char* name, size_t idx, CIPHER data) {
  (void)name, (void)idx;
  Copy_ciph(&Output, data);
  Free_poly_data(&data->_c0_poly), Free_poly_data(&data->_c1_poly);
}

static double Unit(uint64_t* state) { /* in [-1, 1) */
  *state = *state * 6364136223846793005ull + 1442695040888963407ull;
  return (double)(int64_t)(*state >> 11) / (double)(1ull << 52) - 1.0;
}
static uint64_t Image_state(uint64_t seed, int img) { return (seed * 31 + 7) ^ ((uint64_t)img * 0x9E3779B97F4A7C15ull); }

int main(int argc, char** argv) {
  if (argc != 6 && argc != 7) {
    fprintf(stderr, "usage: %s <channels> <height> <width> <outputs to print> <seed> [images]\n", argv[0]);
    return 2;
  }
  size_t   c = strtoul(argv[1], NULL, 0), h = strtoul(argv[2], NULL, 0), w = strtoul(argv[3], NULL, 0);
  int      show = atoi(argv[4]), images = argc == 7 ? atoi(argv[6]) : 1;
  uint64_t seed = strtoull(argv[5], NULL, 0);
  Shadow_slots     = Get_context_params()->_poly_degree / 2;
  Shadow_top_level = (uint32_t)Get_context_params()->_mul_depth + 1;
  Shadow_amplitude = getenv("RT_HIP_SYNTHETIC_WEIGHTS") ? atof(getenv("RT_HIP_SYNTHETIC_WEIGHTS")) : 0.0;
  if (!(Shadow_amplitude > 0) || c * h * w > Shadow_slots) {
    fprintf(stderr, "RT_HIP_SYNTHETIC_WEIGHTS=<amplitude> is required, and the image must fit the slots\n");
    return 2;
  }
  for (int img = 0; img < images; ++img) {
    uint64_t st = Image_state(seed, img);
    memset(&Input, 0, sizeof(Input));
    Alloc_poly_data(&Input._c0_poly, Shadow_slots, 1, 0);
    Alloc_poly_data(&Input._c1_poly, Shadow_slots, 1, 0);
    for (size_t i = 0; i < c * h * w; ++i) Sh(Input._c0_poly._data)[i] = 0.5 * Unit(&st); /* the NORMAL scheme: in order */
    Input._level     = Get_context_params()->_input_level ? (uint32_t)Get_context_params()->_input_level : Shadow_top_level;
    Input._sc_degree = 1;
    memset(&Output, 0, sizeof(Output));
    if (!Main_graph()) return 1;
    printf("output:");
    for (int i = 0; i < show; ++i) printf(" %.6f", Sh(Output._c0_poly._data)[i]);
    printf("\n");
    Free_poly_data(&Input._c0_poly), Free_poly_data(&Input._c1_poly);
    Free_poly_data(&Output._c0_poly), Free_poly_data(&Output._c1_poly);
  }
  return 0;
}

#include MODEL_INC

/* An end-to-end program in the shape the FHE compiler emits for a small network:
 * the harness side (main) prepares the context, generates keys, encrypts the input
 * tensor, runs Main_graph, decrypts and decodes the output; Main_graph evaluates
 *
 *     y = (W x + b)^2        (a Gemm layer by diagonals followed by a square)
 *
 * on ciphertexts with plaintext weights encoded in the program, as generated code
 * does for constants it embeds (cf. the Gemm bodies in
 * rtlib/ant/dataset/resnet20_cifar10_pre.onnx.inc and the harness in
 * rtlib/ant/ckks/src/rtlib.c:66-229, rtlib/include/common/rt_api.h:48-80).
 *
 * Also runs the reference's encode test (rtlib/ant/test/test_ant_encode.c:16-37):
 * Encode_float of four values, Get_msg_from_plain within 1e-7.
 *
 * usage: gemm_program <poly degree> <dim> <seed>
 * prints one line "max_err <e> encode_err <e>" and exits 0 when both are within bounds.
 */
#include <math.h>

#include "rt_ant/rt_ant.h"

#define MAX_DIM 64
static struct {
  CKKS_PARAMS p;
  int32_t     rot[MAX_DIM];
} Params = {.p = {._provider         = LIB_ANT,
                  ._poly_degree      = 4096,
                  ._sec_level        = 0,
                  ._mul_depth        = 3,
                  ._input_level      = 0,
                  ._first_mod_size   = 60,
                  ._scaling_mod_size = 50,
                  ._num_q_parts      = 2,
                  ._hamming_weight   = 192,
                  ._num_rot_idx      = 0}};
static int   Dim;
static float Weight[MAX_DIM][MAX_DIM], Bias[MAX_DIM];

static MAP_DESC    Desc_in  = {NORMAL, 0, 0, 0, 0};
static MAP_DESC    Desc_out = {NORMAL, 0, 0, 0, 0};
static DATA_SCHEME Scheme_in  = {"input", {0, 0, 0, 0}, 1, &Desc_in};
static DATA_SCHEME Scheme_out = {"output", {0, 0, 0, 0}, 1, &Desc_out};

CKKS_PARAMS* Get_context_params(void) { return &Params.p; }
int          Get_input_count(void) { return 1; }
int          Get_output_count(void) { return 1; }
DATA_SCHEME* Get_encode_scheme(int idx) { return idx == 0 ? &Scheme_in : NULL; }
DATA_SCHEME* Get_decode_scheme(int idx) { return idx == 0 ? &Scheme_out : NULL; }

bool Main_graph(void) {
  CIPHERTEXT input = Get_input_data("input", 0);
  CIPHERTEXT dup, rot, term, acc, gemm, sq, out;
  PLAINTEXT  pt;
  memset(&dup, 0, sizeof(dup));
  memset(&rot, 0, sizeof(rot));
  memset(&term, 0, sizeof(term));
  memset(&acc, 0, sizeof(acc));
  memset(&gemm, 0, sizeof(gemm));
  memset(&sq, 0, sizeof(sq));
  memset(&out, 0, sizeof(out));
  memset(&pt, 0, sizeof(pt));

  /* the input sits in slots 0..Dim-1; a second copy in Dim..2Dim-1 makes rotations by i < Dim cyclic */
  Rotate_ciph(&dup, &input, -Dim);
  Add_ciph(&dup, &dup, &input);

  float diag[MAX_DIM];
  for (int i = 0; i < Dim; ++i) {
    for (int j = 0; j < Dim; ++j) diag[j] = Weight[j][(j + i) % Dim];
    Encode_float(&pt, diag, (size_t)Dim, 1, (uint32_t)Level(&dup));
    CIPHER src = &dup;
    if (i) src = Rotate_ciph(&rot, &dup, i);
    if (i == 0) {
      Mul_plain(&acc, src, &pt);
    } else {
      Mul_plain(&term, src, &pt);
      Add_ciph(&acc, &acc, &term);
    }
  }
  Rescale_ciph(&gemm, &acc);
  Encode_float(&pt, Bias, (size_t)Dim, 1, (uint32_t)Level(&gemm));
  Add_plain(&gemm, &gemm, &pt);

  Mul_ciph(&sq, &gemm, &gemm);
  Rescale_ciph(&out, &sq);
  Set_output_data("output", 0, &out);

  Free_plain_poly(&pt);
  Free_ciph_poly(&input, 1);
  Free_ciph_poly(&dup, 1);
  Free_ciph_poly(&rot, 1);
  Free_ciph_poly(&term, 1);
  Free_ciph_poly(&acc, 1);
  Free_ciph_poly(&gemm, 1);
  Free_ciph_poly(&sq, 1);
  return true;
}

static double Unit(uint64_t* state) { /* in [-1, 1) */
  *state = *state * 6364136223846793005ull + 1442695040888963407ull;
  return (double)(int64_t)(*state >> 11) / (double)(1ull << 52) - 1.0;
}

int main(int argc, char** argv) {
  if (argc != 4) {
    fprintf(stderr, "usage: %s <poly degree> <dim> <seed>\n", argv[0]);
    return 2;
  }
  Params.p._poly_degree = (uint32_t)strtoul(argv[1], NULL, 0);
  Dim                   = atoi(argv[2]);
  uint64_t seed         = strtoull(argv[3], NULL, 0);
  if (Dim < 2 || Dim > MAX_DIM || (size_t)2 * Dim > Params.p._poly_degree / 2) {
    fprintf(stderr, "dim out of range\n");
    return 2;
  }
  Params.p._num_rot_idx = (size_t)Dim;
  Params.rot[0]         = -Dim;
  for (int i = 1; i < Dim; ++i) Params.rot[i] = i;
  Scheme_out._shape = (SHAPE){1, 1, 1, (size_t)Dim};

  uint64_t st = seed;
  double   x[MAX_DIM], expect[MAX_DIM];
  for (int i = 0; i < Dim; ++i) {
    for (int j = 0; j < Dim; ++j) Weight[i][j] = (float)(Unit(&st) / sqrt((double)Dim));
    Bias[i] = (float)(0.5 * Unit(&st));
    x[i]    = Unit(&st);
  }
  for (int i = 0; i < Dim; ++i) {
    double s = Bias[i];
    for (int j = 0; j < Dim; ++j) s += (double)Weight[i][j] * x[j];
    expect[i] = s * s;
  }

  Prepare_context();
  Rt_generate_keys(seed);

  /* the reference's encode test */
  float     probe[] = {1.0380784273147583f, -3.1710917949676514f, -0.024826018139719963f, 0.6483810544013977f};
  PLAINTEXT ppt;
  memset(&ppt, 0, sizeof(ppt));
  Encode_float(&ppt, probe, 4, 1, 0);
  double* msg        = Get_msg_from_plain(&ppt);
  double  encode_err = 0;
  for (int i = 0; i < 4; ++i) encode_err = fmax(encode_err, fabs(msg[i] - (double)probe[i]));
  free(msg);
  Free_plain_poly(&ppt);

  TENSOR* in = Alloc_tensor(1, 1, 1, (size_t)Dim, x);
  Prepare_input(in, "input");
  Run_main_graph();
  double* y       = Handle_output("output");
  double  max_err = 0;
  for (int i = 0; i < Dim; ++i) max_err = fmax(max_err, fabs(y[i] - expect[i]));
  printf("max_err %.3e encode_err %.3e\n", max_err, encode_err);
  free(y);
  Free_tensor(in);
  Finalize_context();
  return (max_err < 1e-3 && encode_err < 1e-7) ? 0 : 1;
}

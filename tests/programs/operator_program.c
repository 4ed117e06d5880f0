/* One block of a compiled model at the model's own size, with weights this program knows: a 3x3 convolution laid
 * out the way the compiler lays out ResNet-20's first one (rtlib/ant/dataset/resnet20_cifar10_pre.onnx.inc:
 * 1445-1572: the input's 4096 values repeated over 16384 slots by three rotations, nine rolled copies for the
 * taps, one sum of plaintext products per channel diagonal with the plaintexts read by Pt_from_msg from the weight
 * side-file, the sum's copy into the other half of the slots, the diagonal's rotation by a multiple of 1024, the
 * bias, a rescale), then Bootstrap to level 15 and the compiler's own polynomial ReLU (lines 1577-1597: x and
 * x / 4 into App_relu).  The generated program is included as it is for its Rotate, Relinearize and App_relu and for
 * its parameters (ring degree 65536, depth 33, 197 rotation indices); its Main_graph is not called.  The weights are
 * written by this program into a side-file of the reference's message format before Prepare_context reads it, so
 * the expected values are known: the plain-float operator models of the validation mode (Conv_impl, Relu_impl:
 * rt_validate.c:143-222) give them.
 *
 * usage: operator_block <side-file to write> <seed> [amplitude of the weights, default 0.33]
 * prints "conv_err <e> bootstrap_err <e> relu_err <e> relu_err_away_from_zero <e> level <l> ..." and exits 0 when
 * every error is below its bound (the bounds are in the checks at the end).
 */
#define _GNU_SOURCE
#include <math.h>
#include <time.h>

#include "common/rtlib.h"

#include MODEL_INC

#define SLOTS 32768
#define HALF 16384
#define CH 4 /* channels in and out; the compiler pads ResNet-20's three input channels to four the same way */
#define HW 32
#define PLANE (HW * HW)

static double Unit(uint64_t* state) { /* in [-1, 1) */
  *state = *state * 6364136223846793005ull + 1442695040888963407ull;
  return (double)(int64_t)(*state >> 11) / (double)(1ull << 52) - 1.0;
}
static double Now_ms(void) {
  struct timespec t;
  clock_gettime(CLOCK_MONOTONIC, &t);
  return t.tv_sec * 1e3 + t.tv_nsec * 1e-6;
}

static const int Tap[9] = {-33, -32, -31, -1, 0, 1, 31, 32, 33}; /* dy * 32 + dx, the order of the program's _cst_61 */

/* ---- the side-file (fhe-cmplr/include/fhe/core/rt_data_def.h:62-84): header, entries from 4096 on, lookup table ---- */
typedef struct {
  char            magic[8];
  uint32_t        rt_ver;
  uint16_t        flag;
  uint8_t         ent_type, ent_align;
  uint64_t        ent_count, lut_ofst;
  struct timespec ctime;
  char            model[48], uuid[40];
} FILE_HDR;
typedef struct {
  char     name[16];
  uint32_t index, size;
  uint64_t scale : 8, level : 8, ofst : 48;
} FILE_LUT;

static void Write_side_file(const char* path, float (*entry)[HALF], uint32_t count) {
  FILE* f = fopen(path, "wb");
  if (!f) {
    perror(path);
    exit(2);
  }
  FILE_HDR h;
  memset(&h, 0, sizeof(h));
  memcpy(h.magic, "!ANTFHE\0", 8);
  h.rt_ver    = 1;
  h.ent_type  = DE_MSG_F32;
  h.ent_align = 5;
  h.ent_count = count;
  h.lut_ofst  = 4096 + (uint64_t)count * HALF * sizeof(float);
  snprintf(h.model, sizeof(h.model), "operator block");
  snprintf(h.uuid, sizeof(h.uuid), "%s", Get_rt_data_info()->_file_uuid);
  char page[4096];
  memset(page, 0, sizeof(page));
  memcpy(page, &h, sizeof(h));
  fwrite(page, 1, sizeof(page), f);
  fwrite(entry, sizeof(float) * HALF, count, f);
  for (uint32_t i = 0; i < count; ++i) {
    FILE_LUT e;
    memset(&e, 0, sizeof(e));
    snprintf(e.name, sizeof(e.name), "cst_%u", i);
    e.index = i;
    e.size  = HALF * sizeof(float);
    e.ofst  = 4096 + (uint64_t)i * HALF * sizeof(float);
    fwrite(&e, sizeof(e), 1, f);
  }
  fclose(f);
}

/* ---- ciphertext sums and plaintext products, limb by limb, as the compiler writes them ---- */
static void Add_into(CIPHERTEXT* res, CIPHERTEXT* a, CIPHERTEXT* b) {
  uint32_t degree = Degree();
  Init_ciph_same_scale(res, a, b);
  MODULUS* m = Q_modulus();
  uint32_t n = Poly_level(&res->_c0_poly);
  for (uint32_t i = 0; i < n; ++i, ++m) {
    Hw_modadd(Coeffs(&res->_c0_poly, i, degree), Coeffs(&a->_c0_poly, i, degree), Coeffs(&b->_c0_poly, i, degree), m, degree);
    Hw_modadd(Coeffs(&res->_c1_poly, i, degree), Coeffs(&a->_c1_poly, i, degree), Coeffs(&b->_c1_poly, i, degree), m, degree);
  }
}
static void Free_ct(CIPHERTEXT* c) {
  Free_poly_data(&c->_c1_poly);
  Free_poly_data(&c->_c0_poly);
}
static double* Decrypted(CIPHERTEXT* c) {
  PLAINTEXT p;
  memset(&p, 0, sizeof(p));
  Rt_decrypt(&p, c);
  double* v = Get_msg_from_plain(&p);
  Free_poly_data(&p._poly);
  return v;
}
/* largest difference over the slots that hold the block's result: slot (co, y, x) of every copy of the four planes */
static double Worst(const double* got, const double* want, const double* weight_by, double at_least) {
  double worst = 0;
  for (int s = 0; s < HALF; ++s) {
    if (weight_by && fabs(weight_by[s % (CH * PLANE)]) < at_least) continue;
    worst = fmax(worst, fabs(got[s] - want[s % (CH * PLANE)]));
  }
  return worst;
}

int main(int argc, char** argv) {
  if (argc != 3 && argc != 4) {
    fprintf(stderr, "usage: %s <side-file to write> <seed> [weight amplitude]\n", argv[0]);
    return 2;
  }
  uint64_t seed = strtoull(argv[2], NULL, 0), st = seed * 1000003 + 17;
  double   amp  = argc == 4 ? atof(argv[3]) : 0.33;

  /* weights, bias, image */
  static float weight[CH][CH][3][3], bias[CH];
  static double image[CH * PLANE];
  for (int o = 0; o < CH; ++o)
    for (int i = 0; i < CH; ++i)
      for (int t = 0; t < 9; ++t) weight[o][i][t / 3][t % 3] = (float)(amp * Unit(&st));
  for (int o = 0; o < CH; ++o) bias[o] = (float)(0.1 * Unit(&st));
  for (int i = 0; i < CH * PLANE; ++i) image[i] = 0.5 * Unit(&st);

  /* the side-file: entry d * 9 + t is the plaintext of diagonal d and tap t (slot (c, y, x) of each of the four
   * copies: the weight from input channel c to output channel c - d, zero where the tap leaves the plane), entry 36
   * the bias */
  static float entry[CH * 9 + 1][HALF];
  for (int d = 0; d < CH; ++d)
    for (int t = 0; t < 9; ++t) {
      int dy = t / 3 - 1, dx = t % 3 - 1;
      for (int s = 0; s < HALF; ++s) {
        int c = (s / PLANE) % CH, y = (s % PLANE) / HW, x = s % HW;
        bool inside = y + dy >= 0 && y + dy < HW && x + dx >= 0 && x + dx < HW;
        entry[d * 9 + t][s] = inside ? weight[(c - d + CH) % CH][c][t / 3][t % 3] : 0.0f;
      }
    }
  for (int s = 0; s < HALF; ++s) entry[CH * 9][s] = bias[(s / PLANE) % CH];
  Write_side_file(argv[1], entry, CH * 9 + 1);
  Get_rt_data_info()->_file_name  = argv[1];
  Get_context_params()->_first_mod_size   = 60; /* the chain the reference builds its models with */
  Get_context_params()->_scaling_mod_size = 56; /* (scripts/build_resnet20_cifar10.sh:13-14,32) */

  Prepare_context();
  Rt_generate_keys(seed);
  Rt_sync();
  uint32_t degree = Degree();

  /* expected values: the validation mode's float models */
  double* want_conv = Conv_impl(image, 1, CH, HW, HW, &weight[0][0][0][0], CH, CH, 3, 3, bias, CH, 1, 1, 0, 0, 1, 1);
  double* want_relu = Relu_impl(want_conv, CH * PLANE);

  /* the image in the first 4096 of 32768 slots at level 3: the products use one level, the bootstrap starts from 2 */
  double* slots = (double*)calloc(SLOTS, sizeof(double));
  memcpy(slots, image, sizeof(image));
  PLAINTEXT  pt;
  CIPHERTEXT input;
  memset(&pt, 0, sizeof(pt));
  memset(&input, 0, sizeof(input));
  Encode_double(&pt, slots, SLOTS, 1, 3);
  Encrypt(&input, &pt);
  Free_poly_data(&pt._poly);
  free(slots);

  double t0 = Now_ms();
  /* ---- the convolution ---- */
  CIPHERTEXT r1 = Rotate(input, -4096), r2 = Rotate(input, -8192), r3 = Rotate(input, -12288), s1, s2, dup;
  memset(&s1, 0, sizeof(s1)), memset(&s2, 0, sizeof(s2)), memset(&dup, 0, sizeof(dup));
  Add_into(&s1, &input, &r1);
  Add_into(&s2, &s1, &r2);
  Add_into(&dup, &s2, &r3);
  Free_ct(&r1), Free_ct(&r2), Free_ct(&r3), Free_ct(&s1), Free_ct(&s2), Free_ct(&input);
  CIPHERTEXT roll[9];
  memset(roll, 0, sizeof(roll));
  for (int t = 0; t < 9; ++t) {
    CIPHERTEXT r = Rotate(dup, Tap[t]);
    Copy_ciph(&roll[t], &r);
    Free_ct(&r);
  }
  Free_ct(&dup);
  CIPHERTEXT result, diag, prod, both;
  PLAINTEXT  w;
  memset(&result, 0, sizeof(result)), memset(&prod, 0, sizeof(prod)), memset(&both, 0, sizeof(both)), memset(&w, 0, sizeof(w));
  for (int d = 0; d < CH; ++d) {
    memset(&diag, 0, sizeof(diag));
    for (int t = 0; t < 9; ++t) {
      Pt_from_msg(&w, (uint32_t)(t + d * 9), HALF, Sc_degree(&roll[t]), Level(&roll[t]));
      Init_ciph_up_scale_plain(&prod, &roll[t], &w);
      Init_ciph_same_scale(&diag, &diag, &prod);
      MODULUS* m = Q_modulus();
      uint32_t n = Poly_level(&diag._c0_poly);
      for (uint32_t i = 0; i < n; ++i, ++m) {
        Hw_modmul(Coeffs(&prod._c0_poly, i, degree), Coeffs(&roll[t]._c0_poly, i, degree), Coeffs(&w._poly, i, degree), m, degree);
        Hw_modmul(Coeffs(&prod._c1_poly, i, degree), Coeffs(&roll[t]._c1_poly, i, degree), Coeffs(&w._poly, i, degree), m, degree);
        Hw_modadd(Coeffs(&diag._c0_poly, i, degree), Coeffs(&diag._c0_poly, i, degree), Coeffs(&prod._c0_poly, i, degree), m, degree);
        Hw_modadd(Coeffs(&diag._c1_poly, i, degree), Coeffs(&diag._c1_poly, i, degree), Coeffs(&prod._c1_poly, i, degree), m, degree);
      }
    }
    CIPHERTEXT other = Rotate(diag, -HALF);
    Add_into(&both, &diag, &other);
    CIPHERTEXT turned = Rotate(both, d * PLANE);
    Add_into(&result, &result, &turned);
    Free_ct(&other), Free_ct(&turned), Free_ct(&diag);
  }
  Free_ciph_poly(roll, 9);
  Free_ct(&prod), Free_ct(&both);
  Free_poly_data(&w._poly);
  /* the bias at the products' scale, then one rescale */
  PLAINTEXT b;
  memset(&b, 0, sizeof(b));
  Pt_from_msg(&b, CH * 9, HALF, Sc_degree(&result), Level(&result));
  Init_ciph_same_scale_plain(&result, &result, &b);
  {
    MODULUS* m = Q_modulus();
    uint32_t n = Poly_level(&result._c0_poly);
    for (uint32_t i = 0; i < n; ++i, ++m)
      Hw_modadd(Coeffs(&result._c0_poly, i, degree), Coeffs(&result._c0_poly, i, degree), Coeffs(&b._poly, i, degree), m, degree);
  }
  Free_poly_data(&b._poly);
  CIPHERTEXT conv;
  memset(&conv, 0, sizeof(conv));
  Init_ciph_down_scale(&conv, &result);
  Rescale(&conv._c0_poly, &result._c0_poly);
  Rescale(&conv._c1_poly, &result._c1_poly);
  Free_ct(&result);
  Rt_sync();
  double  t1       = Now_ms();
  double* got_conv = Decrypted(&conv);

  /* ---- bootstrap to level 15, as the program asks for it ---- */
  double     t2 = Now_ms();
  CIPHERTEXT fresh;
  memset(&fresh, 0, sizeof(fresh));
  Bootstrap(&fresh, &conv, 15);
  Rt_sync();
  double t3 = Now_ms();
  Free_ct(&conv);
  double*  got_fresh = Decrypted(&fresh);
  uint32_t level     = Level(&fresh);

  /* ---- the compiler's ReLU on (x, x / 4) ---- */
  double     t4      = Now_ms();
  float      quarter = 0.25f;
  PLAINTEXT  q;
  CIPHERTEXT scaled, scaled_down;
  memset(&q, 0, sizeof(q)), memset(&scaled, 0, sizeof(scaled)), memset(&scaled_down, 0, sizeof(scaled_down));
  Encode_float(&q, &quarter, 1, 1, Level(&fresh));
  Init_ciph_up_scale_plain(&scaled, &fresh, &q);
  {
    MODULUS* m = Q_modulus();
    uint32_t n = Poly_level(&scaled._c0_poly);
    for (uint32_t i = 0; i < n; ++i, ++m) {
      Hw_modmul(Coeffs(&scaled._c0_poly, i, degree), Coeffs(&fresh._c0_poly, i, degree), Coeffs(&q._poly, i, degree), m, degree);
      Hw_modmul(Coeffs(&scaled._c1_poly, i, degree), Coeffs(&fresh._c1_poly, i, degree), Coeffs(&q._poly, i, degree), m, degree);
    }
  }
  Free_poly_data(&q._poly);
  Init_ciph_down_scale(&scaled_down, &scaled);
  Rescale(&scaled_down._c0_poly, &scaled._c0_poly);
  Rescale(&scaled_down._c1_poly, &scaled._c1_poly);
  Free_ct(&scaled);
  CIPHERTEXT relu = App_relu(fresh, scaled_down);
  Rt_sync();
  double  t5       = Now_ms();
  double* got_relu = Decrypted(&relu);

  double conv_err = Worst(got_conv, want_conv, NULL, 0), fresh_err = Worst(got_fresh, want_conv, NULL, 0);
  double relu_err = Worst(got_relu, want_relu, NULL, 0), relu_far = Worst(got_relu, want_relu, want_conv, 0.1);
  double lo = want_conv[0], hi = want_conv[0];
  for (int i = 0; i < CH * PLANE; ++i) lo = fmin(lo, want_conv[i]), hi = fmax(hi, want_conv[i]);
  printf("conv_err %.3e bootstrap_err %.3e relu_err %.3e relu_err_away_from_zero %.3e level %u relu_level %u "
         "range %.3f %.3f conv_ms %.1f bootstrap_ms %.1f relu_ms %.1f\n",
         conv_err, fresh_err, relu_err, relu_far, level, (unsigned)Level(&relu), lo, hi, t1 - t0, t3 - t2, t5 - t4);
  printf("first values:");
  for (int i = 0; i < 6; ++i) printf(" %.6f/%.6f", got_relu[i], want_relu[i]);
  printf("\n");
  free(got_conv), free(got_fresh), free(got_relu), free(want_conv), free(want_relu);
  Finalize_context();
  /* the convolution is exact arithmetic on encoded values (the encoder's and one rescale's rounding); the bootstrap
   * has the bound of its own test; the ReLU is the compiler's polynomial, whose fit is loosest around zero: 1e-3,
   * the bound of the reference's relu example, away from zero (|x| >= 0.1, the example's smallest input is 0.126) */
  return (conv_err < 1e-5 && fresh_err < 1e-3 && relu_far < 1e-3 && relu_err < 1e-2 && level == 15) ? 0 : 1;
}

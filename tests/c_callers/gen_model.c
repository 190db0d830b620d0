/* A model file shaped like the C the HALO code generator emits for
 *   add1 = (input + w0) + w1        (float[3])
 * [ref: lib/target/generic_cpp/generic_cxx_codegen.cc:668-889; expected text in
 *  tests/compile/test_cxx_gen.cc:35-43]: file-scope computation and context,
 * a helper that records the operators, func_init / func / func_fini.  Compiled
 * as C against the library's own header, so that value types, value lists and
 * value ids cross the boundary the way a C compiler passes them. */
#include <odla_hip.h>

extern const float w0[3];
extern const float w1[3];

static odla_computation Comp;
static odla_context Ctx;

static void func_helper(void) {
  odla_CreateComputation(&Comp);
  odla_value input = odla_CreateArgument(
      (odla_value_type){ODLA_FLOAT32, {.size = 1, .dims = {3}}}, (const odla_value_id)("input"));
  odla_value c0 = odla_CreateConstant(
      (odla_value_type){ODLA_FLOAT32, {.size = 1, .dims = {3}}}, w0, (const odla_value_id)("w0"));
  odla_value c1 = odla_CreateConstant(
      (odla_value_type){ODLA_FLOAT32, {.size = 1, .dims = {3}}}, w1, (const odla_value_id)("w1"));
  odla_value add0 = odla_Add(input, c0, (const odla_value_id)"add0");
  odla_value add1 = odla_Add(add0, c1, (const odla_value_id)"add1");
  odla_SetValueAsOutput(add1);
}

void func_fini(void) {
  odla_DestroyContext(Ctx);
  odla_DestroyComputation(Comp);
}

int func_init(void) {
  if (Comp == NULL) {
    func_helper();
  }
  if (Ctx == NULL) {
    odla_status s = odla_CreateContext(&Ctx);
    if (s != ODLA_SUCCESS) return (int)s;
  }
  return 0;
}

int func(const float input[3], float out_add1[3]) {
  int s = func_init();
  if (s != 0) return s;
  odla_BindToArgumentById((const odla_value_id) "input", input, Ctx);
  odla_BindToOutputById((const odla_value_id) "add1", out_add1, Ctx);
  return (int)odla_ExecuteComputation(Comp, Ctx, ODLA_COMPUTE_INFERENCE, NULL);
}

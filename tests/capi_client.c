/* A plain C99 client of include/eclat_hip.h, as the Rust shim's FFI would use it: the header
 * must compile as C, and the library must work without any Python around it.
 *
 *   capi_client render   renders and compiles `a + b` over 4 floats for gfx950; needs no GPU
 *   capi_client run      the reference's known answer [1,2,3,4] + [5,6,7,8] = [6,8,10,12]
 *                        (crates/backend-c/src/lib.rs:183-205) through
 *                        eh_program_execute_positional, and again from the program's binary
 *                        through eh_module_load / eh_module_launch
 * Exit status 0 on success; the failing call and eh_last_error() go to stderr otherwise.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "eclat_hip.h"

static const char* kAdd4 =
    "(program (kernel \"E_4_0\" (params (\"buf0\" (ptr f32 global) imm normal) "
    "(\"buf2\" (ptr f32 global) imm normal) (\"buf4\" (ptr f32 global) mut normal)) "
    "(grid (const i64 1) (const i64 1) (const i64 1)) (tg (const i64 1) (const i64 1) (const i64 1)) "
    "(range \"ridx0\" (const i64 0) (const i64 1) (const i64 4) "
    "(store (var \"buf4\") (var \"ridx0\") (add (load (var \"buf0\") (var \"ridx0\") 1 f32) "
    "(load (var \"buf2\") (var \"ridx0\") 1 f32))) sequential)))";

#define CHECK(call)                                                              \
  do {                                                                           \
    int rc_ = (call);                                                            \
    if (rc_ != EH_OK) {                                                          \
      fprintf(stderr, "%s failed (%d): %s\n", #call, rc_, eh_last_error());      \
      return 1;                                                                  \
    }                                                                            \
  } while (0)

static int render(void) {
  eh_plan* plan = NULL;
  int n = 0;
  eh_launch_info info;
  void* blob = NULL;
  size_t len = 0;
  CHECK(eh_render_program(kAdd4, NULL, &plan));
  CHECK(eh_plan_num_launches(plan, &n));
  if (n != 1) { fprintf(stderr, "expected one launch, got %d\n", n); return 1; }
  CHECK(eh_plan_launch(plan, 0, &info));
  if (!strstr(info.source, "__global__") || info.n_args != 3) { fprintf(stderr, "unexpected rendering\n"); return 1; }
  CHECK(eh_compile_source(info.source, "gfx950", &blob, &len));
  if (len < 64 || memcmp(blob, "\177ELF", 4) != 0) { fprintf(stderr, "not an ELF code object\n"); return 1; }
  printf("render ok: %s %s, %zu bytes of gfx950 code\n", info.entry, info.schedule, len);
  eh_free(blob);
  CHECK(eh_plan_release(plan));
  /* errors are codes plus a message, never a crash */
  if (eh_render_program("(program (kernel", NULL, &plan) != EH_ERR_PARSE || !*eh_last_error()) {
    fprintf(stderr, "malformed text was not reported as EH_ERR_PARSE\n");
    return 1;
  }
  return 0;
}

static int expect(const float* got, const char* what) {
  static const float want[4] = {6, 8, 10, 12};
  if (memcmp(got, want, sizeof want) != 0) {
    fprintf(stderr, "%s: got [%g %g %g %g]\n", what, got[0], got[1], got[2], got[3]);
    return 1;
  }
  return 0;
}

static int run(void) {
  const float a[4] = {1, 2, 3, 4}, b[4] = {5, 6, 7, 8};
  float out[4];
  int count = 0;
  eh_device* dev = NULL;
  eh_buffer *ba = NULL, *bb = NULL, *bo = NULL;
  eh_program* prog = NULL;
  eh_module* mod = NULL;
  eh_launch_info info;
  const void* blob = NULL;
  size_t len = 0;
  eh_buffer* ins[2];
  eh_buffer* outs[1];
  eh_buffer* args[3];
  CHECK(eh_device_count(&count));
  if (count == 0) { fprintf(stderr, "no HIP device\n"); return 2; }
  CHECK(eh_device_open(0, &dev));
  CHECK(eh_buffer_alloc(dev, sizeof a, &ba));
  CHECK(eh_buffer_alloc(dev, sizeof b, &bb));
  CHECK(eh_buffer_alloc(dev, sizeof out, &bo));
  CHECK(eh_buffer_write(ba, a, sizeof a));
  CHECK(eh_buffer_write(bb, b, sizeof b));
  if (eh_buffer_write(bb, b, sizeof b - 4) != EH_ERR_SIZE) { fprintf(stderr, "short write accepted\n"); return 1; }
  CHECK(eh_program_compile(dev, kAdd4, NULL, &prog));
  ins[0] = ba; ins[1] = bb; outs[0] = bo;
  CHECK(eh_program_execute_positional(prog, ins, 2, outs, 1, 1));
  CHECK(eh_buffer_read(bo, out, sizeof out));
  if (expect(out, "program")) return 1;
  /* the same kernel again from its binary */
  CHECK(eh_program_launch(prog, 0, &info));
  CHECK(eh_program_binary(prog, 0, &blob, &len));
  CHECK(eh_module_load(dev, blob, len, info.entry, &mod));
  memset(out, 0, sizeof out);
  CHECK(eh_buffer_write(bo, out, sizeof out));
  args[0] = ba; args[1] = bb; args[2] = bo;
  CHECK(eh_module_launch(mod, info.grid, info.block, info.lds_bytes, args, 3, 1));
  CHECK(eh_buffer_read(bo, out, sizeof out));
  if (expect(out, "module")) return 1;
  CHECK(eh_module_release(mod));
  CHECK(eh_program_release(prog));
  CHECK(eh_buffer_release(ba));
  CHECK(eh_buffer_release(bb));
  CHECK(eh_buffer_release(bo));
  CHECK(eh_device_close(dev));
  printf("run ok: [6 8 10 12] from the program and from its binary\n");
  return 0;
}

int main(int argc, char** argv) {
  if (argc == 2 && strcmp(argv[1], "render") == 0) return render();
  if (argc == 2 && strcmp(argv[1], "run") == 0) return run();
  fprintf(stderr, "usage: %s render|run (library version %d)\n", argv[0], eh_version());
  return 64;
}

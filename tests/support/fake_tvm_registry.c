/* Test double for the three TVM C-API symbols the library resolves with dlsym when a TVM
 * runtime is loaded in the process: a registry that records what was registered and the last
 * error text.  It is not a TVM build and is loaded only by tests/test_capi_cpu.py. */
#include <string.h>

typedef int (*packed_cfunc)(void* args, int* type_codes, int num_args, void* ret, void* resource);

#define MAX_FUNCS 32
static struct { char name[64]; packed_cfunc fn; void* resource; } g_funcs[MAX_FUNCS];
static int g_count = 0;
static char g_last_error[512] = "";
static struct { packed_cfunc fn; void* resource; } g_handles[MAX_FUNCS];
static int g_handle_count = 0;

void TVMAPISetLastError(const char* msg) {
  strncpy(g_last_error, msg, sizeof(g_last_error) - 1);
  g_last_error[sizeof(g_last_error) - 1] = 0;
}

int TVMFuncCreateFromCFunc(packed_cfunc func, void* resource_handle, void (*fin)(void*), void** out) {
  (void)fin;
  if (g_handle_count >= MAX_FUNCS) return -1;
  g_handles[g_handle_count].fn = func;
  g_handles[g_handle_count].resource = resource_handle;
  *out = &g_handles[g_handle_count++];
  return 0;
}

int TVMFuncRegisterGlobal(const char* name, void* f, int override) {
  (void)override;
  if (g_count >= MAX_FUNCS) return -1;
  strncpy(g_funcs[g_count].name, name, 63);
  g_funcs[g_count].fn = ((typeof(&g_handles[0]))f)->fn;
  g_funcs[g_count].resource = ((typeof(&g_handles[0]))f)->resource;
  ++g_count;
  return 0;
}

/* inspection helpers for the test */
int fake_tvm_count(void) { return g_count; }
const char* fake_tvm_name(int i) { return g_funcs[i].name; }
const char* fake_tvm_last_error(void) { return g_last_error; }
int fake_tvm_call(int i, void* args, int* type_codes, int num_args) {
  return g_funcs[i].fn(args, type_codes, num_args, 0, g_funcs[i].resource);
}

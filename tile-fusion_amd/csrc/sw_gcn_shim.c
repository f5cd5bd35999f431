/* libsw_gcn.so: what the reference's Python layers load with
 *     torch.ops.load_library("build/lib/libsw_gcn.so")
 * (binding-project/gcn-e2e-training/FusedGCNLayer.py:3, test_lib.py:6, binding_benchmark.py:6).
 * The reference's library registers torch.ops.sw_gcn.* from C++ (binding-project/main.cpp:133-142).  Here the
 * operators are registered from Python (tile-fusion_amd/torch_ops.py, on top of libtilefusion_hip's C ABI), so
 * this library does one thing when it is loaded into a Python process: it imports that module, which registers
 * the same operator names.  A script of the reference then only needs the path in its load_library line changed.
 * Loaded outside Python (no interpreter in the process) it does nothing.
 * Plain C, no link-time dependency on libpython: the interpreter's symbols are looked up in the running process. */
#define _GNU_SOURCE
#include <dlfcn.h>
#include <stdio.h>
#include <string.h>

typedef int (*is_initialized_fn)(void);
typedef int (*gil_ensure_fn)(void);
typedef void (*gil_release_fn)(int);
typedef int (*run_string_fn)(const char *);

__attribute__((constructor)) static void sw_gcn_register(void) {
  is_initialized_fn is_init = (is_initialized_fn)dlsym(RTLD_DEFAULT, "Py_IsInitialized");
  gil_ensure_fn ensure = (gil_ensure_fn)dlsym(RTLD_DEFAULT, "PyGILState_Ensure");
  gil_release_fn release = (gil_release_fn)dlsym(RTLD_DEFAULT, "PyGILState_Release");
  run_string_fn run = (run_string_fn)dlsym(RTLD_DEFAULT, "PyRun_SimpleString");
  if (!is_init || !ensure || !release || !run || !is_init()) return;
  /* this file sits in <root>/tile-fusion_amd/lib/: the package is imported from <root> */
  Dl_info me;
  if (!dladdr((void *)&sw_gcn_register, &me) || !me.dli_fname) return;
  char root[4096];
  strncpy(root, me.dli_fname, sizeof(root) - 1);
  root[sizeof(root) - 1] = 0;
  for (int up = 0; up < 3; ++up) {
    char *slash = strrchr(root, '/');
    if (!slash) return;
    *slash = 0;
  }
  char code[8192];
  snprintf(code, sizeof(code),
           "import sys, os, importlib\n"
           "_r = os.path.realpath(r'''%s''' or '.')\n"
           "if _r not in sys.path: sys.path.insert(0, _r)\n"
           "importlib.import_module('tile-fusion_amd.torch_ops')\n",
           root);
  const int gil = ensure();
  if (run(code) != 0) fprintf(stderr, "libsw_gcn: importing tile-fusion_amd.torch_ops failed (see the traceback above)\n");
  release(gil);
}

// Plumbing of liblitgpt_seq.so: the thread-local error string and the version.
#include <string.h>

#include "seq_common.h"

static thread_local char g_seq_err[512] = {0};

extern "C" void lga_set_error(const char* msg) {
  strncpy(g_seq_err, msg ? msg : "", sizeof(g_seq_err) - 1);
  g_seq_err[sizeof(g_seq_err) - 1] = 0;
}

extern "C" const char* lgs_last_error_string(void) { return g_seq_err; }

extern "C" int lgs_version(void) { return 1; }

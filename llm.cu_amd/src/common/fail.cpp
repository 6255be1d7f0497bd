#include "common/fail.h"

#include <cstdio>
#include <cstdlib>

#include "llama3_host.h"
#include "llmcu_hip.h"

static llama3_error_fn g_handler = nullptr;

extern "C" void llama3_set_error_handler(llama3_error_fn fn) { g_handler = fn; }

void llama3_fail(const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (g_handler) g_handler(buf);
    printf("Error: %s\n", buf);
    fflush(stdout);
    exit(1);
}

void llama3_check(int status, const char *what) {
    if (status != LLM_OK) llama3_fail("%s failed: %s", what, llm_last_error());
}

#pragma once
#include <vector>
struct StubCall {
    const char *what;
    int batch;
    const void *a, *b, *c;
    int flag;
};
extern std::vector<StubCall> g_calls;
extern int g_capacity;

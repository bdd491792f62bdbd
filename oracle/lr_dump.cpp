// Prints learning-rate schedules as JSON (FP32 bit patterns) for a fixed set of configurations.
// TEST INFRASTRUCTURE.  The LRScheduler class comes from whichever "training/lr_scheduler.h" the
// include path finds first: the reference's (include/training/lr_scheduler.h) to write golden
// vectors, or this repository's mirror to check it against them.
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "training/lr_scheduler.h"

static uint32_t bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static void dump(const char* name, const LRScheduler& s, int steps, bool last) {
    printf("  \"%s\": [", name);
    for (int i = 0; i < steps; i++) printf("%s%u", i ? ", " : "", bits(s.get_lr(i)));
    printf("]%s\n", last ? "" : ",");
}

int main() {
    LRScheduler s;
    printf("{\n");
    s.init_constant(1e-4f);            dump("constant_1e-4", s, 20, false);
    s.init_constant(1e-3f, 10);        dump("constant_1e-3_warmup10", s, 30, false);
    s.init_constant(1e-5f, 1);         dump("constant_1e-5_warmup1", s, 5, false);
    s.init_cosine(1e-3f, 1e-5f, 0, 100);   dump("cosine_1e-3_1e-5_w0_t100", s, 120, false);
    s.init_cosine(1e-3f, 1e-4f, 10, 110);  dump("cosine_1e-3_1e-4_w10_t110", s, 130, false);
    s.init_cosine(1e-5f, 0.0f, 50, 2000);  dump("cosine_1e-5_0_w50_t2000", s, 2100, false);
    s.init_cosine(3e-4f, 3e-5f, 10, 10);   dump("cosine_total_equals_warmup", s, 20, false);
    s.init_cosine(3e-4f, 3e-5f, 10, 5);    dump("cosine_total_below_warmup", s, 20, false);
    LRScheduler d;                     dump("default_constructed", d, 5, true);
    printf("}\n");
    return 0;
}

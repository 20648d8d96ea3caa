// KSEARCH_PROFILE: per-section times of a decode step, as GemmaPrimModel::forward_token prints them
// (crates/ksearch_gemma/src/gemma_prim.rs:885, 924-929, 1203-1213, 1260-1273).  The reference synchronises the
// device between sections and reads the host clock; here an event is recorded on the stream at every section
// boundary and the step is launched kernel by kernel (no graph replay), so the sections keep running back to back
// and the figures are device time.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdio>
#include <vector>

namespace ksh {

struct SectionTimer {
    enum { kEmbed = 0, kPrepass, kAttn, kMlp, kPle, kLogits, kSections };
    bool on = false;
    hipStream_t st = nullptr;
    std::vector<hipEvent_t> ev;
    std::vector<int> sec;
    size_t used = 0;

    ~SectionTimer()
    {
        for (hipEvent_t e : ev) (void)hipEventDestroy(e);
    }
    bool record()
    {
        if (used == ev.size()) {
            hipEvent_t e = nullptr;
            if (hipEventCreate(&e) != hipSuccess) return false;
            ev.push_back(e);
        }
        return hipEventRecord(ev[used++], st) == hipSuccess;
    }
    // start of a step
    void begin(hipStream_t stream)
    {
        if (!on) return;
        st = stream;
        used = 0;
        sec.clear();
        if (!record()) on = false;
    }
    // what was launched since the previous mark belongs to `section`
    void mark(int section)
    {
        if (!on) return;
        if (record()) sec.push_back(section);
        else on = false;
    }
    // waits for the step and prints one line in the reference's format
    void report(const char *what, int pos)
    {
        if (!on || used < 2) return;
        if (hipEventSynchronize(ev[used - 1]) != hipSuccess) return;
        double ms[kSections] = {}, total = 0.0;
        for (size_t i = 0; i + 1 < used; i++) {
            float t = 0.f;
            if (hipEventElapsedTime(&t, ev[i], ev[i + 1]) != hipSuccess) return;
            ms[sec[i]] += t;
            total += t;
        }
        fprintf(stderr, "[profile] %s pos=%d embed=%.3fms prepass=%.3fms attn=%.3fms mlp=%.3fms ple=%.3fms logits+sync=%.3fms total=%.3fms\n", what,
                pos, ms[kEmbed], ms[kPrepass], ms[kAttn], ms[kMlp], ms[kPle], ms[kLogits], total);
    }
};

}  // namespace ksh

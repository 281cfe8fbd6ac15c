// The environment switches of tuning.h: read once, reported once.
#include "tuning.h"

#include <cstdio>
#include <cstring>
#include <cstdlib>
#include <string>

#include "common.h"

namespace {
struct Parsed {
    TurqTuning t;
    std::string set;  // "NAME=value ..." of the variables that were set
};

void parse_INT(int &f, const char *v) { f = atoi(v); }
void parse_TRI(int &f, const char *v) { f = atoi(v) != 0 ? 1 : 0; }
void parse_FLAG(bool &f, const char *) { f = true; }
void parse_OFF(bool &f, const char *v) { f = atoi(v) == 0; }

const Parsed &parsed() {
    static const Parsed p = [] {
        Parsed q;
#define X(f, env, kind, d, doc)                       \
    if (const char *v = getenv(env)) {                \
        parse_##kind(q.t.f, v);                       \
        q.t.overrides++;                              \
        q.set += std::string(" ") + env + "=" + v;    \
    }
        TURQ_TUNING_TABLE(X)
#undef X
        if (q.t.overrides)
            fprintf(stderr, "libturq: %d kernel-selection override(s) from the environment:%s\n", q.t.overrides, q.set.c_str());
        return q;
    }();
    return p;
}
}  // namespace

const TurqTuning &turq_tuning() { return parsed().t; }

// one line per switch: "NAME=value  (default | set)  what it overrides"; returns the bytes the whole text needs
extern "C" int turq_tuning_describe(char *buf, size_t cap, size_t *needed) {
    const TurqTuning &t = turq_tuning();
    std::string s;
    char line[320];
#define X(f, env, kind, d, doc)                                                                                  \
    snprintf(line, sizeof line, "%s=%d  (%s)  %s\n", env, (int)t.f, getenv(env) ? "set" : "default", doc);       \
    s += line;
    TURQ_TUNING_TABLE(X)
#undef X
    if (needed) *needed = s.size() + 1;
    if (buf && cap) {
        const size_t nbytes = s.size() < cap - 1 ? s.size() : cap - 1;
        memcpy(buf, s.data(), nbytes);
        buf[nbytes] = 0;
    }
    return TURQ_OK;
}

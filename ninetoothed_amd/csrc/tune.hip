// The table of tuned choices and its on-disk form.
#include "tune.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <shared_mutex>
#include <unordered_map>
#include <algorithm>
#include <vector>

#include "../../include/ninetoothed_hip.h"

namespace nt {
namespace {

struct TuneKey {
    int device, kind, count;
    int v[kTuneMaxValues];
    bool operator==(const TuneKey &o) const { return device == o.device && kind == o.kind && count == o.count && memcmp(v, o.v, sizeof(v)) == 0; }
};
struct TuneKeyHash {
    size_t operator()(const TuneKey &x) const {
        size_t h = 1469598103934665603ull;
        h = (h ^ (size_t)(unsigned)x.device) * 1099511628211ull;
        h = (h ^ (size_t)(unsigned)x.kind) * 1099511628211ull;
        for (int i = 0; i < x.count; ++i) h = (h ^ (size_t)(unsigned)x.v[i]) * 1099511628211ull;
        return h;
    }
};
std::shared_mutex g_mutex;
struct Choice {
    int index;
    int extras;    // descriptive integers that follow the index in the file (the block sizes of a GEMM instance)
    int extra[3];
};
std::unordered_map<TuneKey, Choice, TuneKeyHash> g_choices;

bool make_key(TuneKey &key, int kind, const int *values, int count) {
    if (kind < 0 || kind >= kTuneKinds || count < 0 || count > kTuneMaxValues || (count > 0 && values == nullptr)) return false;
    key.device = 0;
    (void)hipGetDevice(&key.device);
    key.kind = kind;
    key.count = count;
    memset(key.v, 0, sizeof(key.v));
    for (int i = 0; i < count; ++i) key.v[i] = values[i];
    return true;
}

}  // namespace

int tune_lookup(int kind, const int *values, int count) {
    TuneKey key;
    if (!make_key(key, kind, values, count)) return -1;
    std::shared_lock<std::shared_mutex> lock(g_mutex);
    auto it = g_choices.find(key);
    return it == g_choices.end() ? -1 : it->second.index;
}

void tune_record(int kind, const int *values, int count, int choice, const int *extra, int extras) {
    TuneKey key;
    if (!make_key(key, kind, values, count)) return;
    Choice entry = {choice, 0, {0, 0, 0}};
    for (int i = 0; i < extras && i < 3 && extra != nullptr; ++i) entry.extra[entry.extras++] = extra[i];
    std::unique_lock<std::shared_mutex> lock(g_mutex);
    g_choices[key] = entry;
}

namespace {
TuneChoiceCheck g_checks[kTuneKinds] = {};
}  // namespace

bool tune_register_check(int kind, TuneChoiceCheck check) {
    if (kind < 0 || kind >= kTuneKinds) return false;
    g_checks[kind] = check;
    return true;
}

namespace {
thread_local int t_launch_program = kLaunchNone;
thread_local int t_launch_choice = -1;
thread_local const char *t_launch_name = nullptr;
}  // namespace

void note_launch(int program, int choice, const char *name) {
    t_launch_program = program;
    t_launch_choice = choice;
    t_launch_name = name;
}

}  // namespace nt

using namespace nt;

extern "C" {

// Describes the kernel that served the calling thread's latest launch_nt_* call, e.g.
// "attention variant 3: software-pipelined loop, 64-key blocks, four waves".
NineToothedResult nt_last_launch(char *buffer, int size) {
    if (buffer == nullptr || size <= 0) return hipErrorInvalidValue;
    static const char *const programs[] = {"none", "gemm instance", "attention variant", "conv2d path", "softmax kernel", "tile map"};
    const int program = t_launch_program >= kLaunchNone && t_launch_program <= kLaunchMap ? t_launch_program : kLaunchNone;
    if (program == kLaunchNone) snprintf(buffer, (size_t)size, "none");
    else snprintf(buffer, (size_t)size, "%s %d: %s", programs[program], t_launch_choice, t_launch_name ? t_launch_name : "");
    return 0;
}

int nt_tune_lookup(int kind, const int *values, int count) { return tune_lookup(kind, values, count); }

int nt_tune_file_format(void) { return kTuneFileFormat; }

// On-disk form: the line-pair CSV the reference's AutoTuningCache reads
// (src/ninetoothed/templates/auto_tuning_cache.h:27-75; written by src/ninetoothed/build.py:683-703): a line of
// integers describing the problem, then a line of integers with the choice; the first pair has an empty problem
// line and carries a default.  A problem line is the program (0 = matmul / addmm, 1 = attention, 2 = conv2d)
// followed by the problem's values; a choice line is the variant's index followed by optional descriptive
// integers (the GEMM instances add their block sizes).  The default pair's choice line holds kTuneFileFormat.
NineToothedResult nt_tune_cache_save(const char *path) {
    if (path == nullptr) return hipErrorInvalidValue;
    int device = 0;
    (void)hipGetDevice(&device);
    FILE *file = fopen(path, "w");
    if (file == nullptr) return hipErrorInvalidValue;
    fprintf(file, "\n%d\n", kTuneFileFormat);
    {
        std::shared_lock<std::shared_mutex> lock(g_mutex);
        for (const auto &entry : g_choices) {
            const TuneKey &key = entry.first;
            if (key.device != device) continue;
            fprintf(file, "%d", key.kind);
            for (int i = 0; i < key.count; ++i) fprintf(file, ",%d", key.v[i]);
            fprintf(file, "\n%d", entry.second.index);
            for (int i = 0; i < entry.second.extras; ++i) fprintf(file, ",%d", entry.second.extra[i]);
            fprintf(file, "\n");
        }
    }
    return fclose(file) == 0 ? 0 : (int)hipErrorInvalidValue;
}

// Reads such a file into the table of the current device.  *entries (may be NULL) receives the number of choices
// taken over; lines that do not parse are skipped.  A file whose default pair does not hold this build's
// kTuneFileFormat is ignored whole (0 entries, no error), and so is every choice that the program it belongs to
// does not recognise (a GEMM instance index whose block sizes differ from the ones written next to it): the
// numbering of the variants may differ between builds, and a stale choice would be a valid but slow kernel.
NineToothedResult nt_tune_cache_load(const char *path, int *entries) {
    if (entries) *entries = 0;
    if (path == nullptr) return hipErrorInvalidValue;
    FILE *file = fopen(path, "r");
    if (file == nullptr) return hipErrorInvalidValue;
    auto parse = [](const char *line, std::vector<long> &values) {
        values.clear();
        const char *cursor = line;
        while (*cursor) {
            while (*cursor == ' ' || *cursor == '\t' || *cursor == '\r' || *cursor == '\n' || *cursor == ',') ++cursor;
            if (!*cursor) break;
            char *end = nullptr;
            const long value = strtol(cursor, &end, 10);
            if (end == cursor) return false;
            values.push_back(value);
            cursor = end;
        }
        return true;
    };
    char problem_line[512], choice_line[512];
    std::vector<long> problem, choice;
    bool first = true;
    int taken = 0;
    while (fgets(problem_line, sizeof(problem_line), file) && fgets(choice_line, sizeof(choice_line), file)) {
        const bool parsed = parse(problem_line, problem) && parse(choice_line, choice);
        if (first) {  // the default pair
            first = false;
            if (!parsed || choice.empty() || choice[0] != kTuneFileFormat) break;
            continue;
        }
        if (!parsed || problem.empty() || choice.empty() || problem.size() > (size_t)kTuneMaxValues + 1) continue;
        if (problem[0] < 0 || problem[0] >= kTuneKinds || choice[0] < 0) continue;
        int values[kTuneMaxValues];
        const int count = (int)problem.size() - 1;
        for (int i = 0; i < count; ++i) values[i] = (int)problem[i + 1];
        int extra[3] = {0, 0, 0};
        const int extras = (int)std::min<size_t>(choice.size() - 1, 3);
        for (int i = 0; i < extras; ++i) extra[i] = (int)choice[i + 1];
        const TuneChoiceCheck check = g_checks[problem[0]];
        if (check != nullptr && !check((int)choice[0], extra, extras)) continue;
        tune_record((int)problem[0], values, count, (int)choice[0], extra, extras);
        ++taken;
    }
    fclose(file);
    if (entries) *entries = taken;
    return 0;
}

}  // extern "C"

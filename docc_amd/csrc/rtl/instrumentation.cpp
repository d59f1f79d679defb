// Runtime behind the `__daisy_instrumentation_*` calls of instrumented generated code, with
// the ROCm event set (see include/docc_rocm_rtl.h). It plays the part of the reference's
// rtl/src/instrumentation.cpp for the rocm target: same protocol, same trace layout, HIP
// events and roctx ranges in place of PAPI counters.
#include <dlfcn.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <limits>
#include <map>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include "docc_rocm_rt.h"
#include "docc_rocm_rtl.h"

namespace {

long long wall_ns() {
    timespec ts;
    clock_gettime(CLOCK_REALTIME, &ts);
    return (long long) ts.tv_sec * 1000000000LL + ts.tv_nsec;
}

// running mean / variance / extremes (Welford), the aggregate the reference's trace reports
struct Stats {
    long long n = 0;
    double mean = 0.0, variance = 0.0;
    double min = std::numeric_limits<double>::infinity(), max = -std::numeric_limits<double>::infinity();

    void add(double x) {
        n += 1;
        const double d1 = x - mean;
        mean += d1 / (double) n;
        const double d2 = x - mean;
        variance += (d1 * d2 - variance) / (double) n;
        if (x < min) min = x;
        if (x > max) max = x;
    }
};

struct Metadata {
    std::string file_name, function_name, sdfg_name, sdfg_file, arg_capture_path, features_file, opt_report_file;
    std::string element_type, target_type, region_uuid;
    bool has_sdfg_name = false, has_sdfg_file = false;
    long line_begin = 0, line_end = 0, column_begin = 0, column_end = 0;
    size_t element_id = 0;
    int loopnest_index = -1;
    size_t num_loops = 0, num_maps = 0, num_fors = 0, num_whiles = 0, max_depth = 0;
    bool is_perfectly_nested = false, is_perfectly_parallel = false, is_elementwise = false, has_side_effects = false;
};

std::string str(const char* s) { return s ? s : ""; }

struct Region {
    Metadata md;
    __daisy_event_set event_set = __DAISY_EVENT_SET_NONE;
    // one entry per execution (individual mode)
    std::vector<long long> starts, durations;
    // aggregate mode
    long long first_start = 0, last_start = 0;
    Stats runtime;
    std::map<std::string, Stats> static_counters;
    // ROCm event set: the events of the execution that is open
    docc_rocm_event_t begin = nullptr, end = nullptr;
    bool events_recorded = false;
    bool open = false;
};

// An execution whose events are recorded but not read yet: the device time of a region is taken from its two events
// when the trace is written (or when many are waiting), so that a region costs the host two event records and no
// wait - the stream keeps running under instrumented code as it does without.
struct Pending {
    size_t region;
    size_t index;     // into Region::durations (individual mode)
    docc_rocm_event_t begin, end;
};

std::string json_string(const std::string& s) {
    std::string out = "\"";
    for (unsigned char c : s) {
        switch (c) {
            case '"': out += "\\\""; break;
            case '\\': out += "\\\\"; break;
            case '\n': out += "\\n"; break;
            case '\t': out += "\\t"; break;
            case '\r': out += "\\r"; break;
            default:
                if (c < 0x20) {
                    char buf[8];
                    std::snprintf(buf, sizeof(buf), "\\u%04x", c);
                    out += buf;
                } else {
                    out += (char) c;
                }
        }
    }
    return out + "\"";
}

std::string json_number(double v) {
    if (!std::isfinite(v)) return "null";
    std::ostringstream os;
    os.precision(17);
    os << v;
    return os.str();
}

std::string base_name(const std::string& path) {
    const size_t p = path.find_last_of('/');
    return p == std::string::npos ? path : path.substr(p + 1);
}

void state_flush();

class State {
public:
    State() {
        const char* mode = std::getenv("__DAISY_INSTRUMENTATION_MODE");
        aggregate_ = mode && std::strcmp(mode, "aggregate") == 0;
        const char* file = std::getenv("__DAISY_INSTRUMENTATION_FILE");
        output_file_ = file && *file ? file : "daisy_trace.json";
        // roctx is optional: the ranges only matter under a profiler. rocprofv3 listens to the
        // rocprofiler-sdk implementation, older tools to roctracer's.
        for (const char* name : {"librocprofiler-sdk-roctx.so", "librocprofiler-sdk-roctx.so.1", "libroctx64.so", "libroctx64.so.4"}) {
            void* h = dlopen(name, RTLD_LAZY | RTLD_GLOBAL);
            if (!h) continue;
            range_push_ = reinterpret_cast<int (*)(const char*)>(dlsym(h, "roctxRangePushA"));
            range_pop_ = reinterpret_cast<int (*)()>(dlsym(h, "roctxRangePop"));
            if (range_push_ && range_pop_) break;
            range_push_ = nullptr;
            range_pop_ = nullptr;
        }
        gpu_ = docc_rocm_device_count() > 0;
    }

    ~State() { write(); }

    // events are read while the HIP runtime is still there: at exit before its own tear-down (registered after its
    // start-up, so run before), not from this object's destructor
    static void at_exit() { state_flush(); }

    size_t init(const __daisy_metadata_t* m, __daisy_event_set set) {
        std::lock_guard<std::mutex> lock(mutex_);
        const std::string uuid = str(m->region_uuid);
        auto known = by_uuid_.find(uuid);
        if (known != by_uuid_.end()) return known->second;
        Region r;
        r.event_set = set;
        Metadata& d = r.md;
        d.file_name = str(m->file_name);
        d.function_name = str(m->function_name);
        d.sdfg_name = str(m->sdfg_name);
        d.sdfg_file = str(m->sdfg_file);
        d.has_sdfg_name = m->sdfg_name != nullptr;
        d.has_sdfg_file = m->sdfg_file != nullptr;
        d.arg_capture_path = str(m->arg_capture_path);
        d.features_file = str(m->features_file);
        d.opt_report_file = str(m->opt_report_file);
        d.element_type = str(m->element_type);
        d.target_type = str(m->target_type);
        d.region_uuid = uuid;
        d.line_begin = m->line_begin;
        d.line_end = m->line_end;
        d.column_begin = m->column_begin;
        d.column_end = m->column_end;
        d.element_id = m->element_id;
        d.loopnest_index = m->loopnest_index;
        d.num_loops = m->num_loops;
        d.num_maps = m->num_maps;
        d.num_fors = m->num_fors;
        d.num_whiles = m->num_whiles;
        d.max_depth = m->max_depth;
        d.is_perfectly_nested = m->is_perfectly_nested;
        d.is_perfectly_parallel = m->is_perfectly_parallel;
        d.is_elementwise = m->is_elementwise;
        d.has_side_effects = m->has_side_effects;
        const size_t id = next_id_++;
        regions_[id] = std::move(r);
        by_uuid_[uuid] = id;
        return id;
    }

    void enter(size_t id) {
        std::lock_guard<std::mutex> lock(mutex_);
        Region& r = region(id, "entering");
        if (r.event_set == __DAISY_EVENT_SET_NONE) return;
        r.events_recorded = false;
        if (r.event_set == __DAISY_EVENT_SET_ROCM) {
            if (range_push_) range_push_(r.md.region_uuid.c_str());
            if (gpu_) {
                // the begin event completes when what is already queued on the stream has: that work is not part of
                // the region, and the host does not wait for it
                if (!exit_hook_) {
                    exit_hook_ = true;
                    std::atexit(&State::at_exit);
                }
                r.begin = take_event();
                r.end = take_event();
                if (r.begin && r.end && docc_rocm_event_record(r.begin, nullptr) == 0) r.events_recorded = true;
            }
        }
        const long long now = wall_ns();
        if (aggregate_) {
            if (r.first_start == 0) r.first_start = now;
            r.last_start = now;
        } else {
            r.starts.push_back(now);
        }
        r.open = true;
    }

    void exit(size_t id) {
        std::lock_guard<std::mutex> lock(mutex_);
        Region& r = region(id, "exiting");
        if (r.event_set == __DAISY_EVENT_SET_NONE || !r.open) return;
        r.open = false;
        bool deferred = false;
        if (r.event_set == __DAISY_EVENT_SET_ROCM) {
            if (r.events_recorded && docc_rocm_event_record(r.end, nullptr) == 0) {
                if (!aggregate_) r.durations.push_back(-1);
                pending_.push_back(Pending{id, aggregate_ ? 0 : r.durations.size() - 1, r.begin, r.end});
                deferred = true;
            } else {
                give_event(r.begin);
                give_event(r.end);
            }
            r.begin = r.end = nullptr;
            if (range_pop_) range_pop_();
        }
        if (!deferred) {
            const long long duration = wall_ns() - (aggregate_ ? r.last_start : r.starts.back());
            if (aggregate_)
                r.runtime.add((double) duration);
            else
                r.durations.push_back(duration);
        }
        if (pending_.size() >= kMaxPending) resolve();
    }

    void metric(size_t id, const char* name, double value) {
        std::lock_guard<std::mutex> lock(mutex_);
        region(id, "metric for").static_counters[str(name)].add(value);
    }

    void finalize(size_t id) {
        std::lock_guard<std::mutex> lock(mutex_);
        Region& r = region(id, "finalizing");
        // the events stay with the region: it is usually entered again by the next call
        (void) r;
    }

    int write() {
        std::lock_guard<std::mutex> lock(mutex_);
        resolve();
        if (regions_.empty() && written_) return 0;
        FILE* f = std::fopen(output_file_.c_str(), "w");
        if (!f) {
            std::perror("[docc-rtl-rocm] cannot open the trace file");
            return -1;
        }
        std::fputs("{\"traceEvents\":[\n", f);
        bool first = true;
        for (auto& kv : regions_) {
            const Region& r = kv.second;
            if (aggregate_) {
                if (r.runtime.n == 0 && r.static_counters.empty()) continue;
                if (!first) std::fputs(",\n", f);
                first = false;
                std::fputs(event(r, 0, true).c_str(), f);
                continue;
            }
            for (size_t i = 0; i < r.durations.size(); i++) {
                if (!first) std::fputs(",\n", f);
                first = false;
                std::fputs(event(r, i, false).c_str(), f);
            }
        }
        std::fputs("\n]}\n", f);
        std::fclose(f);
        written_ = true;
        return 0;
    }

private:
    static constexpr size_t kMaxPending = 4096;

    docc_rocm_event_t take_event() {
        if (!free_events_.empty()) {
            docc_rocm_event_t e = free_events_.back();
            free_events_.pop_back();
            return e;
        }
        docc_rocm_event_t e = nullptr;
        return docc_rocm_event_create(&e) == 0 ? e : nullptr;
    }
    void give_event(docc_rocm_event_t e) {
        if (e) free_events_.push_back(e);
    }

    // reads the events of the executions that are waiting (the caller holds the lock); an execution whose events cannot
    // be read is reported with a duration of 0
    void resolve() {
        for (auto& p : pending_) {
            float ms = 0.f;
            const long long duration = docc_rocm_event_elapsed_ms(p.begin, p.end, &ms) == 0 ? (long long) ((double) ms * 1e6) : 0;
            Region& r = regions_.at(p.region);
            if (aggregate_)
                r.runtime.add((double) duration);
            else
                r.durations[p.index] = duration;
            give_event(p.begin);
            give_event(p.end);
        }
        pending_.clear();
    }

    Region& region(size_t id, const char* what) {
        auto it = regions_.find(id);
        if (it == regions_.end()) {
            std::fprintf(stderr, "[docc-rtl-rocm] %s unknown region %zu\n", what, id);
            std::exit(EXIT_FAILURE);
        }
        return it->second;
    }

    // one row of the Chrome trace; field order and names follow the reference's writer
    std::string event(const Region& r, size_t index, bool aggregated) const {
        const Metadata& md = r.md;
        std::ostringstream e;
        e << "{\"ph\":\"X\",\"cat\":\"" << (aggregated ? "aggregated_region,daisy" : "region,daisy") << "\",";
        e << "\"name\":" << json_string(md.function_name + " [L" + std::to_string(md.line_begin) + "-" + std::to_string(md.line_end) + "]") << ",";
        e << "\"pid\":" << getpid() << ",\"tid\":" << (long) syscall(SYS_gettid) << ",";
        if (aggregated) {
            e << "\"ts\":" << r.first_start / 1000 << ",\"dur\":" << json_number(r.runtime.mean * (double) r.runtime.n / 1000.0) << ",";
        } else {
            e << "\"ts\":" << r.starts[index] / 1000 << ",\"dur\":" << json_number((double) r.durations[index] / 1000.0) << ",";
        }
        e << "\"args\":{\"function\":" << json_string(md.function_name) << ",\"module\":" << json_string(base_name(md.file_name)) << ",";
        e << "\"source_ranges\":[{\"file\":" << json_string(md.file_name) << ",\"from\":{\"line\":" << md.line_begin << ",\"col\":"
          << md.column_begin << "},\"to\":{\"line\":" << md.line_end << ",\"col\":" << md.column_end << "}}],";
        e << "\"docc\":{\"sdfg_name\":" << json_string(md.sdfg_name) << ",\"sdfg_file\":" << json_string(md.sdfg_file)
          << ",\"arg_capture_path\":" << json_string(md.arg_capture_path) << ",\"features_file\":" << json_string(md.features_file)
          << ",\"opt_report_file\":" << json_string(md.opt_report_file);
        if (md.has_sdfg_name && md.has_sdfg_file) {
            e << ",\"element_id\":" << md.element_id << ",\"element_type\":" << json_string(md.element_type)
              << ",\"loopnest_index\":" << md.loopnest_index << ",\"loop_info\":{\"loopnest_index\":" << md.loopnest_index
              << ",\"num_loops\":" << md.num_loops << ",\"num_maps\":" << md.num_maps << ",\"num_fors\":" << md.num_fors
              << ",\"num_whiles\":" << md.num_whiles << ",\"max_depth\":" << md.max_depth
              << ",\"is_perfectly_nested\":" << (md.is_perfectly_nested ? "true" : "false")
              << ",\"is_perfectly_parallel\":" << (md.is_perfectly_parallel ? "true" : "false")
              << ",\"is_elementwise\":" << (md.is_elementwise ? "true" : "false")
              << ",\"has_side_effects\":" << (md.has_side_effects ? "true" : "false") << "}";
        }
        e << "},\"target_type\":" << json_string(md.target_type) << ",\"metrics\":{";
        bool first = true;
        for (auto& kv : r.static_counters) {
            if (!first) e << ",";
            first = false;
            const Stats& s = kv.second;
            e << json_string("static:::" + kv.first) << ":";
            if (aggregated)
                e << "{\"mean\":" << json_number(s.mean) << ",\"variance\":" << json_number(s.variance) << ",\"count\":" << s.n
                  << ",\"min\":" << json_number(s.min) << ",\"max\":" << json_number(s.max) << "}";
            else
                e << json_number(s.mean);
        }
        if (aggregated) {
            if (!first) e << ",";
            e << "\"runtime\":{\"mean\":" << json_number(r.runtime.mean / 1000.0) << ",\"variance\":" << json_number(r.runtime.variance / 1000.0)
              << ",\"count\":" << r.runtime.n << ",\"min\":" << json_number(r.runtime.min / 1000.0)
              << ",\"max\":" << json_number(r.runtime.max / 1000.0) << "}";
        }
        e << "}}}";
        return e.str();
    }

    std::mutex mutex_;
    size_t next_id_ = 1;
    std::map<size_t, Region> regions_;
    std::map<std::string, size_t> by_uuid_;
    std::vector<Pending> pending_;
    std::vector<docc_rocm_event_t> free_events_;
    bool aggregate_ = false, gpu_ = false, written_ = false, exit_hook_ = false;
    std::string output_file_;
    int (*range_push_)(const char*) = nullptr;
    int (*range_pop_)() = nullptr;
};

State& state() {
    static State s;
    return s;
}

void state_flush() { (void) state().write(); }

} // namespace

extern "C" {

size_t __daisy_instrumentation_init(__daisy_metadata_t* metadata, enum __daisy_event_set event_set) {
    if (!metadata) {
        std::fprintf(stderr, "[docc-rtl-rocm] __daisy_instrumentation_init without metadata\n");
        std::exit(EXIT_FAILURE);
    }
    return state().init(metadata, event_set);
}

void __daisy_instrumentation_finalize(size_t region_id) { state().finalize(region_id); }

void __daisy_instrumentation_enter(size_t region_id) { state().enter(region_id); }

void __daisy_instrumentation_exit(size_t region_id) { state().exit(region_id); }

void __daisy_instrumentation_increment(size_t region_id, const char* name, long long value) {
    state().metric(region_id, name, (double) value);
}

void __daisy_instrumentation_metric(size_t region_id, const char* name, double value) { state().metric(region_id, name, value); }

int docc_rocm_rtl_flush(void) { return state().write(); }

} // extern "C"

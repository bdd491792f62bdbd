// Training-metrics logger with JSON-lines output: the interface of the reference's Logger
// (include/training/logger.h:27-128) without its third-party JSON dependency.
//
//   Logger logger("checkpoints/run_001");   // appends to run_001/train_log.jsonl
//   logger.log(step, "loss", 2.34f);         // several calls per key before commit() are averaged
//   logger.commit(step);                     // one JSON object per line, also a summary on stdout
//
// A line looks like {"grad_norm":1.5,"loss":2.3399999141693115,"lr":9.999999747378752e-06,"step":100}:
// keys sorted, values the float means widened to double and printed in their shortest form.
#pragma once
#include <charconv>
#include <cmath>
#include <cstdio>
#include <filesystem>
#include <limits>
#include <map>
#include <string>
#include <vector>

class Logger {
public:
    struct Entry {
        int step = 0;
        std::map<std::string, float> values;
        bool contains(const std::string& k) const { return values.count(k) != 0; }
    };

    Logger() = default;
    explicit Logger(const std::string& log_dir) { open(log_dir); }
    ~Logger() { if (file_) fclose(file_); }
    Logger(const Logger&) = delete;
    Logger& operator=(const Logger&) = delete;

    void open(const std::string& log_dir) {
        if (log_dir.empty()) return;
        std::filesystem::create_directories(log_dir);
        log_path_ = log_dir + "/train_log.jsonl";
        file_ = fopen(log_path_.c_str(), "a");   // append: a restarted run continues the same file
        if (!file_) fprintf(stderr, "[Logger] WARNING: cannot open %s for writing\n", log_path_.c_str());
    }

    void log(int step, const std::string& key, float value) {
        Window& w = pending_[key];
        w.sum += value;
        w.count += 1;
        pending_step_ = step;
    }

    void log(int step, const std::map<std::string, float>& metrics) {
        for (const auto& kv : metrics) log(step, kv.first, kv.second);
    }

    void commit(int step) {
        if (pending_.empty()) return;
        Entry e;
        e.step = step;
        printf("[step %d]", step);
        for (const auto& kv : pending_) {
            const float val = kv.second.count > 0 ? kv.second.sum / kv.second.count : 0.0f;
            e.values[kv.first] = val;
            if (fabsf(val) < 0.01f && val != 0.0f) printf("  %s=%.3e", kv.first.c_str(), val);
            else printf("  %s=%.4f", kv.first.c_str(), val);
        }
        printf("\n");
        if (file_) {
            fputs((to_json(e) + "\n").c_str(), file_);
            fflush(file_);
        }
        history_.push_back(e);
        pending_.clear();
    }

    const std::vector<Entry>& history() const { return history_; }

    float last(const std::string& key) const {
        for (int i = (int)history_.size() - 1; i >= 0; i--)
            if (history_[i].contains(key)) return history_[i].values.at(key);
        return std::numeric_limits<float>::quiet_NaN();
    }

    const std::string& log_path() const { return log_path_; }

    static std::string number(double x) {
        if (!std::isfinite(x)) return "null";
        char buf[64];
        auto r = std::to_chars(buf, buf + sizeof(buf), x);
        std::string s(buf, r.ptr);
        if (s.find_first_of(".e") == std::string::npos) s += ".0";
        return s;
    }

    static std::string to_json(const Entry& e) {
        std::map<std::string, std::string> fields;
        for (const auto& kv : e.values) fields[kv.first] = number((double)kv.second);
        fields["step"] = std::to_string(e.step);
        std::string out = "{";
        bool first = true;
        for (const auto& kv : fields) {
            if (!first) out += ",";
            first = false;
            out += "\"" + kv.first + "\":" + kv.second;
        }
        return out + "}";
    }

private:
    struct Window {
        float sum = 0.0f;
        int count = 0;
    };
    FILE* file_ = nullptr;
    std::string log_path_;
    std::map<std::string, Window> pending_;
    int pending_step_ = 0;
    std::vector<Entry> history_;
};

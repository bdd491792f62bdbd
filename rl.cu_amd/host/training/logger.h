// Training-metrics logger writing JSON lines: the interface of the reference's Logger
// (include/training/logger.h:27-128: open / log / commit / history / last / log_path) without its
// third-party JSON dependency.
//
//   Logger logger("checkpoints/run_001");   // appends to run_001/train_log.jsonl
//   logger.log(step, "loss", 2.34f);         // values logged for one key before commit() are averaged
//   logger.commit(step);                     // one JSON object per line, and a summary on stdout
//
// A committed line looks like
//   {"grad_norm":1.5,"loss":2.3399999141693115,"lr":9.999999747378752e-06,"step":100}
// with keys in sorted order ("step" among them) and every value the FP32 mean of its window, widened
// to double and printed in its shortest round-trip form.
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
    // One committed line.
    struct Entry {
        int step = 0;
        std::map<std::string, float> values;
        bool contains(const std::string& key) const { return values.find(key) != values.end(); }
    };

    Logger() = default;
    explicit Logger(const std::string& log_dir) { open(log_dir); }
    Logger(const Logger&) = delete;
    Logger& operator=(const Logger&) = delete;
    ~Logger() {
        if (sink_) fclose(sink_);
    }

    // log_dir empty: stdout only.  The file is opened for append so that a restarted run continues it.
    void open(const std::string& log_dir) {
        if (log_dir.empty()) return;
        std::filesystem::create_directories(log_dir);
        path_ = log_dir + "/train_log.jsonl";
        sink_ = fopen(path_.c_str(), "a");
        if (!sink_) fprintf(stderr, "[Logger] WARNING: cannot open %s for writing\n", path_.c_str());
    }

    void log(int /*step*/, const std::string& key, float value) {
        Mean& m = window_[key];
        m.total += value;
        m.samples += 1;
    }

    void log(int step, const std::map<std::string, float>& metrics) {
        for (const auto& item : metrics) log(step, item.first, item.second);
    }

    // Closes the current window: averages, prints, appends one line, remembers it.
    void commit(int step) {
        if (window_.empty()) return;
        Entry entry;
        entry.step = step;
        std::string summary = "[step " + std::to_string(step) + "]";
        for (const auto& item : window_) {
            const Mean& m = item.second;
            const float mean = m.samples > 0 ? m.total / (float)m.samples : 0.0f;
            entry.values[item.first] = mean;
            char text[96];
            const bool tiny = fabsf(mean) < 0.01f && mean != 0.0f;       // small values in scientific notation
            snprintf(text, sizeof(text), tiny ? "  %s=%.3e" : "  %s=%.4f", item.first.c_str(), mean);
            summary += text;
        }
        puts(summary.c_str());
        if (sink_) {
            const std::string line = to_json(entry) + "\n";
            fwrite(line.data(), 1, line.size(), sink_);
            fflush(sink_);
        }
        history_.push_back(entry);
        window_.clear();
    }

    const std::vector<Entry>& history() const { return history_; }

    // Most recent committed value of `key`, NaN if there is none.
    float last(const std::string& key) const {
        for (auto it = history_.rbegin(); it != history_.rend(); ++it)
            if (it->contains(key)) return it->values.at(key);
        return std::numeric_limits<float>::quiet_NaN();
    }

    const std::string& log_path() const { return path_; }

    // Shortest decimal text that reads back as the same double; integers keep a ".0".
    static std::string number(double x) {
        if (!std::isfinite(x)) return "null";
        char buf[64];
        const auto res = std::to_chars(buf, buf + sizeof(buf), x);
        std::string text(buf, res.ptr);
        if (text.find_first_of(".e") == std::string::npos) text += ".0";
        return text;
    }

    static std::string to_json(const Entry& entry) {
        std::map<std::string, std::string> fields;
        fields["step"] = std::to_string(entry.step);
        for (const auto& item : entry.values) fields[item.first] = number((double)item.second);
        std::string out;
        for (const auto& field : fields) {
            out += out.empty() ? "{\"" : ",\"";
            out += field.first + "\":" + field.second;
        }
        return out + "}";
    }

private:
    struct Mean {
        float total = 0.0f;
        int samples = 0;
    };
    FILE* sink_ = nullptr;
    std::string path_;
    std::map<std::string, Mean> window_;      // metrics logged since the last commit
    std::vector<Entry> history_;
};

#include "chrome_tracing.h"

#include <fstream>

#include "log.h"

namespace chainer_compiler {
namespace runtime {

ChromeTracingEmitter::ChromeTracingEmitter() : base_time_(Clock::now()) {
}

size_t ChromeTracingEmitter::Begin(const std::string& category, const std::string& name, int pc, int64_t flops) {
    events_.push_back(Event{category, name, pc, flops, Clock::now(), Clock::time_point()});
    return events_.size() - 1;
}

void ChromeTracingEmitter::End(size_t event) {
    events_[event].end = Clock::now();
}

void ChromeTracingEmitter::Emit(const std::string& output_filename) const {
    std::ofstream ofs(output_filename);
    CHECK(ofs) << "cannot write " << output_filename;
    auto us = [](Clock::duration d) { return static_cast<int64_t>(std::chrono::duration_cast<std::chrono::microseconds>(d).count()); };
    ofs << "[\n";
    for (size_t i = 0; i < events_.size(); ++i) {
        const Event& e = events_[i];
        if (i) ofs << ",\n";
        ofs << "{\"cat\":\"" << e.category << "\",\"name\":\"" << e.name << "\",\"ts\":" << us(e.start - base_time_)
            << ",\"dur\":" << us(e.end - e.start) << ",\"tid\":1,\"pid\":1,\"args\":{\"pc\":" << e.pc;
        if (e.flops > 0) ofs << ",\"flops\":" << e.flops;
        ofs << "},\"ph\":\"X\"}";
    }
    ofs << "\n]\n";
}

}  // namespace runtime
}  // namespace chainer_compiler

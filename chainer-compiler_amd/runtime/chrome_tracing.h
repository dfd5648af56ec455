// Per-instruction timeline in the Chrome tracing format (chrome://tracing, Perfetto), the
// --chrome_tracing output of the reference's run_onnx (runtime/chrome_tracing.{h,cc} of the
// chainer-compiler tree): one complete event ("ph":"X") per executed instruction with the op name,
// the program counter, start and duration in microseconds.
#pragma once

#include <chrono>
#include <cstdint>
#include <string>
#include <vector>

namespace chainer_compiler {
namespace runtime {

class ChromeTracingEmitter {
public:
    ChromeTracingEmitter();

    // Opens an event; the returned index closes it.
    size_t Begin(const std::string& category, const std::string& name, int pc, int64_t flops);
    void End(size_t event);

    void Emit(const std::string& output_filename) const;
    size_t size() const {
        return events_.size();
    }

private:
    using Clock = std::chrono::system_clock;
    struct Event {
        std::string category, name;
        int pc;
        int64_t flops;
        Clock::time_point start, end;
    };
    Clock::time_point base_time_;
    std::vector<Event> events_;
};

}  // namespace runtime
}  // namespace chainer_compiler

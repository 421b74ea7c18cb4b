// Time markers for the reference library's own benchmark harness on the GPU_AMD architecture.
//
// The harness (benchmarks/fkBenchmarksCommon.h of the reference) times executions through TimeMarkerOne<ARCH> and
// TimeMarkerTwo<ARCH>, which it specialises per architecture; this header supplies the ParArch::GPU_AMD ones on top of
// the event calls of the C ABI (fklhip.h).  Include order in the benchmark's translation unit:
//     #include <benchmarks/fkBenchmarksCommon.h>      // the reference's harness: declares the marker templates
//     #include <fused_kernel/amd/benchmark_markers.h>  // this file
//     #include <benchmarks/...benchmark...h>           // the benchmark itself, unchanged
#ifndef FK_AMD_BENCHMARK_MARKERS_H
#define FK_AMD_BENCHMARK_MARKERS_H

#include <array>
#include <fklhip.h>
#include <fused_kernel/core/execution_model/stream.h>
#include <fused_kernel/core/utils/utils.h>

namespace fk::amd {
// A start/stop event pair on one stream: lap() closes the running interval and returns its length in milliseconds.
class EventPair {
    void* m_start{nullptr};
    void* m_stop{nullptr};
    void* m_stream{nullptr};

public:
    explicit EventPair(fk::Stream stream) : m_stream(stream.getNativeStream()) {
        gpuErrchk(fklhip_event_create(&m_start));
        gpuErrchk(fklhip_event_create(&m_stop));
    }
    EventPair(const EventPair&) = delete;
    EventPair& operator=(const EventPair&) = delete;
    ~EventPair() {
        fklhip_event_destroy(m_start);
        fklhip_event_destroy(m_stop);
    }
    void begin() { gpuErrchk(fklhip_event_record(m_start, m_stream)); }
    float lap() {
        float ms = 0.f;
        gpuErrchk(fklhip_event_record(m_stop, m_stream));
        gpuErrchk(fklhip_event_sync(m_stop));
        gpuErrchk(fklhip_event_elapsed_ms(&ms, m_start, m_stop));
        return ms;
    }
};
inline void account(const float ms, float& longest, float& shortest, float& total) {
    if (ms > longest) longest = ms;
    if (ms < shortest) shortest = ms;
    total += ms;
}
} // namespace fk::amd

template <> class TimeMarkerOne<fk::ParArch::GPU_AMD> final : public TimeMarkerInterfaceOne {
    fk::amd::EventPair m_events;
    std::array<float, ITERS> m_elapsedTime{};

public:
    TimeMarkerOne(fk::Stream stream) : m_events(stream) {}
    void start() final { m_events.begin(); }
    void stop(BenchmarkResultsNumbersOne& resF, const int& idx) final {
        m_elapsedTime[idx] = m_events.lap();
        fk::amd::account(m_elapsedTime[idx], resF.fkElapsedTimeMax, resF.fkElapsedTimeMin, resF.fkElapsedTimeAcum);
    }
    std::array<float, ITERS> getElapsedTime() const final { return m_elapsedTime; }
};

template <> class TimeMarkerTwo<fk::ParArch::GPU_AMD> final : public TimeMarkerInterfaceTwo {
    fk::amd::EventPair m_events;
    std::array<float, ITERS> m_firstElapsedTime{};
    std::array<float, ITERS> m_secondElapsedTime{};

public:
    TimeMarkerTwo(fk::Stream stream) : m_events(stream) {}
    void startFirst() final { m_events.begin(); }
    void stopFirstStartSecond(BenchmarkResultsNumbersTwo& resF, const int& idx) final {
        m_firstElapsedTime[idx] = m_events.lap();
        fk::amd::account(m_firstElapsedTime[idx], resF.firstElapsedTimeMax, resF.firstElapsedTimeMin, resF.firstElapsedTimeAcum);
        m_events.begin();
    }
    void stopSecond(BenchmarkResultsNumbersTwo& resF, const int& idx) final {
        m_secondElapsedTime[idx] = m_events.lap();
        fk::amd::account(m_secondElapsedTime[idx], resF.secondElapsedTimeMax, resF.secondElapsedTimeMin, resF.secondElapsedTimeAcum);
    }
    std::array<float, ITERS> getFirstElapsedTime() const final { return m_firstElapsedTime; }
    std::array<float, ITERS> getSecondElapsedTime() const final { return m_secondElapsedTime; }
};

#endif

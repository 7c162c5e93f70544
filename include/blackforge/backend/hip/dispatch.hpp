#pragma once
// Device dispatch for the HIP backend: what `blackforge run|train|devices --device ...` needs in order to reach
// hip::Executor, hip::Model and hip::runTraining; likewise the GPU branches of `generate` and `benchmark`.  The reference's CLI parses `cpu | cuda | cuda:N` into a DeviceSpec
// and branches on it (src/main.cpp:118-186 parse, :298-395 run, :397-476 train, :86-112 devices); its runtime has
// DeviceKind{CPU, CUDA} (include/blackforge/runtime/device.hpp:8) and its semantic analyser a closed list of target
// names (src/sema/semantic_analyzer.cpp:12-17,139-144).  This header supplies the same pieces with `hip | hip:N` added:
// the parser (same diagnostics, same exit-code meaning), the device family, the target-name check, the `devices`
// listing, and the bodies of the run / train branches as functions over the reference's own ir / ast types, so the
// CLI's edit is one `else if (spec.family == DeviceFamily::Hip)` per command.  Nothing here parses .bf programs or
// text: `generate` starts from token ids (the tokenizer stays on the host side of the CLI).
#include <algorithm>
#include <cctype>
#include <chrono>
#include <cstddef>
#include <cstdint>
#include <iosfwd>
#include <ostream>
#include <string>
#include <vector>

#include "blackforge/backend/hip/device_query.hpp"

namespace blackforge::backend::hip {

// runtime::DeviceKind with the third family (device.hpp:8 has CPU and CUDA).
enum class DeviceFamily { Cpu, Cuda, Hip };

struct DeviceSpec {
    DeviceFamily family = DeviceFamily::Cpu;
    int index = 0;
    [[nodiscard]] bool isGpu() const { return family != DeviceFamily::Cpu; }
    [[nodiscard]] std::string toString() const {
        if (family == DeviceFamily::Cpu) return "cpu";
        return std::string(family == DeviceFamily::Cuda ? "cuda:" : "hip:") + std::to_string(index);
    }
};

// `--device cpu | cuda | cuda:N | hip | hip:N`.  Returns false and fills `error` (the text main.cpp prints after
// "errore: " before exiting with status 2) for anything else; a bare family name means device 0.
inline bool parseDeviceSpec(const std::string& device, DeviceSpec& spec, std::string& error) {
    if (device == "cpu") {
        spec = DeviceSpec{DeviceFamily::Cpu, 0};
        return true;
    }
    for (const auto& [prefix, family] : {std::pair<const char*, DeviceFamily>{"cuda", DeviceFamily::Cuda}, {"hip", DeviceFamily::Hip}}) {
        const std::string name(prefix);
        if (device == name) {
            spec = DeviceSpec{family, 0};
            return true;
        }
        if (device.compare(0, name.size() + 1, name + ":") != 0) continue;
        const std::string digits = device.substr(name.size() + 1);
        const bool numeric = !digits.empty() && digits.size() <= 6 &&
                             std::all_of(digits.begin(), digits.end(), [](unsigned char c) { return std::isdigit(c) != 0; });
        if (!numeric) {
            error = "indice GPU non valido in '" + device + "'";
            return false;
        }
        spec = DeviceSpec{family, std::stoi(digits)};
        return true;
    }
    error = "dispositivo sconosciuto '" + device + "' (valori validi: cpu, cuda, cuda:N, hip, hip:N)";
    return false;
}

// Target names of the `target` declaration that select this backend, to be added to the analyser's known targets
// (semantic_analyzer.cpp:12-17 lists nvidia.blackwell, nvidia.hopper, nvidia.ampere, nvidia.ada, cpu).
inline const std::vector<std::string>& hipTargetNames() {
    static const std::vector<std::string> names = {"amd.cdna4", "amd.mi355x", "amd.gfx950"};
    return names;
}
inline bool isHipTarget(const std::string& target) {
    const auto& names = hipTargetNames();
    return std::find(names.begin(), names.end(), target) != names.end();
}

// The `blackforge devices` lines for this backend (main.cpp:86-112 prints "cuda:N: name (compute capability ...)").
inline void listDevices(std::ostream& out) {
    const std::vector<HipDeviceInfo> devices = enumerateDevices();
    if (devices.empty()) out << "hip: nessuna GPU AMD rilevata (nessun dispositivo visibile al driver)\n";
    for (const HipDeviceInfo& d : devices)
        out << "hip:" << d.index << ": " << d.name << " (" << d.arch << ", " << d.computeUnits << " CU, "
            << (d.totalMemoryBytes / (1024ULL * 1024ULL)) << " MiB)\n";
}

// Makes the device of a parsed spec current.  Throws std::invalid_argument for a family this backend does not serve or
// an index that does not exist (setActiveDevice, device_query.cu:34-40).
inline void selectDevice(const DeviceSpec& spec) {
    require(spec.family == DeviceFamily::Hip, "hip::selectDevice: '" + spec.toString() + "' is not a HIP device");
    setActiveDevice(spec.index);
}

}  // namespace blackforge::backend::hip

// The run / train branches need the IR, the AST and the seeded generators: available inside a BlackForge build.
#if __has_include("blackforge/ir/module.hpp") && __has_include("blackforge/ast/ast.hpp") && \
    __has_include("blackforge/backend/cpu/random_init.hpp")
#include "blackforge/backend/hip/checkpoint.hpp"
#include "blackforge/backend/hip/executor.hpp"
#include "blackforge/backend/hip/train_runner.hpp"

namespace blackforge::backend::hip {

struct RunOutcome {
    runtime::Tensor input;
    runtime::Tensor output;
    bool loadedCheckpoint = false;
};

// The GPU branch of runRun (main.cpp:356-382): synthetic input for `batchSize`, then either the executor with
// regenerated seed-42 weights or, with a checkpoint, a Model of the module's precision policy that loads it.
inline RunOutcome runOnDevice(const DeviceSpec& spec, const ir::Module& module, std::size_t batchSize, const std::string& fromCheckpoint = "") {
    require(!module.models.empty(), "il programma non definisce alcun modello da eseguire");
    selectDevice(spec);
    const ir::ModelIR& model = module.models.front();
    Executor executor;
    RunOutcome outcome;
    outcome.input = executor.makeSyntheticInput(model, batchSize);
    if (fromCheckpoint.empty()) {
        outcome.output = executor.run(model, outcome.input);
    } else {
        Model loaded(model, 42U, module.precision);
        loadCheckpoint(loaded, fromCheckpoint);
        outcome.loadedCheckpoint = true;
        outcome.output = loaded.forward(DeviceTensor::fromHost(outcome.input)).toHost();
    }
    return outcome;
}

// The GPU branch of runTrain (main.cpp:464-467).
inline TrainRunResult trainOnDevice(const DeviceSpec& spec, const ast::Program& program, const ir::Module& module,
                                    const std::string& fromCheckpoint, const std::string& saveCheckpointPath, std::ostream* progress) {
    selectDevice(spec);
    return runTraining(program, module, fromCheckpoint, saveCheckpointPath, progress);
}

// The GPU branch of runGenerate (main.cpp:594-617), from token ids to token ids: the model of the module's precision
// policy loads the checkpoint, the prompt goes through forwardIncremental once and every further token alone, each
// chosen as the first maximum of the last position's logits (main.cpp:504-518).  The choice is made on the device; for a
// pipeline from token ids to logits over the same vocabulary the token never leaves it (Model::generateGreedy: the ids
// are read back once, at the end), otherwise one index per token crosses to the host instead of the logits.  Like the CLI, generation stops quietly when the model
// refuses a further position (its positional table is exhausted); `stoppedAtCapacity` reports that.
struct GenerateOutcome {
    std::vector<std::uint32_t> tokens;   // the prompt followed by the generated ids
    bool stoppedAtCapacity = false;
};

inline GenerateOutcome generateOnDevice(const DeviceSpec& spec, const ir::Module& module, const std::string& fromCheckpoint,
                                        const std::vector<std::uint32_t>& promptIds, std::size_t maxNewTokens) {
    require(!module.models.empty(), "il programma non definisce alcun modello da eseguire");
    require(!promptIds.empty(), "il prompt codificato e' vuoto (prompt vuoto?)");
    selectDevice(spec);
    Model loaded(module.models.front(), 42U, module.precision);
    loadCheckpoint(loaded, fromCheckpoint);
    loaded.resetGenerationState();
    GenerateOutcome outcome;
    outcome.tokens = promptIds;
    const std::vector<float> promptFloats(promptIds.begin(), promptIds.end());
    const std::size_t promptLen = promptIds.size(), limit = loaded.maxPositions();
    if (maxNewTokens > 0 && promptLen <= limit && loaded.supportsGenerateGreedy()) {
        // the same loop with token and position kept on the device (Model::generateGreedy): the step that would feed a token
        // at position `limit` is the one the loop below stops at
        const std::size_t untilFull = limit - promptLen + 1;
        const std::size_t count = std::min(maxNewTokens, untilFull);
        outcome.stoppedAtCapacity = maxNewTokens >= untilFull;
        for (std::size_t id : loaded.generateGreedy(DeviceTensor::fromHost(runtime::Tensor({1, promptLen}, promptFloats)), count))
            outcome.tokens.push_back(static_cast<std::uint32_t>(id));
        return outcome;
    }
    DeviceTensor logits = loaded.forwardIncremental(DeviceTensor::fromHost(runtime::Tensor({1, promptIds.size()}, promptFloats)));
    for (std::size_t step = 0; step < maxNewTokens; ++step) {
        const auto best = static_cast<std::uint32_t>(argmaxLastPosition(logits));
        outcome.tokens.push_back(best);
        try {
            logits = loaded.forwardIncremental(DeviceTensor::fromHost(runtime::Tensor({1, 1}, {static_cast<float>(best)})));
        } catch (const std::exception&) {
            outcome.stoppedAtCapacity = true;
            break;
        }
    }
    return outcome;
}

// The GPU branch of runBenchmark (main.cpp:801-850): the executor on a synthetic batch, `warmupIterations` untimed runs,
// then `measuredIterations` timed with the host clock (each run ends in a device-to-host copy, so the clock sees
// finished work), mean milliseconds and examples per second, and the last output for the comparison with the CPU run.
struct BenchmarkOutcome {
    std::string deviceName;
    std::vector<std::size_t> inputShape;
    double meanMilliseconds = 0.0;
    double throughputSamplesPerSecond = 0.0;
    runtime::Tensor output;
};

inline BenchmarkOutcome benchmarkOnDevice(const DeviceSpec& spec, const ir::ModelIR& model, std::size_t batchSize,
                                          std::size_t warmupIterations, std::size_t measuredIterations) {
    require(measuredIterations > 0, "benchmarkOnDevice: needs at least one measured iteration");
    selectDevice(spec);
    BenchmarkOutcome outcome;
    outcome.deviceName = "GPU sconosciuta";
    for (const HipDeviceInfo& d : enumerateDevices())
        if (d.index == spec.index) outcome.deviceName = d.name.empty() ? d.arch : d.name;   // some drivers report no marketing name
    Executor executor;
    const runtime::Tensor input = executor.makeSyntheticInput(model, batchSize);
    outcome.inputShape = input.shape();
    for (std::size_t i = 0; i < warmupIterations; ++i) (void)executor.run(model, input);
    const auto start = std::chrono::steady_clock::now();
    for (std::size_t i = 0; i < measuredIterations; ++i) outcome.output = executor.run(model, input);
    const auto end = std::chrono::steady_clock::now();
    outcome.meanMilliseconds = std::chrono::duration<double, std::milli>(end - start).count() / static_cast<double>(measuredIterations);
    outcome.throughputSamplesPerSecond = outcome.meanMilliseconds > 0.0 ? static_cast<double>(batchSize) * 1000.0 / outcome.meanMilliseconds : 0.0;
    return outcome;
}

}  // namespace blackforge::backend::hip
#endif

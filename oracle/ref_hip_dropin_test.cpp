// Drop-in check of the HIP operator layer against the REAL reference front end and CPU backend -- TEST
// INFRASTRUCTURE ONLY.  Built by oracle/Makefile into oracle/_ref/hip_dropin_test together with the reference's own
// source files (where they lie); runs on a GPU box.  The same ir::ModelIR / ast::Program objects are handed to
// blackforge::backend::cpu and blackforge::backend::hip:
//   1. Executor: same synthetic input, outputs equal within 1e-4 (weights come from the same seeded generators);
//   2. Model(ir, 42): same parameter names, shapes and initial values as cpu::Model;
//   3. runTraining(program, module, "", save): same epoch losses (1e-4) and final checkpoints (tolerance below),
//      both backends starting from their own seed-42 initialisation and reading the same BFDATA1 file;
//   4. checkpoint interop: the CPU run's file loads into hip::Model and the other way round;
//   5. device dispatch (hip/dispatch.hpp): `--device hip` / `hip:0` reach hip::Executor, hip::Model and hip::runTraining
//      through runOnDevice / trainOnDevice with the results of steps 1 and 3; `hip:99` and `cuda` are refused;
//   6. generate: greedy decoding from a trained checkpoint through generateOnDevice gives the token ids of the CPU
//      model's forwardIncremental + first-maximum loop, including the stop when the positional table is exhausted;
//   7. benchmark: benchmarkOnDevice times the executor and its last output matches the CPU executor's.
// Prints one line per check and exits non-zero on the first failure.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "blackforge/ast/ast.hpp"
#include "blackforge/backend/cpu/checkpoint.hpp"
#include "blackforge/backend/cpu/executor.hpp"
#include "blackforge/backend/cpu/model.hpp"
#include "blackforge/backend/cpu/train_runner.hpp"
#include "blackforge/backend/hip/checkpoint.hpp"
#include "blackforge/backend/hip/dispatch.hpp"
#include "blackforge/backend/hip/executor.hpp"
#include "blackforge/backend/hip/model.hpp"
#include "blackforge/backend/hip/train_runner.hpp"
#include "blackforge/data/dataset.hpp"
#include "blackforge/ir/module.hpp"

namespace bf = blackforge;
namespace cpu = blackforge::backend::cpu;
namespace hip = blackforge::backend::hip;
namespace ir = blackforge::ir;
namespace ast = blackforge::ast;

static int failures = 0;
static void report(bool ok, const std::string& what) {
    std::printf("[%s] %s\n", ok ? "  OK  " : " FAIL ", what.c_str());
    std::fflush(stdout);
    if (!ok) ++failures;
}
static double maxRelError(const std::vector<float>& got, const std::vector<float>& want, double floor) {
    if (got.size() != want.size()) return 1e30;
    double rms = 0.0;
    for (float w : want) rms += double(w) * w;
    rms = std::sqrt(rms / double(want.empty() ? 1 : want.size()));
    double worst = 0.0;
    for (std::size_t i = 0; i < got.size(); ++i) {
        double err = std::fabs(double(got[i]) - double(want[i])) / (std::fabs(double(want[i])) + std::max(rms, floor));
        if (!(err <= worst)) worst = err;
    }
    return worst;
}

struct LayerDesc { ir::OpKind kind; long long a0, a1; };
static ir::ModelIR makeModel(const std::string& name, const std::vector<LayerDesc>& layers, std::vector<ir::Dim> inputShape) {
    ir::ModelIR m;
    m.name = name;
    auto value = [&](std::size_t id, std::vector<ir::Dim> shape) {
        ir::Value v;
        v.id = id;
        v.dtype = bf::sema::DType::FP32;
        v.shape = std::move(shape);
        return v;
    };
    m.values.push_back(value(0, inputShape));
    m.inputValue = 0;
    ir::Pipeline p;
    p.sourceValue = 0;
    long long features = inputShape.back().literalValue;   // last dimension of the running value
    for (std::size_t i = 0; i < layers.size(); ++i) {
        ir::Operation op{};
        op.input = i;
        op.output = i + 1;
        op.kind = layers[i].kind;
        switch (op.kind) {
            case ir::OpKind::Linear: op.linearOutFeatures = layers[i].a0; features = layers[i].a0; break;
            case ir::OpKind::Embedding: op.embeddingVocabSize = layers[i].a0; op.embeddingDim = layers[i].a1; features = layers[i].a1; break;
            case ir::OpKind::PositionalEmbedding: op.positionalMaxSeqLen = layers[i].a0; break;
            case ir::OpKind::Attention:
            case ir::OpKind::BidirectionalAttention: op.attentionNumHeads = layers[i].a0; break;
            case ir::OpKind::FeedForward: op.feedForwardHiddenDim = layers[i].a0; break;
            default: break;
        }
        m.values.push_back(value(i + 1, {ir::Dim{true, "batch", 0}, ir::Dim{false, "", features}}));
        p.operations.push_back(op);
    }
    m.pipelines.push_back(std::move(p));
    return m;
}

static ast::Program makeProgram(const std::string& model, const std::string& datasetPath, const std::string& loss, const std::string& optimizer,
                                long long epochs, long long batch, double lr, bool cosine) {
    ast::Program program;
    ast::DatasetDecl dataset;
    dataset.name = "data";
    dataset.fields.push_back(ast::DatasetPathField{datasetPath, {}});
    program.declarations.push_back(dataset);
    ast::TrainDecl train;
    train.fields.push_back(ast::TrainModelField{model, {}});
    train.fields.push_back(ast::TrainDatasetField{"data", {}});
    train.fields.push_back(ast::TrainLossField{loss, {}});
    train.fields.push_back(ast::TrainOptimizerField{optimizer, {}});
    train.fields.push_back(ast::TrainEpochsField{epochs, {}});
    train.fields.push_back(ast::TrainBatchSizeField{batch, {}});
    train.fields.push_back(ast::TrainLearningRateField{lr, {}});
    if (cosine) train.fields.push_back(ast::TrainLrScheduleField{"cosine", {}});
    program.declarations.push_back(train);
    return program;
}

int main(int argc, char** argv) {
    const std::string tmp = argc > 1 ? argv[1] : "/tmp";
    const ir::Dim batchDim{true, "batch", 0};
    auto lit = [](long long v) { return ir::Dim{false, "", v}; };
    ir::ModelIR lm = makeModel("tiny_lm",
                               {{ir::OpKind::Embedding, 48, 32}, {ir::OpKind::PositionalEmbedding, 12, 0}, {ir::OpKind::Attention, 4, 0},
                                {ir::OpKind::FeedForward, 64, 0}, {ir::OpKind::RmsNorm, 0, 0}, {ir::OpKind::Linear, 48, 0}},
                               {batchDim, lit(12)});
    ir::ModelIR mlp = makeModel("mlp", {{ir::OpKind::Linear, 24, 0}, {ir::OpKind::Silu, 0, 0}, {ir::OpKind::Linear, 24, 0}, {ir::OpKind::Gelu, 0, 0},
                                       {ir::OpKind::Linear, 5, 0}, {ir::OpKind::Softmax, 0, 0}},
                                {batchDim, lit(10)});
    // a masked language model: the CPU backend runs it, the CUDA backend refuses it (model.cu:151-160)
    ir::ModelIR mlm = makeModel("tiny_mlm",
                                {{ir::OpKind::Embedding, 48, 32}, {ir::OpKind::PositionalEmbedding, 12, 0}, {ir::OpKind::BidirectionalAttention, 4, 0},
                                 {ir::OpKind::FeedForward, 64, 0}, {ir::OpKind::Linear, 48, 0}},
                                {batchDim, lit(12)});
    try {
        // 1. executors
        for (const ir::ModelIR* m : {&lm, &mlp, &mlm}) {
            cpu::Executor cx(42);
            hip::Executor hx(42);
            bf::runtime::Tensor in = cx.makeSyntheticInput(*m, 6), inHip = hx.makeSyntheticInput(*m, 6);
            report(in.shape() == inHip.shape() && in.data() == inHip.data(), m->name + ": Executor::makeSyntheticInput identical");
            bf::runtime::Tensor want = cx.run(*m, in), got = hx.run(*m, in);
            double err = maxRelError(got.data(), want.data(), 1e-6);
            report(want.shape() == got.shape() && err <= 1e-4, m->name + ": Executor::run matches the CPU executor (max rel err " + std::to_string(err) + ")");
        }
        // 2. model initialisation
        {
            cpu::Model cm(lm, 42U);
            hip::Model hm(lm, 42U);
            auto cp = cm.parameters();
            auto hp = hm.parameters();
            bool same = cp.size() == hp.size();
            for (std::size_t i = 0; same && i < cp.size(); ++i) {
                same = cp[i]->name == hp[i]->name && cp[i]->value.shape() == hp[i]->value.shape() && cp[i]->value.data() == hp[i]->value.toHost().data();
            }
            report(same, "Model(ir, 42): parameter names, shapes and initial values identical to cpu::Model");
        }
        // 3. training runs from the same program
        struct Run { const ir::ModelIR* model; std::string loss, optimizer; long long epochs, batch; double lr; bool cosine; };
        std::vector<float> ids(30 * 12), tgt(30 * 12), x(40 * 10), y(40 * 5);
        unsigned s = 7;
        auto next = [&]() { s = s * 1664525u + 1013904223u; return (s >> 8) & 0xffffu; };
        for (auto& v : ids) v = float(next() % 48);
        for (auto& v : tgt) v = float(next() % 48);
        for (auto& v : x) v = float(next()) / 32768.0f - 1.0f;
        for (std::size_t i = 0; i < 40; ++i) {
            float sum = 0.0f;
            for (int j = 0; j < 5; ++j) { y[i * 5 + j] = float(next() % 100 + 1); sum += y[i * 5 + j]; }
            for (int j = 0; j < 5; ++j) y[i * 5 + j] /= sum;
        }
        std::vector<float> maskedTgt(ids.size());
        for (std::size_t i = 0; i < ids.size(); ++i) maskedTgt[i] = next() % 4 == 0 ? ids[i] : -1.0f;   // a quarter of the positions count
        bf::data::saveDataset(tmp + "/dropin_mlm.bfdata", {12}, {12}, ids, maskedTgt, 30);
        bf::data::saveDataset(tmp + "/dropin_lm.bfdata", {12}, {12}, ids, tgt, 30);
        bf::data::saveDataset(tmp + "/dropin_mlp.bfdata", {10}, {5}, x, y, 40);
        std::vector<Run> runs = {{&lm, "cross_entropy_sparse", "adamw", 3, 5, 5e-3, true}, {&mlp, "mse", "sgd", 3, 8, 0.1, false},
                                 {&mlm, "cross_entropy_masked", "adamw", 3, 5, 5e-3, false}};
        for (const Run& r : runs) {
            const std::string data = tmp + (r.model == &lm ? "/dropin_lm.bfdata" : r.model == &mlm ? "/dropin_mlm.bfdata" : "/dropin_mlp.bfdata");
            ast::Program program = makeProgram(r.model->name, data, r.loss, r.optimizer, r.epochs, r.batch, r.lr, r.cosine);
            ir::Module module;
            module.models.push_back(*r.model);
            const std::string cpuCkpt = tmp + "/dropin_" + r.model->name + "_cpu.bfckpt", hipCkpt = tmp + "/dropin_" + r.model->name + "_hip.bfckpt";
            cpu::TrainRunResult want = cpu::runTraining(program, module, "", cpuCkpt, nullptr);
            hip::TrainRunResult got = hip::runTraining(program, module, "", hipCkpt, nullptr);
            bool lossesOk = want.epochLosses.size() == got.epochLosses.size() && want.modelName == got.modelName;
            double worst = 0.0;
            for (std::size_t e = 0; lossesOk && e < want.epochLosses.size(); ++e) {
                worst = std::max(worst, std::fabs(got.epochLosses[e] - want.epochLosses[e]) / std::fabs(want.epochLosses[e]));
            }
            report(lossesOk && worst <= 1e-4, r.model->name + ": runTraining(program, module) epoch losses match cpu::runTraining (max rel diff " + std::to_string(worst) + ")");
            // 4. interop both ways + final weights
            cpu::Model cm(*r.model, 42U);
            hip::Model hm(*r.model, 42U);
            cpu::loadCheckpoint(cm, hipCkpt);   // HIP file into the CPU model
            hip::loadCheckpoint(hm, cpuCkpt);   // CPU file into the HIP model
            auto cp = cm.parameters();
            auto hp = hm.parameters();
            double werr = 0.0;
            for (std::size_t i = 0; i < cp.size(); ++i) werr = std::max(werr, maxRelError(cp[i]->value.data(), hp[i]->value.toHost().data(), 2e-2));
            report(werr <= 2e-2, r.model->name + ": checkpoints interchange between the backends; trained weights agree (max rel err " + std::to_string(werr) + ")");
        }
        // 5. the dispatch a CLI would go through
        {
            hip::DeviceSpec spec;
            std::string error;
            ir::Module module;
            module.models.push_back(lm);
            for (const char* name : {"hip", "hip:0"}) {
                bool parsed = hip::parseDeviceSpec(name, spec, error);
                hip::RunOutcome outcome = hip::runOnDevice(spec, module, 6);
                cpu::Executor cx(42);
                bf::runtime::Tensor want = cx.run(lm, cx.makeSyntheticInput(lm, 6));
                double err = maxRelError(outcome.output.data(), want.data(), 1e-6);
                report(parsed && outcome.output.shape() == want.shape() && err <= 1e-4,
                       std::string("--device ") + name + ": runOnDevice gives the CPU executor's output (max rel err " + std::to_string(err) + ")");
            }
            const std::string ckpt = tmp + "/dropin_tiny_lm_cpu.bfckpt";   // written by the CPU training run above
            hip::parseDeviceSpec("hip:0", spec, error);
            hip::RunOutcome fromFile = hip::runOnDevice(spec, module, 4, ckpt);
            cpu::Model cm(lm, 42U);
            cpu::loadCheckpoint(cm, ckpt);
            double err = maxRelError(fromFile.output.data(), cm.forward(fromFile.input).data(), 1e-6);
            report(fromFile.loadedCheckpoint && err <= 1e-4, "--device hip:0 --from-checkpoint: output of the loaded weights matches cpu::Model (max rel err " + std::to_string(err) + ")");
            ast::Program program = makeProgram(lm.name, tmp + "/dropin_lm.bfdata", "cross_entropy_sparse", "adamw", 2, 5, 5e-3, false);
            cpu::TrainRunResult want = cpu::runTraining(program, module, "", "", nullptr);
            hip::TrainRunResult got = hip::trainOnDevice(spec, program, module, "", "", nullptr);
            double worst = 0.0;
            for (std::size_t e = 0; e < want.epochLosses.size() && e < got.epochLosses.size(); ++e)
                worst = std::max(worst, std::fabs(got.epochLosses[e] - want.epochLosses[e]) / std::fabs(want.epochLosses[e]));
            report(got.epochLosses.size() == want.epochLosses.size() && worst <= 1e-4, "--device hip:0: trainOnDevice epoch losses match cpu::runTraining");
            auto refused = [&](const char* name) {
                if (!hip::parseDeviceSpec(name, spec, error)) return false;
                try { (void)hip::runOnDevice(spec, module, 2); } catch (const std::invalid_argument&) { return true; }
                return false;
            };
            report(refused("hip:99"), "--device hip:99 parses and is refused at selection (std::invalid_argument)");
            report(refused("cuda"), "--device cuda parses and is refused by the HIP backend");
            report(!hip::parseDeviceSpec("hip:x", spec, error) && error == "indice GPU non valido in 'hip:x'", "--device hip:x is a parse error");
        }
        // 6. greedy generation from the CPU run's checkpoint (the loop of runGenerate, src/main.cpp:575-592)
        {
            hip::DeviceSpec spec;
            std::string error;
            hip::parseDeviceSpec("hip:0", spec, error);
            ir::Module module;
            module.models.push_back(lm);
            const std::string ckpt = tmp + "/dropin_tiny_lm_cpu.bfckpt";
            auto cpuGenerate = [&](const std::vector<std::uint32_t>& prompt, std::size_t maxNew, bool& stopped) {
                cpu::Model cm(lm);
                cpu::loadCheckpoint(cm, ckpt);
                cm.resetGenerationState();
                std::vector<std::uint32_t> out = prompt;
                std::vector<float> pf(prompt.begin(), prompt.end());
                bf::runtime::Tensor logits = cm.forwardIncremental(bf::runtime::Tensor({1, prompt.size()}, pf));
                stopped = false;
                for (std::size_t step = 0; step < maxNew; ++step) {
                    const std::size_t vocab = logits.dim(2), last = logits.dim(1) - 1;
                    std::size_t best = 0;
                    for (std::size_t v = 1; v < vocab; ++v)
                        if (logits.at(last * vocab + v) > logits.at(last * vocab + best)) best = v;
                    out.push_back(static_cast<std::uint32_t>(best));
                    try {
                        logits = cm.forwardIncremental(bf::runtime::Tensor({1, 1}, {static_cast<float>(best)}));
                    } catch (const std::exception&) { stopped = true; break; }
                }
                return out;
            };
            for (const auto& [prompt, maxNew] : std::vector<std::pair<std::vector<std::uint32_t>, std::size_t>>{{{3, 17, 40}, 4}, {{5}, 8}, {{1, 2, 3, 4, 5, 6, 7}, 20}}) {
                bool stopped = false;
                std::vector<std::uint32_t> want = cpuGenerate(prompt, maxNew, stopped);
                hip::GenerateOutcome got = hip::generateOnDevice(spec, module, ckpt, prompt, maxNew);
                report(got.tokens == want && got.stoppedAtCapacity == stopped,
                       "generate: " + std::to_string(prompt.size()) + " prompt tokens + " + std::to_string(maxNew) + " requested -> " +
                           std::to_string(got.tokens.size()) + " ids identical to the CPU loop" + (stopped ? " (both stop at the positional table's end)" : ""));
            }
        }
        // 7. the benchmark command's GPU branch (src/main.cpp:801-850)
        {
            hip::DeviceSpec spec;
            std::string error;
            hip::parseDeviceSpec("hip", spec, error);
            hip::BenchmarkOutcome outcome = hip::benchmarkOnDevice(spec, mlp, 16, 2, 5);
            cpu::Executor cx;
            bf::runtime::Tensor want = cx.run(mlp, cx.makeSyntheticInput(mlp, 16));
            float maxAbsDiff = 0.0F;
            for (std::size_t i = 0; i < want.elementCount() && i < outcome.output.elementCount(); ++i)
                maxAbsDiff = std::max(maxAbsDiff, std::fabs(want.at(i) - outcome.output.at(i)));
            report(outcome.output.shape() == want.shape() && maxAbsDiff <= 1e-5F && outcome.meanMilliseconds > 0.0 && outcome.throughputSamplesPerSecond > 0.0 &&
                       outcome.inputShape == std::vector<std::size_t>{16, 10} && !outcome.deviceName.empty(),
                   "benchmark: benchmarkOnDevice on '" + outcome.deviceName + "' " + std::to_string(outcome.meanMilliseconds) + " ms per run, max abs diff vs the CPU executor " +
                       std::to_string(maxAbsDiff));
        }
    } catch (const std::exception& e) {
        report(false, std::string("exception: ") + e.what());
    }
    std::printf("%d failure(s)\n", failures);
    return failures == 0 ? 0 : 1;
}

#pragma once
// One training step of hip::Model recorded as a HIP graph and replayed.
//
// The reference's training loop (src/backend/cuda/train_runner.cu:203-236) launches every kernel of every step from the
// host: zeroGrad, forward, loss, backward, optimizer.  For a small model (the tiny language model of the reference's
// own tests runs ~95 kernels of a few microseconds each) the step is bounded by those launches, not by the GPU.
// CapturedTrainStep runs the same calls once while the library records them (bf_hip_capture_begin/end) and then
// replays the recording: one submission per step.  The replay executes the kernels the eager loop would have launched,
// with the same arguments, so parameters, gradients and the accumulated loss are bit-identical to the eager loop's.
//
// What a recording fixes, and what it therefore asks of the caller:
//   * the input and target tensors are read where they lay when the step was recorded: write each batch INTO them
//     (same shapes), do not replace them;
//   * token ids are not range-checked on the device during the step (that check reads a flag back to the host):
//     validate them on the host first, as the reference's runner does (train_runner.cu:210-212);
//   * the learning rate and AdamW's step count are read from device memory (Optimizer::publishStep), so schedules
//     and the bias corrections work as in the eager loop;
//   * the model's parameters must not be reallocated while the recording lives (loadCheckpoint writes in place).
// Replays are asynchronous on the recording's stream, which eager work on the default stream waits for.
#include <stdexcept>
#include <string>

#include "blackforge/backend/hip/loss.hpp"
#include "blackforge/backend/hip/model.hpp"
#include "blackforge/backend/hip/optimizer.hpp"

namespace blackforge::backend::hip {

// The loss names of the `train` block (cpu/train_runner.cpp:128-133) -> gradient of the loss, its value added to
// lossAccumulator on the device.
inline DeviceTensor lossGradientAccumulate(const std::string& loss, const DeviceTensor& output, const DeviceTensor& target,
                                           DeviceTensor& lossAccumulator, bool gradImage) {
    if (loss == "cross_entropy_sparse") return softmaxCrossEntropySparseAccumulate(output, target, lossAccumulator, gradImage);
    if (loss == "cross_entropy_masked") return softmaxCrossEntropyMaskedAccumulate(output, target, lossAccumulator);
    if (loss == "cross_entropy") return softmaxCrossEntropyAccumulate(output, target, lossAccumulator);
    return meanSquaredErrorAccumulate(output, target, lossAccumulator, gradImage);   // every other name, as in the runner
}

// Loss (added to lossAccumulator) and backward pass of one step.  A bf16 model that ends in a linear head takes the
// sparse cross-entropy through the fused form (softmaxCrossEntropySparseHeadAccumulate: gradient as a bf16 image plus the
// head's bias gradient, no fp32 gradient), every other combination through lossGradientAccumulate.  Everyone who runs a
// training step (the runner, the recorded step, the harness) comes through here, so that their steps agree bit for bit.
inline void lossAndBackward(Model& model, const std::string& loss, const DeviceTensor& output, const DeviceTensor& target,
                            DeviceTensor& lossAccumulator, bool inputRangeTrusted) {
    if (loss == "cross_entropy_sparse" && model.headTakesImageGradient()) {
        DeviceTensor grad, biasGrad;
        if (softmaxCrossEntropySparseHeadAccumulate(output, target, lossAccumulator, grad, biasGrad)) {
            model.backward(grad, inputRangeTrusted, &biasGrad);
            return;
        }
    }
    DeviceTensor grad = lossGradientAccumulate(loss, output, target, lossAccumulator, model.usesBf16());
    model.backward(grad, inputRangeTrusted);
}

class CapturedTrainStep {
public:
    // Records zeroGrad + forward + loss + backward + optimizer update for tensors of these shapes.  Nothing is executed:
    // parameters, optimizer state and lossAccumulator are as they were when the constructor returns.  The model's
    // activation caches are NOT: recording walked the layers for their host side effects and left the caches pointing at
    // buffers no kernel has written, so the constructor marks them invalid (Model::invalidateCaches): an eager backward()
    // needs an eager forward() after the recording, and throws otherwise.  The same holds after a recording that failed.
    CapturedTrainStep(Model& model, Optimizer& optimizer, const std::string& loss, const DeviceTensor& input, const DeviceTensor& target,
                      DeviceTensor& lossAccumulator)
        : optimizer_(optimizer) {
        optimizer.prepareRecording(model.parameters());
        check(bf_hip_stream_create(&stream_));
        int status = bf_hip_capture_begin(stream_);
        if (status != BF_OK) {
            bf_hip_stream_destroy(stream_);
            check(status);
        }
        try {
            model.zeroGrad(/*deferred=*/true);
            DeviceTensor output = model.forward(input, /*inputRangeTrusted=*/true);
            outputRows_ = output.elementCount() / output.shape().back();
            outputElements_ = output.elementCount();
            lossAndBackward(model, loss, output, target, lossAccumulator, /*inputRangeTrusted=*/true);
            optimizer.recordStep(model.parameters());
        } catch (...) {
            bf_hip_capture_end(nullptr);   // abandon the recording, return its memory
            bf_hip_stream_destroy(stream_);
            model.invalidateCaches();
            throw;
        }
        model.invalidateCaches();
        status = bf_hip_capture_end(&graph_);
        if (status != BF_OK) {
            bf_hip_stream_destroy(stream_);
            check(status);
        }
    }

    CapturedTrainStep(const CapturedTrainStep&) = delete;
    CapturedTrainStep& operator=(const CapturedTrainStep&) = delete;

    ~CapturedTrainStep() {
        bf_hip_graph_destroy(graph_);   // waits for replays in flight
        bf_hip_stream_destroy(stream_);
    }

    // One step on whatever the input and target tensors hold now.  Returns at once; the default stream, and so toHost(),
    // waits for it.
    void run() {
        optimizer_.publishStep(stream_);
        check(bf_hip_graph_launch(graph_, stream_));
    }

    void synchronize() { check(bf_hip_stream_synchronize(stream_)); }

    // rows of the model output (the divisor of a cross-entropy loss sum) and its element count (that of mse)
    [[nodiscard]] std::size_t outputRows() const { return outputRows_; }
    [[nodiscard]] std::size_t outputElements() const { return outputElements_; }

private:
    Optimizer& optimizer_;
    bf_stream_t stream_ = nullptr;
    bf_graph_t graph_ = nullptr;
    std::size_t outputRows_ = 0, outputElements_ = 0;
};

}  // namespace blackforge::backend::hip

// Tests of the device dispatch of the HIP backend (include/blackforge/backend/hip/dispatch.hpp): the `--device` parser with
// the reference's diagnostics (src/main.cpp:163-186), the target names, the device listing and device selection.
// Runs with or without a GPU: `dispatch_test <expectedDeviceCount>` (-1 = whatever the driver reports).
#include <cstdio>
#include <cstdlib>
#include <sstream>
#include <stdexcept>
#include <string>

#include "blackforge/backend/hip/dispatch.hpp"

namespace hip = blackforge::backend::hip;

static int failures = 0;
static void expect(bool ok, const char* what) {
    std::printf("[%s] %s\n", ok ? "  OK  " : " FAIL ", what);
    if (!ok) ++failures;
}

int main(int argc, char** argv) {
    const int expectedDevices = argc > 1 ? std::atoi(argv[1]) : -1;
    hip::DeviceSpec spec;
    std::string error;
    expect(hip::parseDeviceSpec("cpu", spec, error) && spec.family == hip::DeviceFamily::Cpu && !spec.isGpu(), "cpu");
    expect(hip::parseDeviceSpec("hip", spec, error) && spec.family == hip::DeviceFamily::Hip && spec.index == 0, "hip alone is device 0");
    expect(hip::parseDeviceSpec("hip:0", spec, error) && spec.family == hip::DeviceFamily::Hip && spec.index == 0, "hip:0");
    expect(hip::parseDeviceSpec("hip:7", spec, error) && spec.index == 7 && spec.toString() == "hip:7", "hip:7");
    expect(hip::parseDeviceSpec("cuda", spec, error) && spec.family == hip::DeviceFamily::Cuda && spec.index == 0, "cuda still parses (main.cpp:168-171)");
    expect(hip::parseDeviceSpec("cuda:3", spec, error) && spec.family == hip::DeviceFamily::Cuda && spec.index == 3, "cuda:3");
    for (const char* bad : {"hip:", "hip:x", "hip:-1", "hip:1a", "cuda:", "hip:1234567"}) {
        error.clear();
        expect(!hip::parseDeviceSpec(bad, spec, error) && error == std::string("indice GPU non valido in '") + bad + "'", bad);
    }
    for (const char* bad : {"", "gpu", "hipp", "HIP", "rocm:0", "cpu:0"}) {
        error.clear();
        expect(!hip::parseDeviceSpec(bad, spec, error) && error.rfind(std::string("dispositivo sconosciuto '") + bad + "'", 0) == 0 &&
                   error.find("hip:N") != std::string::npos, bad[0] ? bad : "(empty)");
    }
    expect(hip::isHipTarget("amd.cdna4") && hip::isHipTarget("amd.mi355x") && !hip::isHipTarget("nvidia.hopper") && !hip::isHipTarget("cpu"), "target names");

    const auto devices = hip::enumerateDevices();
    if (expectedDevices >= 0) expect(int(devices.size()) == expectedDevices, "device count as expected");
    std::ostringstream listing;
    hip::listDevices(listing);
    if (devices.empty()) expect(listing.str().find("nessuna GPU AMD") != std::string::npos, "listing without devices");
    else expect(listing.str().rfind("hip:0: ", 0) == 0 && listing.str().find(" CU, ") != std::string::npos, "listing names hip:0");

    auto throwsInvalid = [](const hip::DeviceSpec& s) {
        try { hip::selectDevice(s); } catch (const std::invalid_argument&) { return true; }
        return false;
    };
    expect(throwsInvalid({hip::DeviceFamily::Hip, 99}), "hip:99 is refused with std::invalid_argument");
    expect(throwsInvalid({hip::DeviceFamily::Cuda, 0}), "a cuda spec is refused by the HIP backend");
    expect(throwsInvalid({hip::DeviceFamily::Cpu, 0}), "a cpu spec is refused by the HIP backend");
    if (devices.empty()) {
        expect(throwsInvalid({hip::DeviceFamily::Hip, 0}), "hip:0 without a device is refused");
    } else {
        expect(!throwsInvalid({hip::DeviceFamily::Hip, 0}), "hip:0 is selected");
        int current = -1;
        expect(bf_hip_get_device(&current) == BF_OK && current == 0, "device 0 is current");
    }
    std::printf("%d failure(s)\n", failures);
    return failures == 0 ? 0 : 1;
}

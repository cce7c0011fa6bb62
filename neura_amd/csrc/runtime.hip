// Device handle, memory, timing and the weight arena: the part of the library that stands
// where the reference's GPU abstraction (device / queue / buffer / submission) stands.
#include "common.hpp"

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <vector>

namespace nh {

static thread_local char last_error[512] = "";

int32_t fail(int32_t code, const char *format, ...) {
    va_list args;
    va_start(args, format);
    vsnprintf(last_error, sizeof(last_error), format, args);
    va_end(args);
    return code;
}

int32_t hip_fail(hipError_t error, const char *what) {
    return fail(NH_E_DEVICE, "%s failed: %s", what, hipGetErrorString(error));
}

void *scratch(nh_device *device, size_t bytes) {
    if (bytes <= device->scratch_bytes) return device->scratch;
    // The block that is outgrown is kept until nh_close: work already queued on the stream, and any recorded
    // decode step that has not been recorded again yet, still holds its address, and nothing is released
    // in the middle of a process (no synchronize, no free).
    // It grows to at least twice its size, so that all the retired blocks together stay smaller than the live one.
    size_t wanted = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
    if (wanted < 2 * device->scratch_bytes) wanted = 2 * device->scratch_bytes;
    void *held = nullptr;
    if (hipMalloc(&held, wanted) != hipSuccess) {
        fail(NH_E_MEMORY, "device %d holds no %zu bytes of scratch", device->index, wanted);
        return nullptr;
    }
    if (device->scratch) device->retired.push_back(device->scratch);
    device->scratch = held;
    device->scratch_bytes = wanted;
    device->moved++;
    return held;
}

const float *rope_frequencies(nh_device *device, float base, uint32_t width) {
    // one table per (base, width) the device has met, kept until nh_close: a table never moves, so decoders of
    // different head widths or bases can step in turn, each from its own recorded graph
    for (const nh_device::RopeTable &known : device->rope_tables)
        if (known.base == base && known.width == width) return known.table;
    // pow(base, -2c/width) in fp32 on the host: crates/neura-kernel/src/task/rope.rs:48-50
    std::vector<float> table(width / 2);
    for (uint32_t c = 0; c < width / 2; c++) table[c] = powf(base, -2.0f * (float)c / (float)width);
    float *held = nullptr;
    if (hipMalloc((void **)&held, table.size() * sizeof(float)) != hipSuccess) {
        fail(NH_E_MEMORY, "device %d holds no rope table of %u channels", device->index, width);
        return nullptr;
    }
    if (hipMemcpy(held, table.data(), table.size() * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipFree(held);
        fail(NH_E_DEVICE, "device %d takes no rope table", device->index);
        return nullptr;
    }
    device->rope_tables.push_back({base, width, held});
    return held;
}

int32_t check_refusal(nh_device *device, const char *what) {
    uint32_t word = 0;
    NH_HIP(hipMemcpyAsync(&word, device->refusal, sizeof(word), hipMemcpyDeviceToHost, device->stream));
    NH_HIP(hipStreamSynchronize(device->stream));
    if (word == REFUSAL_NONE) return NH_OK;
    NH_HIP(hipMemsetAsync(device->refusal, 0, sizeof(word), device->stream));
    NH_HIP(hipStreamSynchronize(device->stream));
    switch (word) {
    case REFUSAL_SEAM: return fail(NH_E_DEVICE, "%s: a product of a chained launch gave up waiting for the numbers of the product before", what);
    case REFUSAL_INDEX: return fail(NH_E_REFUSAL, "%s: a token id walks past the rows its table holds", what);
    case REFUSAL_ORIGIN: return fail(NH_E_REFUSAL, "%s: a cursor walks past the keys its cache holds", what);
    default: return fail(NH_E_REFUSAL, "%s: the device refused with code %u", what, word);
    }
}

void profile_mark(nh_device *device) {
    if (!device->profile) return;
    if (device->profile_used == device->profile_events.size()) {
        hipEvent_t event;
        if (hipEventCreate(&event) != hipSuccess) return;
        device->profile_events.push_back(event);
    }
    (void)hipEventRecord(device->profile_events[device->profile_used++], device->stream);
}

}  // namespace nh

using namespace nh;

extern "C" {

const char *nh_last_error(void) { return last_error; }

nh_device *nh_open(int32_t device_index) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || device_index < 0 || device_index >= count) {
        fail(NH_E_DEVICE, "no HIP device %d is present (%d devices)", device_index, count);
        return nullptr;
    }
    hipDeviceProp_t properties;
    if (hipGetDeviceProperties(&properties, device_index) != hipSuccess) {
        fail(NH_E_DEVICE, "device %d reports no properties", device_index);
        return nullptr;
    }
    if (strncmp(properties.gcnArchName, "gfx950", 6) != 0) {
        fail(NH_E_DEVICE, "device %d is %s, and this library carries gfx950 code only", device_index, properties.gcnArchName);
        return nullptr;
    }
    if (hipSetDevice(device_index) != hipSuccess) {
        fail(NH_E_DEVICE, "device %d cannot be made current", device_index);
        return nullptr;
    }
    nh_device *device = new nh_device();
    device->index = device_index;
    device->compute_units = properties.multiProcessorCount;
    bool ok = hipStreamCreateWithFlags(&device->stream, hipStreamNonBlocking) == hipSuccess &&
              hipEventCreate(&device->started) == hipSuccess && hipEventCreate(&device->stopped) == hipSuccess &&
              hipMalloc((void **)&device->refusal, 256) == hipSuccess && hipMemset(device->refusal, 0, 256) == hipSuccess &&
              hipMalloc((void **)&device->tick, 256) == hipSuccess && hipMemset(device->tick, 0, 256) == hipSuccess;
    if (!ok) {
        fail(NH_E_DEVICE, "device %d opens no stream, events or refusal word", device_index);
        nh_close(device);
        return nullptr;
    }
    if (argmax_static_setup(device) != NH_OK) {  // the error names the call that failed
        nh_close(device);
        return nullptr;
    }
    return device;
}

void nh_close(nh_device *device) {
    if (!device) return;
    (void)hipSetDevice(device->index);
    if (device->stream) (void)hipStreamSynchronize(device->stream);
    if (device->scratch) (void)hipFree(device->scratch);
    for (void *block : device->retired) (void)hipFree(block);
    if (device->refusal) (void)hipFree(device->refusal);
    if (device->tick) (void)hipFree(device->tick);
    for (const nh_device::RopeTable &known : device->rope_tables) (void)hipFree(known.table);
    for (hipEvent_t event : device->profile_events) (void)hipEventDestroy(event);
    if (device->started) (void)hipEventDestroy(device->started);
    if (device->stopped) (void)hipEventDestroy(device->stopped);
    if (device->stream) (void)hipStreamDestroy(device->stream);
    delete device;
}

void *nh_alloc(nh_device *device, size_t bytes) {
    if (!device) {
        fail(NH_E_ARGUMENT, "an allocation names no device");
        return nullptr;
    }
    void *held = nullptr;
    size_t wanted = bytes ? bytes : 4;
    if (hipMalloc(&held, wanted) != hipSuccess) {
        fail(NH_E_MEMORY, "device %d holds no %zu bytes", device->index, wanted);
        return nullptr;
    }
    if (hipMemsetAsync(held, 0, wanted, device->stream) != hipSuccess || hipStreamSynchronize(device->stream) != hipSuccess) {
        (void)hipFree(held);
        fail(NH_E_DEVICE, "device %d clears no %zu bytes", device->index, wanted);
        return nullptr;
    }
    return held;
}

int32_t nh_free(nh_device *device, void *dev) {
    NH_REQUIRE(device, "a release names no device");
    if (!dev) return NH_OK;
    NH_HIP(hipStreamSynchronize(device->stream));
    NH_HIP(hipFree(dev));
    return NH_OK;
}

int32_t nh_upload(nh_device *device, void *dev_dst, const void *host_src, size_t bytes) {
    NH_REQUIRE(device && (bytes == 0 || (dev_dst && host_src)), "an upload of %zu bytes names no buffer", bytes);
    if (!bytes) return NH_OK;
    NH_HIP(hipMemcpyAsync(dev_dst, host_src, bytes, hipMemcpyHostToDevice, device->stream));
    NH_HIP(hipStreamSynchronize(device->stream));
    return NH_OK;
}

int32_t nh_download(nh_device *device, void *host_dst, const void *dev_src, size_t bytes) {
    NH_REQUIRE(device && (bytes == 0 || (host_dst && dev_src)), "a download of %zu bytes names no buffer", bytes);
    if (!bytes) return NH_OK;
    NH_HIP(hipMemcpyAsync(host_dst, dev_src, bytes, hipMemcpyDeviceToHost, device->stream));
    NH_HIP(hipStreamSynchronize(device->stream));
    return NH_OK;
}

int32_t nh_copy(nh_device *device, void *dev_dst, const void *dev_src, size_t bytes) {
    NH_REQUIRE(device && (bytes == 0 || (dev_dst && dev_src)), "a copy of %zu bytes names no buffer", bytes);
    if (!bytes) return NH_OK;
    NH_HIP(hipMemcpyAsync(dev_dst, dev_src, bytes, hipMemcpyDeviceToDevice, device->stream));
    return NH_OK;
}

int32_t nh_clear(nh_device *device, void *dev, size_t bytes) {
    NH_REQUIRE(device && (bytes == 0 || dev), "a clear of %zu bytes names no buffer", bytes);
    if (!bytes) return NH_OK;
    NH_HIP(hipMemsetAsync(dev, 0, bytes, device->stream));
    return NH_OK;
}

int32_t nh_sync(nh_device *device) {
    NH_REQUIRE(device, "a wait names no device");
    NH_HIP(hipStreamSynchronize(device->stream));
    return NH_OK;
}

int32_t nh_timer_start(nh_device *device) {
    NH_REQUIRE(device, "a timer names no device");
    NH_HIP(hipEventRecord(device->started, device->stream));
    return NH_OK;
}

int32_t nh_timer_stop(nh_device *device, double *seconds_out) {
    NH_REQUIRE(device && seconds_out, "a timer names no device or no result");
    NH_HIP(hipEventRecord(device->stopped, device->stream));
    NH_HIP(hipEventSynchronize(device->stopped));
    float milliseconds = 0.0f;
    NH_HIP(hipEventElapsedTime(&milliseconds, device->started, device->stopped));
    *seconds_out = (double)milliseconds * 1e-3;
    return NH_OK;
}

int32_t nh_profile_begin(nh_device *device) {
    NH_REQUIRE(device, "a profile names no device");
    NH_HIP(hipStreamSynchronize(device->stream));
    device->profile = true;
    device->profile_used = 0;
    device->profile_bytes = 0;
    return NH_OK;
}

int32_t nh_profile_end(nh_device *device, double *seconds_out, uint64_t *launches_out, uint64_t *bytes_out) {
    NH_REQUIRE(device && seconds_out && launches_out && bytes_out, "a profile names no device or no result");
    device->profile = false;
    NH_HIP(hipStreamSynchronize(device->stream));
    double total = 0.0;
    for (size_t at = 0; at + 1 < device->profile_used; at += 2) {
        float milliseconds = 0.0f;
        NH_HIP(hipEventElapsedTime(&milliseconds, device->profile_events[at], device->profile_events[at + 1]));
        total += (double)milliseconds * 1e-3;
    }
    *seconds_out = total;
    *launches_out = device->profile_used / 2;
    *bytes_out = device->profile_bytes;
    return NH_OK;
}

}  // extern "C"

// ---- weight arena -----------------------------------------------------------------------

struct nh_weights {
    nh_device *device = nullptr;
    uint8_t *base = nullptr;
    size_t bytes = 0;
};

extern "C" {

nh_weights *nh_weights_create(nh_device *device, size_t bytes) {
    if (!device || !bytes) {
        fail(NH_E_ARGUMENT, "an arena of %zu bytes names no device or no byte", bytes);
        return nullptr;
    }
    // 256 spare bytes so a 16-byte load that starts inside the last block never leaves the arena
    uint8_t *base = nullptr;
    if (hipMalloc((void **)&base, bytes + 256) != hipSuccess) {
        fail(NH_E_MEMORY, "device %d holds no arena of %zu bytes", device->index, bytes);
        return nullptr;
    }
    if (hipMemsetAsync(base + bytes, 0, 256, device->stream) != hipSuccess) {
        (void)hipFree(base);
        fail(NH_E_DEVICE, "device %d clears no arena tail", device->index);
        return nullptr;
    }
    nh_weights *weights = new nh_weights();
    weights->device = device;
    weights->base = base;
    weights->bytes = bytes;
    return weights;
}

void nh_weights_destroy(nh_weights *weights) {
    if (!weights) return;
    (void)hipStreamSynchronize(weights->device->stream);
    (void)hipFree(weights->base);
    delete weights;
}

int32_t nh_weights_put(nh_weights *weights, size_t at, const void *host_bytes, size_t bytes) {
    NH_REQUIRE(weights && host_bytes, "a pour names no arena or no bytes");
    NH_REQUIRE(at <= weights->bytes && bytes <= weights->bytes - at, "a pour of %zu bytes at %zu leaves an arena of %zu bytes", bytes, at,
               weights->bytes);
    if (!bytes) return NH_OK;
    NH_HIP(hipMemcpyAsync(weights->base + at, host_bytes, bytes, hipMemcpyHostToDevice, weights->device->stream));
    NH_HIP(hipStreamSynchronize(weights->device->stream));
    return NH_OK;
}

void *nh_weights_at(nh_weights *weights, size_t at) {
    if (!weights || at > weights->bytes) {
        fail(NH_E_ARGUMENT, "an arena holds no byte %zu", at);
        return nullptr;
    }
    return weights->base + at;
}

size_t nh_weights_bytes(const nh_weights *weights) { return weights ? weights->bytes : 0; }

}  // extern "C"

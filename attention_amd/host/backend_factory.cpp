// BackendFactory: registry of creators and capabilities, with the HIP backend built in.
#include "api/backend_factory.hpp"

#include <algorithm>
#include <cctype>
#include <iostream>
#include <sstream>

#include "ahpc_hip.h"
#include "algorithms/flash_attention.hpp"
#include "algorithms/paged_attention.hpp"

namespace attention_hpc {

namespace {
int key(BackendType t) { return static_cast<int>(t); }

const char* builtin_name(BackendType type) {
    switch (type) {
        case BackendType::CPU: return "CPU";
        case BackendType::CUDA: return "CUDA";
        case BackendType::OPENCL: return "OpenCL";
        case BackendType::OPENGL: return "OpenGL";
        case BackendType::VULKAN: return "Vulkan";
        case BackendType::AUTO: return "AUTO";
        case BackendType::HIP: return "HIP";
        default: return "Unknown";
    }
}
}  // namespace

BackendFactory& BackendFactory::getInstance() {
    static BackendFactory instance;
    return instance;
}

BackendFactory::BackendFactory() {
    // Runs once, inside the function-local static's initialisation: nothing here goes back through
    // getInstance() (the reference's constructor does, src/api/backend_factory.cpp:55-58, :90, :499).
    priority_ = {BackendType::HIP, BackendType::CUDA, BackendType::VULKAN, BackendType::OPENCL, BackendType::OPENGL,
                 BackendType::CPU};
    for (BackendType t : {BackendType::CPU, BackendType::CUDA, BackendType::OPENCL, BackendType::OPENGL, BackendType::VULKAN})
        capabilities_[key(t)] = BackendCapability{};  // known, not available
    probe_hip();
    flash_creators_[key(BackendType::HIP)] = [] { return std::unique_ptr<AttentionInterface>(new FlashAttention()); };
    paged_creators_[key(BackendType::HIP)] = [] { return std::unique_ptr<AttentionInterface>(new PagedAttention()); };
}

// Capability record of the first HIP device (reference: detectBackendCapabilities and BackendCapability,
// src/api/backend_factory.hpp:24-37).
void BackendFactory::probe_hip() {
    BackendCapability cap;
    int n = 0;
    ahpc_hip_device_count(&n);
    ahpc_device_info info;
    if (n > 0 && ahpc_hip_device_info(0, &info) == 0) {
        cap.available = true;
        cap.version = "HIP runtime " + std::to_string(info.runtime_version);
        cap.device_name = std::string(info.name[0] ? info.name : "AMD GPU") + " (" + info.arch + ")";
        cap.memory_size = static_cast<size_t>(info.total_memory_bytes);
        // "compute capability" carries the gfx number: gfx950 -> 9.50
        int gfx = 0;
        for (const char* p = info.arch; *p; ++p)
            if (std::isdigit(static_cast<unsigned char>(*p))) gfx = gfx * 10 + (*p - '0');
        cap.compute_capability_major = gfx / 100;
        cap.compute_capability_minor = gfx % 100;
        cap.supported_data_types = {DataType::FLOAT32, DataType::FLOAT16, DataType::BFLOAT16};
        cap.supported_layouts = {MemoryLayout::ROW_MAJOR};
        cap.max_threads = static_cast<size_t>(info.max_threads_per_workgroup);
        cap.max_shared_memory = static_cast<size_t>(info.lds_bytes_per_workgroup);
        cap.supports_mixed_precision = true;
        cap.supports_tensor_cores = true;  // MFMA matrix cores
    }
    capabilities_[key(BackendType::HIP)] = cap;
}

bool BackendFactory::available_locked(BackendType type) const {
    auto it = capabilities_.find(key(type));
    return it != capabilities_.end() && it->second.available;
}

std::string BackendFactory::name_locked(BackendType type) const {
    auto it = names_.find(key(type));
    return it != names_.end() ? it->second : std::string(builtin_name(type));
}

// First available backend in priority order that has a creator.  (The reference scores backends by
// sequence length and memory, src/api/backend_factory.cpp:446-470, :600-720; with one real backend the
// order alone decides.)
BackendType BackendFactory::best_locked(const AttentionParams&) const {
    for (BackendType t : priority_)
        if (available_locked(t) && flash_creators_.count(key(t))) return t;
    return BackendType::CPU;
}

std::unique_ptr<AttentionInterface> BackendFactory::create_locked(BackendType type, bool paged) {
    if (type == BackendType::AUTO) {
        type = default_backend_ != BackendType::AUTO ? default_backend_ : best_locked(AttentionParams{});
    }
    // Returns null when the backend cannot be had; the callers throw BackendException only after the lock is
    // released, because that exception's constructor asks the factory for the backend's name.
    if (!available_locked(type)) return nullptr;
    auto& map = paged ? paged_creators_ : flash_creators_;
    auto it = map.find(key(type));
    if (it == map.end()) return nullptr;
    return it->second();
}

namespace {
[[noreturn]] void throw_unavailable(BackendType type, const std::string& why) { throw BackendException(type, why); }
}  // namespace

std::unique_ptr<AttentionInterface> BackendFactory::createFlashAttention(BackendType type) {
    auto& f = getInstance();
    std::unique_ptr<AttentionInterface> obj;
    std::string failure;
    {
        std::lock_guard<std::mutex> lock(f.mutex_);
        try {
            obj = f.create_locked(type, false);
        } catch (const std::exception& e) {
            failure = std::string("Failed to create backend: ") + e.what();
        }
    }
    if (!failure.empty()) throw_unavailable(type, failure);
    if (!obj) throw_unavailable(type, "Backend not available");
    return obj;
}

std::unique_ptr<AttentionInterface> BackendFactory::createPagedAttention(BackendType type) {
    auto& f = getInstance();
    std::unique_ptr<AttentionInterface> obj;
    std::string failure;
    {
        std::lock_guard<std::mutex> lock(f.mutex_);
        try {
            obj = f.create_locked(type, true);
        } catch (const std::exception& e) {
            failure = std::string("Failed to create backend: ") + e.what();
        }
    }
    if (!failure.empty()) throw_unavailable(type, failure);
    if (!obj) throw_unavailable(type, "PagedAttention backend not available");
    return obj;
}

std::unique_ptr<AttentionInterface> BackendFactory::createBackend(BackendType type) { return createFlashAttention(type); }

bool BackendFactory::isBackendAvailable(BackendType type) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    if (type == BackendType::AUTO) return f.available_locked(f.best_locked(AttentionParams{}));
    return f.available_locked(type);
}

std::vector<BackendType> BackendFactory::getAvailableBackends() {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    std::vector<BackendType> out;
    for (BackendType t : {BackendType::CPU, BackendType::CUDA, BackendType::OPENCL, BackendType::OPENGL, BackendType::VULKAN,
                          BackendType::HIP})
        if (f.available_locked(t)) out.push_back(t);
    return out;
}

BackendCapability BackendFactory::getBackendCapability(BackendType type) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    auto it = f.capabilities_.find(key(type));
    return it != f.capabilities_.end() ? it->second : BackendCapability{};
}

BackendType BackendFactory::selectBestBackend(const AttentionParams& params) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    return f.best_locked(params);
}

BackendType BackendFactory::selectBestBackend(const std::vector<BackendType>& preferred) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    for (BackendType t : preferred)
        if (f.available_locked(t)) return t;
    return f.best_locked(AttentionParams{});
}

void BackendFactory::setBackendPriority(const std::vector<BackendType>& order) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    f.priority_ = order;
}

std::vector<BackendType> BackendFactory::getBackendPriority() {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    return f.priority_;
}

// Plug-in point (reference: src/api/backend_factory.cpp:497-513).  Registering a creator for a type that had
// no capability record marks it available, so a plug-in becomes usable with this one call.
void BackendFactory::registerBackend(BackendType type, const std::string& name, BackendCreator creator) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    f.flash_creators_[key(type)] = std::move(creator);
    f.names_[key(type)] = name;
    auto& cap = f.capabilities_[key(type)];
    if (!cap.available) {
        cap.available = true;
        if (cap.version.empty()) cap.version = "plugin";
        if (cap.device_name.empty()) cap.device_name = name;
        if (cap.supported_data_types.empty()) cap.supported_data_types = {DataType::FLOAT32};
        if (cap.supported_layouts.empty()) cap.supported_layouts = {MemoryLayout::ROW_MAJOR};
    }
}

void BackendFactory::registerPagedBackend(BackendType type, const std::string& name, BackendCreator creator) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    f.paged_creators_[key(type)] = std::move(creator);
    if (!f.names_.count(key(type))) f.names_[key(type)] = name;
}

void BackendFactory::registerBackendCapability(BackendType type, const BackendCapability& capability) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    f.capabilities_[key(type)] = capability;
}

void BackendFactory::unregisterBackend(BackendType type) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    f.flash_creators_.erase(key(type));
    f.paged_creators_.erase(key(type));
    f.names_.erase(key(type));
    if (type != BackendType::HIP) f.capabilities_[key(type)] = BackendCapability{};
}

std::string BackendFactory::backendTypeToString(BackendType type) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    return f.name_locked(type);
}

BackendType BackendFactory::stringToBackendType(const std::string& type_str) {
    std::string s = type_str;
    std::transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return static_cast<char>(std::tolower(c)); });
    if (s == "cpu") return BackendType::CPU;
    if (s == "cuda") return BackendType::CUDA;
    if (s == "opencl") return BackendType::OPENCL;
    if (s == "opengl") return BackendType::OPENGL;
    if (s == "vulkan") return BackendType::VULKAN;
    if (s == "auto") return BackendType::AUTO;
    if (s == "hip" || s == "rocm") return BackendType::HIP;
    throw std::invalid_argument("Unknown backend type: " + type_str);
}

std::vector<std::string> BackendFactory::getSupportedBackendNames() {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    std::vector<std::string> names;
    for (const auto& kv : f.flash_creators_) names.push_back(f.name_locked(static_cast<BackendType>(kv.first)));
    std::sort(names.begin(), names.end());
    return names;
}

std::string BackendFactory::getSystemInfo() {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    std::ostringstream os;
    os << "AttentionHPC (MI355X build)\n";
    for (const auto& kv : f.capabilities_) {
        const BackendCapability& c = kv.second;
        os << "  " << f.name_locked(static_cast<BackendType>(kv.first)) << ": " << (c.available ? "available" : "not available");
        if (c.available) os << ", " << c.device_name << ", " << (c.memory_size >> 20) << " MiB, " << c.version;
        os << "\n";
    }
    return os.str();
}

void BackendFactory::printAvailableBackends() { std::cout << getSystemInfo(); }

// Reference: validateBackendCompatibility / isBackendSuitable, src/api/backend_factory.cpp:590-720.  For HIP:
// dimensions positive, head_dimension within the kernels' range, K+V+Q+O of the batch fit in device memory.
bool BackendFactory::validateBackendCompatibility(BackendType type, const AttentionParams& p) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    if (type == BackendType::AUTO) type = f.best_locked(p);
    if (!f.available_locked(type)) return false;
    if (p.batch_size == 0 || p.sequence_length == 0 || p.num_heads == 0 || p.head_dimension == 0) return false;
    if (type != BackendType::HIP) return true;
    if (p.head_dimension > 256) return false;
    if (p.key_value_heads != 0 && (p.key_value_heads > p.num_heads || p.num_heads % p.key_value_heads)) return false;
    const auto& cap = f.capabilities_.at(key(type));
    const double bytes = 4.0 * 4.0 * (double)p.batch_size * (double)p.sequence_length * (double)p.num_heads * (double)p.head_dimension;
    return bytes < (double)cap.memory_size;
}

void BackendFactory::enableDebugMode(bool enable) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    f.debug_mode_ = enable;
}
bool BackendFactory::isDebugModeEnabled() {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    return f.debug_mode_;
}
void BackendFactory::setDefaultBackend(BackendType type) {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    f.default_backend_ = type;
}
BackendType BackendFactory::getDefaultBackend() {
    auto& f = getInstance();
    std::lock_guard<std::mutex> lock(f.mutex_);
    return f.default_backend_;
}

}  // namespace attention_hpc

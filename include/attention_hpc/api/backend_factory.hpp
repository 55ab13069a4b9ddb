// Backend registry and factory.  Keeps the reference's public surface
// (src/api/backend_factory.hpp:14-115 and :167-178): BackendType, BackendCapability, the static
// create*/availability/selection/registration calls, BackendException - with three repairs:
//   * BackendType::HIP is appended after AUTO (existing enumerator values are unchanged) and is the
//     one built-in backend; the CUDA/OpenCL/OpenGL/Vulkan enumerators stay so that callers compile,
//     but are never available.  There is no built-in CPU backend either: a caller that wants one
//     registers it through registerBackend (tests do, with a reference implementation).
//   * FlashAttention and PagedAttention have separate creators.  In the reference both create calls
//     alias createBackend (src/api/backend_factory.cpp:390-396), so a type could only ever be one of
//     them.  registerBackend keeps its signature and registers the flash creator;
//     registerPagedBackend is the new sibling.
//   * AUTO resolves through selectBestBackend, and no public call re-enters the factory lock (the
//     reference locks a non-recursive mutex recursively, src/api/backend_factory.cpp:366-374, :499).
#pragma once

#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "attention_interface.hpp"

namespace attention_hpc {

enum class BackendType {
    CPU,
    CUDA,
    OPENCL,
    OPENGL,
    VULKAN,
    AUTO,
    HIP  // AMD gfx950 (MI355X): the backend this library implements
};

struct BackendCapability {
    bool available = false;
    std::string version;
    std::string device_name;
    size_t memory_size = 0;
    int compute_capability_major = 0;
    int compute_capability_minor = 0;
    std::vector<DataType> supported_data_types;
    std::vector<MemoryLayout> supported_layouts;
    size_t max_threads = 0;
    size_t max_shared_memory = 0;
    bool supports_mixed_precision = false;
    bool supports_tensor_cores = false;
};

class BackendFactory {
public:
    using BackendCreator = std::function<std::unique_ptr<AttentionInterface>()>;

    static BackendFactory& getInstance();
    BackendFactory(const BackendFactory&) = delete;
    BackendFactory& operator=(const BackendFactory&) = delete;

    static std::unique_ptr<AttentionInterface> createBackend(BackendType type);        // = createFlashAttention
    static std::unique_ptr<AttentionInterface> createFlashAttention(BackendType type);
    static std::unique_ptr<AttentionInterface> createPagedAttention(BackendType type);

    static bool isBackendAvailable(BackendType type);
    static std::vector<BackendType> getAvailableBackends();
    static BackendCapability getBackendCapability(BackendType type);

    static BackendType selectBestBackend(const AttentionParams& params = AttentionParams{});
    static BackendType selectBestBackend(const std::vector<BackendType>& preferred_backends);
    static void setBackendPriority(const std::vector<BackendType>& priority_order);
    static std::vector<BackendType> getBackendPriority();

    static void registerBackend(BackendType type, const std::string& name, BackendCreator creator);
    static void registerPagedBackend(BackendType type, const std::string& name, BackendCreator creator);
    static void registerBackendCapability(BackendType type, const BackendCapability& capability);
    static void unregisterBackend(BackendType type);

    static std::string backendTypeToString(BackendType type);
    static BackendType stringToBackendType(const std::string& type_str);
    static std::vector<std::string> getSupportedBackendNames();

    static void printAvailableBackends();
    static std::string getSystemInfo();
    static bool validateBackendCompatibility(BackendType type, const AttentionParams& params);

    static void enableDebugMode(bool enable = true);
    static bool isDebugModeEnabled();
    static void setDefaultBackend(BackendType type);
    static BackendType getDefaultBackend();

private:
    BackendFactory();
    ~BackendFactory() = default;

    // *_locked helpers assume mutex_ is held and never take it
    bool available_locked(BackendType type) const;
    BackendType best_locked(const AttentionParams& params) const;
    std::string name_locked(BackendType type) const;
    std::unique_ptr<AttentionInterface> create_locked(BackendType type, bool paged);
    void probe_hip();

    mutable std::mutex mutex_;
    std::unordered_map<int, BackendCapability> capabilities_;
    std::unordered_map<int, BackendCreator> flash_creators_;
    std::unordered_map<int, BackendCreator> paged_creators_;
    std::unordered_map<int, std::string> names_;
    std::vector<BackendType> priority_;
    BackendType default_backend_ = BackendType::AUTO;
    bool debug_mode_ = false;
};

class BackendException : public AttentionException {
public:
    explicit BackendException(BackendType backend_type, const std::string& message)
        : AttentionException(AttentionError::BACKEND_NOT_AVAILABLE,
                             "Backend " + BackendFactory::backendTypeToString(backend_type) + ": " + message),
          backend_type_(backend_type) {}
    BackendType backend_type() const noexcept { return backend_type_; }

private:
    BackendType backend_type_;
};

}  // namespace attention_hpc

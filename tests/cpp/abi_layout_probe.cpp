// Prints the layout facts a backend plugin and the library that loads it must agree on:
// sizes and member offsets of the types that cross the plugin boundary by value or by
// reference, and the virtual-table slot of every public virtual function of
// nixlBackendEngine.  The test builds this file twice, against the reference's own headers
// and against this repository's restatement of them, and compares the two outputs.
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "backend/backend_engine.h"
#include "backend/backend_plugin.h"
#include "nixl_descriptors.h"

#define SIZE(T) std::printf("sizeof(%s) = %zu align %zu\n", #T, sizeof(T), alignof(T))
#define OFF(T, m) std::printf("offsetof(%s, %s) = %zu\n", #T, #m, offsetof(T, m))

// Itanium C++ ABI: a pointer to a virtual member function holds 1 + the byte offset of its
// slot in the virtual table.
template<typename F>
static void
slot(const char *name, F f) {
    std::uintptr_t raw[2] = {0, 0};
    static_assert(sizeof(f) <= sizeof(raw));
    std::memcpy(raw, &f, sizeof(f));
    std::printf("vtable slot of %s = %zu\n", name, static_cast<size_t>((raw[0] - 1) / sizeof(void *)));
}
#define SLOT(m) slot(#m, &nixlBackendEngine::m)

int
main() {
    SIZE(nixlBasicDesc);
    OFF(nixlBasicDesc, addr);
    OFF(nixlBasicDesc, len);
    OFF(nixlBasicDesc, devId);
    SIZE(nixlBlobDesc);
    OFF(nixlBlobDesc, metaInfo);
    SIZE(nixlMetaDesc);
    OFF(nixlMetaDesc, metadataP);
    SIZE(nixlStrideDesc);
    OFF(nixlStrideDesc, stride);
    OFF(nixlStrideDesc, count);
    OFF(nixlStrideDesc, start_idx);
    SIZE(nixlBackendInitParams);
    OFF(nixlBackendInitParams, localAgent);
    OFF(nixlBackendInitParams, type);
    OFF(nixlBackendInitParams, customParams);
    OFF(nixlBackendInitParams, enableProgTh);
    OFF(nixlBackendInitParams, pthrDelay);
    OFF(nixlBackendInitParams, syncMode);
    OFF(nixlBackendInitParams, enableTelemetry_);
    SIZE(nixlBackendPlugin);
    OFF(nixlBackendPlugin, api_version);
    OFF(nixlBackendPlugin, create_engine);
    OFF(nixlBackendPlugin, destroy_engine);
    OFF(nixlBackendPlugin, get_plugin_name);
    OFF(nixlBackendPlugin, get_plugin_version);
    OFF(nixlBackendPlugin, get_backend_options);
    OFF(nixlBackendPlugin, get_backend_mems);
    SIZE(nixlDescList<nixlMetaDesc>);
    SIZE(nixlDescList<nixlBasicDesc>);
    SIZE(nixlDescList<nixlBlobDesc>);
    SIZE(nixlStrideDescList);
    SIZE(nixlBackendEngine);
    SIZE(nixlBackendOptionalArgs);
    slot("releaseMemView", &nixlBackendEngine::releaseMemView);
    slot("estimateXferCost", &nixlBackendEngine::estimateXferCost);
    slot("queryMem", &nixlBackendEngine::queryMem);
    std::printf("NIXL_PLUGIN_API_VERSION = %d\n", static_cast<int>(NIXL_PLUGIN_API_VERSION));
    std::printf("status: SUCCESS %d IN_PROG %d INVALID_PARAM %d BACKEND %d NOT_FOUND %d NOT_SUPPORTED %d\n", NIXL_SUCCESS,
                NIXL_IN_PROG, NIXL_ERR_INVALID_PARAM, NIXL_ERR_BACKEND, NIXL_ERR_NOT_FOUND, NIXL_ERR_NOT_SUPPORTED);
    std::printf("mem: DRAM %d VRAM %d BLK %d OBJ %d FILE %d; op: READ %d WRITE %d\n", DRAM_SEG, VRAM_SEG, BLK_SEG, OBJ_SEG,
                FILE_SEG, NIXL_READ, NIXL_WRITE);
    SLOT(supportsRemote);
    SLOT(supportsLocal);
    SLOT(supportsNotif);
    SLOT(getSupportedMems);
    SLOT(registerMem);
    SLOT(deregisterMem);
    SLOT(connect);
    SLOT(disconnect);
    SLOT(unloadMD);
    SLOT(prepXfer);
    SLOT(postXfer);
    SLOT(checkXfer);
    SLOT(releaseReqH);
    SLOT(getPublicData);
    SLOT(getConnInfo);
    SLOT(loadRemoteConnInfo);
    SLOT(loadRemoteMD);
    SLOT(loadLocalMD);
    SLOT(getNotifs);
    SLOT(genNotif);
    return 0;
}

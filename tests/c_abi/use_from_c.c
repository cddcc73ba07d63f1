/* include/infmoe.h used from plain C (C99, no HIP headers, no C++): what a cgo / JNI / ctypes-free C caller
 * sees.  Built by tests/test_host_api.py with gcc and linked against libinfmoe.so; run without a GPU it
 * exercises the host-only part of the life cycle (create with the creator's fields, configure, workspace
 * size, serialise / deserialise, clone, error reporting) and prints what the Python side checks. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "infmoe.h"

static infmoe_field field(const char* name, const void* data, int type, int length) {
    infmoe_field f;
    f.name = name, f.data = data, f.type = type, f.length = length;
    return f;
}

int main(void) {
    const int E = 4, d = 64, h = 256, mc = 2;
    float centroids[4 * 64], gamma[64];
    for (int i = 0; i < E * d; ++i) centroids[i] = (float)(i % 7) * 0.125f;
    for (int i = 0; i < d; ++i) gamma[i] = 1.0f;
    infmoe_field fields[9];
    int n = 0;
    fields[n++] = field("expert_count", &E, INFMOE_FIELD_INT32, 1);
    fields[n++] = field("embedding_size", &d, INFMOE_FIELD_INT32, 1);
    fields[n++] = field("hidden_size", &h, INFMOE_FIELD_INT32, 1);
    fields[n++] = field("max_concurrency", &mc, INFMOE_FIELD_INT32, 1);
    fields[n++] = field("expert_centroids", centroids, INFMOE_FIELD_FLOAT32, E * d);
    fields[n++] = field("layernorm_weight", gamma, INFMOE_FIELD_FLOAT32, d);
    fields[n++] = field("expert_sublayer_type", "T5_FF", INFMOE_FIELD_UNKNOWN, 5);
    fields[n++] = field("moe_variant", "cpm_2", INFMOE_FIELD_UNKNOWN, 5);

    infmoe_plugin* p = NULL;
    if (infmoe_create("layer0", fields, n, &p) != INFMOE_OK) {
        printf("create failed: %s\n", infmoe_last_error());
        return 1;
    }
    const int32_t dims[3] = {2, 16, 64};
    size_t ws = 0, blob_bytes = 0;
    if (infmoe_configure(p, dims, 3) != INFMOE_OK || infmoe_workspace_size(p, dims, 3, &ws) != INFMOE_OK) {
        printf("configure failed: %s\n", infmoe_last_error());
        return 1;
    }
    if (infmoe_serialization_size(p, &blob_bytes) != INFMOE_OK) return 1;
    void* blob = malloc(blob_bytes);
    if (infmoe_serialize(p, blob, blob_bytes) != INFMOE_OK) return 1;
    infmoe_plugin* back = NULL;
    if (infmoe_deserialize("layer0", blob, blob_bytes, &back) != INFMOE_OK) {
        printf("deserialize failed: %s\n", infmoe_last_error());
        return 1;
    }
    size_t again = 0;
    if (infmoe_serialization_size(back, &again) != INFMOE_OK || again != blob_bytes) return 1;
    infmoe_plugin* twin = NULL;
    if (infmoe_clone(p, &twin) != INFMOE_OK) return 1;

    /* errors are codes and messages, never aborts */
    const int32_t bad_dims[3] = {2, 16, 65};
    const int32_t status = infmoe_workspace_size(p, bad_dims, 3, &ws);
    printf("name=%s version=%s workspace=%zu blob=%zu bad_dims_status=%d message=%s\n", infmoe_plugin_name(),
           infmoe_plugin_version(), ws, blob_bytes, (int)status, infmoe_last_error());
    fields[7] = field("moe_variant", "no_such_variant", INFMOE_FIELD_UNKNOWN, 15);
    infmoe_plugin* none = NULL;
    printf("bad_variant_status=%d\n", (int)infmoe_create("layer1", fields, n, &none));

    free(blob);
    infmoe_destroy(twin);
    infmoe_destroy(back);
    infmoe_destroy(p);
    return 0;
}

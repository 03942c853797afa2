// Binary-layout mirror of the parts of the reference's ggml that a dlopen'ed backend touches.
//
// A ggml backend plugin is handed `ggml_tensor` / `ggml_cgraph` objects by the host and hands back vtable
// objects, so both sides must agree on struct layouts and enum ordinals -- not on names.  This header restates
// those layouts (x86-64, LP64) in namespace ggml_abi so that the backend builds without the reference tree.
// Every struct carries static_asserts with the sizes/offsets measured from the reference's headers:
//   ggml/include/ggml.h:218-225 (limits), :324-329 (status), :360-401 (types), :438-549 (ops), :597-631 (tensor)
//   ggml/include/ggml-backend.h:48-52, :135-164 (usage, device type, caps, props)
//   ggml/src/ggml-backend-impl.h:11 (API version), :17-35, :41-69, :89-135, :143-192, :198-214 (vtables/objects)
//   ggml/src/ggml-impl.h:184-188, :287-304 (hash set, cgraph incl. the fork's flags/graph_name_by_time/n_ctx)
// tests/test_abi.py compares mla_ggml_abi_table() (built from THIS header) entry by entry with the same table
// produced from the real headers.
#pragma once

#include <stddef.h>
#include <stdint.h>

namespace ggml_abi {

constexpr int MAX_DIMS      = 4;
constexpr int MAX_SRC       = 10;
constexpr int MAX_OP_PARAMS = 64;
constexpr int MAX_NAME      = 64;
constexpr int KQ_MASK_PAD   = 64;
constexpr int BACKEND_API_VERSION = 1;

enum status : int { STATUS_ALLOC_FAILED = -2, STATUS_FAILED = -1, STATUS_SUCCESS = 0, STATUS_ABORTED = 1 };

enum type : int {
    TYPE_F32 = 0, TYPE_F16 = 1, TYPE_Q8_0 = 8, TYPE_I8 = 24, TYPE_I16 = 25, TYPE_I32 = 26, TYPE_I64 = 27, TYPE_F64 = 28,
    TYPE_BF16 = 30, TYPE_COUNT = 39,
};

// only the ordinals the backend acts on; the fork appended 13 ops after upstream's list, so COUNT is 94
enum op : int {
    OP_NONE = 0, OP_CONCAT = 20, OP_MUL_MAT = 26, OP_CPY = 31, OP_CONT = 32, OP_RESHAPE = 33, OP_VIEW = 34, OP_PERMUTE = 35, OP_TRANSPOSE = 36,
    OP_ROPE = 44, OP_FLASH_ATTN_EXT = 61, OP_SCATTER_UPDATE = 92, OP_COUNT = 94,
};

enum prec : int { PREC_DEFAULT = 0, PREC_F32 = 1 };
enum tensor_flag : int { TENSOR_FLAG_INPUT = 1, TENSOR_FLAG_OUTPUT = 2 };
enum dev_type : int { DEVICE_TYPE_CPU = 0, DEVICE_TYPE_GPU = 1, DEVICE_TYPE_ACCEL = 2 };
enum buffer_usage : int { BUFFER_USAGE_ANY = 0, BUFFER_USAGE_WEIGHTS = 1, BUFFER_USAGE_COMPUTE = 2 };

struct backend_buffer;
struct backend_buffer_type;
struct backend;
struct backend_device;
struct backend_reg;
struct backend_event;

struct tensor {
    int32_t          type;
    backend_buffer * buffer;
    int64_t          ne[MAX_DIMS];
    size_t           nb[MAX_DIMS];
    int32_t          op;
    int32_t          op_params[MAX_OP_PARAMS / sizeof(int32_t)];
    int32_t          flags;
    tensor *         src[MAX_SRC];
    tensor *         view_src;
    size_t           view_offs;
    void *           data;
    char             name[MAX_NAME];
    void *           extra;
    char             padding[8];
};
static_assert(sizeof(tensor) == 336, "ggml_tensor size");
static_assert(offsetof(tensor, buffer) == 8 && offsetof(tensor, ne) == 16 && offsetof(tensor, nb) == 48, "ggml_tensor layout");
static_assert(offsetof(tensor, op) == 80 && offsetof(tensor, op_params) == 84 && offsetof(tensor, flags) == 148, "ggml_tensor layout");
static_assert(offsetof(tensor, src) == 152 && offsetof(tensor, view_src) == 232 && offsetof(tensor, view_offs) == 240, "ggml_tensor layout");
static_assert(offsetof(tensor, data) == 248 && offsetof(tensor, name) == 256 && offsetof(tensor, extra) == 320, "ggml_tensor layout");

struct hash_set {
    size_t     size;
    uint32_t * used;
    tensor **  keys;
};

struct cgraph {
    int       size;
    int       n_nodes;
    int       n_leafs;
    int       flags;  // fork addition: bit 0 = GE mode, bit 1 = compile only
    tensor ** nodes;
    tensor ** grads;
    tensor ** grad_accs;
    tensor ** leafs;
    hash_set  visited_hash_set;
    int       order;
    char *    graph_name_by_time;  // fork addition
    int       n_ctx;               // fork addition
};
static_assert(sizeof(cgraph) == 96 && offsetof(cgraph, nodes) == 16, "ggml_cgraph layout");

struct dev_caps {
    bool async, host_buffer, buffer_from_host_ptr, events;
};
struct dev_props {
    const char * name;
    const char * description;
    size_t       memory_free;
    size_t       memory_total;
    int32_t      type;
    dev_caps     caps;
};
static_assert(sizeof(dev_props) == 40, "ggml_backend_dev_props layout");

struct backend_buffer_type_i {
    const char *     (*get_name)(backend_buffer_type * buft);
    backend_buffer * (*alloc_buffer)(backend_buffer_type * buft, size_t size);
    size_t           (*get_alignment)(backend_buffer_type * buft);
    size_t           (*get_max_size)(backend_buffer_type * buft);
    size_t           (*get_alloc_size)(backend_buffer_type * buft, const tensor * t);
    bool             (*is_host)(backend_buffer_type * buft);
};
struct backend_buffer_type {
    backend_buffer_type_i iface;
    backend_device *      device;
    void *                context;
};
static_assert(sizeof(backend_buffer_type_i) == 48 && sizeof(backend_buffer_type) == 64, "buffer type layout");

struct backend_buffer_i {
    void   (*free_buffer)(backend_buffer * buffer);
    void * (*get_base)(backend_buffer * buffer);
    int    (*init_tensor)(backend_buffer * buffer, tensor * t);
    void   (*memset_tensor)(backend_buffer * buffer, tensor * t, uint8_t value, size_t offset, size_t size);
    void   (*set_tensor)(backend_buffer * buffer, tensor * t, const void * data, size_t offset, size_t size);
    void   (*get_tensor)(backend_buffer * buffer, const tensor * t, void * data, size_t offset, size_t size);
    bool   (*cpy_tensor)(backend_buffer * buffer, const tensor * src, tensor * dst);
    void   (*clear)(backend_buffer * buffer, uint8_t value);
    void   (*reset)(backend_buffer * buffer);
};
struct backend_buffer {
    backend_buffer_i      iface;
    backend_buffer_type * buft;
    void *                context;
    size_t                size;
    int32_t               usage;
};
static_assert(sizeof(backend_buffer_i) == 72 && sizeof(backend_buffer) == 104, "buffer layout");

typedef void * graph_plan_t;
struct backend_i {
    const char * (*get_name)(backend * be);
    void         (*free)(backend * be);
    void         (*set_tensor_async)(backend * be, tensor * t, const void * data, size_t offset, size_t size);
    void         (*get_tensor_async)(backend * be, const tensor * t, void * data, size_t offset, size_t size);
    bool         (*cpy_tensor_async)(backend * src_be, backend * dst_be, const tensor * src, tensor * dst);
    void         (*synchronize)(backend * be);
    graph_plan_t (*graph_plan_create)(backend * be, const cgraph * g);
    void         (*graph_plan_free)(backend * be, graph_plan_t plan);
    void         (*graph_plan_update)(backend * be, graph_plan_t plan, const cgraph * g);
    int          (*graph_plan_compute)(backend * be, graph_plan_t plan);
    int          (*graph_compute)(backend * be, cgraph * g);
    void         (*event_record)(backend * be, backend_event * ev);
    void         (*event_wait)(backend * be, backend_event * ev);
};
typedef uint8_t guid_t[16];
struct backend {
    guid_t *         guid;
    backend_i        iface;
    backend_device * device;
    void *           context;
};
static_assert(sizeof(backend_i) == 104 && sizeof(backend) == 128, "backend layout");

struct backend_event {
    backend_device * device;
    void *           context;
};

struct backend_device_i {
    const char *          (*get_name)(backend_device * dev);
    const char *          (*get_description)(backend_device * dev);
    void                  (*get_memory)(backend_device * dev, size_t * free, size_t * total);
    int                   (*get_type)(backend_device * dev);
    void                  (*get_props)(backend_device * dev, dev_props * props);
    backend *             (*init_backend)(backend_device * dev, const char * params);
    backend_buffer_type * (*get_buffer_type)(backend_device * dev);
    backend_buffer_type * (*get_host_buffer_type)(backend_device * dev);
    backend_buffer *      (*buffer_from_host_ptr)(backend_device * dev, void * ptr, size_t size, size_t max_tensor_size);
    bool                  (*supports_op)(backend_device * dev, const tensor * op);
    bool                  (*supports_buft)(backend_device * dev, backend_buffer_type * buft);
    bool                  (*offload_op)(backend_device * dev, const tensor * op);
    backend_event *       (*event_new)(backend_device * dev);
    void                  (*event_free)(backend_device * dev, backend_event * ev);
    void                  (*event_synchronize)(backend_device * dev, backend_event * ev);
};
struct backend_device {
    backend_device_i iface;
    backend_reg *    reg;
    void *           context;
};
static_assert(sizeof(backend_device_i) == 120 && sizeof(backend_device) == 136, "device layout");

struct backend_reg_i {
    const char *     (*get_name)(backend_reg * reg);
    size_t           (*get_device_count)(backend_reg * reg);
    backend_device * (*get_device)(backend_reg * reg, size_t index);
    void *           (*get_proc_address)(backend_reg * reg, const char * name);
};
struct backend_reg {
    int           api_version;
    backend_reg_i iface;
    void *        context;
};
static_assert(sizeof(backend_reg_i) == 32 && sizeof(backend_reg) == 48, "reg layout");

// Q8_0 block: fp16 scale + 32 int8 (ggml/src/ggml-common.h:217-224)
struct block_q8_0 {
    uint16_t d;
    int8_t   qs[32];
};
static_assert(sizeof(block_q8_0) == 34, "block_q8_0 layout");

}  // namespace ggml_abi

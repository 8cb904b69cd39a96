/*
 * PHI backend seam of the MI355X articulation-step library, as plain C function-pointer tables.
 *
 * Shape, member order and meaning follow the reference's PHI v2 interface so that a maintainer can register this
 * backend next to (or instead of) the CUDA one:
 *   nuka_phi_buffer_type_i / nuka_phi_buffer_i   <- src/phi/buffer.hpp:36-58   (BufferTypeI, BufferI)
 *   nuka_phi_backend_i                           <- src/phi/backend.hpp:86-103 (BackendI, 15 entries)
 *   nuka_phi_device_i                            <- src/phi/backend.hpp:108-115 (DeviceI)
 *   nuka_phi_registry_entry_i                    <- src/phi/backend.hpp:120-125 (RegistryEntryI)
 * Every concrete handle begins with a pointer to its table (src/phi/backend.hpp:127-136, buffer.hpp:60-72).
 * C++ references of the reference signatures (const ModelView&, const DataView&, const OpCall&) are pointers here,
 * which is the same ABI.  Ops return a status and never throw across the seam.
 */
#ifndef NUKA_PHI_H_
#define NUKA_PHI_H_

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* src/phi/status.hpp */
typedef enum nuka_phi_status { NUKA_PHI_OK = 0, NUKA_PHI_UNSUPPORTED = 1, NUKA_PHI_FAILED = 2, NUKA_PHI_OUT_OF_MEMORY = 3,
                               NUKA_PHI_INVALID_ARGUMENT = 4 } nuka_phi_status;

typedef struct nuka_phi_backend nuka_phi_backend;
typedef struct nuka_phi_device nuka_phi_device;
typedef struct nuka_phi_registry_entry nuka_phi_registry_entry;
typedef struct nuka_phi_buffer_type nuka_phi_buffer_type;
typedef struct nuka_phi_buffer nuka_phi_buffer;
typedef struct nuka_phi_plan nuka_phi_plan;
typedef struct nuka_phi_event nuka_phi_event;
typedef struct nuka_phi_model_view nuka_phi_model_view;   /* flat aggregate of device pointers, one per template table */
typedef struct nuka_phi_data_view nuka_phi_data_view;     /* flat aggregate of device pointers, one per state field */

/* src/phi/backend.hpp:47-52 */
typedef struct nuka_phi_execution_error {
    uint8_t status;
    uint16_t failed_op;
    int32_t native_code;
    char message[256];
} nuka_phi_execution_error;

/* src/phi/backend.hpp:54-62 */
typedef struct nuka_phi_resource_info {
    uint64_t free_bytes, total_bytes, thread_stack_limit_bytes, graph_used_bytes, graph_reserved_bytes;
    uint32_t compute_units, threads_per_unit;
} nuka_phi_resource_info;

/* src/phi/backend.hpp:64-72 */
typedef struct nuka_phi_plan_metrics {
    uint64_t nodes, kernels, clears, copies, early_launch_dependencies, capture_lanes, forked_operators;
} nuka_phi_plan_metrics;

/* src/phi/backend.hpp:78-81: an op id and its parameter POD, owned by the caller for the plan's lifetime */
typedef struct nuka_phi_op_call {
    uint16_t op;
    const void* params;
} nuka_phi_op_call;

typedef struct nuka_phi_buffer_type_i {
    const char* (*get_name)(nuka_phi_buffer_type*);
    nuka_phi_buffer* (*alloc)(nuka_phi_buffer_type*, size_t bytes, uint8_t* status);
    size_t (*alignment)(nuka_phi_buffer_type*);
    int (*is_host)(nuka_phi_buffer_type*);
} nuka_phi_buffer_type_i;

typedef struct nuka_phi_buffer_i {
    void (*free)(nuka_phi_buffer*);
    void* (*base)(nuka_phi_buffer*);
    uint8_t (*upload)(nuka_phi_buffer*, const void* src, size_t off, size_t n);
    uint8_t (*download)(nuka_phi_buffer*, void* dst, size_t off, size_t n);
    uint8_t (*memset)(nuka_phi_buffer*, uint8_t v, size_t off, size_t n);
    uint8_t (*copy_from)(nuka_phi_buffer* dst, nuka_phi_buffer* src, size_t doff, size_t soff, size_t n);
} nuka_phi_buffer_i;

typedef struct nuka_phi_backend_i {
    const char* (*get_name)(nuka_phi_backend*);
    void (*free)(nuka_phi_backend*);
    uint8_t (*dispatch)(nuka_phi_backend*, const nuka_phi_model_view*, const nuka_phi_data_view*, const nuka_phi_op_call*);
    uint8_t (*synchronize)(nuka_phi_backend*, nuka_phi_execution_error*);
    nuka_phi_plan* (*plan_create)(nuka_phi_backend*, const nuka_phi_model_view*, const nuka_phi_data_view*,
                                  const nuka_phi_op_call* calls, int n_calls, nuka_phi_execution_error*);
    uint8_t (*plan_execute)(nuka_phi_backend*, nuka_phi_plan*, nuka_phi_execution_error*);
    void (*plan_free)(nuka_phi_backend*, nuka_phi_plan*);
    nuka_phi_event* (*event_new)(nuka_phi_backend*);
    void (*event_record)(nuka_phi_backend*, nuka_phi_event*);
    void (*event_wait)(nuka_phi_backend*, nuka_phi_event*);
    void (*event_free)(nuka_phi_backend*, nuka_phi_event*);
    float (*event_elapsed_ms)(nuka_phi_backend*, nuka_phi_event*, nuka_phi_event*);
    nuka_phi_resource_info (*resource_info)(nuka_phi_backend*);
    nuka_phi_plan_metrics (*plan_metrics)(nuka_phi_backend*, nuka_phi_plan*);
    uint8_t (*plan_execute_repeated)(nuka_phi_backend*, nuka_phi_plan*, uint32_t count, uint32_t* submitted,
                                     nuka_phi_execution_error*);
} nuka_phi_backend_i;

typedef struct nuka_phi_device_i {
    const char* (*get_name)(nuka_phi_device*);
    void (*get_memory)(nuka_phi_device*, size_t* free_b, size_t* total_b);
    nuka_phi_backend* (*init_backend)(nuka_phi_device*, const char* params_json);
    nuka_phi_buffer_type* (*get_buffer_type)(nuka_phi_device*);
    nuka_phi_buffer_type* (*get_host_buffer_type)(nuka_phi_device*);
    bool (*supports_op)(nuka_phi_device*, uint16_t op);   /* bool, as DeviceI::supports_op (src/phi/backend.hpp:114) */
} nuka_phi_device_i;

typedef struct nuka_phi_registry_entry_i {
    const char* (*get_name)(nuka_phi_registry_entry*);
    size_t (*device_count)(nuka_phi_registry_entry*);
    nuka_phi_device* (*get_device)(nuka_phi_registry_entry*, size_t i);
    void* (*get_proc_address)(nuka_phi_registry_entry*, const char* name);
} nuka_phi_registry_entry_i;

/* Opaque-handle layout contract: the first member of every handle is its table. */
typedef struct nuka_phi_backend_head { const nuka_phi_backend_i* iface; } nuka_phi_backend_head;
typedef struct nuka_phi_device_head { const nuka_phi_device_i* iface; } nuka_phi_device_head;
typedef struct nuka_phi_registry_entry_head { const nuka_phi_registry_entry_i* iface; } nuka_phi_registry_entry_head;
typedef struct nuka_phi_buffer_type_head { const nuka_phi_buffer_type_i* iface; } nuka_phi_buffer_type_head;
typedef struct nuka_phi_buffer_head { const nuka_phi_buffer_i* iface; } nuka_phi_buffer_head;

/* The one registration hook, the counterpart of RegisterCudaBackendEntry() (src/phi/backend_cuda/cuda_backend.cu:714):
 * returns the process-wide registry entry of the HIP backend; hand it to RegisterBackend(RegistryEntry*)
 * (src/phi/registry.cpp:29-31). */
nuka_phi_registry_entry* nuka_hip_register_backend_entry(void);

/* Op ids of this backend in catalog order (subset of src/phi/op_catalog.inc), and their names. */
uint16_t nuka_hip_op_count(void);
const char* nuka_hip_op_name(uint16_t op);
/* -1 when the name is not an op of this backend. */
int nuka_hip_op_from_name(const char* name);

/* ModelView / DataView (src/nk/model/generated/views.hpp:34-36; forward-declared in src/phi/backend.hpp) are flat
 * aggregates of device pointers, one per field of src/nk/model/fields.yaml.  This backend's two views hold the fields
 * its ops touch under the same names, element types and per-entity widths, plus a few of its own; a host that keeps
 * the reference's field table fills them through the calls below instead of by struct layout.  All of them are also
 * reached through RegistryEntryI::get_proc_address under their own names (src/phi/backend.hpp:124).
 *
 * One member of a view.  `reference_name` is the field of fields.yaml the member stands for (mostly the member's own
 * name; dof_link is dof_to_link there), NULL for a member of this backend's own, which a host gives memory from its
 * solver scratch (block_descent_scratch in fields.yaml).  `dtype` is the scalar the elements are made of (0 float32,
 * 1 uint32, 2 uint64, 3 uint8), `per` the entity the field has one element group for, `scalars_per_entity` the scalars
 * of a group (a transform per link: 7), 0 where the field is sized by a count of its own (per scalar).  Model fields
 * are read for one environment: where the host replicates them per environment, the first copy serves. */
enum { NUKA_HIP_PER_ENV = 0, NUKA_HIP_PER_LINK, NUKA_HIP_PER_BODY, NUKA_HIP_PER_DOF, NUKA_HIP_PER_DOF2, NUKA_HIP_PER_CONTACT_SLOT,
       NUKA_HIP_PER_ROW_SLOT, NUKA_HIP_PER_ROW_DOF, NUKA_HIP_PER_SCALAR };
typedef struct nuka_hip_view_field_t {
    const char* name;
    const char* reference_name;
    uint8_t owner;   /* 0 model view, 1 data view */
    uint8_t dtype;
    uint8_t per;
    uint32_t scalars_per_entity;
} nuka_hip_view_field_t;
uint32_t nuka_hip_view_field_count(void);
/* 0 on success, -1 past the last field */
int nuka_hip_view_field(uint32_t index, nuka_hip_view_field_t* out);
/* bytes of the two view structs, for a host that allocates them as opaque storage (zero them first) */
size_t nuka_hip_model_view_bytes(void);
size_t nuka_hip_data_view_bytes(void);
/* Sets the member of either view that stands for each named field (`names[i]`: a name of fields.yaml, or a member's own
 * name) to `pointers[i]`; names no member stands for are ignored.  Returns the number of members still null afterwards
 * and writes their names, comma separated, to `missing` (as far as `missing_bytes` allows; may be NULL). */
int nuka_hip_bind_views(const char* const* names, void* const* pointers, uint32_t count, nuka_phi_model_view* model, nuka_phi_data_view* data,
                        char* missing, size_t missing_bytes);
/* The per-environment counts at the head of the model view, by name (links_per_env, bodies_per_env, dof, max_dof,
 * max_depth, contact_slots, rows_per_env, contact_rows_per_env, profile_count, floating_root, max_points_per_slot,
 * excluded_pair_count, joint_limit_rows, joint_friction_rows, joint_drive_rows, drive_mode, any_mujoco, contact_cone,
 * integrator, contact_dof_end, rows_from_links, free_body).  0 on success, -1 for an unknown name. */
int nuka_hip_model_view_set_count(nuka_phi_model_view* model, const char* name, uint32_t value);

#ifdef __cplusplus
}
#endif
#endif

// ifa_model_api.hip (profile "layered") -- the ifa_model_* entry points of a library that holds ONLY the layer-list worker class
// (libinferflow_amd_layered.so: ifa_runtime + the fp32-activation ops + ifa_engine_layered + the host engine).  It is what a first
// start in a fresh checkout builds when all it has to serve is a layer-list model: seconds instead of the minutes the per-format
// decode kernels of the standard network take.  The shared entry points hand over to the handle's class exactly like the full
// library's (csrc/ifa_engine*.hip); everything that belongs to the standard network alone reports that it is not in this library.
// Never linked into libinferflow_amd.so (inferflow_amd/build.py keeps this directory out of the full build).
#include "ifa_engine_state.h"

#define IFA_NEED_CLASS(m, who) do { if (!(m) || !(m)->vt) return ifa_fail(IFA_ERR_STATE, who ": this library holds the layer-list worker only"); } while (0)
#define IFA_NOT_HERE(who) return ifa_fail(IFA_ERR_STATE, who ": the standard network is not part of this library (build the full library)")

extern "C" {

int ifa_model_create(const ifa_model_config *, ifa_model **) { IFA_NOT_HERE("ifa_model_create"); }
int ifa_model_set_tensor(ifa_model *, int, int, int, int, const void *, size_t, size_t) { IFA_NOT_HERE("ifa_model_set_tensor"); }
int ifa_model_set_tensor_f16(ifa_model *, int, int, int, int, const void *, size_t, size_t) { IFA_NOT_HERE("ifa_model_set_tensor_f16"); }
int ifa_model_perf_stat(ifa_model *, int *, float *, int, int *, int) { IFA_NOT_HERE("ifa_model_perf_stat"); }
int ifa_model_tp_decode(ifa_model *, const ifa_tp_topology *, int, int, int, int *, float *) { IFA_NOT_HERE("ifa_model_tp_decode"); }
int ifa_model_tp_prefill(ifa_model *, const ifa_tp_topology *, const int *, int, int, void *, int *) { IFA_NOT_HERE("ifa_model_tp_prefill"); }
int ifa_model_tp_decode_batch(ifa_model *, const ifa_tp_topology *, int, const int *, const int *, const int *, int *, void *) { IFA_NOT_HERE("ifa_model_tp_decode_batch"); }
int ifa_comm_init_all(const int *, int, ifa_comm **) { IFA_NOT_HERE("ifa_comm_init_all"); }
int ifa_comm_abort(ifa_comm *) { IFA_NOT_HERE("ifa_comm_abort"); }
int ifa_comm_destroy(ifa_comm *) { return IFA_OK; }

int ifa_model_destroy(ifa_model *m) { return m && m->vt ? m->vt->destroy(m) : IFA_OK; }
int ifa_model_finalize(ifa_model *m) { IFA_NEED_CLASS(m, "ifa_model_finalize"); return m->vt->finalize(m); }
int ifa_model_reset(ifa_model *m) { IFA_NEED_CLASS(m, "ifa_model_reset"); return m->vt->reset(m); }
int ifa_model_kv_slots(ifa_model *m, int n_slots) { IFA_NEED_CLASS(m, "ifa_model_kv_slots"); return m->vt->kv_slots(m, n_slots); }
int ifa_model_select_kv(ifa_model *m, int slot) { IFA_NEED_CLASS(m, "ifa_model_select_kv"); return m->vt->select_kv(m, slot); }
int ifa_model_set_option(ifa_model *m, const char *name, int value)
{
    IFA_NEED_CLASS(m, "ifa_model_set_option");
    IFA_REQUIRE(name, "ifa_model_set_option: null pointer");
    return m->vt->set_option(m, name, value);
}
int ifa_model_set_excluded_tokens(ifa_model *m, const int *ids_host, int n) { IFA_NEED_CLASS(m, "ifa_model_set_excluded_tokens"); return m->vt->set_excluded_tokens(m, ids_host, n); }
int ifa_model_get_buffer(ifa_model *m, const char *name, int layer, void **dptr, size_t *bytes)
{
    IFA_NEED_CLASS(m, "ifa_model_get_buffer");
    IFA_REQUIRE(name && dptr, "ifa_model_get_buffer: null pointer");
    return m->vt->get_buffer(m, name, layer, dptr, bytes);
}
void *ifa_model_stream(ifa_model *m) { return m ? (void *)m->stream : nullptr; }
int ifa_model_forward(ifa_model *m, const int *tokens_host, int n_tokens, int prefix_len, void *logits_out_dev, int *next_token_host)
{
    IFA_NEED_CLASS(m, "ifa_model_forward");
    IFA_REQUIRE(m->finalized, "ifa_model_forward: model not finalized");
    return m->vt->forward(m, tokens_host, n_tokens, prefix_len, logits_out_dev, next_token_host);
}
int ifa_model_decode(ifa_model *m, int first_token, int start_pos, int n_steps, int *out_tokens_host, float *elapsed_ms)
{
    IFA_NEED_CLASS(m, "ifa_model_decode");
    return m->vt->decode(m, first_token, start_pos, n_steps, out_tokens_host, elapsed_ms, false);
}
int ifa_model_decode_prepare(ifa_model *m, int start_pos, int n_steps)
{
    IFA_NEED_CLASS(m, "ifa_model_decode_prepare");
    return m->vt->decode(m, 0, start_pos, n_steps, nullptr, nullptr, true);
}
int ifa_model_decode_batch(ifa_model *m, int n, const int *tokens_host, const int *positions_host, const int *kv_slots_host, int *next_tokens_host,
                           void *logits_out_dev)
{
    IFA_NEED_CLASS(m, "ifa_model_decode_batch");
    IFA_REQUIRE(m->finalized, "ifa_model_decode_batch: model not finalized");
    return m->vt->decode_batch(m, n, tokens_host, positions_host, kv_slots_host, next_tokens_host, logits_out_dev);
}

} // extern "C"

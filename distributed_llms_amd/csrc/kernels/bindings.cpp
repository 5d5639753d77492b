// pybind11 bindings for the gfx950 kernel launchers.
// Tensors cross the boundary as raw device pointers (uintptr_t) plus explicit
// shapes; the Python wrappers in distributed_llms_amd/ops check dtype/contiguity
// and pass torch's current HIP stream, so every launch is graph-capturable.
#include <pybind11/pybind11.h>

#include "launchers.h"

namespace py = pybind11;

PYBIND11_MODULE(_C_kernels, m) {
  m.doc() = "distributed_llms_amd HIP kernels (gfx950 / CDNA4)";
  m.attr("arch") = "gfx950";
  m.def("rms_norm", &dllm::rms_norm, py::arg("y"), py::arg("x"), py::arg("residual"), py::arg("w"),
        py::arg("rows"), py::arg("hidden"), py::arg("eps"), py::arg("stream"));
  m.def("embedding", &dllm::embedding);
  m.def("rope_cache_append", &dllm::rope_cache_append);
  m.def("silu_mul", &dllm::silu_mul);
  m.def("argmax", &dllm::argmax);
  m.def("add_inplace", &dllm::add_inplace);
  m.def("moe_route", &dllm::moe_route);
  m.def("moe_grouped_gemm", &dllm::moe_grouped_gemm);
  m.def("splitk_add_rms_norm", &dllm::splitk_add_rms_norm);
  m.def("splitk_reduce", &dllm::splitk_reduce);
  m.def("gemm_wide", &dllm::gemm_wide);
  m.def("gemm_wide_fp8", &dllm::gemm_wide_fp8);
  m.def("quant_fp8_rows", &dllm::quant_fp8_rows);
  m.def("rms_norm_q8", &dllm::rms_norm_q8);
  m.def("moe_wide_gemm_fp8", &dllm::moe_wide_gemm_fp8);
  m.def("splitk_add_rms_norm_q8", &dllm::splitk_add_rms_norm_q8);
  m.def("gemm_sq", &dllm::gemm_sq);
  m.def("gemm_pp_moe", &dllm::gemm_pp_moe);
  m.def("gemm_pp", &dllm::gemm_pp);
  m.def("gemm_pf", &dllm::gemm_pf);
  m.def("moe_combine", &dllm::moe_combine);
  m.def("moe_wide_gemm", &dllm::moe_wide_gemm);
  m.def("moe_router_route", &dllm::moe_router_route);
  m.def("paged_attention_decode", &dllm::paged_attention_decode);
  m.def("paged_attention_decode_rope", &dllm::paged_attention_decode_rope);
  m.def("paged_attention_prefill", &dllm::paged_attention_prefill);
  m.def("sm_embed_f32", &dllm::sm_embed_f32);
  m.def("sm_rms_norm", &dllm::sm_rms_norm);
  m.def("sm_post_norm_add", &dllm::sm_post_norm_add);
  m.def("sm_causal_conv", &dllm::sm_causal_conv);
  m.def("sm_rglru_gates", &dllm::sm_rglru_gates);
  m.def("sm_rglru_scan", &dllm::sm_rglru_scan);
  m.def("sm_clipped_glu", &dllm::sm_clipped_glu);
  m.def("sm_softcap", &dllm::sm_softcap);
  m.def("sm_attn_prep", &dllm::sm_attn_prep);
  m.def("sm_window_attn_decode", &dllm::sm_window_attn_decode);
  m.def("sm_window_attn_prefill", &dllm::sm_window_attn_prefill);
  m.def("lat_prep", &dllm::lat_prep);
  m.def("lat_q_pack", &dllm::lat_q_pack);
  m.def("lat_head_gate", &dllm::lat_head_gate);
  m.def("lat_q_fold", &dllm::lat_q_fold);
  m.def("lat_v_unfold", &dllm::lat_v_unfold);
  m.def("par_add", &dllm::par_add);
  m.def("stream_cat", &dllm::stream_cat);
  m.def("stream_set", &dllm::stream_set);
  m.def("side_gate", &dllm::side_gate);
  m.def("silu_glu", &dllm::silu_glu);
  m.def("moe_route_groups", &dllm::moe_route_groups);
  m.def("moe_router_groups", &dllm::moe_router_groups);
  m.def("relu_sq", &dllm::relu_sq);
  m.def("sm_embed_norm", &dllm::sm_embed_norm);
  m.def("sm_rownorm_rope", &dllm::sm_rownorm_rope);
  m.def("sm_stream_enter", &dllm::sm_stream_enter);
  m.def("sm_mix_add", &dllm::sm_mix_add);
  m.def("sm_token_shift", &dllm::sm_token_shift);
  m.def("sm_pool_blocks", &dllm::sm_pool_blocks);
  m.def("la_scan", &dllm::la_scan);
  m.def("dr_prep", &dllm::dr_prep);
  m.def("dr_conv_prep", &dllm::dr_conv_prep);
  m.def("sm_conv_tail", &dllm::sm_conv_tail);
  m.def("dr_scan", &dllm::dr_scan);
  m.def("dr_out_norm", &dllm::dr_out_norm);
  m.def("moe_combine_gated", &dllm::moe_combine_gated);
  m.def("p2p_inbox_bytes", &dllm::p2p_inbox_bytes);
  m.def("p2p_standin", &dllm::p2p_standin);
  m.def("p2p_host_words", &dllm::p2p_host_words);
  m.def("p2p_host_words_free", &dllm::p2p_host_words_free);
}

// XLA FFI handlers (jax.ffi custom calls) over the C ABI of librpa_hip.so: one handler per operator entry point.
//
// A handler unpacks XLA buffers into device pointers and static sizes and calls the entry point of include/rpa_hip.h
// that replaces the reference's kernel call (cited there); it holds no logic of its own and no state.  All work goes
// to the stream XLA hands over; launch shapes depend on static dimensions only, so the targets can run inside one
// compiled serving step (the reference builds one executable per token bucket,
// easydel/inference/esurge/runners/model_runner.py:629-660).  Buffers that the operation updates in place (kv_pages,
// kv_scales) must be donated and aliased to the result of the same name (input_output_aliases on the Python side,
// easydel_amd/ffi_calls.py); the scratch memory is an extra result, so that XLA owns it.
//
// Built by easydel_amd/build.py::build_ffi() where jax is installed (it needs jaxlib's xla/ffi/api headers):
//   hipcc -shared -fPIC -std=c++17 -I$(python -c "import jax.ffi; print(jax.ffi.include_dir())") -Iinclude \
//         easydel_amd/csrc/rpa_ffi.cc -Leasydel_amd/lib -lrpa_hip -Wl,-rpath,'$ORIGIN' -o easydel_amd/lib/librpa_ffi.so
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/rpa_hip.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

int Tag(ffi::DataType t) {
  switch (t) {
    case ffi::F32: return RPA_F32;
    case ffi::BF16: return RPA_BF16;
    case ffi::F16: return RPA_F16;
    case ffi::F8E4M3FN: return RPA_FP8_E4M3;
    case ffi::S8: return RPA_INT8;
    default: return -1;
  }
}

int ElemBytes(int tag) { return tag == RPA_F32 ? 4 : (tag == RPA_BF16 || tag == RPA_F16) ? 2 : 1; }

ffi::Error Done(int rc) { return rc == 0 ? ffi::Error::Success() : ffi::Error::Internal(rpa_last_error()); }

// (P, page_size, C, Dp) of a v2 [P, pg, 2*Hkv, D] or v3 [P, pg, groups, packing, Dp] page buffer: token rows of C
// combined heads of Dp stored elements.  The v3 shape for head size 64 packs K_h | V_h into one 128-wide row, the same
// bytes as rows of 64; every other head size is stored in rows of align(D, 128) elements
// (easydel/caching/ragged_page/cache.py:616-647, 695-729).
struct PageGeometry {
  int P, page_size, C, Dp;
  bool ok;
};
PageGeometry Geometry(const ffi::AnyBuffer& pages, int D) {
  auto d = pages.dimensions();
  PageGeometry g{0, 0, 0, 0, false};
  if (d.size() != 4 && d.size() != 5) return g;
  int64_t stored = d[d.size() - 1], per_token = 1;
  for (size_t a = 2; a < d.size(); ++a) per_token *= d[a];
  if (stored < D) return g;
  if (D == 64 && stored == 128 && d.size() == 5) stored = 64;
  g.P = (int)d[0];
  g.page_size = (int)d[1];
  g.C = (int)(per_token / stored);
  g.Dp = (int)stored;
  g.ok = true;
  return g;
}

bool Aliased(const ffi::AnyBuffer& in, ffi::Result<ffi::AnyBuffer>& out) { return out->untyped_data() == in.untyped_data(); }

// ---- ragged_page_attention_v2: read-only attention (ragged_page_attention.py:281-313) ----------------------------------
ffi::Error AttentionV2Impl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer kv_pages, ffi::Buffer<ffi::S32> context_lens,
                           ffi::Buffer<ffi::S32> block_tables, ffi::Buffer<ffi::S32> qsl, ffi::Buffer<ffi::S32> num_seqs,
                           ffi::Buffer<ffi::F32> softmax_aux, ffi::Result<ffi::AnyBuffer> out,
                           ffi::Result<ffi::AnyBuffer> workspace, float softmax_scale, int32_t sliding_window,
                           float logits_soft_cap, int32_t num_kv_heads, bool use_softmax_aux) {
  auto qd = q.dimensions();
  if (qd.size() != 3) return ffi::Error::InvalidArgument("query must be [T, Hq, D]");
  const int T = (int)qd[0], Hq = (int)qd[1], D = (int)qd[2], S = (int)context_lens.element_count();
  const PageGeometry g = Geometry(kv_pages, D);
  if (!g.ok || S <= 0) return ffi::Error::InvalidArgument("kv_pages must be [P, pg, 2*Hkv, D] or [P, pg, groups, packing, Dp]");
  const int M = (int)(block_tables.element_count() / S);
  return Done(rpa_ragged_paged_attention(stream, q.untyped_data(), kv_pages.untyped_data(), /*kv_scales=*/nullptr,
                                         context_lens.typed_data(), block_tables.typed_data(), qsl.typed_data(),
                                         num_seqs.typed_data(), out->untyped_data(), workspace->untyped_data(),
                                         workspace->size_bytes(), T, S, M, g.P, g.page_size, Hq, num_kv_heads, D, g.Dp, g.C,
                                         Tag(q.element_type()), Tag(kv_pages.element_type()), softmax_scale, sliding_window,
                                         logits_soft_cap, use_softmax_aux ? softmax_aux.typed_data() : nullptr));
}

// ---- ragged_page_attention_v3: fused page write + attention, pages in place (:684-695, :732-746) ------------------------
ffi::Error AttentionV3Impl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer kv_pages,
                           ffi::Buffer<ffi::S32> context_lens, ffi::Buffer<ffi::S32> block_tables, ffi::Buffer<ffi::S32> qsl,
                           ffi::Buffer<ffi::S32> distribution, ffi::Buffer<ffi::F32> softmax_aux,
                           ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> kv_pages_out,
                           ffi::Result<ffi::AnyBuffer> workspace, float softmax_scale, int32_t sliding_window,
                           float logits_soft_cap, bool use_softmax_aux) {
  auto qd = q.dimensions();
  if (qd.size() != 3 || k.dimensions().size() != 3) return ffi::Error::InvalidArgument("query / key must be [T, H, D]");
  if (!Aliased(kv_pages, kv_pages_out)) return ffi::Error::Internal("kv_pages must be donated and aliased to the second result");
  const int T = (int)qd[0], Hq = (int)qd[1], D = (int)qd[2], Hkv = (int)k.dimensions()[1], S = (int)context_lens.element_count();
  const PageGeometry g = Geometry(kv_pages, D);
  if (!g.ok || S <= 0) return ffi::Error::InvalidArgument("kv_pages must be [P, pg, 2*Hkv, D] or [P, pg, groups, packing, Dp]");
  if (k.element_type() != kv_pages.element_type() || v.element_type() != kv_pages.element_type())
    return ffi::Error::InvalidArgument("key / value must be cast to the cache dtype first (ragged_page_attention.py:570-580)");
  const int M = (int)(block_tables.element_count() / S);
  return Done(rpa_ragged_paged_attention_v3(stream, q.untyped_data(), k.untyped_data(), v.untyped_data(), kv_pages.untyped_data(),
                                            context_lens.typed_data(), block_tables.typed_data(), qsl.typed_data(),
                                            distribution.typed_data(), out->untyped_data(), workspace->untyped_data(),
                                            workspace->size_bytes(), T, S, M, g.P, g.page_size, Hq, Hkv, D, g.Dp, g.C,
                                            Tag(q.element_type()), Tag(kv_pages.element_type()), softmax_scale, sliding_window,
                                            logits_soft_cap, use_softmax_aux ? softmax_aux.typed_data() : nullptr));
}

// ---- the same over scaled 8-bit pages: quantising write + attention; pages and scales in place ---------------------------
ffi::Error AttentionV3QuantisedImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v,
                                    ffi::AnyBuffer kv_pages, ffi::Buffer<ffi::F32> kv_scales, ffi::Buffer<ffi::S32> context_lens,
                                    ffi::Buffer<ffi::S32> block_tables, ffi::Buffer<ffi::S32> qsl,
                                    ffi::Buffer<ffi::S32> distribution, ffi::Buffer<ffi::F32> softmax_aux,
                                    ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> kv_pages_out,
                                    ffi::Result<ffi::Buffer<ffi::F32>> kv_scales_out, ffi::Result<ffi::AnyBuffer> workspace,
                                    float softmax_scale, int32_t sliding_window, float logits_soft_cap, bool use_softmax_aux) {
  auto qd = q.dimensions();
  if (qd.size() != 3 || k.dimensions().size() != 3) return ffi::Error::InvalidArgument("query / key must be [T, H, D]");
  if (!Aliased(kv_pages, kv_pages_out) || kv_scales_out->typed_data() != kv_scales.typed_data())
    return ffi::Error::Internal("kv_pages and kv_scales must be donated and aliased to the results of the same name");
  const int T = (int)qd[0], Hq = (int)qd[1], D = (int)qd[2], Hkv = (int)k.dimensions()[1], S = (int)context_lens.element_count();
  const PageGeometry g = Geometry(kv_pages, D);
  if (!g.ok || S <= 0) return ffi::Error::InvalidArgument("kv_pages must be [P, pg, 2*Hkv, D] or [P, pg, groups, packing, Dp]");
  const int M = (int)(block_tables.element_count() / S);
  return Done(rpa_ragged_paged_attention_v3_quantised(
      stream, q.untyped_data(), k.untyped_data(), v.untyped_data(), kv_pages.untyped_data(), kv_scales_out->typed_data(),
      context_lens.typed_data(), block_tables.typed_data(), qsl.typed_data(), distribution.typed_data(), out->untyped_data(),
      workspace->untyped_data(), workspace->size_bytes(), T, S, M, g.P, g.page_size, Hq, Hkv, D, g.Dp, g.C, Tag(q.element_type()),
      Tag(k.element_type()), Tag(kv_pages.element_type()), softmax_scale, sliding_window, logits_soft_cap,
      use_softmax_aux ? softmax_aux.typed_data() : nullptr));
}

// ---- unified_attention: separate K and V pools [P, pg, Hkv, D] (unified_attention.py:363-388) -------------------------------
ffi::Error UnifiedAttentionImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer key_cache, ffi::AnyBuffer value_cache,
                                ffi::Buffer<ffi::S32> context_lens, ffi::Buffer<ffi::S32> block_tables,
                                ffi::Buffer<ffi::S32> qsl, ffi::Buffer<ffi::F32> softmax_aux, ffi::Result<ffi::AnyBuffer> out,
                                ffi::Result<ffi::AnyBuffer> workspace, float softmax_scale, int32_t sliding_window,
                                float logits_soft_cap, bool use_softmax_aux) {
  auto qd = q.dimensions(), kd = key_cache.dimensions();
  if (qd.size() != 3 || kd.size() != 4) return ffi::Error::InvalidArgument("query [T, Hq, D], key_cache [P, pg, Hkv, D]");
  const int T = (int)qd[0], Hq = (int)qd[1], D = (int)qd[2], S = (int)context_lens.element_count();
  if (S <= 0 || kd[3] != D) return ffi::Error::InvalidArgument("cache head size differs from the query's");
  const int M = (int)(block_tables.element_count() / S);
  // the reference passes no live-row count to this kernel: every row of context_lens is live (num_seqs = NULL)
  return Done(rpa_unified_attention(stream, q.untyped_data(), key_cache.untyped_data(), value_cache.untyped_data(),
                                    /*kv_scales=*/nullptr, context_lens.typed_data(), block_tables.typed_data(),
                                    qsl.typed_data(), /*num_seqs=*/nullptr, out->untyped_data(), workspace->untyped_data(),
                                    workspace->size_bytes(), T, S, M, (int)kd[0], (int)kd[1], Hq, (int)kd[2], D,
                                    Tag(q.element_type()), Tag(key_cache.element_type()), softmax_scale, sliding_window,
                                    logits_soft_cap, use_softmax_aux ? softmax_aux.typed_data() : nullptr));
}

// ---- kv_cache_update_jax: slice-form page scatter, pages in place (caching/ragged_page/utils.py:302-387) -----------------
ffi::Error ScatterSlicesImpl(hipStream_t stream, ffi::AnyBuffer new_kv, ffi::Buffer<ffi::S32> slice_indices,
                             ffi::AnyBuffer kv_cache_pages, ffi::Buffer<ffi::S32> total_update_slices,
                             ffi::Result<ffi::AnyBuffer> pages_out, int32_t page_size, int32_t page_shard_index) {
  if (!Aliased(kv_cache_pages, pages_out)) return ffi::Error::Internal("kv_cache_pages must be donated and aliased to the result");
  auto nd = new_kv.dimensions(), pd = kv_cache_pages.dimensions(), sd = slice_indices.dimensions();
  if (nd.size() < 2 || pd.size() != nd.size() || sd.size() != 2 || sd[0] != 3)
    return ffi::Error::InvalidArgument("new_kv [T, ...], kv_cache_pages [positions, ...] with equal token rows, slice_indices [3, N]");
  int64_t row = ElemBytes(Tag(new_kv.element_type()));
  for (size_t a = 1; a < nd.size(); ++a) row *= nd[a];
  return Done(rpa_page_scatter_slices(stream, new_kv.untyped_data(), slice_indices.typed_data(), total_update_slices.typed_data(),
                                      kv_cache_pages.untyped_data(), (int)nd[0], (int)sd[1], pd[0], page_size, row,
                                      page_shard_index));
}

// ---- the write half of the v3 operation on its own ----------------------------------------------------------------------------
ffi::Error ScatterRaggedImpl(hipStream_t stream, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer kv_pages,
                             ffi::Buffer<ffi::S32> context_lens, ffi::Buffer<ffi::S32> block_tables, ffi::Buffer<ffi::S32> qsl,
                             ffi::Buffer<ffi::S32> num_seqs, ffi::Result<ffi::AnyBuffer> kv_pages_out) {
  if (!Aliased(kv_pages, kv_pages_out)) return ffi::Error::Internal("kv_pages must be donated and aliased to the result");
  auto kd = k.dimensions();
  if (kd.size() != 3) return ffi::Error::InvalidArgument("key must be [T, Hkv, D]");
  const int T = (int)kd[0], Hkv = (int)kd[1], D = (int)kd[2], S = (int)context_lens.element_count();
  const PageGeometry g = Geometry(kv_pages, D);
  if (!g.ok || S <= 0) return ffi::Error::InvalidArgument("kv_pages must be [P, pg, 2*Hkv, D] or [P, pg, groups, packing, Dp]");
  return Done(rpa_page_scatter_ragged(stream, k.untyped_data(), v.untyped_data(), kv_pages.untyped_data(),
                                      context_lens.typed_data(), block_tables.typed_data(), qsl.typed_data(),
                                      num_seqs.typed_data(), T, S, (int)(block_tables.element_count() / S), g.P, g.page_size,
                                      Hkv, D, g.Dp, g.C, ElemBytes(Tag(kv_pages.element_type()))));
}

// ---- multi_latent_ragged_page_attention (v1 and v2: same operands; multi_latent_ragged_page_attention.py:495-511) --------
ffi::Error MlaAttentionImpl(hipStream_t stream, ffi::AnyBuffer qn, ffi::AnyBuffer qp, ffi::AnyBuffer kv, ffi::AnyBuffer pe,
                            ffi::AnyBuffer kv_pages, ffi::Buffer<ffi::S32> context_lens, ffi::Buffer<ffi::S32> block_tables,
                            ffi::Buffer<ffi::S32> qsl, ffi::Buffer<ffi::S32> distribution, ffi::Buffer<ffi::F32> softmax_aux,
                            ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> kv_pages_out,
                            ffi::Result<ffi::AnyBuffer> workspace, float softmax_scale, int32_t sliding_window,
                            float logits_soft_cap, bool use_softmax_aux) {
  auto qd = qn.dimensions(), pd = kv_pages.dimensions();  // pages [P, pg / packing, packing, row] or [P, pg, row]
  if (qd.size() != 3 || qp.dimensions().size() != 3 || (pd.size() != 3 && pd.size() != 4))
    return ffi::Error::InvalidArgument("queries [T, Hq, rank] / [T, Hq, rope], latent pages 3-D or 4-D");
  if (!Aliased(kv_pages, kv_pages_out)) return ffi::Error::Internal("kv_pages must be donated and aliased to the second result");
  const int T = (int)qd[0], Hq = (int)qd[1], rank = (int)qd[2], rope = (int)qp.dimensions()[2];
  const int S = (int)context_lens.element_count();
  if (S <= 0) return ffi::Error::InvalidArgument("empty context_lens");
  const int P = (int)pd[0], pg = pd.size() == 4 ? (int)(pd[1] * pd[2]) : (int)pd[1], row = (int)pd[pd.size() - 1];
  return Done(rpa_mla_ragged_paged_attention(stream, qn.untyped_data(), qp.untyped_data(), kv.untyped_data(), pe.untyped_data(),
                                             kv_pages.untyped_data(), context_lens.typed_data(), block_tables.typed_data(),
                                             qsl.typed_data(), distribution.typed_data(), out->untyped_data(),
                                             workspace->untyped_data(), workspace->size_bytes(), T, S,
                                             (int)(block_tables.element_count() / S), P, pg, Hq, rank, rope, row,
                                             Tag(qn.element_type()), Tag(kv_pages.element_type()), softmax_scale, sliding_window,
                                             logits_soft_cap, use_softmax_aux ? softmax_aux.typed_data() : nullptr));
}

}  // namespace

#define RPA_ATTENTION_ATTRS \
  .Attr<float>("softmax_scale").Attr<int32_t>("sliding_window").Attr<float>("logits_soft_cap")

XLA_FFI_DEFINE_HANDLER_SYMBOL(RpaAttentionV2Ffi, AttentionV2Impl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // query
                                  .Arg<ffi::AnyBuffer>()          // kv_pages
                                  .Arg<ffi::Buffer<ffi::S32>>()   // context_lens
                                  .Arg<ffi::Buffer<ffi::S32>>()   // block_tables
                                  .Arg<ffi::Buffer<ffi::S32>>()   // query_start_loc
                                  .Arg<ffi::Buffer<ffi::S32>>()   // num_seqs
                                  .Arg<ffi::Buffer<ffi::F32>>()   // softmax_aux [Hq] (read only with use_softmax_aux)
                                  .Ret<ffi::AnyBuffer>()          // out
                                  .Ret<ffi::AnyBuffer>()          // workspace
                                  RPA_ATTENTION_ATTRS.Attr<int32_t>("num_kv_heads")
                                  .Attr<bool>("use_softmax_aux"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(RpaAttentionV3Ffi, AttentionV3Impl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // query
                                  .Arg<ffi::AnyBuffer>()          // key
                                  .Arg<ffi::AnyBuffer>()          // value
                                  .Arg<ffi::AnyBuffer>()          // kv_pages (operand 3, aliased to result 1)
                                  .Arg<ffi::Buffer<ffi::S32>>()   // context_lens
                                  .Arg<ffi::Buffer<ffi::S32>>()   // block_tables
                                  .Arg<ffi::Buffer<ffi::S32>>()   // query_start_loc
                                  .Arg<ffi::Buffer<ffi::S32>>()   // distribution
                                  .Arg<ffi::Buffer<ffi::F32>>()   // softmax_aux
                                  .Ret<ffi::AnyBuffer>()          // out
                                  .Ret<ffi::AnyBuffer>()          // kv_pages
                                  .Ret<ffi::AnyBuffer>()          // workspace
                                  RPA_ATTENTION_ATTRS.Attr<bool>("use_softmax_aux"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(RpaAttentionV3QuantisedFfi, AttentionV3QuantisedImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // query
                                  .Arg<ffi::AnyBuffer>()          // key (float32 or bfloat16)
                                  .Arg<ffi::AnyBuffer>()          // value
                                  .Arg<ffi::AnyBuffer>()          // kv_pages (operand 3, aliased to result 1)
                                  .Arg<ffi::Buffer<ffi::F32>>()   // kv_scales (operand 4, aliased to result 2)
                                  .Arg<ffi::Buffer<ffi::S32>>()   // context_lens
                                  .Arg<ffi::Buffer<ffi::S32>>()   // block_tables
                                  .Arg<ffi::Buffer<ffi::S32>>()   // query_start_loc
                                  .Arg<ffi::Buffer<ffi::S32>>()   // distribution
                                  .Arg<ffi::Buffer<ffi::F32>>()   // softmax_aux
                                  .Ret<ffi::AnyBuffer>()          // out
                                  .Ret<ffi::AnyBuffer>()          // kv_pages
                                  .Ret<ffi::Buffer<ffi::F32>>()   // kv_scales
                                  .Ret<ffi::AnyBuffer>()          // workspace
                                  RPA_ATTENTION_ATTRS.Attr<bool>("use_softmax_aux"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(RpaUnifiedAttentionFfi, UnifiedAttentionImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // query
                                  .Arg<ffi::AnyBuffer>()          // key_cache
                                  .Arg<ffi::AnyBuffer>()          // value_cache
                                  .Arg<ffi::Buffer<ffi::S32>>()   // context_lens
                                  .Arg<ffi::Buffer<ffi::S32>>()   // block_tables
                                  .Arg<ffi::Buffer<ffi::S32>>()   // query_start_loc
                                  .Arg<ffi::Buffer<ffi::F32>>()   // softmax_aux
                                  .Ret<ffi::AnyBuffer>()          // out
                                  .Ret<ffi::AnyBuffer>()          // workspace
                                  RPA_ATTENTION_ATTRS.Attr<bool>("use_softmax_aux"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(RpaScatterSlicesFfi, ScatterSlicesImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // new_kv_tokens
                                  .Arg<ffi::Buffer<ffi::S32>>()   // slice_indices [3, N]
                                  .Arg<ffi::AnyBuffer>()          // kv_cache_pages (operand 2, aliased to result 0)
                                  .Arg<ffi::Buffer<ffi::S32>>()   // total_update_slices [1]
                                  .Ret<ffi::AnyBuffer>()          // kv_cache_pages
                                  .Attr<int32_t>("page_size")
                                  .Attr<int32_t>("page_shard_index"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(RpaScatterRaggedFfi, ScatterRaggedImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // key
                                  .Arg<ffi::AnyBuffer>()          // value
                                  .Arg<ffi::AnyBuffer>()          // kv_pages (operand 2, aliased to result 0)
                                  .Arg<ffi::Buffer<ffi::S32>>()   // context_lens
                                  .Arg<ffi::Buffer<ffi::S32>>()   // block_tables
                                  .Arg<ffi::Buffer<ffi::S32>>()   // query_start_loc
                                  .Arg<ffi::Buffer<ffi::S32>>()   // num_seqs
                                  .Ret<ffi::AnyBuffer>());        // kv_pages

XLA_FFI_DEFINE_HANDLER_SYMBOL(RpaMlaAttentionFfi, MlaAttentionImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // queries_nope
                                  .Arg<ffi::AnyBuffer>()          // queries_pe
                                  .Arg<ffi::AnyBuffer>()          // keys_values
                                  .Arg<ffi::AnyBuffer>()          // keys_pe
                                  .Arg<ffi::AnyBuffer>()          // kv_pages (operand 4, aliased to result 1)
                                  .Arg<ffi::Buffer<ffi::S32>>()   // context_lens
                                  .Arg<ffi::Buffer<ffi::S32>>()   // block_tables
                                  .Arg<ffi::Buffer<ffi::S32>>()   // query_start_loc
                                  .Arg<ffi::Buffer<ffi::S32>>()   // distribution
                                  .Arg<ffi::Buffer<ffi::F32>>()   // softmax_aux
                                  .Ret<ffi::AnyBuffer>()          // out
                                  .Ret<ffi::AnyBuffer>()          // kv_pages
                                  .Ret<ffi::AnyBuffer>()          // workspace
                                  RPA_ATTENTION_ATTRS.Attr<bool>("use_softmax_aux"));

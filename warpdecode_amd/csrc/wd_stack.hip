// A stack of MoE layers fed from the expert-slot cache: what a decode step does when the routed experts do
// not all fit in HBM (or are kept in a bounded pool on purpose).  The cache's device slot tables stand in for
// the reference's per-layer pointer-table upload (src/qwen38_moe.cuh:3288-3303).
//
// With a routing trace known to the host and a pool that holds at least two tokens' experts, the experts of all
// layers are acquired before the first layer is launched and every layer waits for its own fills only: the host
// link streams the token's misses back to back under the layers' compute.  With a smaller pool the fills of layer
// l+1 are queued before layer l is launched and waited for after it.  Without one, every layer
// does what the reference does (src/qwen38_moe.cuh:2323-2380): router and selection, ids to pinned host
// memory, stream synchronisation, acquire, expert dispatches.
using namespace wd;

extern "C" int wd_moe_stack_cached_f32(const wd_moe_layer *layers, int n_layers, wd_expert_cache *cache, float *d_x,
                                       float *d_layer_out, wd_moe_scratch *s, const int32_t *h_ids_trace,
                                       const int32_t *d_ids_trace, float residual_scale, unsigned flags, void *stream) {
    WD_REQUIRE(layers && n_layers > 0 && cache && s, "cached MoE stack: null layers, cache or scratch");
    WD_REQUIRE(d_x && d_layer_out, "cached MoE stack: null activation or output pointer");
    WD_REQUIRE(n_layers <= cache->n_layers, "cached MoE stack: %d layers exceed the cache's %d", n_layers, cache->n_layers);
    WD_REQUIRE((h_ids_trace == nullptr) == (d_ids_trace == nullptr), "cached MoE stack: the routing trace needs its host and device copy");
    WD_REQUIRE(!(flags & (WD_MOE_ONLY_A | WD_MOE_ONLY_B | WD_MOE_ONLY_C | WD_MOE_STAGED)), "cached MoE stack: unsupported flags");
    const bool per_layer = (flags & WD_MOE_PER_LAYER) != 0;
    flags &= ~WD_MOE_PER_LAYER;
    const hipStream_t st = as_stream(stream);
    SiteScope total_site(WD_SITE_STACK_TOTAL, st);
    auto bind = [&](int l) {
        wd_moe_layer L = layers[l];
        L.slot_of_expert = cache->d_table + static_cast<size_t>(l) * cache->n_experts;
        L.slot_pool = cache->pool;
        L.slot_bytes = cache->slot_bytes, L.slot_gate_bytes = cache->gate_bytes, L.slot_up_bytes = cache->up_bytes;
        return L;
    };
    for (int l = 0; l < n_layers; ++l) {
        const wd_moe_layer L = bind(l);
        if (const int rc = check_layer(&L, s, flags)) return rc;
        WD_REQUIRE(L.n_experts == cache->n_experts, "cached MoE stack: layer %d has %d experts, the cache %d", l, L.n_experts, cache->n_experts);
    }
    const int k = layers[0].top_k;
    const size_t part_slots = cache->parts[0].end - cache->parts[0].begin;
    const bool ahead = h_ids_trace != nullptr && part_slots >= static_cast<size_t>(4 * k);
    const bool token_ahead = h_ids_trace != nullptr && !cache->partitioned &&
                             part_slots >= 2 * static_cast<size_t>(n_layers) * k;

    if (token_ahead) {
        if (cache->fills_pending)
            if (const int rc = wait_fills(cache, st)) return rc;
        // One launch for the whole stack where its shape allows (wd_resident.cuh): to that launch the pool is one tensor of
        // slots, the routing trace names slots, and the fills of a layer that are still on their way when the launch begins
        // count the layer off when they are there (they run beside the launch, on the cache's stream).
        std::vector<wd_moe_layer> pooled;
        bool one_launch = !per_layer && flags == 0 && n_layers <= kRowsLayers && k <= kRowsK && cache->n_slots < (1u << 31);
        if (one_launch) {
            pooled.assign(layers, layers + n_layers);
            for (wd_moe_layer &L : pooled) {
                L.gate = cache->pool, L.up = cache->pool + cache->gate_bytes, L.down = cache->pool + cache->gate_bytes + cache->up_bytes;
                L.gate_stride = L.up_stride = L.down_stride = cache->slot_bytes;
                L.slot_of_expert = nullptr, L.slot_pool = nullptr;
            }
            one_launch = resident_shape(pooled.data(), n_layers, s, 0) && s->res_fits != 0 && rows_prepare(cache) == WD_OK;
        }
        cache->mark_seq = one_launch ? rows_begin_token(cache) : 0u;
        const int rc_acquire = acquire_token_ahead(cache, n_layers, h_ids_trace, k, stream);
        cache->mark_seq = 0u;
        if (rc_acquire) return rc_acquire;
        if (one_launch) {
            ResidentSlots slots{};
            if (const int rc = rows_upload(cache, n_layers, h_ids_trace, k, st, &slots.rows_trace, &slots.fill_need)) return rc;
            slots.fill_done = cache->d_fill_done, slots.n_slots = static_cast<unsigned>(cache->n_slots);
            const int rc = stack_resident(pooled.data(), n_layers, d_x, d_layer_out, s, d_ids_trace, residual_scale, st, &slots);
            if (rc != kTakePerLayer) {
                if (rc == WD_OK) ++cache->resident_tokens;
                return rc;
            }
        }
        for (int l = 0; l < n_layers; ++l) {
            const wd_moe_layer L = bind(l);
            if (const int rc = wait_layer_fills(cache, l, st)) return rc;
            if (const int rc = layer_fused(&L, d_x, d_layer_out, s, flags, d_ids_trace + static_cast<size_t>(l) * k, d_x, residual_scale, st))
                return rc;
        }
        return WD_OK;
    }
    if (h_ids_trace) {
        if (const int rc = wd_expert_cache_acquire(cache, 0, h_ids_trace, k, nullptr, stream)) return rc;
        for (int l = 0; l < n_layers; ++l) {
            const wd_moe_layer L = bind(l);
            if (ahead && l + 1 < n_layers) {
                if (const int rc = acquire_impl(cache, l + 1, h_ids_trace + static_cast<size_t>(l + 1) * k, k, nullptr, stream, true)) return rc;
            }
            if (const int rc = layer_fused(&L, d_x, d_layer_out, s, flags, d_ids_trace + static_cast<size_t>(l) * k, d_x, residual_scale, st))
                return rc;
            if (l + 1 < n_layers) {
                if (ahead) {
                    if (const int rc = wait_fills(cache, st)) return rc;
                } else if (const int rc = wd_expert_cache_acquire(cache, l + 1, h_ids_trace + static_cast<size_t>(l + 1) * k, k, nullptr, stream)) {
                    return rc;
                }
            }
        }
        return WD_OK;
    }

    for (int l = 0; l < n_layers; ++l) {
        const wd_moe_layer L = bind(l);
        // dispatch A also carries the shared expert's gate/up rows and its gate: it runs whenever there is something in it
        // (with ids given by the caller it leaves the router rows out)
        SiteScope layer_site(WD_SITE_ROUTED_TOTAL, st);
        {   // the reference's router_select bracket: router and selection, ids to the host, the synchronisation that closes it
            SiteScope select_site(WD_SITE_ROUTER, st);
            if (!(flags & WD_MOE_PRESELECTED) || L.shared_gate_inp) {
                if (const int rc = layer_fused(&L, d_x, d_layer_out, s, flags | WD_MOE_ONLY_A, nullptr, d_x, residual_scale, st)) return rc;
            }
            {
                SiteScope d2h_site(WD_SITE_ROUTER_D2H, st);
                WD_HIP(hipMemcpyAsync(s->h_ids, s->ids, sizeof(int32_t) * L.top_k, hipMemcpyDeviceToHost, st));
            }
            SiteScope sync_site(WD_SITE_ROUTER_SYNC, st);
            WD_HIP(hipStreamSynchronize(st));
        }
        if (const int rc = wd_expert_cache_acquire(cache, l, s->h_ids, L.top_k, nullptr, stream)) return rc;
        if (const int rc = layer_fused(&L, d_x, d_layer_out, s, flags | WD_MOE_ONLY_B | WD_MOE_ONLY_C, nullptr, d_x, residual_scale, st))
            return rc;
    }
    return WD_OK;
}

// Looking into a plan: its device arrays copied down, the host-side layout of the same plan for a
// machine of any size, and the facts mx_plan_get_info reports.
#include <algorithm>
#include <atomic>
#include <chrono>
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <numeric>
#include <omp.h>
#include <parallel/algorithm>
#include <queue>
#include <vector>

#include "mx_plan_parts.h"

using namespace mxp;

// Every device array of a plan copied to host memory, with a name: for tests that hold the routes
// of making a plan against each other.
extern "C" void mx_plan_arrays_free(mx_plan_array *a, int n)
{
    if (!a) return;
    for (int i = 0; i < n; ++i) {
        free(a[i].data);
        a[i].data = nullptr;
    }
}
extern "C" int mx_plan_arrays(const mx_plan *plan, mx_plan_array *out, int cap, int *n)
{
    if (!plan || !out || !n || cap < 1) {
        set_error("mx_plan_arrays: bad argument");
        return MX_ERR_ARG;
    }
    *n = 0;
    const size_t es = (size_t)mx::elem_size(plan->dtype);
    int rc = MX_OK;
    auto add = [&](const char *name, const void *dev, size_t bytes) {
        if (rc || !dev) return;
        if (*n >= cap) {
            set_error("mx_plan_arrays: more arrays than the caller has room for");
            rc = MX_ERR_ARG;
            return;
        }
        void *p = malloc(std::max<size_t>(bytes, 1));
        if (!p || (bytes && hipMemcpy(p, dev, bytes, hipMemcpyDeviceToHost) != hipSuccess)) {
            free(p);
            set_error("mx_plan_arrays: out of memory or copy failed");
            rc = MX_ERR_ALLOC;
            return;
        }
        out[*n].name = name;
        out[*n].bytes = bytes;
        out[*n].data = p;
        ++*n;
    };
    if (plan->csr_variant != 1) {
        const mx::DeviceCsr &A = plan->csr;
        add("csr.rowPtr", A.rowPtr, ((size_t)A.rows + 1) * 4);
        add("csr.col", A.col, (size_t)A.nnz * 4);
        add("csr.col16", A.col16, (size_t)A.nnz * 2);
        add("csr.colBase", A.colBase, (size_t)A.nBlocks * 4);
        add("csr.val", A.val, (size_t)A.nnz * es);
        add("csr.blockDesc", A.blockDesc, (size_t)A.nBlocks * 16);
        add("csr.codes", A.codes, (size_t)A.nnz);
        add("csr.dict", A.dict, 256 * es);
    }
    if (plan->csr_variant != 0) {
        const mx::DeviceSlices &D = plan->slices;
        const size_t nEcol = ((size_t)D.steps + mx::kSlicePadSteps) * 64 * mx::slice_step_entries(plan->dtype);
        add("slices.wgDesc", D.wgDesc, ((size_t)D.nWG * 4 + 4) * 4);
        add("slices.waveDesc", D.waveDesc, ((size_t)D.nWG * mx::kSliceWaves * 4 + 4) * 4);
        add("slices.chunkEnd", D.chunkEnd, ((size_t)D.chunks + 64) * 4);
        add("slices.ecol", D.ecol, nEcol * 2);
        add("slices.eval", D.eval, nEcol * es);
        add("slices.ecode", D.ecode, nEcol);
        add("slices.dict", D.dict, 256 * es);
        add("slices.rowInfo", D.rowInfo, (((size_t)D.rows + 3) / 4 * 4 + 4) * 4);
        add("slices.segIdx", D.segIdx, ((size_t)D.vrows + 1) * 4);
        add("slices.lightRow", D.lightRow, (size_t)D.nLight * 4);
        add("slices.lightIdx", D.lightIdx, (size_t)D.nLight * 4 * D.lightQuads * 4);
        add("slices.heavyInfo", D.heavyInfo, ((size_t)D.nHeavy * 4 + 4) * 4);
        if (D.fused) {
            add("slices.wgGroups", D.wgGroups, ((size_t)D.nWG * 2 + 2) * 4);
            add("slices.groupNeed", D.groupNeed, ((size_t)D.nGroups + 1) * 4);
            add("slices.fusedTarget", D.fusedTarget, (size_t)D.chunks * 64 * 4);
        }
    }
    const mx::DeviceTiles *two[2] = {&plan->tiles, &plan->strips};
    static const char *const names[2][5] = {{"tiles.waveDesc", "tiles.hdr", "tiles.atox", "tiles.tcVal", "tiles.vidx"},
                                            {"strips.waveDesc", "strips.hdr", "strips.atox", "strips.tcVal", "strips.vidx"}};
    for (int t = 0; t < 2; ++t) {
        const mx::DeviceTiles &T = *two[t];
        if (T.nWaves <= 0) continue;
        add(names[t][0], T.waveDesc, (size_t)T.nWaves * 8 * 4);
        add(names[t][1], T.hdr, (size_t)T.steps * mx::kTileHdr * 4);
        add(names[t][2], T.atox, (size_t)T.steps * 64 * 4);
        add(names[t][3], T.tcVal, (size_t)T.stored * es);
        add(names[t][4], T.vidx, (size_t)T.steps * 128 * 4);
    }
    if (rc) {
        mx_plan_arrays_free(out, *n);
        *n = 0;
    }
    return rc;
}

extern "C" void mx_plan_layout_free(mx_plan_layout_view *v)
{
    if (!v) return;
    free(v->csrRowPtr);
    free(v->csrColInd);
    free(v->csrVal);
    free(v->stripRows);
    for (int t = 0; t < 2; ++t) {
        free(v->tiles[t].hdr);
        free(v->tiles[t].atox);
        free(v->tiles[t].waveDesc);
        free(v->tiles[t].valOffset);
        free(v->tiles[t].val);
    }
    std::memset(v, 0, sizeof(*v));
}

extern "C" int mx_plan_layout(const mx_partition *P, int flags, int nCU, mx_plan_layout_view *out)
{
    mx::refresh_options();
    if (!P || !out || nCU < 1) {
        set_error("mx_plan_layout: bad argument");
        return MX_ERR_ARG;
    }
    std::memset(out, 0, sizeof(*out));
    if (int rc = mx::partition_host(P)) return rc;
    const int es = mx::elem_size(P->dtype);
    auto give = [](const auto *p, size_t n) {
        typedef typename std::remove_cv<typename std::remove_pointer<decltype(p)>::type>::type T;
        T *q = (T *)malloc(std::max<size_t>(n, 1) * sizeof(T));
        if (q && n) std::memcpy(q, p, n * sizeof(T));
        return q;
    };
    try {
        out->rows = P->rows;
        out->cols = P->cols;
        out->fragM = P->fragM;
        out->fragK = P->fragK;
        out->slots = mx::tile_slots(P->dtype);
        HostPlanParts H;
        HostTiles T[2];
        if (!P->extracted) {
            out->csr_nnz = P->cdRowPtr[P->rows];
            out->csrRowPtr = give(P->cdRowPtr.data(), (size_t)P->rows + 1);
            out->csrColInd = give(P->cdColInd.data(), (size_t)out->csr_nnz);
            out->csrVal = give((const unsigned char *)P->cdVal.data(), (size_t)out->csr_nnz * es);
        } else {
            PhaseLog quiet;
            quiet.on = false;
            int rc = plan_host_parts(P, flags, H, quiet);
            if (rc) return rc;
            out->csr_nnz = H.rowPtr[P->rows];
            out->csrRowPtr = give(H.rowPtr.data(), H.rowPtr.size());
            out->csrColInd = give(H.col.data(), H.col.size());
            out->csrVal = give(H.val.data(), H.val.size());
            const void *bits = P->dtype == MX_F64 ? (const void *)P->fragBit32.data() : (const void *)P->fragBit64.data();
            rc = build_tiles(P->dtype, P->chunkNum, H.sel.data(), P->dRows, P->chunkPtr.data(), P->fragPtr.data(), bits,
                             P->tcVal.data(), P->sparse_AToX_index.data(), P->descColId.data(), P->rId.data(), nCU, T[0],
                             H.taken.empty() ? nullptr : H.taken.data());
            if (rc) return rc;
            if (!H.stripChunks.empty()) {
                rc = build_tiles(P->dtype, P->chunkNum, H.sel.data(), P->dRows, P->chunkPtr.data(), P->fragPtr.data(), bits,
                                 P->tcVal.data(), P->sparse_AToX_index.data(), P->descColId.data(), P->rId.data(), nCU, T[1],
                                 nullptr, &H.stripChunks);
                if (rc) return rc;
            }
        }
        {
            // the form of the CSR part a plan on a device with nCU compute units takes for it
            const int *rp = P->extracted ? H.rowPtr.data() : P->cdRowPtr.data();
            const int *ci = P->extracted ? H.col.data() : P->cdColInd.data();
            const void *va = P->extracted ? (const void *)H.val.data() : P->cdVal.data();
            const int S = slice_count(P->dtype, P->rows, P->cols, rp[P->rows], nCU);
            const CsrChoice pick = choose_csr_form(P->dtype, P->rows, P->cols, rp, ci, va, flags, nCU, S, H.stripRows.empty());
            out->csr_variant = pick.want[2] ? 2 : pick.want[0] && pick.want[1] ? -1 : pick.want[1] ? 1 : 0;
            out->est_rows_us = pick.usRows;
            out->est_slices_us = pick.usSlices;
        }
        std::vector<unsigned char> sr((size_t)P->rows, 0);
        if (!H.stripRows.empty()) std::memcpy(sr.data(), H.stripRows.data(), sr.size());
        out->stripRows = give(sr.data(), sr.size());
        bool ok = out->csrRowPtr && out->csrColInd && out->csrVal && out->stripRows;
        for (int t = 0; t < 2; ++t) {
            mx_tile_layout_view &V = out->tiles[t];
            V.steps = T[t].steps;
            V.nWaves = T[t].nWaves;
            V.chunks = T[t].chunkNum;
            V.nnz = T[t].vals;
            V.dense = T[t].dense ? 1 : 0;
            V.nVal = (long long)(T[t].val.size() / (size_t)es);
            V.hdr = give(T[t].hdr.data(), T[t].hdr.size());
            V.atox = give(T[t].atox.data(), T[t].atox.size());
            V.waveDesc = give(T[t].waveDesc.data(), T[t].waveDesc.size());
            V.valOffset = give(T[t].valOffset.data(), T[t].valOffset.size());
            V.val = give(T[t].val.data(), T[t].val.size());
            ok = ok && V.hdr && V.atox && V.waveDesc && V.valOffset && V.val;
        }
        if (!ok) {
            mx_plan_layout_free(out);
            set_error("mx_plan_layout: out of memory");
            return MX_ERR_ALLOC;
        }
    } catch (const std::bad_alloc &) {
        mx_plan_layout_free(out);
        set_error("mx_plan_layout: out of memory");
        return MX_ERR_ALLOC;
    }
    return MX_OK;
}

extern "C" int mx_plan_get_info(const mx_plan *plan, mx_plan_info *info)
{
    if (!plan || !info) {
        set_error("mx_plan_get_info: null argument");
        return MX_ERR_ARG;
    }
    const double es = mx::elem_size(plan->dtype);
    const int fragK = mx::frag_k(plan->dtype);
    const double bitBytes = plan->dtype == MX_F64 ? 4 : 8;
    info->dtype = plan->dtype;
    info->rows = plan->rows;
    info->cols = plan->cols;
    info->nnz = plan->nnz;
    info->tile_chunks = plan->tiles.chunkNum + plan->strips.chunkNum;
    info->tile_frags = plan->tiles.frags + plan->strips.frags;
    info->tile_nnz = plan->tile_nnz;
    info->csr_nnz = plan->csr_nnz;
    info->csr_blocks = plan->csr_variant == 1 ? plan->slices.nWG : plan->csr.nBlocks;
    info->csr_variant = plan->csr_variant;
    // what each kernel has to move at least once: its arrays, x once, its y rows
    info->csr_bytes = (double)plan->csr_nnz * (es + 4) + ((double)plan->rows + 1) * 4 + (double)plan->cols * es +
                      (double)plan->rows * es;
    // what the tile kernel reads and writes per launch: headers, column ids, values, x once per
    // column id, y once per row
    info->tile_bytes = 0.0;
    if (plan->tiles.steps)
        info->tile_bytes += (double)plan->tiles.steps * (mx::kTileHdr * 4.0 + 64 * 4.0) + (double)plan->tiles.stored * es +
                            (double)plan->tiles.frags * fragK * es + (double)plan->tiles.chunkNum * 8 * 2 * es;
    if (plan->strips.steps)  // no column ids, no old y
        info->tile_bytes += (double)plan->strips.steps * (mx::kTileHdr * 4.0) + (double)plan->strips.stored * es +
                            (double)plan->strips.frags * 8 * es + (double)plan->strips.chunkNum * 8 * es;
    (void)bitBytes;
    const bool sliceMain = plan->csr_variant == 1 || (plan->csr_variant == 2 && plan->slices.nnz > plan->csr.nnz);
    info->csr_main_kernel = sliceMain ? 1 : 0;
    info->csr_main_nnz = plan->csr_variant == 2 ? (sliceMain ? plan->slices.nnz : plan->csr.nnz) : plan->csr_nnz;
    info->tile_variant = plan->strips.steps > 0 ? (plan->dtype == MX_F64 ? 2 : 1) : 0;
    info->tile_strip_nnz = plan->strips.vals;
    info->csr_value_dict = plan->csr_variant == 1 ? (plan->slices.useDict ? plan->slices.nDict : 0)
                                                  : (plan->csr.useDict ? plan->csr.nDict : 0);
    info->est_rows_us = plan->est_rows_us;
    info->est_slices_us = plan->est_slices_us;
    info->prep_route = plan->prep_route;
    info->ext_dCols = plan->ext_dCols;
    info->ext_dRows = plan->ext_dRows;
    info->ext_nnzRowD = plan->ext_nnzRowD;
    info->ext_frags = plan->ext_frags;
    info->csr_fused = plan->csr_variant == 1 && plan->fused ? 1 : 0;
    info->opt_flags = plan->opt_flags;
    info->opt_tile_gate = plan->opt_tile_gate;
    info->csr_keep = plan->csr_variant != 0 && plan->slices.keep ? 1 : 0;
    info->touched_bytes = mxp::touched_bytes(plan);
    return MX_OK;
}



// pipeline.hip -- frame pipeline: VoxelGenerator -> conv stack -> Sparse2Dense on one stream.
//
// Counterpart of the graph the reference wires in createEngine (se-ssd-ai-trt.cpp:1138-1252) and of
// what TensorRT's executor does at run time: it owns every intermediate tensor and workspace and
// calls each plugin's enqueue in order.  BatchNorm1d + ReLU (se-ssd-ai-trt.cpp:808-856) is folded
// into each conv's epilogue.  Everything is allocated in create(); enqueue only launches kernels,
// optionally by replaying a hipGraph captured from the same enqueue sequence.
#include <memory>

#include "plugins.h"

namespace sessd {

namespace {

sessd_tensor_desc make_desc(std::initializer_list<int> dims, int type) {
    sessd_tensor_desc t;
    std::memset(&t, 0, sizeof(t));
    t.nbDims = (int)dims.size();
    int i = 0;
    for (int v : dims) t.d[i++] = v;
    t.type = type;
    t.scale = 1.0f;
    return t;
}

struct DeviceBuffer {
    void* p = nullptr;
    size_t bytes = 0;
    int alloc(size_t n) {
        bytes = n;
        SESSD_HIP_TRY(hipMalloc(&p, n ? n : 16));
        return SESSD_OK;
    }
    ~DeviceBuffer() {
        if (p) (void)hipFree(p);
    }
};

}  // namespace

struct ConvStage {
    sessd_layer_spec spec;
    std::unique_ptr<SubmConv3dLayerPlugin> subm;
    std::unique_ptr<SparseConv3dLayerPlugin> sparse;
    DeviceBuffer ws, feat, coors, num;  // coors/num only for sparse layers (they produce new ones)
    int rulebook_from = -1;             // SubM layer whose workspace holds this layer's rulebook
    sessd_tensor_desc in_desc[3], out_desc[3];
    void* coors_ptr = nullptr;  // coordinates valid AFTER this layer
    void* num_ptr = nullptr;
};

// a captured enqueue sequence, replayed while the pointers it was captured with stay the same
struct CapturedGraph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    const void* points = nullptr;
    const void* size = nullptr;
    void* dense = nullptr;
    int nodes = -1;
    void reset() {
        if (exec) (void)hipGraphExecDestroy(exec);
        if (graph) (void)hipGraphDestroy(graph);
        exec = nullptr;
        graph = nullptr;
    }
    ~CapturedGraph() { reset(); }
};

struct Pipeline {
    sessd_pipeline_desc desc;
    std::unique_ptr<VoxelGeneratorPlugin> vg;
    std::unique_ptr<Sparse2DensePlugin> s2d;
    std::vector<std::unique_ptr<ConvStage>> stages;
    DeviceBuffer vg_ws, vg_voxels, vg_coors, vg_num, s2d_ws;
    sessd_tensor_desc vg_in[2], vg_out[3], s2d_in[3], s2d_out[1];
    int max_voxels = 0;
    size_t device_bytes = 0;
    CapturedGraph captured;  // graph replay

    // Frames in flight (desc.frames_in_flight = R >= 2): R complete replicas of this pipeline (tensors, workspaces,
    // graph), used in turn, each on a stream of its own: frame t + 1 starts on the next replica while frame t is
    // still running on its own, so that the head of one frame and the launch gaps between its kernels fill with the
    // other frames' work.  `ev_in` / `ev_frame_done` tie a replica's frame to the caller's streams.
    std::vector<std::unique_ptr<Pipeline>> replicas;
    hipStream_t frame_stream = nullptr;  // (replica) the stream its frames run on
    hipEvent_t ev_in = nullptr, ev_frame_done = nullptr;
    int64_t next_ticket = 0;
    int last_replica = 0;                       // replica of the last submitted frame (layer_io, status, stats)

    // two-stream schedule: the frame's clears and the rulebook builds on `aux`; the voxelizer, the lookups on its
    // voxels and the feature chain on the caller's stream; ev_build[l] = "rulebook of layer l is ready"
    hipStream_t aux = nullptr;
    hipEvent_t ev_start = nullptr, ev_vg = nullptr, ev_fill = nullptr;
    std::vector<hipEvent_t> ev_build;

    // profiling: one event per segment boundary (see sessd_pipeline_enqueue_timed)
    std::vector<hipEvent_t> events;
    DeviceBuffer stats;  // u32[32] scratch for per-offset pair counts

    ~Pipeline() {
        replicas.clear();
        for (hipEvent_t e : {ev_in, ev_frame_done})
            if (e) (void)hipEventDestroy(e);
        if (frame_stream) (void)hipStreamDestroy(frame_stream);
        for (hipEvent_t e : events) (void)hipEventDestroy(e);
        for (hipEvent_t e : ev_build)
            if (e) (void)hipEventDestroy(e);
        if (ev_start) (void)hipEventDestroy(ev_start);
        if (ev_vg) (void)hipEventDestroy(ev_vg);
        if (ev_fill) (void)hipEventDestroy(ev_fill);
        if (aux) (void)hipStreamDestroy(aux);
    }

    // The rulebooks depend only on coordinates, the GEMMs on rulebooks + features.  The coordinate chain
    // (voxelizer, then every layer's rulebook build in order) runs on `aux`; the GEMM chain on `stream`
    // waits per layer for the rulebook it needs, so the small build kernels of later layers overlap the
    // GEMMs of earlier ones.  Under stream capture the fork/join becomes two branches of the graph.
    // Whether the last layer's gather-GEMM scatters into the dense tensor itself (overlapped schedule, matrix-core
    // kernel, same element type).  The tensor is then cleared on the fill branch, beside the GEMMs, and nothing
    // follows the last GEMM; the plugin's own cell-major pass writes fewer bytes but puts two more launches at the
    // end of the critical path (measured: frames 20-40 us longer).
    bool denseByEpilogue() const {
        if (stages.empty() || !aux) return false;
        const ConvStage& st = *stages.back();
        const ConvPluginBase* cp = st.subm ? static_cast<const ConvPluginBase*>(st.subm.get()) : st.sparse.get();
        return cp->out_type_ == s2d->out_type_ && cp->out_channel_ == s2d->feature_map_channel_ && cp->gemmOnMatrixCores();
    }

    int enqueueOverlapped(const void* points, const void* points_size, void* dense, hipStream_t stream) {
        SESSD_HIP_TRY(hipEventRecord(ev_start, stream));
        SESSD_HIP_TRY(hipStreamWaitEvent(aux, ev_start, 0));
        // The kernel that produced a coors tensor has left a cell -> row hash behind (the voxelizer's, or a
        // strided layer's): a SubM layer on the same grid looks its neighbours up in that table and skips its
        // own insert pass (and the clear of its own table).  Keys are (z*Y + y)*X + x: the same number in both
        // grids when X and Y agree; cells of the layer's grid beyond the table's z extent are simply absent.
        // (Beyond 2^20 slots -- 4 MB of keys, one XCD's L2 -- probing the upstream table costs more than the
        // insert pass it saves.)  The first 3x3x3 SubM rulebook behind a producer is built with the symmetric
        // lookup (13 probes per row instead of 27): the producer initialises the mirrored entries of the rows
        // it creates (MirrorInit).
        std::vector<char> probes_upstream(stages.size(), 0), mirrored(stages.size(), 0);
        std::vector<MirrorInit> mirror_of(stages.size() + 1);  // [0]: the voxelizer, [l + 1]: strided stage l
        {
            uint32_t mask = vg->cellTable(vg_ws.p, desc.max_points).mask;
            int cx = vg->grid_x_size_, cy = vg->grid_y_size_, cz = vg->grid_z_size_;
            size_t producer = 0;
            for (size_t l = 0; l < stages.size(); ++l) {
                ConvStage& st = *stages[l];
                if (st.subm) {
                    probes_upstream[l] = st.rulebook_from < 0 && st.subm->out_shape_x_ == cx &&
                                         st.subm->out_shape_y_ == cy && st.subm->out_shape_z_ >= cz && mask < (1u << 20);
                    if (probes_upstream[l] && !mirror_of[producer].nbr) {
                        const MirrorInit m = st.subm->mirrorInit(st.ws.p);
                        if (m.nbr) {
                            mirror_of[producer] = m;
                            mirrored[l] = 1;
                        }
                    }
                } else {
                    mask = st.sparse->cellTable(st.ws.p).mask;
                    cx = st.sparse->out_shape_x_;
                    cy = st.sparse->out_shape_y_;
                    cz = st.sparse->out_shape_z_;
                    producer = l + 1;
                }
            }
        }
        // The head of the frame -- the voxelizer and the lookups of the SubM layers on its voxels, which the first
        // GEMMs wait for -- runs on the caller's stream itself, in front of those GEMMs: a kernel starts 1-2 us
        // behind its producer on the same branch of the graph and 5-10 us behind one on another branch.  The
        // status words of those SubM layers are cleared in the voxelizer's own clear launch.
        const bool head_off = false;
        std::vector<char> on_head(stages.size(), 0);
        FillArgs head_clears;
        for (size_t l = 0; l < stages.size() && !head_off; ++l) {
            ConvStage& st = *stages[l];
            if (!st.subm) break;
            if (st.rulebook_from >= 0) continue;
            if (!probes_upstream[l] || !st.ws.p) break;
            on_head[l] = 1;
            st.subm->collectFill(st.ws.p, head_clears, false);
        }
        hipStream_t head = head_off ? aux : stream;
        const void* vin[2] = {points, points_size};
        void* vout[3] = {vg_voxels.p, vg_coors.p, vg_num.p};
        SESSD_TRY(vg->enqueue(vg_in, vg_out, vin, vout, vg_ws.p, head, mirror_of[0].nbr ? &mirror_of[0] : nullptr, &head_clears));
        SESSD_HIP_TRY(hipEventRecord(ev_vg, head));
        // every other clear of the frame (hash tables, neighbour tables, status words, the dense tensor) has no
        // input: they run batched at the head of `aux`, which has nothing else to do while the voxelizer works (a
        // stream of their own measured the same)
        {
            FillArgs f;
            auto flush = [&]() -> int {
                const int rc = launch_fill(f, aux);
                f = FillArgs();
                return rc;
            };
            for (size_t l = 0; l < stages.size(); ++l) {
                auto& st = stages[l];
                if (!st->ws.p || on_head[l]) continue;
                if (f.n + 6 > FillArgs::kMaxRegions) SESSD_TRY(flush());
                if (st->subm) st->subm->collectFill(st->ws.p, f, !probes_upstream[l]);
                else st->sparse->collectFill(st->ws.p, static_cast<int32_t*>(st->coors.p), f);
            }
            if (f.n + 2 > FillArgs::kMaxRegions) SESSD_TRY(flush());
            if (denseByEpilogue()) s2d->collectFill(dense, s2d_ws.p, f);
            SESSD_TRY(flush());
            SESSD_HIP_TRY(hipEventRecord(ev_fill, aux));
        }
        if (!head_off) SESSD_HIP_TRY(hipStreamWaitEvent(aux, ev_vg, 0));
        const int32_t* coors = static_cast<const int32_t*>(vg_coors.p);
        const int32_t* num = static_cast<const int32_t*>(vg_num.p);
        HashTable cells = vg->cellTable(vg_ws.p, desc.max_points);  // the table upstream of the current layer
        for (size_t l = 0; l < stages.size(); ++l) {
            ConvStage& st = *stages[l];
            if (st.subm) {
                if (st.rulebook_from >= 0) continue;
                SESSD_TRY(st.subm->enqueueBuild(coors, num, st.ws.p, on_head[l] ? stream : aux, true,
                                                probes_upstream[l] ? &cells : nullptr, mirrored[l] != 0));
                if (on_head[l]) continue;  // (its GEMM follows on the same stream: no event)
            } else {
                SESSD_TRY(st.sparse->enqueueBuild(coors, num, static_cast<int32_t*>(st.coors.p),
                                                  static_cast<int32_t*>(st.num.p), st.ws.p, aux, true,
                                                  mirror_of[l + 1].nbr ? &mirror_of[l + 1] : nullptr));
                coors = static_cast<const int32_t*>(st.coors.p);
                num = static_cast<const int32_t*>(st.num.p);
                cells = st.sparse->cellTable(st.ws.p);
            }
            SESSD_HIP_TRY(hipEventRecord(ev_build[l], aux));
        }
        if (head_off) SESSD_HIP_TRY(hipStreamWaitEvent(stream, ev_vg, 0));
        const void* feat = vg_voxels.p;
        coors = static_cast<const int32_t*>(vg_coors.p);
        num = static_cast<const int32_t*>(vg_num.p);
        int last_waited = -1;
        bool scattered = false;
        for (size_t l = 0; l < stages.size(); ++l) {
            ConvStage& st = *stages[l];
            const int owner = st.rulebook_from >= 0 ? st.rulebook_from : (int)l;
            if (owner > last_waited) {
                if (!on_head[(size_t)owner]) SESSD_HIP_TRY(hipStreamWaitEvent(stream, ev_build[owner], 0));
                last_waited = owner;
            }
            // the last layer's epilogue also writes the dense tensor when it runs on the matrix cores and its
            // rows have the dense tensor's element type: the scatter kernel and its launch drop off the end
            // of the critical path
            DenseTarget dt;
            const bool fuse = l + 1 == stages.size() && denseByEpilogue();
            if (fuse) {
                SESSD_HIP_TRY(hipStreamWaitEvent(stream, ev_fill, 0));
                const int32_t* oc = st.subm ? coors : static_cast<const int32_t*>(st.coors.p);
                dt = s2d->denseTarget(dense, oc, s2d_ws.p);
                scattered = true;
            }
            if (st.subm) {
                SESSD_TRY(st.subm->enqueueGemm(feat, st.feat.p, num, stages[owner]->ws.p, stream, fuse ? &dt : nullptr));
            } else {
                SESSD_TRY(st.sparse->enqueueGemm(feat, st.feat.p, static_cast<const int32_t*>(st.num.p), st.ws.p, stream,
                                                 fuse ? &dt : nullptr));
                coors = static_cast<const int32_t*>(st.coors.p);
                num = static_cast<const int32_t*>(st.num.p);
            }
            feat = st.feat.p;
        }
        if (scattered) return SESSD_OK;
        // every event of `aux` has been waited on by now (the last build is the last aux operation)
        if (stages.empty()) SESSD_HIP_TRY(hipStreamWaitEvent(stream, ev_vg, 0));
        SESSD_HIP_TRY(hipStreamWaitEvent(stream, ev_fill, 0));
        const void* din[3] = {feat, coors, num};
        void* dout[1] = {dense};
        return s2d->enqueue(s2d_in, s2d_out, din, dout, s2d_ws.p, stream);
    }

    int enqueueDirect(const void* points, const void* points_size, void* dense, hipStream_t stream) {
        const void* vin[2] = {points, points_size};
        void* vout[3] = {vg_voxels.p, vg_coors.p, vg_num.p};
        SESSD_TRY(vg->enqueue(vg_in, vg_out, vin, vout, vg_ws.p, stream));
        return enqueueAfterVoxelizer(dense, stream);
    }

    int enqueueAfterVoxelizer(void* dense, hipStream_t stream) {
        const void* feat = vg_voxels.p;
        const void* coors = vg_coors.p;
        const void* num = vg_num.p;
        for (auto& st : stages) {
            const void* in[3] = {feat, coors, num};
            if (st->subm) {
                void* out[1] = {st->feat.p};
                if (st->rulebook_from >= 0)
                    SESSD_TRY(st->subm->enqueueShared(st->in_desc, st->out_desc, in, out,
                                                      stages[st->rulebook_from]->ws.p, stream));
                else
                    SESSD_TRY(st->subm->enqueue(st->in_desc, st->out_desc, in, out, st->ws.p, stream));
            } else {
                void* out[3] = {st->feat.p, st->coors.p, st->num.p};
                SESSD_TRY(st->sparse->enqueue(st->in_desc, st->out_desc, in, out, st->ws.p, stream));
                coors = st->coors.p;
                num = st->num.p;
            }
            feat = st->feat.p;
        }
        const void* din[3] = {feat, coors, num};
        void* dout[1] = {dense};
        return s2d->enqueue(s2d_in, s2d_out, din, dout, s2d_ws.p, stream);
    }
};

static int build_pipeline(const sessd_pipeline_desc& d, Pipeline* P) {
    if (d.n_layers < 0 || (d.n_layers && (!d.layers || !d.weights)))
        return fail(SESSD_E_INVALID, "pipeline: layers/weights missing");
    if (d.feature_dtype != SESSD_FLOAT && d.feature_dtype != SESSD_HALF)
        return fail(SESSD_E_UNSUPPORTED, "pipeline: feature_dtype must be FP32 or FP16");
    if (d.max_points <= 0 || d.point_features < 4) return fail(SESSD_E_INVALID, "pipeline: bad points shape");
    P->desc = d;
    // rows of every conv-layer tensor; the voxelizer's own cap (voxelgen.max_voxels) may be lower: strided
    // layers can produce more sites than they are given
    const int V = d.layer_max_voxels > 0 ? d.layer_max_voxels : d.voxelgen.max_voxels;
    if (V < d.voxelgen.max_voxels) return fail(SESSD_E_INVALID, "pipeline: layer_max_voxels below the voxelizer's cap");
    const int VG = d.voxelgen.max_voxels;
    P->max_voxels = V;
    const int ft = d.feature_dtype;
    size_t total = 0;

    VoxelGeneratorPlugin* vg = nullptr;
    SESSD_TRY(VoxelGeneratorPlugin::create(d.voxelgen, &vg));
    P->vg.reset(vg);
    vg->flags_ = d.flags;
    P->vg_in[0] = make_desc({1, d.max_points, d.point_features}, SESSD_FLOAT);
    P->vg_in[1] = make_desc({1}, SESSD_INT32);
    P->vg_out[0] = make_desc({1, VG, 4}, SESSD_FLOAT);
    P->vg_out[1] = make_desc({1, VG, 4}, SESSD_INT32);
    P->vg_out[2] = make_desc({1}, SESSD_INT32);
    SESSD_TRY(vg->configurePlugin(P->vg_in, 2, P->vg_out, 3));
    SESSD_TRY(P->vg_ws.alloc(vg->getWorkspaceSize(P->vg_in, 2, P->vg_out, 3)));
    SESSD_TRY(P->vg_voxels.alloc((size_t)V * 4 * sizeof(float)));
    SESSD_TRY(P->vg_coors.alloc((size_t)V * 4 * sizeof(int32_t)));
    SESSD_TRY(P->vg_num.alloc(256));
    total += P->vg_ws.bytes + P->vg_voxels.bytes + P->vg_coors.bytes + 256;

    int in_type = SESSD_FLOAT;  // the voxelizer's means are FP32
    int in_ch = 4;
    int last_subm_with_rulebook = -1;
    for (int l = 0; l < d.n_layers; ++l) {
        const sessd_layer_spec& s = d.layers[l];
        if (s.in_channel != in_ch)
            return fail(SESSD_E_INVALID, "pipeline: layer %d expects %d input channels, previous layer has %d", l,
                        s.in_channel, in_ch);
        auto st = std::make_unique<ConvStage>();
        st->spec = s;
        st->in_desc[0] = make_desc({1, V, s.in_channel}, in_type);
        st->in_desc[1] = make_desc({1, V, 4}, SESSD_INT32);
        st->in_desc[2] = make_desc({1}, SESSD_INT32);
        st->out_desc[0] = make_desc({1, V, s.out_channel}, ft);
        st->out_desc[1] = make_desc({1, V, 4}, SESSD_INT32);
        st->out_desc[2] = make_desc({1}, SESSD_INT32);
        ConvPluginBase* base = nullptr;
        if (s.type == SESSD_LAYER_SUBM) {
            sessd_submconv3d_desc cd;
            std::memset(&cd, 0, sizeof(cd));
            cd.in_channel = s.in_channel;
            cd.out_channel = s.out_channel;
            cd.max_voxels = V;
            cd.feature_num = s.in_channel;  // se-ssd-ai-trt.cpp:739
            for (int a = 0; a < 3; ++a) cd.out_shape[a] = cd.spatial_shape[a] = s.out_shape[a];
            cd.ksize = s.ksize[0];
            cd.stride = s.stride[0];
            cd.padding = s.padding[0];
            cd.dilation = 1;
            SubmConv3dLayerPlugin* p = nullptr;
            SESSD_TRY(SubmConv3dLayerPlugin::create(cd, d.weights[l], &p));
            st->subm.reset(p);
            base = p;
            SESSD_TRY(p->configurePlugin(st->in_desc, 3, st->out_desc, 1));
            if (d.share_rulebooks && last_subm_with_rulebook >= 0) {
                const sessd_layer_spec& o = d.layers[last_subm_with_rulebook];
                bool same = o.ksize[0] == s.ksize[0] && o.padding[0] == s.padding[0];
                for (int a = 0; a < 3; ++a) same = same && o.out_shape[a] == s.out_shape[a];
                if (same) st->rulebook_from = last_subm_with_rulebook;
            }
            if (st->rulebook_from < 0) {
                SESSD_TRY(st->ws.alloc(p->getWorkspaceSize(st->in_desc, 3, st->out_desc, 1)));
                last_subm_with_rulebook = l;
            }
        } else if (s.type == SESSD_LAYER_SPARSE) {
            sessd_sparseconv3d_desc cd;
            std::memset(&cd, 0, sizeof(cd));
            cd.in_channel = s.in_channel;
            cd.out_channel = s.out_channel;
            cd.max_voxels = V;
            cd.feature_num = s.in_channel;
            for (int a = 0; a < 3; ++a) {
                cd.out_shape[a] = s.out_shape[a];
                cd.ksize[a] = s.ksize[a];
                cd.stride[a] = s.stride[a];
                cd.padding[a] = s.padding[a];
            }
            cd.dilation = 1;
            SparseConv3dLayerPlugin* p = nullptr;
            SESSD_TRY(SparseConv3dLayerPlugin::create(cd, d.weights[l], &p));
            st->sparse.reset(p);
            base = p;
            SESSD_TRY(p->configurePlugin(st->in_desc, 3, st->out_desc, 3));
            SESSD_TRY(st->ws.alloc(p->getWorkspaceSize(st->in_desc, 3, st->out_desc, 3)));
            SESSD_TRY(st->coors.alloc((size_t)V * 4 * sizeof(int32_t)));
            SESSD_TRY(st->num.alloc(256));
            last_subm_with_rulebook = -1;  // new coordinates: earlier rulebooks no longer apply
        } else {
            return fail(SESSD_E_INVALID, "pipeline: layer %d has unknown type %d", l, s.type);
        }
        base->flags_ = d.flags;
        SESSD_TRY(base->setEpilogue(d.scale ? d.scale[l] : nullptr, d.shift ? d.shift[l] : nullptr, d.relu));
        SESSD_TRY(st->feat.alloc((size_t)V * s.out_channel * dtype_size(ft)));
        total += st->ws.bytes + st->feat.bytes + st->coors.bytes + st->num.bytes;
        in_type = ft;
        in_ch = s.out_channel;
        P->stages.push_back(std::move(st));
    }

    if (d.dense.feature_map_channel != in_ch)
        return fail(SESSD_E_INVALID, "pipeline: sparse2dense expects %d channels, backbone ends with %d",
                    d.dense.feature_map_channel, in_ch);
    Sparse2DensePlugin* s2d = nullptr;
    SESSD_TRY(Sparse2DensePlugin::create(d.dense, &s2d));
    P->s2d.reset(s2d);
    SESSD_TRY(s2d->setPadding(d.dense_padding[0], d.dense_padding[1], d.dense_padding[2], d.dense_padding[3]));
    P->s2d_in[0] = make_desc({1, V, in_ch}, in_type);
    P->s2d_in[1] = make_desc({1, V, 4}, SESSD_INT32);
    P->s2d_in[2] = make_desc({1}, SESSD_INT32);
    P->s2d_out[0] = make_desc({1, d.dense.feature_map_channel * d.dense.feature_map_size[2], s2d->outHeight(),
                               s2d->outWidth()}, ft);
    SESSD_TRY(s2d->configurePlugin(P->s2d_in, 3, P->s2d_out, 1));
    SESSD_TRY(P->s2d_ws.alloc(s2d->getWorkspaceSize(P->s2d_in, 3, P->s2d_out, 1)));
    total += P->s2d_ws.bytes;
    P->device_bytes = total;
    if (d.overlap_streams) {
        SESSD_HIP_TRY(hipStreamCreateWithFlags(&P->aux, hipStreamNonBlocking));
        SESSD_HIP_TRY(hipEventCreateWithFlags(&P->ev_fill, hipEventDisableTiming));
        SESSD_HIP_TRY(hipEventCreateWithFlags(&P->ev_start, hipEventDisableTiming));
        SESSD_HIP_TRY(hipEventCreateWithFlags(&P->ev_vg, hipEventDisableTiming));
        P->ev_build.assign(P->stages.size(), nullptr);
        for (auto& e : P->ev_build) SESSD_HIP_TRY(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    }
    // the layer array of the caller need not outlive create()
    P->desc.layers = nullptr;
    P->desc.weights = P->desc.scale = P->desc.shift = nullptr;
    return SESSD_OK;
}

}  // namespace sessd

using namespace sessd;

extern "C" {

int sessd_reference_backbone(sessd_layer_spec* layers, int max_layers, sessd_voxelgen_desc* voxelgen,
                             sessd_sparse2dense_desc* dense) {
    // params.h:39-192: {type, cin, cout, ksize zyx, stride zyx, padding zyx, out_shape xyz}
    static const sessd_layer_spec table[14] = {
        {SESSD_LAYER_SUBM, 4, 16, {3, 3, 3}, {1, 1, 1}, {1, 1, 1}, {1408, 1600, 41}},
        {SESSD_LAYER_SUBM, 16, 16, {3, 3, 3}, {1, 1, 1}, {1, 1, 1}, {1408, 1600, 41}},
        {SESSD_LAYER_SPARSE, 16, 32, {3, 3, 3}, {2, 2, 2}, {1, 1, 1}, {704, 800, 21}},
        {SESSD_LAYER_SUBM, 32, 32, {3, 3, 3}, {1, 1, 1}, {1, 1, 1}, {704, 800, 21}},
        {SESSD_LAYER_SUBM, 32, 32, {3, 3, 3}, {1, 1, 1}, {1, 1, 1}, {704, 800, 21}},
        {SESSD_LAYER_SPARSE, 32, 64, {3, 3, 3}, {2, 2, 2}, {1, 1, 1}, {352, 400, 11}},
        {SESSD_LAYER_SUBM, 64, 64, {3, 3, 3}, {1, 1, 1}, {1, 1, 1}, {352, 400, 11}},
        {SESSD_LAYER_SUBM, 64, 64, {3, 3, 3}, {1, 1, 1}, {1, 1, 1}, {352, 400, 11}},
        {SESSD_LAYER_SUBM, 64, 64, {3, 3, 3}, {1, 1, 1}, {1, 1, 1}, {352, 400, 11}},
        {SESSD_LAYER_SPARSE, 64, 64, {3, 3, 3}, {2, 2, 2}, {0, 1, 1}, {176, 200, 5}},
        {SESSD_LAYER_SUBM, 64, 64, {3, 3, 3}, {1, 1, 1}, {1, 1, 1}, {176, 200, 5}},
        {SESSD_LAYER_SUBM, 64, 64, {3, 3, 3}, {1, 1, 1}, {1, 1, 1}, {176, 200, 5}},
        {SESSD_LAYER_SUBM, 64, 64, {3, 3, 3}, {1, 1, 1}, {1, 1, 1}, {176, 200, 5}},
        {SESSD_LAYER_SPARSE, 64, 64, {3, 1, 1}, {2, 1, 1}, {0, 0, 0}, {176, 200, 2}},
    };
    int n = 0;
    if (layers)
        for (; n < 14 && n < max_layers; ++n) layers[n] = table[n];
    if (voxelgen) {  // params.h:19-36
        voxelgen->max_num_points_per_voxel = 5;
        voxelgen->max_voxels = 60000;
        const float r[6] = {0.0f, -40.0f, -3.0f, 70.4f, 40.0f, 1.0f};
        for (int i = 0; i < 6; ++i) voxelgen->point_cloud_range[i] = r[i];
        voxelgen->voxel_feature_num = 4;
        voxelgen->voxel_size[0] = 0.05f;
        voxelgen->voxel_size[1] = 0.05f;
        voxelgen->voxel_size[2] = 0.1f;
    }
    if (dense) {  // params.h:194-197
        dense->feature_map_size[0] = 176;
        dense->feature_map_size[1] = 200;
        dense->feature_map_size[2] = 2;
        dense->feature_map_channel = 64;
    }
    return n;
}

static int pipeline_create_unguarded(const sessd_pipeline_desc* desc, sessd_pipeline** out) {
    std::unique_ptr<Pipeline> P(new Pipeline());
    if (desc->frames_in_flight >= 2) {
        // R replicas, each a complete pipeline with a stream of its own; this object only holds them and the turn
        if (desc->frames_in_flight > 8) return fail(SESSD_E_INVALID, "pipeline: at most 8 frames in flight");
        if (!desc->overlap_streams)
            return fail(SESSD_E_INVALID, "pipeline: frames_in_flight needs overlap_streams");
        sessd_pipeline_desc one = *desc;
        one.frames_in_flight = 0;
        for (int r = 0; r < desc->frames_in_flight; ++r) {
            std::unique_ptr<Pipeline> rep(new Pipeline());
            SESSD_TRY(build_pipeline(one, rep.get()));
            for (hipEvent_t* e : {&rep->ev_in, &rep->ev_frame_done})
                SESSD_HIP_TRY(hipEventCreateWithFlags(e, hipEventDisableTiming));
            SESSD_HIP_TRY(hipStreamCreateWithFlags(&rep->frame_stream, hipStreamNonBlocking));
            P->device_bytes += rep->device_bytes;
            P->max_voxels = rep->max_voxels;
            P->replicas.push_back(std::move(rep));
        }
        P->desc = *desc;
        P->desc.layers = nullptr;
        P->desc.weights = P->desc.scale = P->desc.shift = nullptr;
    } else {
        SESSD_TRY(build_pipeline(*desc, P.get()));
    }
    *out = reinterpret_cast<sessd_pipeline*>(P.release());
    return SESSD_OK;
}

int sessd_pipeline_create(const sessd_pipeline_desc* desc, sessd_pipeline** out) {
    if (!desc || !out) return fail(SESSD_E_INVALID, "pipeline_create: null argument");
    return guarded(__func__, [&]() -> int { return pipeline_create_unguarded(desc, out); });
}

// the pipeline whose tensors a query is about: with frames in flight, the replica of the last submitted frame
static Pipeline* current(sessd_pipeline* h) {
    auto* P = reinterpret_cast<Pipeline*>(h);
    return P->replicas.empty() ? P : P->replicas[(size_t)P->last_replica].get();
}

// one frame on `stream`: a replay of the captured graph when the pipeline uses graphs (re-captured when a pointer
// changed), direct launches otherwise
static int run_frame(Pipeline* P, const void* points, const void* points_size, void* dense, hipStream_t stream) {
    auto run = [&](hipStream_t st) {
        return P->aux ? P->enqueueOverlapped(points, points_size, dense, st) : P->enqueueDirect(points, points_size, dense, st);
    };
    if (!P->desc.use_graph || stream == nullptr) return run(stream);
    CapturedGraph& g = P->captured;
    if (!g.exec || g.points != points || g.size != points_size || g.dense != dense) {
        g.reset();
        SESSD_HIP_TRY(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
        const int rc = run(stream);
        hipGraph_t captured = nullptr;
        const hipError_t e = hipStreamEndCapture(stream, &captured);
        if (rc != SESSD_OK) {
            if (captured) (void)hipGraphDestroy(captured);
            return rc;
        }
        if (e != hipSuccess) return fail(SESSD_E_HIP, "pipeline: stream capture failed: %s", hipGetErrorString(e));
        g.graph = captured;
        SESSD_HIP_TRY(hipGraphInstantiate(&g.exec, g.graph, nullptr, nullptr, 0));
        size_t nodes = 0;
        if (hipGraphGetNodes(g.graph, nullptr, &nodes) == hipSuccess) g.nodes = (int)nodes;
        g.points = points;
        g.size = points_size;
        g.dense = dense;
    }
    SESSD_HIP_TRY(hipGraphLaunch(g.exec, stream));
    return SESSD_OK;
}

int sessd_pipeline_submit(sessd_pipeline* h, const void* points, const void* points_size, void* dense,
                          sessd_stream_t stream_, int64_t* ticket) {
    if (!h || !points || !points_size || !dense) return fail(SESSD_E_INVALID, "pipeline_submit: null argument");
    auto* P = reinterpret_cast<Pipeline*>(h);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t t = P->next_ticket;
    if (P->replicas.empty()) {  // one frame at a time: the frame runs on the caller's stream, join has nothing to add
        if (stream_ == SESSD_STREAM_NONE) return fail(SESSD_E_INVALID, "pipeline_submit: SESSD_STREAM_NONE needs frames_in_flight >= 2");
        SESSD_TRY(run_frame(P, points, points_size, dense, stream));
    } else {
        const int r = (int)(t % (int64_t)P->replicas.size());
        Pipeline* R = P->replicas[(size_t)r].get();
        // the frame starts on the replica's own stream once the caller's inputs are ready (the replica's previous
        // frame precedes it on that stream)
        if (stream_ != SESSD_STREAM_NONE) {
            SESSD_HIP_TRY(hipEventRecord(R->ev_in, stream));
            SESSD_HIP_TRY(hipStreamWaitEvent(R->frame_stream, R->ev_in, 0));
        }
        SESSD_TRY(run_frame(R, points, points_size, dense, R->frame_stream));
        SESSD_HIP_TRY(hipEventRecord(R->ev_frame_done, R->frame_stream));
        P->last_replica = r;
    }
    P->next_ticket = t + 1;
    if (ticket) *ticket = t;
    return SESSD_OK;
}

int sessd_pipeline_join(sessd_pipeline* h, int64_t ticket, sessd_stream_t stream_) {
    if (!h) return fail(SESSD_E_INVALID, "pipeline_join: null handle");
    auto* P = reinterpret_cast<Pipeline*>(h);
    if (ticket < 0 || ticket >= P->next_ticket) return fail(SESSD_E_INVALID, "pipeline_join: no frame with ticket %lld", (long long)ticket);
    if (P->replicas.empty()) return SESSD_OK;  // the frame ran on the stream it was submitted on
    const int64_t R = (int64_t)P->replicas.size();
    // (a ticket older than the last R frames: its replica has been reused since; waiting for the later frame on
    // it is at least as strong)
    Pipeline* rep = P->replicas[(size_t)(ticket % R)].get();
    // no stream to make wait: the calling thread waits (SESSD_STREAM_NONE is not a stream handle)
    if (stream_ == SESSD_STREAM_NONE) SESSD_HIP_TRY(hipEventSynchronize(rep->ev_frame_done));
    else SESSD_HIP_TRY(hipStreamWaitEvent(static_cast<hipStream_t>(stream_), rep->ev_frame_done, 0));
    return SESSD_OK;
}

// Queries (status, layer statistics, layer tensors read back by the caller on `stream`) are about the last submitted
// frame: with frames in flight that frame runs on its replica's own stream, which the caller's stream has to wait
// for first.
static int order_after_last_frame(sessd_pipeline* h, hipStream_t stream) {
    auto* P = reinterpret_cast<Pipeline*>(h);
    if (P->replicas.empty() || P->next_ticket == 0) return SESSD_OK;
    Pipeline* rep = P->replicas[(size_t)P->last_replica].get();
    SESSD_HIP_TRY(hipStreamWaitEvent(stream, rep->ev_frame_done, 0));
    return SESSD_OK;
}

int sessd_pipeline_wait(sessd_pipeline* h, int64_t ticket) {
    if (!h) return fail(SESSD_E_INVALID, "pipeline_wait: null handle");
    auto* P = reinterpret_cast<Pipeline*>(h);
    if (ticket < 0 || ticket >= P->next_ticket) return fail(SESSD_E_INVALID, "pipeline_wait: no frame with ticket %lld", (long long)ticket);
    if (P->replicas.empty()) return fail(SESSD_E_INVALID, "pipeline_wait: this pipeline runs its frames on the caller's stream; synchronise that");
    Pipeline* rep = P->replicas[(size_t)(ticket % (int64_t)P->replicas.size())].get();
    SESSD_HIP_TRY(hipEventSynchronize(rep->ev_frame_done));
    return SESSD_OK;
}

int sessd_pipeline_enqueue(sessd_pipeline* h, const void* points, const void* points_size, void* dense,
                           sessd_stream_t stream) {
    int64_t ticket = 0;
    SESSD_TRY(sessd_pipeline_submit(h, points, points_size, dense, stream, &ticket));
    return sessd_pipeline_join(h, ticket, stream);
}

int sessd_pipeline_layer_io(sessd_pipeline* h, int layer, void** feat, void** coors, void** voxel_num,
                            void** workspace, int32_t* channels) {
    if (!h) return fail(SESSD_E_INVALID, "pipeline_layer_io: null handle");
    Pipeline* P = current(h);
    if (layer < -1 || layer >= (int)P->stages.size()) return fail(SESSD_E_INVALID, "pipeline_layer_io: no layer %d", layer);
    void* f = P->vg_voxels.p;
    void* c = P->vg_coors.p;
    void* n = P->vg_num.p;
    void* w = P->vg_ws.p;
    int ch = 4;
    for (int l = 0; l <= layer; ++l) {
        ConvStage& st = *P->stages[l];
        f = st.feat.p;
        ch = st.spec.out_channel;
        if (st.sparse) {
            c = st.coors.p;
            n = st.num.p;
        }
        w = st.rulebook_from >= 0 ? P->stages[st.rulebook_from]->ws.p : st.ws.p;
    }
    if (feat) *feat = f;
    if (coors) *coors = c;
    if (voxel_num) *voxel_num = n;
    if (workspace) *workspace = w;
    if (channels) *channels = ch;
    return SESSD_OK;
}

int sessd_pipeline_status(sessd_pipeline* h, sessd_stream_t stream_, int32_t* status) {
    if (!h || !status) return fail(SESSD_E_INVALID, "pipeline_status: null argument");
    Pipeline* P = current(h);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    SESSD_TRY(order_after_last_frame(h, stream));
    int32_t acc = 0, s = 0;
    SESSD_TRY(read_status_word(P->vg_ws.p, P->vg->statusOffset(P->desc.max_points), stream, &s));
    acc |= s;
    for (auto& st : P->stages) {
        if (!st->ws.p) continue;
        const size_t off = st->subm ? st->subm->statusOffset() : st->sparse->statusOffset();
        SESSD_TRY(read_status_word(st->ws.p, off, stream, &s));
        acc |= s;
    }
    SESSD_TRY(read_status_word(P->s2d_ws.p, 0, stream, &s));
    acc |= s;
    *status = acc;
    return SESSD_OK;
}

int sessd_pipeline_enqueue_timed(sessd_pipeline* h, const void* points, const void* points_size, void* dense,
                                 sessd_stream_t stream_, float* segment_ms, int max_segments, int* n_segments) {
    if (!h || !points || !points_size || !dense || !segment_ms || !n_segments)
        return fail(SESSD_E_INVALID, "pipeline_enqueue_timed: null argument");
    if (!reinterpret_cast<Pipeline*>(h)->replicas.empty())
        return fail(SESSD_E_INVALID, "pipeline_enqueue_timed: per-segment timing runs one frame on the caller's stream; "
                                     "create the pipeline without frames_in_flight for it");
    Pipeline* P = current(h);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int L = (int)P->stages.size();
    const int n_seg = 2 * L + 2;  // voxelizer, {rulebook build, gather-GEMM} per layer, sparse2dense
    if (max_segments < n_seg) return fail(SESSD_E_INVALID, "pipeline_enqueue_timed: need room for %d segments", n_seg);
    if (P->events.empty()) {
        P->events.resize(n_seg + 3);  // + two back-to-back events that bracket nothing (timer overhead)
        for (auto& e : P->events) SESSD_HIP_TRY(hipEventCreate(&e));
    }
    for (int l = 0; l < L; ++l) {
        ConvPluginBase* b = P->stages[l]->subm ? static_cast<ConvPluginBase*>(P->stages[l]->subm.get())
                                               : static_cast<ConvPluginBase*>(P->stages[l]->sparse.get());
        b->ev_gemm_begin_ = P->events[2 + 2 * l];
        b->ev_gemm_end_ = P->events[3 + 2 * l];
    }
    // boundaries: e0 | voxelizer | e1 | build_0 | gb_0 | gemm_0 | ge_0 | build_1 | ... | ge_{L-1} | s2d | e_last
    // the voxelizer/first-build boundary e1 is recorded by enqueueing the voxelizer separately
    SESSD_HIP_TRY(hipEventRecord(P->events[n_seg + 1], stream));
    SESSD_HIP_TRY(hipEventRecord(P->events[n_seg + 2], stream));
    SESSD_HIP_TRY(hipEventRecord(P->events[0], stream));
    int rc;
    {
        const void* vin[2] = {points, points_size};
        void* vout[3] = {P->vg_voxels.p, P->vg_coors.p, P->vg_num.p};
        rc = P->vg->enqueue(P->vg_in, P->vg_out, vin, vout, P->vg_ws.p, stream);
    }
    if (rc == SESSD_OK) rc = hipEventRecord(P->events[1], stream) == hipSuccess ? SESSD_OK : SESSD_E_HIP;
    if (rc == SESSD_OK) rc = P->enqueueAfterVoxelizer(dense, stream);
    if (rc == SESSD_OK) rc = hipEventRecord(P->events[n_seg], stream) == hipSuccess ? SESSD_OK : SESSD_E_HIP;
    for (int l = 0; l < L; ++l) {
        ConvPluginBase* b = P->stages[l]->subm ? static_cast<ConvPluginBase*>(P->stages[l]->subm.get())
                                               : static_cast<ConvPluginBase*>(P->stages[l]->sparse.get());
        b->ev_gemm_begin_ = b->ev_gemm_end_ = nullptr;
    }
    SESSD_TRY(rc);
    SESSD_HIP_TRY(hipStreamSynchronize(stream));
    for (int i = 0; i < n_seg; ++i)
        SESSD_HIP_TRY(hipEventElapsedTime(&segment_ms[i], P->events[i], P->events[i + 1]));
    if (max_segments > n_seg)  // optional extra slot: what an empty segment measures on this stream
        SESSD_HIP_TRY(hipEventElapsedTime(&segment_ms[n_seg], P->events[n_seg + 1], P->events[n_seg + 2]));
    *n_segments = n_seg;
    return SESSD_OK;
}

int sessd_pipeline_layer_stats(sessd_pipeline* h, int layer, sessd_stream_t stream_, int64_t* n_out,
                               int64_t* pairs) {
    if (!h || !n_out || !pairs) return fail(SESSD_E_INVALID, "pipeline_layer_stats: null argument");
    Pipeline* P = current(h);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (layer < -1 || layer >= (int)P->stages.size()) return fail(SESSD_E_INVALID, "pipeline_layer_stats: no layer %d", layer);
    SESSD_TRY(order_after_last_frame(h, stream));
    void* num = nullptr;
    void* ws = nullptr;
    SESSD_TRY(sessd_pipeline_layer_io(h, layer, nullptr, nullptr, &num, &ws, nullptr));  // (of the same replica)
    int32_t n = 0;
    SESSD_HIP_TRY(hipMemcpyAsync(&n, num, sizeof(n), hipMemcpyDeviceToHost, stream));
    SESSD_HIP_TRY(hipStreamSynchronize(stream));
    *n_out = n;
    *pairs = 0;
    if (layer < 0) return SESSD_OK;
    if (!P->stats.p) SESSD_TRY(P->stats.alloc(32 * sizeof(uint32_t)));
    ConvStage& st = *P->stages[layer];
    uint32_t* dev_num = static_cast<uint32_t*>(P->stats.p);
    const int K = st.spec.ksize[0] * st.spec.ksize[1] * st.spec.ksize[2];
    if (st.subm) SESSD_TRY(st.subm->countPairs(ws, dev_num, stream));
    else SESSD_TRY(st.sparse->countPairs(ws, dev_num, stream));
    uint32_t host[32] = {0};
    SESSD_HIP_TRY(hipMemcpyAsync(host, dev_num, K * sizeof(uint32_t), hipMemcpyDeviceToHost, stream));
    SESSD_HIP_TRY(hipStreamSynchronize(stream));
    for (int k = 0; k < K; ++k) *pairs += host[k];
    return SESSD_OK;
}

size_t sessd_pipeline_device_bytes(const sessd_pipeline* h) {
    return h ? reinterpret_cast<const Pipeline*>(h)->device_bytes : 0;
}

int sessd_pipeline_num_launches(const sessd_pipeline* h) {
    if (!h) return -1;
    const Pipeline* P = reinterpret_cast<const Pipeline*>(h);
    if (!P->replicas.empty()) P = P->replicas[(size_t)P->last_replica].get();
    return P->captured.nodes;
}

void sessd_pipeline_destroy(sessd_pipeline* h) { delete reinterpret_cast<Pipeline*>(h); }

}  // extern "C"

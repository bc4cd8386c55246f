// Exercises the C++ veneer (neutronbench_amd/host/ntsHIP.hpp) the way the reference's operators do
// (core/ntsMiniBatchGraphOp.hpp:288-375, core/ntsSampler.hpp:353-529): raw device pointers, a
// Cuda_Stream, pre-zeroed outputs.  Results are compared with plain loops written here (a binding
// test; numerical parity against the oracle lives in the Python tests).  Exit status 0 = pass.
#include <math.h>
#include <string.h>

#include <algorithm>
#include <vector>

#include "ntsHIP.hpp"
#include "compat/utils/cuda_memory.hpp"

static int failures = 0;
#define EXPECT(cond)                                            \
  do {                                                          \
    if (!(cond)) {                                              \
      printf("FAILED line %d: %s\n", __LINE__, #cond);          \
      ++failures;                                               \
    }                                                           \
  } while (0)

int main() {
  const VertexId_CUDA Vd = 300, Vs = 500, F = 100;
  std::vector<VertexId_CUDA> co(Vd + 1, 0), ri;
  uint64_t state = 12345;
  auto next = [&]() {
    state = state * 6364136223846793005ull + 1442695040888963407ull;
    return (uint32_t)(state >> 33);
  };
  for (VertexId_CUDA d = 0; d < Vd; ++d) {
    const uint32_t deg = next() % 20;
    for (uint32_t k = 0; k < deg; ++k) ri.push_back(next() % Vs);
    co[d + 1] = (VertexId_CUDA)ri.size();
  }
  const VertexId_CUDA E = (VertexId_CUDA)ri.size();
  std::vector<float> x((size_t)Vs * F), w(E), ref((size_t)Vd * F, 0.f), got((size_t)Vd * F);
  for (auto &v : x) v = (float)(next() % 2001) / 1000.f - 1.f;
  for (auto &v : w) v = (float)(next() % 1000) / 1000.f;
  for (VertexId_CUDA d = 0; d < Vd; ++d)
    for (VertexId_CUDA e = co[d]; e < co[d + 1]; ++e)
      for (VertexId_CUDA f = 0; f < F; ++f) ref[(size_t)d * F + f] = fmaf(x[(size_t)ri[e] * F + f], w[e], ref[(size_t)d * F + f]);

  Cuda_Stream cs;
  deviceCSC csc;
  csc.init(Vd, E);
  csc.load_from_host(co.data(), ri.data());
  float *dx, *dw, *dout;
  allocate_gpu_buffer(&dx, (int)x.size());
  allocate_gpu_buffer(&dw, (int)E);
  allocate_gpu_buffer(&dout, (int)got.size());
  move_data_in(dx, x.data(), 0, Vs, F);
  move_data_in(dw, w.data(), 0, E, 1);
  zero_buffer(dout, (int)got.size());
  cs.Gather_By_Dst_From_Src(dx, dout, dw, csc.row_indices, csc.column_offset, 0, 0, 0, 0, E, Vd, F, true, false);
  cs.CUDA_DEVICE_SYNCHRONIZE();
  move_result_out(got.data(), dout, 0, Vd, F);
  EXPECT(memcmp(got.data(), ref.data(), got.size() * sizeof(float)) == 0);

  // second call accumulates into the same buffer (the reference's += semantics)
  cs.Gather_By_Dst_From_Src_Optim(dx, dout, dw, csc.row_indices, csc.column_offset, 0, 0, 0, 0, E, Vd, F, true, false);
  cs.CUDA_DEVICE_SYNCHRONIZE();
  move_result_out(got.data(), dout, 0, Vd, F);
  bool twice = true;
  for (size_t i = 0; i < got.size(); ++i) twice = twice && fabsf(got[i] - 2.f * ref[i]) <= 1e-5f * (1.f + fabsf(ref[i]));
  EXPECT(twice);

  // An output that was cleared with zero_buffer and then written through this header before the call is
  // not taken for zeros: the call still adds to what the buffer holds.
  {
    std::vector<float> ones(got.size(), 1.f);
    zero_buffer(dout, (int)got.size());
    move_data_in(dout, ones.data(), 0, Vd, F);
    cs.Gather_By_Dst_From_Src(dx, dout, dw, csc.row_indices, csc.column_offset, 0, 0, 0, 0, E, Vd, F, true, false);
    cs.CUDA_DEVICE_SYNCHRONIZE();
    move_result_out(got.data(), dout, 0, Vd, F);
    bool added = true;
    for (size_t i = 0; i < got.size(); ++i) added = added && fabsf(got[i] - (1.f + ref[i])) <= 1e-5f * (1.f + fabsf(ref[i]));
    EXPECT(added);
    // and a cleared output of another size or address is not confused with this one
    zero_buffer(dx, 4);
    move_data_in(dx, x.data(), 0, Vs, F);
    zero_buffer(dout, (int)got.size());
    cs.Gather_By_Src_From_Dst(dx, dout, dw, csc.column_offset, csc.row_indices, 0, 0, 0, 0, E, Vd, F, true, false);
    cs.CUDA_DEVICE_SYNCHRONIZE();
    move_result_out(got.data(), dout, 0, Vd, F);
    EXPECT(memcmp(got.data(), ref.data(), got.size() * sizeof(float)) == 0);
  }

  // zero-copy feature gather from mapped pinned host memory + label gather
  float *pinned = (float *)cudaMallocPinned((long)x.size() * sizeof(float));
  memcpy(pinned, x.data(), x.size() * sizeof(float));
  float *pinned_dev = (float *)getDevicePointer(pinned);
  std::vector<VertexId_CUDA> ids(200);
  for (auto &v : ids) v = next() % Vs;
  VertexId_CUDA *dids;
  allocate_gpu_edge(&dids, (int)ids.size());
  move_edge_in(dids, ids.data(), 0, (VertexId_CUDA)ids.size(), 1);
  float *dbatch;
  allocate_gpu_buffer(&dbatch, (int)(ids.size() * F));
  cs.zero_copy_feature_move_gpu(dbatch, pinned_dev, dids, F, (VertexId_CUDA)ids.size());
  std::vector<float> batch(ids.size() * F);
  move_result_out(batch.data(), dbatch, 0, (int)ids.size(), F);
  bool rows_ok = true;
  for (size_t i = 0; i < ids.size(); ++i)
    rows_ok = rows_ok && memcmp(&batch[i * F], &x[(size_t)ids[i] * F], F * sizeof(float)) == 0;
  EXPECT(rows_ok);
  std::vector<long> labels(Vs), lab_out(ids.size());
  for (VertexId_CUDA v = 0; v < Vs; ++v) labels[v] = (long)(v * 7 % 41);
  long *dlab, *dlab_out;
  alloc_gpu_data(&dlab, (int)Vs);
  alloc_gpu_data(&dlab_out, (int)ids.size());
  move_bytes_in(dlab, labels.data(), (long)labels.size() * sizeof(long));
  cs.global_copy_label_move_gpu(dlab_out, dlab, dids, (VertexId_CUDA)ids.size());
  NTS_VENEER_CHECK(nts_memcpy_d2h(lab_out.data(), dlab_out, lab_out.size() * sizeof(long), 1));
  bool lab_ok = true;
  for (size_t i = 0; i < ids.size(); ++i) lab_ok = lab_ok && lab_out[i] == labels[ids[i]];
  EXPECT(lab_ok);

  // edge softmax through the veneer, with a separate cache buffer
  std::vector<float> logits(E), alpha(E), cached(E);
  for (auto &v : logits) v = (float)(next() % 4001) / 1000.f - 2.f;
  float *dlog, *dalpha, *dcache;
  allocate_gpu_buffer(&dlog, (int)E);
  allocate_gpu_buffer(&dalpha, (int)E);
  allocate_gpu_buffer(&dcache, (int)E);
  move_data_in(dlog, logits.data(), 0, E, 1);
  cs.Edge_Softmax_Forward_Block(dalpha, dlog, dcache, csc.row_indices, csc.column_offset, Vd, 1);
  cs.CUDA_DEVICE_SYNCHRONIZE();
  move_result_out(alpha.data(), dalpha, 0, E, 1);
  move_result_out(cached.data(), dcache, 0, E, 1);
  bool sm_ok = memcmp(alpha.data(), cached.data(), E * sizeof(float)) == 0;
  for (VertexId_CUDA d = 0; d < Vd; ++d) {
    double s = 0;
    for (VertexId_CUDA e = co[d]; e < co[d + 1]; ++e) s += alpha[e];
    if (co[d + 1] > co[d]) sm_ok = sm_ok && fabs(s - 1.0) < 1e-5;
  }
  EXPECT(sm_ok);

  double used = 0, total = 0;
  get_gpu_mem(used, total);
  EXPECT(total > 1024.0 && used >= 0.0);

  // Schedules for static structures: a chunk of >= 2^22 edges whose arrays are uploaded once gets a
  // schedule on the third identical call; re-uploading an array drops it and the results follow the
  // new contents; structures that name no source range (the mini-batch operators) never get one.
  {
    const VertexId_CUDA Vb = 3000, Fb = 16;
    std::vector<VertexId_CUDA> cob(Vb + 1, 0), rib;
    for (VertexId_CUDA d = 0; d < Vb; ++d) {
      const uint32_t deg = d == 7 ? 600000 : 1200 + next() % 200;  // one hub, the rest medium rows
      for (uint32_t k = 0; k < deg; ++k) rib.push_back(next() % Vb);
      std::sort(rib.end() - deg, rib.end());
      cob[d + 1] = (VertexId_CUDA)rib.size();
    }
    const VertexId_CUDA Eb = (VertexId_CUDA)rib.size();
    EXPECT(Eb >= (1u << 22));
    std::vector<float> xb((size_t)Vb * Fb), outb((size_t)Vb * Fb), refb;
    for (auto &v : xb) v = (float)(next() % 2001) / 1000.f - 1.f;
    auto reference = [&]() {
      std::vector<double> r((size_t)Vb * Fb, 0.0);
      for (VertexId_CUDA d = 0; d < Vb; ++d)
        for (VertexId_CUDA e = cob[d]; e < cob[d + 1]; ++e)
          for (VertexId_CUDA f = 0; f < Fb; ++f) r[(size_t)d * Fb + f] += xb[(size_t)rib[e] * Fb + f];
      return r;
    };
    VertexId_CUDA *dco = (VertexId_CUDA *)cudaMallocGPU((long)(Vb + 1) * sizeof(VertexId_CUDA));
    VertexId_CUDA *dri = (VertexId_CUDA *)cudaMallocGPU((long)Eb * sizeof(VertexId_CUDA));
    move_bytes_in(dco, cob.data(), (long)(Vb + 1) * sizeof(VertexId_CUDA));
    move_bytes_in(dri, rib.data(), (long)Eb * sizeof(VertexId_CUDA));
    float *dxb, *doutb;
    allocate_gpu_buffer(&dxb, (int)xb.size());
    allocate_gpu_buffer(&doutb, (int)outb.size());
    move_data_in(dxb, xb.data(), 0, Vb, Fb);
    auto run_and_check = [&](const std::vector<double> &want) {
      zero_buffer(doutb, (int)outb.size());
      cs.Gather_By_Dst_From_Src(dxb, doutb, NULL, dri, dco, 0, Vb, 0, Vb, Eb, Vb, Fb, false, false);
      cs.CUDA_DEVICE_SYNCHRONIZE();
      move_result_out(outb.data(), doutb, 0, Vb, Fb);
      bool ok = true;
      for (size_t i = 0; i < outb.size(); ++i) ok = ok && fabs(outb[i] - want[i]) <= 2e-3 + 1e-4 * fabs(want[i]);
      return ok;
    };
    std::vector<double> want = reference();
    const long built0 = nts_veneer::plans_built();
    EXPECT(run_and_check(want));
    EXPECT(run_and_check(want));
    EXPECT(nts_veneer::plans_built() == built0);  // not yet: two sightings
    EXPECT(run_and_check(want));
    EXPECT(nts_veneer::plans_built() == built0 + 1);
    const long planned0 = nts_veneer::planned_calls();
    EXPECT(run_and_check(want));
    EXPECT(nts_veneer::planned_calls() == planned0 + 1);
    // new contents at the same addresses: the schedule must not survive
    for (VertexId_CUDA e = cob[7]; e < cob[8]; ++e) rib[e] = (rib[e] * 7 + 3) % Vb;
    std::sort(rib.begin() + cob[7], rib.begin() + cob[8]);
    move_bytes_in(dri, rib.data(), (long)Eb * sizeof(VertexId_CUDA));
    want = reference();
    const long planned1 = nts_veneer::planned_calls();
    EXPECT(run_and_check(want));
    EXPECT(nts_veneer::planned_calls() == planned1);
    // A write the veneer cannot see (what a libtorch operator or a kernel of the caller's own would be:
    // here a copy through the C ABI directly): the schedule that exists by now must not be used on the
    // new contents.  It is found out by the checksum taken before every scheduled call.
    EXPECT(run_and_check(want));
    EXPECT(run_and_check(want));
    const long built2 = nts_veneer::plans_built();
    EXPECT(run_and_check(want));  // third sighting of the re-uploaded arrays: scheduled again
    EXPECT(nts_veneer::plans_built() == built2 + 1 || nts_veneer::plans_built() == built2);
    EXPECT(run_and_check(want));
    const long planned2 = nts_veneer::planned_calls(), dropped0 = nts_veneer::plans_dropped_by_checksum();
    EXPECT(planned2 > planned1);
    for (VertexId_CUDA e = cob[7]; e < cob[8]; ++e) rib[e] = (rib[e] * 5 + 11) % Vb;
    std::sort(rib.begin() + cob[7], rib.begin() + cob[8]);
    EXPECT(nts_memcpy_h2d(dri, rib.data(), (size_t)Eb * sizeof(VertexId_CUDA), 1) == NTS_OK);
    want = reference();
    EXPECT(run_and_check(want));  // correct on the new contents ...
    EXPECT(nts_veneer::planned_calls() == planned2);  // ... because the schedule was not used
    EXPECT(nts_veneer::plans_dropped_by_checksum() == dropped0 + 1);
    EXPECT(nts_veneer::deferred_checks() > 0);  // the checksums ran on the side stream, next to the aggregation
    EXPECT(run_and_check(want));
    EXPECT(run_and_check(want));  // and a new schedule follows once the new contents have repeated
    EXPECT(run_and_check(want));
    EXPECT(nts_veneer::planned_calls() > planned2);
    // without a source range (as SingleGPUSampleGraphOp calls it) no schedule is ever made
    const long built1 = nts_veneer::plans_built();
    for (int rep = 0; rep < 4; ++rep) {
      zero_buffer(doutb, (int)outb.size());
      cs.Gather_By_Dst_From_Src(dxb, doutb, NULL, dri, dco, 0, 0, 0, 0, Eb, Vb, Fb, false, false);
    }
    cs.CUDA_DEVICE_SYNCHRONIZE();
    EXPECT(nts_veneer::plans_built() == built1);
    FreeEdge(dco); FreeEdge(dri); FreeBuffer(dxb); FreeBuffer(doutb);
  }

  // A whole mini-batch built on the device (nts_batch_builder_*), the way Sampler::sample_one's
  // replacement calls it, with whole neighbourhoods (fanout -1) so that plain host loops give the
  // expected layers; then the layer is aggregated through Cuda_Stream as SingleGPUSampleGraphOp does.
  {
    const VertexId_CUDA Vg = 400;
    std::vector<VertexId_CUDA> gco(Vg + 1, 0), gri;
    for (VertexId_CUDA d = 0; d < Vg; ++d) {
      std::vector<VertexId_CUDA> nb;
      const uint32_t deg = next() % 7;  // some vertices have no in-edge
      for (uint32_t k = 0; k < deg; ++k) nb.push_back(next() % Vg);
      std::sort(nb.begin(), nb.end());
      gri.insert(gri.end(), nb.begin(), nb.end());
      gco[d + 1] = (VertexId_CUDA)gri.size();
    }
    const VertexId_CUDA Eg = (VertexId_CUDA)gri.size();
    VertexId_CUDA *dgco = (VertexId_CUDA *)cudaMallocGPU((Vg + 1) * sizeof(VertexId_CUDA));
    VertexId_CUDA *dgri = (VertexId_CUDA *)cudaMallocGPU(Eg * sizeof(VertexId_CUDA));
    move_bytes_in(dgco, gco.data(), (Vg + 1) * sizeof(VertexId_CUDA));
    move_bytes_in(dgri, gri.data(), Eg * sizeof(VertexId_CUDA));
    const int32_t fanouts[2] = {-1, -1};
    const uint32_t hops = 2, max_batch = 32;
    const size_t bytes = nts_batch_builder_arena_bytes(Vg, Eg, fanouts, hops, max_batch, 0);
    EXPECT(bytes > 0);
    void *arena = cudaMallocGPU(bytes);
    nts_batch_builder_t *builder = NULL;
    NTS_VENEER_CHECK(nts_batch_builder_create(&builder, dgco, dgri, Vg, Eg, fanouts, hops, max_batch, 0, arena, bytes));
    std::vector<VertexId_CUDA> batch;
    for (VertexId_CUDA v = 3; batch.size() < 20; v += 17) batch.push_back(v % Vg);  // distinct ids
    VertexId_CUDA *dbatch_ids = (VertexId_CUDA *)cudaMallocGPU(batch.size() * sizeof(VertexId_CUDA));
    move_bytes_in(dbatch_ids, batch.data(), batch.size() * sizeof(VertexId_CUDA));
    for (int rep = 0; rep < 2; ++rep) {  // the second batch re-uses the arena
      NTS_VENEER_CHECK(nts_batch_builder_sample(builder, dbatch_ids, (uint32_t)batch.size(), 7 + rep, cs.stream));
      nts_sampled_layer_t L[2];
      NTS_VENEER_CHECK(nts_batch_builder_layers(builder, L));
      std::vector<VertexId_CUDA> dst = batch;
      for (int hop = 0; hop < 2; ++hop) {
        const nts_sampled_layer_t &l = L[1 - hop];  // L[0] is the input-side layer
        // expected: all in-neighbours of every destination, sources = sorted distinct ids
        std::vector<VertexId_CUDA> eco(dst.size() + 1, 0), eglob;
        for (size_t i = 0; i < dst.size(); ++i) {
          eglob.insert(eglob.end(), gri.begin() + gco[dst[i]], gri.begin() + gco[dst[i] + 1]);
          eco[i + 1] = (VertexId_CUDA)eglob.size();
        }
        std::vector<VertexId_CUDA> esrc = eglob;
        std::sort(esrc.begin(), esrc.end());
        esrc.erase(std::unique(esrc.begin(), esrc.end()), esrc.end());
        EXPECT(l.v_size == dst.size() && l.e_size == eglob.size() && l.src_size == esrc.size());
        if (l.v_size != dst.size() || l.e_size != eglob.size() || l.src_size != esrc.size()) break;
        std::vector<VertexId_CUDA> gotco(l.v_size + 1), gotri(l.e_size), gotsrc(l.src_size), gotro(l.src_size + 1),
            gotci(l.e_size), gotdst(l.v_size);
        std::vector<float> gotwf(l.e_size), gotwb(l.e_size);
        NTS_VENEER_CHECK(nts_memcpy_d2h(gotco.data(), l.column_offset, gotco.size() * 4, 1));
        NTS_VENEER_CHECK(nts_memcpy_d2h(gotdst.data(), l.destination, gotdst.size() * 4, 1));
        if (l.e_size) {
          NTS_VENEER_CHECK(nts_memcpy_d2h(gotri.data(), l.row_indices, gotri.size() * 4, 1));
          NTS_VENEER_CHECK(nts_memcpy_d2h(gotsrc.data(), l.source, gotsrc.size() * 4, 1));
          NTS_VENEER_CHECK(nts_memcpy_d2h(gotci.data(), l.column_indices, gotci.size() * 4, 1));
          NTS_VENEER_CHECK(nts_memcpy_d2h(gotwf.data(), l.edge_weight_forward, gotwf.size() * 4, 1));
          NTS_VENEER_CHECK(nts_memcpy_d2h(gotwb.data(), l.edge_weight_backward, gotwb.size() * 4, 1));
        }
        NTS_VENEER_CHECK(nts_memcpy_d2h(gotro.data(), l.row_offset, gotro.size() * 4, 1));
        EXPECT(gotco == eco && gotsrc == esrc && gotdst == dst);
        bool ok = true;
        std::vector<VertexId_CUDA> outdeg(esrc.size(), 0);
        for (size_t e = 0; e < eglob.size(); ++e) {
          ok = ok && gotri[e] < esrc.size() && esrc[gotri[e]] == eglob[e];
          if (ok) ++outdeg[gotri[e]];
        }
        EXPECT(ok);
        for (size_t s2 = 0; ok && s2 < esrc.size(); ++s2) ok = gotro[s2 + 1] - gotro[s2] == outdeg[s2];
        EXPECT(ok && gotro[0] == 0);
        // CSR rows list the destinations of a source in ascending edge order; weights follow
        // nts_norm_degree on the layer's own degrees
        for (size_t s2 = 0; ok && s2 < esrc.size(); ++s2) {
          VertexId_CUDA k = gotro[s2];
          for (size_t i = 0; i < dst.size(); ++i)
            for (VertexId_CUDA e = eco[i]; e < eco[i + 1]; ++e)
              if (gotri[e] == s2) {
                ok = ok && gotci[k] == i;
                const float wgt = 1.0f / ((float)sqrt((double)outdeg[s2]) * (float)sqrt((double)(eco[i + 1] - eco[i])));
                ok = ok && gotwb[k] == wgt && gotwf[e] == wgt;
                ++k;
              }
          ok = ok && k == gotro[s2 + 1];
        }
        EXPECT(ok);
        // aggregate the layer as SingleGPUSampleGraphOp::forward does
        if (l.e_size) {
          const VertexId_CUDA Fl = 24;
          std::vector<float> xl((size_t)l.src_size * Fl), want((size_t)l.v_size * Fl, 0.f), have(want.size());
          for (auto &v : xl) v = (float)(next() % 2001) / 1000.f - 1.f;
          for (size_t i = 0; i < dst.size(); ++i)
            for (VertexId_CUDA e = eco[i]; e < eco[i + 1]; ++e)
              for (VertexId_CUDA f = 0; f < Fl; ++f)
                want[i * Fl + f] = fmaf(xl[(size_t)gotri[e] * Fl + f], gotwf[e], want[i * Fl + f]);
          float *dxl, *dyl;
          allocate_gpu_buffer(&dxl, (int)xl.size());
          allocate_gpu_buffer(&dyl, (int)want.size());
          move_data_in(dxl, xl.data(), 0, l.src_size, Fl);
          zero_buffer(dyl, (int)want.size());
          cs.Gather_By_Dst_From_Src(dxl, dyl, l.edge_weight_forward, l.row_indices, l.column_offset, 0, 0, 0, 0, l.e_size,
                                    l.v_size, Fl, true, false);
          cs.CUDA_DEVICE_SYNCHRONIZE();
          move_result_out(have.data(), dyl, 0, l.v_size, Fl);
          EXPECT(memcmp(have.data(), want.data(), want.size() * sizeof(float)) == 0);
          FreeBuffer(dxl); FreeBuffer(dyl);
        }
        dst = esrc;
      }
      std::reverse(batch.begin(), batch.end());  // another order of the same ids for the second batch
      move_bytes_in(dbatch_ids, batch.data(), batch.size() * sizeof(VertexId_CUDA));
    }
    NTS_VENEER_CHECK(nts_batch_builder_destroy(builder));
    FreeEdge(dgco); FreeEdge(dgri); FreeEdge(dbatch_ids); FreeEdge((VertexId_CUDA *)arena);
  }

  csc.release();
  FreeBuffer(dx); FreeBuffer(dw); FreeBuffer(dout); FreeBuffer(dbatch); FreeBuffer(dlog); FreeBuffer(dalpha);
  FreeBuffer(dcache); FreeEdge(dids); free_gpu_data(dlab); free_gpu_data(dlab_out); ntsFreeHost(pinned);
  printf(failures ? "veneer test: %d failure(s)\n" : "veneer test: ok\n", failures);
  return failures ? 1 : 0;
}

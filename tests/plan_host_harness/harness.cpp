// Runs flagcxLocalPlanExecute (the real flagcx_amd/csrc/host_c2c_local.cpp) over host buffers
// through device_double.cpp.  Every buffer is a heap block of exactly its size, so a build with
// AddressSanitizer reports any access past an end.
// usage: harness <manifest>; one case per line:
//   prefix nranks c0 .. c{n-1} totalCount chunks commOp redOp algorithm fused dtype root scratch inDir outDir [v]
// with v: 4 * nranks * nranks more numbers follow, the counts and displacements of an AlltoAllv
// (sendCounts, sDispls, recvCounts, rDispls, row r = rank r's arrays)
#include "../../include/flagcx_amd.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

static std::vector<char> slurp(const std::string &p, size_t want) {
  std::ifstream f(p, std::ios::binary);
  std::vector<char> v(want);
  f.read(v.data(), (std::streamsize)want);
  if ((size_t)f.gcount() != want) { fprintf(stderr, "harness: %s is short\n", p.c_str()); exit(3); }
  return v;
}

int main(int argc, char **argv) {
  if (argc < 2) return 2;
  std::ifstream man(argv[1]);
  std::string line;
  int cases = 0;
  while (std::getline(man, line)) {
    if (line.empty()) continue;
    std::istringstream in(line);
    std::string prefix, inDir, outDir;
    int nr;
    in >> prefix >> nr;
    std::vector<int> cl(nr);
    for (auto &c : cl) in >> c;
    size_t total, chunks;
    int commOp, redOp, algo, fused, dt, root, useScratch;
    in >> total >> chunks >> commOp >> redOp >> algo >> fused >> dt >> root >> useScratch >> inDir >> outDir;
    std::string tag;
    std::vector<size_t> v;
    if (in >> tag && tag == "v") {
      v.resize(4 * (size_t)nr * nr);
      for (auto &x : v) in >> x;
    }
    const size_t ts = flagcxLocalGetDataTypeSize((flagcxDataType_t)dt), nbytes = total * ts;
    flagcxLocalPlan_t plan = nullptr;
    if (flagcxLocalPlanCreate(&plan, nr, cl.data(), nullptr, total, (flagcxCommOp_t)commOp, (flagcxRedOp_t)redOp) != flagcxSuccess) return 4;
    if (chunks) flagcxLocalPlanSetChunks(plan, chunks);
    flagcxResult_t r = flagcxLocalPlanImportXml(plan, prefix.c_str());
    if (r == flagcxSuccess) r = flagcxLocalPlanSetAlgorithm(plan, algo);
    if (r == flagcxSuccess) r = flagcxLocalPlanSetFused(plan, fused);
    if (r == flagcxSuccess && !v.empty()) {
      const size_t m = (size_t)nr * nr;
      r = flagcxLocalPlanSetAlltoAllv(plan, v.data(), v.data() + m, v.data() + 2 * m, v.data() + 3 * m);
    }
    std::vector<void *> send(nr), recv(nr), scr(nr, nullptr);
    for (int k = 0; k < nr; k++) {
      std::vector<char> h = slurp(inDir + "/in_" + std::to_string(k) + ".bin", nbytes);
      send[k] = malloc(nbytes);
      recv[k] = malloc(nbytes);
      memcpy(send[k], h.data(), nbytes);
      memset(recv[k], 0x55, nbytes);
      if (useScratch) {
        scr[k] = malloc(nbytes);
        memset(scr[k], 0x33, nbytes);
      }
    }
    if (r == flagcxSuccess)
      r = flagcxLocalPlanExecute(plan, (const void *const *)send.data(), recv.data(), useScratch ? scr.data() : nullptr,
                                 (flagcxDataType_t)dt, root, nullptr);
    std::ofstream st(outDir + "/status.txt");
    st << (int)r << " " << flagcxLocalPlanGetLastError(plan) << "\n";
    for (int k = 0; k < nr; k++) {
      std::ofstream o(outDir + "/out_" + std::to_string(k) + ".bin", std::ios::binary);
      o.write((const char *)recv[k], (std::streamsize)nbytes);
      std::ofstream s(outDir + "/send_" + std::to_string(k) + ".bin", std::ios::binary);
      s.write((const char *)send[k], (std::streamsize)nbytes);
      free(send[k]);
      free(recv[k]);
      free(scr[k]);
    }
    flagcxLocalPlanDestroy(plan);
    cases++;
  }
  printf("harness: %d cases\n", cases);
  return 0;
}

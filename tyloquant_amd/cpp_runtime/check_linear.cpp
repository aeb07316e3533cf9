// mfq-check-linear: the --check-linear micro-benchmark of the reference's mfq-decode
// (cpp_runtime/mfq_decode.cpp:16510-16638) for one tensor of an .mfq file.
//
//   mfq-check-linear model.mfq <tensor-name> [M=1] [reps=200]
//
// Prints key=value lines: production_ms, production_weight_gbps (device-layout bytes, the
// reference's convention), payload_gbps (compact MFQ payload bytes), production_rel,
// production_mean_abs, production_max_abs against a full dequant times x in fp64.
#include <cstdio>
#include <cstdlib>
#include <exception>

#include "mfq_runtime.h"

int main(int argc, char **argv) {
    if (argc < 3) {
        std::fprintf(stderr, "usage: %s file.mfq tensor [M] [reps]\n", argv[0]);
        return 2;
    }
    try {
        mfq_rt::MfqFile file(argv[1]);
        const mfq_rt::MfqRecord &rec = file.find(argv[2]);
        const int M = argc > 3 ? std::atoi(argv[3]) : 1, reps = argc > 4 ? std::atoi(argv[4]) : 200;
        mfq_rt::QuantLinear lin = mfq_rt::load_quant_linear(rec.dtype, file.data(rec), rec.nbytes);
        const mfq_rt::LinearCheckResult r = mfq_rt::run_linear_check(lin, M, reps);
        std::printf("check_linear tensor=%s dtype=%s out=%lld neuron_len=%lld m=%d reps=%d\n", rec.name.c_str(),
                    rec.dtype.c_str(), (long long)lin.out(), (long long)lin.neuron_len(), M, reps);
        std::printf("production_ms=%.6f production_weight_gbps=%.2f payload_gbps=%.2f weight_bytes=%lld payload_bytes=%lld\n",
                    r.production_ms, r.production_weight_gbps, r.payload_gbps, (long long)r.weight_bytes,
                    (long long)r.payload_bytes);
        std::printf("production_rel=%.3e production_mean_abs=%.3e production_max_abs=%.3e\n", r.production_rel,
                    r.production_mean_abs, r.production_max_abs);
        return 0;
    } catch (const std::exception &e) {
        std::fprintf(stderr, "error: %s\n", e.what());
        return 1;
    }
}

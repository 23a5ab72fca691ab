// Driver (ours) around the reference host operator classes: runs a .one model on the CPU with the reference's own
// operator objects (fill_operands, prepare, shape_infer, rt_prepare, forward of host/ops/*.h and host/op.h) and
// the reference's own x86 kernels, loaded by op::find_handle from $ONENEW_REF_OP_DIR/<Op>/lib<Op>_x86.so.
// The reference's net class (host/net.h) cannot be compiled here, it pulls in OpenCV through common/utils_cpp.hpp;
// this file does what net and extractor do between those calls: walk the file, order the operators, keep the
// operand descriptors and allocate one buffer per operand.  Test infrastructure: compiled only by
// `make -C oracle ref`, includes the reference headers in place.
//
//   ref_run_one model.one out_dir input0.bin [input1.bin ...]     raw fp32 inputs in io order
// writes out_dir/<n>.bin for output number n, and out_dir/shapes.txt with "<name> <ndim> <dims...>" per output;
// REF_DUMP_ALL=1 also writes every operand as out_dir/op_<index>.bin with its name in shapes.txt;
// REF_REPEAT=n times n further inferences and prints "forward_ms <median>".
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>
#include <set>
#include <unordered_map>
#include <algorithm>
#include <omp.h>

#include "io.h"
#include "conv.h"
#include "gemm.h"
#include "mat_mul.h"
#include "add.h"
#include "relu.h"
#include "maxpool.h"
#include "global_avgpool.h"
#include "gelu.h"
#include "layer_normalization.h"
#include "softmax.h"
#include "transpose.h"
#include "flatten.h"
#include "reshape.h"

static int align64(int n) { return (n + 63) & ~63; }

int main(int argc, char **argv) {
    if (argc < 3) {
        fprintf(stderr, "usage: %s model.one out_dir [input.bin ...]\n", argv[0]);
        return 2;
    }
    FILE *f = fopen(argv[1], "rb");
    if (!f) { fprintf(stderr, "cannot open %s\n", argv[1]); return 2; }
    fseek(f, 0, SEEK_END);
    const long size = ftell(f);
    fseek(f, 0, SEEK_SET);
    char *one = (char *) aligned_alloc(64, (size_t) align64((int) size) + 64);
    if (fread(one, 1, (size_t) size, f) != (size_t) size) { fprintf(stderr, "short read\n"); return 2; }
    fclose(f);
    ONE_MODEL_DESC_S *desc = (ONE_MODEL_DESC_S *) one;
    if (desc->one_model_magic_num != ONE_MAGIC_NUM) { fprintf(stderr, "not a .one file\n"); return 2; }
    // the shared scratch buffer some x86 kernels use (extractor::new_output_buf)
    PUBLIC_BUF_INFO_S *pub = &desc->useful_info.public_buf_info;
    pub->public_buf_ptr = (int64_t) aligned_alloc(32, (size_t) pub->public_buf_size);

    Manager &m = Manager::getInstance();
    std::vector<std::shared_ptr<op>> ops;
    std::vector<std::shared_ptr<op>> io_ops;
    char *p = one + desc->io_cfg_offset;
    for (int i = 0; i < desc->io_cfg_cnt; ++i) {
        std::shared_ptr<op> o;
        m.Opmap[std::string(p)](o, p);
        o->fill_operands(one);
        io_ops.push_back(o);
        p += align64(m.op_cfg_size_map[std::string(p)]);
    }
    p = one + desc->node_cfg_offset;
    for (int i = 0; i < desc->node_cnt; ++i) {
        const std::string type(p);
        if (m.Opmap.find(type) == m.Opmap.end()) { fprintf(stderr, "no reference operator class for %s\n", type.c_str()); return 3; }
        std::shared_ptr<op> o;
        m.Opmap[type](o, p);
        o->fill_operands(one);
        o->prepare(p);
        if (!o->evla_impl) { fprintf(stderr, "no x86 kernel for %s under %s\n", type.c_str(), getenv("ONENEW_REF_OP_DIR")); return 3; }
        ops.push_back(o);
        p += align64(m.op_cfg_size_map[type]);
    }

    // initialisers that some operator reads
    std::set<std::string> init_list;
    p = one + desc->init_info_offset;
    for (int i = 0; i < desc->init_cnt; ++i) {
        OPERAND_S *od = (OPERAND_S *) p;
        for (auto &o : ops)
            for (auto &name : o->in_operands)
                if (name == od->operand_name) init_list.insert(name);
        p += align64((int) sizeof(OPERAND_S) + operand_buf_size(od));
    }

    // operand descriptors: the inputs' come from the io configs
    std::unordered_map<std::string, OPERAND_S> stu;
    std::set<std::string> ready(init_list);
    std::vector<std::string> in_names, out_names;
    for (auto &o : io_ops) {
        io *iop = dynamic_cast<io *>(o.get());
        const std::string name(iop->io_cfg.operand.operand_name);
        if (std::string(iop->io_cfg.op_name) == "input") {
            stu[name] = iop->io_cfg.operand;
            ready.insert(name);
            in_names.push_back(name);
        } else {
            out_names.push_back(name);
        }
    }
    // execution order: the first operator in file order whose inputs all exist
    std::vector<std::shared_ptr<op>> order;
    std::vector<bool> placed(ops.size(), false);
    for (size_t done = 0; done < ops.size(); ++done) {
        int pick = -1;
        for (size_t i = 0; i < ops.size() && pick < 0; ++i) {
            if (placed[i]) continue;
            bool ok = true;
            for (auto &name : ops[i]->in_operands)
                if (!name.empty() && !ready.count(name)) ok = false;
            if (ok) pick = (int) i;
        }
        if (pick < 0) { fprintf(stderr, "graph cannot be ordered\n"); return 3; }
        placed[pick] = true;
        order.push_back(ops[pick]);
        for (auto &name : ops[pick]->out_operands) {
            ready.insert(name);
            OPERAND_S od;
            memset(&od, 0, sizeof(od));
            strncpy(od.operand_name, name.c_str(), OPERAND_NAME_LEN - 1);
            stu[name] = od;
        }
    }
    for (auto &o : order) o->shape_infer(stu);

    // one buffer per operand (fp32 elements, a little slack for kernels that read whole vectors)
    std::unordered_map<std::string, BUFFER_INFO_S> bufs;
    for (auto &kv : stu) {
        if (kv.second.not_need_buf == TRUE) continue;
        const int32_t elems = operand_elem_size(&kv.second);
        BUFFER_INFO_S b;
        b.addr = (int64_t) aligned_alloc(32, (size_t) align64(elems * 4) + 64);
        memset((void *) b.addr, 0, (size_t) align64(elems * 4) + 64);
        b.elem_size = elems;
        b.buf_size = elems * 4;
        bufs[kv.first] = b;
    }
    if ((int) in_names.size() != argc - 3) { fprintf(stderr, "the model has %zu inputs, %d files given\n", in_names.size(), argc - 3); return 2; }
    for (size_t i = 0; i < in_names.size(); ++i) {
        FILE *fi = fopen(argv[3 + i], "rb");
        if (!fi) { fprintf(stderr, "cannot open %s\n", argv[3 + i]); return 2; }
        const size_t want = (size_t) bufs[in_names[i]].buf_size;
        if (fread((void *) bufs[in_names[i]].addr, 1, want, fi) != want) { fprintf(stderr, "input %zu is short\n", i); return 2; }
        fclose(fi);
    }
    for (auto &o : order) o->rt_prepare(bufs, stu, init_list);
    for (auto &o : order) o->forward(bufs, stu, init_list);
    // REF_REPEAT=n: n more inferences, the median time of one goes to stdout (the CPU baseline of the benchmark)
    if (const char *rep = getenv("REF_REPEAT")) {
        std::vector<double> ms;
        for (int r = 0; r < atoi(rep); ++r) {
            const double t0 = omp_get_wtime();
            for (auto &o : order) o->forward(bufs, stu, init_list);
            ms.push_back((omp_get_wtime() - t0) * 1e3);
        }
        std::sort(ms.begin(), ms.end());
        if (!ms.empty()) printf("forward_ms %.4f\n", ms[ms.size() / 2]);
    }

    const std::string dir(argv[2]);
    FILE *fs = fopen((dir + "/shapes.txt").c_str(), "w");
    auto dump = [&](const std::string &file, const std::string &name) {
        OPERAND_S &od = stu[name];
        FILE *fo = fopen((dir + "/" + file).c_str(), "wb");
        fwrite((void *) bufs[name].addr, 4, (size_t) operand_elem_size(&od), fo);
        fclose(fo);
        fprintf(fs, "%s %s %d", file.c_str(), name.c_str(), od.dim_num_of_shapes);
        for (int d = 0; d < od.dim_num_of_shapes; ++d) fprintf(fs, " %d", od.shapes[d]);
        fprintf(fs, "\n");
    };
    for (size_t i = 0; i < out_names.size(); ++i) dump(std::to_string(i) + ".bin", out_names[i]);
    if (getenv("REF_DUMP_ALL")) {
        int k = 0;
        for (auto &o : order)
            for (auto &name : o->out_operands) dump("op_" + std::to_string(k++) + ".bin", name);
    }
    fclose(fs);
    return 0;
}

// Driver (ours) around the reference host classes: builds the SiLU and GELU activation tables
// with the reference's own code and writes them as raw float32 to the two files named on the
// command line.  Compiled only by `make -C oracle ref`; includes the reference headers in place.
#include <cstdio>
#include "conv.h"
#include "gelu.h"

int main(int argc, char **argv) {
    if (argc != 3) {
        fprintf(stderr, "usage: %s silu.bin gelu.bin\n", argv[0]);
        return 2;
    }
    Conv conv;
    conv.conv_cfg.act_type = SILU;
    conv.other_prepare();
    Gelu gelu;
    gelu.inputs_vec.resize(BUF_MAXNUM);
    gelu.other_prepare();
    FILE *f = fopen(argv[1], "wb");
    fwrite(conv.lut.data(), sizeof(float), conv.lut.size(), f);
    fclose(f);
    f = fopen(argv[2], "wb");
    fwrite(gelu.lut.data(), sizeof(float), gelu.lut.size(), f);
    fclose(f);
    printf("silu %zu gelu %zu\n", conv.lut.size(), gelu.lut.size());
    return 0;
}

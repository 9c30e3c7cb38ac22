/* Host-only driver for the sanitizer build of the library's C files: parse-only mode, so no
 * device is touched.  Each argument is "cfg" or "cfg@weights": parse, optionally read the weights
 * file and write it back to argv[1], query every layer, shrink the batch, free. */
#include <stdio.h>
#include <string.h>
#include "darknet_amd.h"
#include "darknet_hip.h"

int main(int argc, char **argv)
{
    hip_set_parse_only(1);
    network_set_verbose(0);
    for (int i = 2; i < argc; ++i) {
        char *cfg = argv[i];
        char *weights = strchr(cfg, '@');
        if (weights) *weights++ = 0;
        network *net = parse_network_cfg(cfg);
        if (weights) {
            load_weights(net, weights);
            save_weights(net, argv[1]);
        }
        int iv[64];
        float fv[16];
        const int n = network_num_layers(net);
        for (int k = 0; k < n; ++k) network_layer_info(net, k, iv, fv);
        set_batch_network(net, 1);
        free_network(net);
        printf("ok %s %d\n", cfg, n);
    }
    return 0;
}

/*
 * A C program written against include/aspen.h alone, in the shape of the reference's command-line
 * driver (reference main.c:60-151): build the model from a cfg + weight file, save it as .aspen and load it
 * back, create the tile graph, run `iterations` inferences in the reset / run / wait / stop loop with the
 * input read from an NCHW float file, write the final layer in {BATCH, OUT_C, OUT_H, OUT_W} order.
 *
 *   caller <cfg> <weights.bin> <input.bin> <batch> <min_ninst> <iterations> <out.bin> <tmp.aspen>
 */
#include "aspen.h"

static double now_sec (void)
{
    struct timeval tv;
    gettimeofday (&tv, NULL);
    return (double)tv.tv_sec + 1e-6 * (double)tv.tv_usec;
}

int main (int argc, char **argv)
{
    if (argc != 9)
    {
        fprintf (stderr, "usage: %s cfg weights input batch min_ninst iterations out tmp_aspen\n", argv[0]);
        return 2;
    }
    const unsigned int batch = (unsigned int)atoi (argv[4]), min_ninst = (unsigned int)atoi (argv[5]);
    const int iterations = atoi (argv[6]);
    print_aspen_build_info ();
    aspen_dnn_t *built = apu_create_dnn (argv[1], argv[2]);
    if (built == NULL) { ERROR_PRTF ("cannot build the model from %s\n", argv[1]); return 1; }
    apu_save_dnn_to_file (built, argv[8]);
    apu_destroy_dnn (built);
    aspen_dnn_t *dnn = apu_load_dnn_from_file (argv[8]);
    if (dnn == NULL) { ERROR_PRTF ("cannot load %s\n", argv[8]); return 1; }
    nasm_t *nasm = apu_create_nasm (dnn, min_ninst, batch);
    if (nasm == NULL) { ERROR_PRTF ("cannot create the tile graph\n"); return 1; }
    rpool_t *rpool = rpool_init ();
    dse_group_t *dse_group = dse_group_init (4);
    dse_group_set_rpool (dse_group, rpool);
    rpool_add_nasm (rpool, nasm, argv[3]);
    const double t0 = now_sec ();
    for (int i = 0; i < iterations; i++)
    {
        if (i > 0)
        {
            rpool_reset_queue (rpool);
            rpool_reset_nasm (rpool, nasm);
        }
        dse_group_run (dse_group);
        dse_wait_for_nasm_completion (nasm);
        dse_group_stop (dse_group);
    }
    PRTF ("%s: %d iterations, %f s each\n", layer_type_str[INPUT_LAYER], iterations, (now_sec () - t0) / (iterations > 0 ? iterations : 1));
    if (!dse_check_nasm_completion (nasm)) { ERROR_PRTF ("the run did not complete\n"); return 1; }
    LAYER_PARAMS order[] = {BATCH, OUT_C, OUT_H, OUT_W};
    void *result = NULL;
    const ssize_t bytes = dse_get_nasm_result (nasm, order, &result);
    if (bytes <= 0 || result == NULL) { ERROR_PRTF ("no result\n"); return 1; }
    FILE *f = fopen (argv[7], "wb");
    if (f == NULL || fwrite (result, (size_t)bytes, 1, f) != 1) { ERROR_PRTF ("cannot write %s\n", argv[7]); return 1; }
    fclose (f);
    free (result);
    aspen_flush_dynamic_memory ();
    dse_group_destroy (dse_group);
    rpool_destroy (rpool);
    apu_destroy_nasm (nasm);
    apu_destroy_dnn (dnn);
    return 0;
}

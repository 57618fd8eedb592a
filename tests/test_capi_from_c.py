"""The C ABI called from C: a small program compiled by gcc against include/born_rocm.h and linked with
born_amd/lib/libborn_rocm.so exercises the argument-error paths that need no GPU (status codes, the
per-thread error text, the config defaults' validation).  ctypes is not involved: what the header declares is
what a C (or cgo) caller gets."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

C_SOURCE = r"""
#include <stdio.h>
#include <string.h>
#include "born_rocm.h"

static int failures = 0;
#define EXPECT(cond)                                                        \
    do {                                                                    \
        if (!(cond)) {                                                      \
            printf("FAILED line %d: %s   (last error: %s)\n", __LINE__, #cond, born_rocm_last_error()); \
            failures++;                                                     \
        }                                                                   \
    } while (0)

int main(void) {
    born_sampler *s = (born_sampler *)0;
    born_sampler_config cfg;
    float x[4] = {0.0f, 1.0f, 2.0f, 3.0f}, u[1] = {0.5f};
    int32_t tok[1];
    int64_t shape_a[2] = {2, 3}, shape_b[2] = {4, 3}, out_shape[2];

    /* handle creation: every rejected configuration is an argument error with a "sampler: ..." message */
    EXPECT(born_rocm_sampler_create(0, 1, 10, 0) == BORN_ROCM_ERR_ARGUMENT);
    EXPECT(born_rocm_sampler_create(0, 0, 10, &s) == BORN_ROCM_ERR_ARGUMENT && s == 0);
    EXPECT(strncmp(born_rocm_last_error(), "sampler: ", 9) == 0);
    memset(&cfg, 0, sizeof cfg);
    cfg.temperature = -1.0f;
    EXPECT(born_rocm_sampler_create(&cfg, 1, 10, &s) == BORN_ROCM_ERR_ARGUMENT && strstr(born_rocm_last_error(), "temperature"));
    cfg.temperature = 0.7f;
    cfg.top_p = 1.5f;                                   /* (0, 1] on the handle path as on the per-row path */
    EXPECT(born_rocm_sampler_create(&cfg, 1, 10, &s) == BORN_ROCM_ERR_ARGUMENT && strstr(born_rocm_last_error(), "top_p"));
    cfg.top_p = 0.9f;
    cfg.min_p = 1.0f;
    EXPECT(born_rocm_sampler_create(&cfg, 1, 10, &s) == BORN_ROCM_ERR_ARGUMENT && strstr(born_rocm_last_error(), "min_p"));
    cfg.min_p = 0.0f;
    cfg.repetition_penalty = -2.0f;
    EXPECT(born_rocm_sampler_create(&cfg, 1, 10, &s) == BORN_ROCM_ERR_ARGUMENT && strstr(born_rocm_last_error(), "repetition_penalty"));
    cfg.repetition_penalty = 1.1f;
    EXPECT(born_rocm_sampler_create(&cfg, 1, ((int64_t)1 << 20), &s) == BORN_ROCM_ERR_UNSUPPORTED);   /* vocabulary beyond the kernels */

    /* calls on a null handle or with null buffers fail before any device work */
    EXPECT(born_rocm_sample(0, x, 1, 4, 4, 0, 0, 0, u, tok, 0, 0, 0, 0, 0, 0) == BORN_ROCM_ERR_ARGUMENT);
    EXPECT(born_rocm_argmax(0, x, 1, 4, 4, tok, 0) == BORN_ROCM_ERR_ARGUMENT);
    EXPECT(born_rocm_sampler_set_path(0, 0) == BORN_ROCM_ERR_ARGUMENT);
    EXPECT(born_rocm_sampler_set_step(0, 0) == BORN_ROCM_ERR_ARGUMENT);
    EXPECT(born_rocm_sampler_get_step(0, 0) == BORN_ROCM_ERR_ARGUMENT);
    EXPECT(born_rocm_sampler_destroy(0) == BORN_ROCM_OK);
    EXPECT(born_rocm_exp(0, 0, 4, 0) == BORN_ROCM_ERR_ARGUMENT);
    EXPECT(born_rocm_exp(x, x, -1, 0) == BORN_ROCM_ERR_ARGUMENT);
    EXPECT(born_rocm_exp(x, x, 0, 0) == BORN_ROCM_OK);  /* nothing to do: no launch */

    /* the entry point that allocates nothing states its limits */
    EXPECT(born_rocm_sample_static(&cfg, x, 1, 4, 4, 0, 0, 0, 0, tok, 0, 0, 0) == BORN_ROCM_ERR_ARGUMENT && strstr(born_rocm_last_error(), "uniforms"));
    EXPECT(born_rocm_sample_static(&cfg, x, 4097, 4, 4, 0, 0, 0, u, tok, 0, 0, 0) == BORN_ROCM_ERR_UNSUPPORTED && strstr(born_rocm_last_error(), "4096"));
    cfg.top_p = 2.0f;
    EXPECT(born_rocm_sample_static(&cfg, x, 1, 4, 4, 0, 0, 0, u, tok, 0, 0, 0) == BORN_ROCM_ERR_ARGUMENT && strstr(born_rocm_last_error(), "top_p"));

    /* host-side shape logic: tensor.BroadcastShapes (internal/tensor/shape.go:83-118) */
    EXPECT(born_rocm_broadcast_shape(shape_a, 2, shape_b, 2, out_shape) == BORN_ROCM_ERR_ARGUMENT);
    shape_b[0] = 1;
    EXPECT(born_rocm_broadcast_shape(shape_a, 2, shape_b, 2, out_shape) == BORN_ROCM_OK && out_shape[0] == 2 && out_shape[1] == 3);

    printf(failures ? "%d failure(s)\n" : "all C-side checks passed\n", failures);
    return failures ? 1 : 0;
}
"""


def test_c_program_against_the_header(tmp_path):
    lib_dir = os.path.join(ROOT, "born_amd", "lib")
    assert os.path.exists(os.path.join(lib_dir, "libborn_rocm.so")), "build the library first (python -m born_amd.build)"
    src = tmp_path / "capi.c"
    src.write_text(C_SOURCE)
    exe = tmp_path / "capi"
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
                           "-L", lib_dir, "-lborn_rocm", "-L", "/opt/rocm/lib", "-Wl,-rpath," + lib_dir, "-Wl,-rpath,/opt/rocm/lib",
                           "-Wl,--allow-shlib-undefined"])
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "all C-side checks passed" in run.stdout

"""The code paths that the default launch policy reaches only at benchmark sizes, exercised at test sizes with the
exact checks of the other GPU tests: the non-temporal kernel variants (policy threshold set to zero, so every
array takes them) and the grid-stride loops (grid capped at one workgroup per compute unit, so every thread walks
several groups).  Also the plain variants with the non-temporal policy switched off.
"""
import pytest

import test_gpu_additive as T_add
import test_gpu_batch_norm as T_bn
import test_gpu_flat as T_flat
import test_gpu_softmax as T_sm
from anode_amd import gpu

pytestmark = pytest.mark.gpu

# knob numbers of anode_gpu_set_tuning: 0 workgroups per CU of a streaming map (0 = full grid), 3 / 4 non-temporal
# masks of the maps / reductions, 5 smallest array read with non-temporal loads, 7 smallest array written with
# streaming stores (the variants with streaming stores only sit between the two)
PROFILES = {
    "nontemporal_everywhere": {5: 0},
    "streaming_stores_only": {7: 0},
    "nontemporal_off": {3: 0, 4: 0},
    "one_workgroup_per_cu": {0: 1},
    "one_workgroup_per_cu_nontemporal": {0: 1, 5: 0},
    # knob 14: the n-d NLL backward pass walks planes of up to this many pixels as a flat array; 0 sends every shape
    # to the kernel that gives a thread four pixels and walks their classes (the default only does so from 131073 on)
    "nd_backward_by_pixel_groups": {14: 0},
    "nd_backward_by_pixel_groups_nontemporal": {14: 0, 5: 0},
    # knob 15: rows of 16385 to 65536 classes held half in LDS, half in registers; 0 sends them to the streaming kernel
    "long_rows_streamed": {15: 0},
    "long_rows_streamed_nontemporal": {15: 0, 5: 0},
    "long_rows_half_in_lds_nontemporal": {5: 0},
    # knob 17: n-d softmax over short planes with more than 32 classes keeps whole samples in registers; 0 sends
    # them to the LDS tiles, the column tiles and the register kernels that split a pixel group over lanes
    "nd_short_planes_through_tiles": {17: 0},
    "nd_short_planes_through_tiles_nontemporal": {17: 0, 5: 0},
    # knob 18: n-d softmax with 33 to 512 classes on planes of 128 pixels and more takes column tiles in registers; 0
    # sends them to the kernels with eight lanes per pixel group, the LDS column tiles and the two-pass kernel
    "nd_many_classes_without_register_tiles": {18: 0},
    "nd_many_classes_without_register_tiles_nontemporal": {18: 0, 17: 0, 5: 0},
}


@pytest.fixture(params=sorted(PROFILES))
def tuned(request):
    saved = {k: gpu.set_tuning(k, v) for k, v in PROFILES[request.param].items()}
    yield request.param
    for k, v in saved.items():
        gpu.set_tuning(k, v)


def test_batch_norm_under_tuning(tuned, oracle):
    # 401 408 and 802 816 elements: more than one pass of a 256-workgroup grid; S odd; element-aligned pointers
    for S, C, N in [(784, 16, 32), (12544, 4, 8), (49, 300, 4), (5001, 2, 3)]:
        for offset in (0, 1):
            T_bn.test_batch_norm_all_symbols(oracle, S, C, N, offset)


def test_flat_maps_under_tuning(tuned, oracle):
    for name in sorted(T_flat.MAPS):
        T_flat.test_flat_maps(oracle, name)
    T_flat.test_two_input_maps_and_in_place_backward(oracle)
    T_flat.test_positive_clip_in_place_and_sign_rules(oracle)
    T_flat.test_upcast(oracle)
    T_flat.test_dequantize_all_codes_and_ragged_lengths(oracle, -1.0, 1.0)
    T_flat.test_one_hot(oracle, 4096, 5, 2)
    T_flat.test_f1_loss_and_bwd(oracle, 70000, 2, 2)


def test_softmax_under_tuning(tuned, oracle):
    for K, R in [(10, 4000), (1000, 256), (4096, 3), (40000, 1), (16388, 3), (32768, 2), (65536, 2)]:
        for name in T_sm.ROW_ENTRY_POINTS:
            T_sm.test_softmax_rows(oracle, name, K, R)
    T_sm.test_softmax_cat_nll_and_bwd_rows(oracle, 1000, 256)
    for P, C, N in [(2048, 19, 2), (1300, 19, 3), (8, 64, 3), (7, 40, 3), (16, 200, 2), (1024, 256, 2),
                    (196, 70, 3), (100, 100, 3), (196, 150, 2), (64, 300, 3), (196, 200, 2), (256, 65, 2), (324, 70, 2),
                    (1028, 48, 2), (1032, 65, 2), (1028, 129, 1), (1024, 192, 1), (1056, 200, 2), (1028, 300, 1),
                    (784, 100, 2), (2048, 472, 1), (900, 65, 1), (1025, 19, 2), (515, 40, 2)]:
        T_sm.test_softmax_nd_all_symbols(oracle, P, C, N)


def test_additive_under_tuning(tuned, oracle):
    T_add.test_arg_max_rows(oracle)
    T_add.test_quantize_u8(oracle, -4.0, 4.0)
    T_add.test_bcast_affine_family(oracle, 3136, 3, 40)
    T_add.test_channel_sums_and_mean_var(oracle, 784, 16, 32)
    for masked in (False, True):
        T_add.test_fused_batch_norm_equals_the_launch_sequence(oracle, 784, 16, 32, masked)
    T_add.test_fused_softmax_nd_nll_equals_the_two_launches(oracle, 2048, 19, 2)
    for P, C, N in [(196, 82, 2), (64, 300, 3), (196, 200, 2), (1056, 200, 1), (1028, 300, 1)]:
        T_add.test_fused_softmax_nd_nll_equals_the_two_launches(oracle, P, C, N)

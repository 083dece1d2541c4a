// Host build of the attention kernels' work order (dl4s_amd/csrc/work_order.h) for tests/test_work_order.py.
#include "../dl4s_amd/csrc/work_order.h"

extern "C" int work_item_at(int block, int nunits, int total_blocks, int lpt, int snake, int *bh, int *unit) {
    return dl4s_work_order::work_item_at(block, nunits, total_blocks, lpt, *bh, *unit, snake) ? 1 : 0;
}

extern "C" void split_item_at(int bx, int by, int gx, int nsplit, int *blk, int *sp) {
    dl4s_work_order::split_item_at(bx, by, gx, nsplit, *blk, *sp);
}

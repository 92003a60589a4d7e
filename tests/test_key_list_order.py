"""The order the 16-token dK/dV kernel requires of caller-built key-centric lists, and the host-side check of it
(``ops.key_lists_ascending``, used by ``ops.attn_bwd(check_lists=True)`` / ``S3R_CHECK_LISTS=1``).  The kernel merges
the lists of four neighbouring key blocks a window at a time and treats the entries below a threshold as a prefix of
each list: a list that is not ascending makes it skip entries, and dk / dv come out incomplete without any error."""
import torch

from speed3r_amd.sparse_attn.ops import key_lists_ascending


def _lists(groups, tail=()):
    flat = [x for g in groups for x in g] + list(tail)
    offs = [0]
    for g in groups:
        offs.append(offs[-1] + len(g))
    return torch.tensor(flat, dtype=torch.int32).view(1, 1, -1), torch.tensor(offs, dtype=torch.int32).view(1, 1, -1)


def test_ascending_groups_pass_and_a_swapped_pair_fails():
    assert key_lists_ascending(*_lists([[0, 3, 3, 7], [], [1, 2], [5]]))
    assert not key_lists_ascending(*_lists([[0, 3, 2, 7], [], [1, 2], [5]]))
    assert not key_lists_ascending(*_lists([[0, 3, 3, 7], [], [2, 1], [5]]))


def test_group_borders_and_the_unspecified_tail_are_free():
    assert key_lists_ascending(*_lists([[8, 9], [0, 1], [0]]))                    # every border steps down
    assert key_lists_ascending(*_lists([[1, 2], [3]], tail=(9, 4, 0, -7)))       # entries behind the last offset


def test_batched_heads_each_with_their_own_offsets():
    la, oa = _lists([[0, 1, 2], [4]])
    lb, ob = _lists([[2], [0, 1, 9]])
    lists, offs = torch.cat((la, lb), dim=1), torch.cat((oa, ob), dim=1)
    assert key_lists_ascending(lists, offs)
    lists[0, 1, 1] = 5                                                            # 5, 1 inside head 1's second group
    assert not key_lists_ascending(lists, offs)

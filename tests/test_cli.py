"""The command line's options, without a GPU: names and meanings follow the reference's `arle` and `infer`
(crates/cli/src/args.rs:188-302, infer/src/main.rs:26-236)."""
import pytest

from arle_amd.cli import build_parser, main


def test_global_options_and_run():
    args = build_parser().parse_args(["--model-path", "/m", "--max-tokens", "auto", "--temperature", "0.7", "--no-cuda-graph",
                                      "--num-slots", "8", "--chunked-prefill-size", "2048", "run", "--prompt-ids", "1, 2,3",
                                      "--json"])
    assert args.command == "run" and args.model_path == "/m" and args.max_tokens == 0 and args.temperature == 0.7
    assert args.no_cuda_graph and not args.no_weight_tiles and args.num_slots == 8 and args.chunked_prefill_size == 2048
    assert args.prompt_ids == "1, 2,3" and args.json


def test_defaults_are_the_reference_library_defaults():
    args = build_parser().parse_args(["--model-path", "/m", "run", "--prompt", "hi"])
    # infer/src/main.rs:90-105: slots 4, 16384 tokens a step, the portion and the prompt tokens of a step left to be
    # settled by the GPU's memory (infer/src/scheduler/types.rs:315-334); greedy (crates/cli/src/args.rs)
    assert (args.num_slots, args.chunked_prefill_size, args.max_num_batched_tokens, args.max_prefill_tokens) == (4, None, 16384, None)
    assert args.temperature == 0.0 and args.top_k == -1 and args.top_p == 1.0 and args.min_p == 0.0 and args.seed == 42
    assert not args.no_cuda_graph and not args.no_weight_tiles and args.dtype == "bfloat16"


def test_bad_values_are_refused(capsys):
    with pytest.raises(SystemExit):
        build_parser().parse_args(["--max-tokens", "-3", "run", "--prompt", "x"])
    with pytest.raises(SystemExit):
        build_parser().parse_args(["--dtype", "float16", "run", "--prompt", "x"])
    with pytest.raises(SystemExit):   # one source of the prompt only
        build_parser().parse_args(["run", "--prompt", "x", "--stdin"])
    assert main(["run", "--prompt", "x"]) == 2          # no model folder
    assert "--model-path" in capsys.readouterr().err


def test_stop_strings_are_found_in_list_order_and_their_length_is_held_back():
    """The reading of infer/src/scheduler/cuda/request.rs:396-413 (the reference holds no vectors for it): the first
    stop string of the list that the text holds decides, not the one that comes first in the text; empty ones do
    not count; without a hit all but the longest stop string's bytes may go out, cut back to a whole character."""
    from arle_amd.engine.api import check_stop_sequences

    assert check_stop_sequences("one two three", ["three", "two"]) == (True, 8)
    assert check_stop_sequences("one two three", ["", "two"]) == (True, 4)
    assert check_stop_sequences("one two", ["three"]) == (False, 2)          # 7 - 5
    assert check_stop_sequences("on", ["three"]) == (False, 0)
    assert check_stop_sequences("one two", []) == (False, 7) and check_stop_sequences("one two", [""]) == (False, 7)
    assert check_stop_sequences("aé", ["xy"]) == (False, 1)                 # 3 bytes - 2 falls inside the é: back to "a"
    assert check_stop_sequences("ab\u00e9\u00e9", ["\u00e9x"]) == (False, 2)    # 6 bytes - 3: inside the first é


def test_slots_left_to_the_engine_follow_what_the_cache_holds():
    """--num-slots auto (the reference's flag left unset, infer/src/main.rs:782-855): as many requests of the longest
    length as the cache holds, from 4 to 128."""
    from arle_amd.cache.manager import slots_for_tokens

    assert build_parser().parse_args(["--num-slots", "auto", "run", "--prompt", "x"]).num_slots is None
    assert build_parser().parse_args(["--num-slots", "7", "run", "--prompt", "x"]).num_slots == 7
    with pytest.raises(SystemExit):
        build_parser().parse_args(["--num-slots", "0", "run", "--prompt", "x"])
    assert [slots_for_tokens(t, 64) for t in (0, 128, 256, 2048, 64 * 128, 10 ** 9)] == [4, 4, 4, 32, 128, 128]

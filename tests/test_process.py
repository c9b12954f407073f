"""The process entry point's request rules and result file, with stand-in child
processes and no model (/root/reference/tools/nnis_hub_hf_generate.py:309-411
tests its wrapper the same way)."""

import json
import sys

import pytest

from nnis_amd import process


def test_request_rules(tmp_path):
    model = tmp_path / "m"
    model.mkdir()
    (model / "tokenizer.json").write_text("{}")
    ok = dict(model=str(model), tokenizer=None, prompt="hi", prompt_ids=None, device=0, max_new_tokens=4,
              result=str(tmp_path / "r.json"))
    process.validate_request(**ok)
    process.validate_request(**{**ok, "prompt": None, "prompt_ids": "1,2"})
    for change in (dict(model=str(tmp_path / "none")), dict(prompt=None), dict(prompt_ids="1"), dict(prompt=""),
                   dict(prompt="a\0b"), dict(device=-1), dict(max_new_tokens=0), dict(max_new_tokens=65537),
                   dict(tokenizer=str(tmp_path / "missing.json")), dict(result=str(model))):
        with pytest.raises(process.RequestError):
            process.validate_request(**{**ok, **change})
    link = tmp_path / "link"
    link.symlink_to(model)
    with pytest.raises(process.RequestError, match="symbolic links are refused"):
        process.validate_request(**{**ok, "model": str(link)})


def test_child_and_result_file(tmp_path):
    child = process.run_child([sys.executable, "-c", "print('7,8,9')"], 30)
    assert child["status"] == "generated" and child["stdout"] == b"7,8,9\n"
    assert process.run_child([sys.executable, "-c", "import sys; sys.exit(3)"], 30)["status"] == "failed"
    assert process.run_child([sys.executable, "-c", "import time; time.sleep(5)"], 0.2)["status"] == "timeout"
    assert process.run_child([str(tmp_path / "no-such-binary")], 5)["status"] == "not_started"
    # the cap holds while the child is read: a child that would write without end is stopped at the cap
    endless = "import sys\nwhile True: sys.stdout.write('x' * 65536)"
    cut = process.run_child([sys.executable, "-c", endless], 60, capture_limit=1 << 20)
    assert cut["status"] == "output_too_large" and cut["stdout"] == b"" and b"1048576" in cut["stderr"]
    noisy = process.run_child([sys.executable, "-c", "import sys; sys.stderr.write('e' * 5000); print('ok')"], 30, capture_limit=4096)
    assert noisy["status"] == "output_too_large"
    exact = process.run_child([sys.executable, "-c", "import sys; sys.stdout.write('y' * 4096)"], 30, capture_limit=4096)
    assert exact["status"] == "generated" and len(exact["stdout"]) == 4096
    result = process.build_result({"prompt": "x"}, child)
    assert result["stdout"]["bytes"] == 6 and len(result["stdout"]["sha256"]) == 64 and result["sampling"] == "greedy"
    path = tmp_path / "out" / "r.json"
    process.write_new_json(str(path), result)
    assert json.loads(path.read_text())["stdout"]["utf8"] == "7,8,9\n"
    with pytest.raises(process.RequestError, match="already exists"):
        process.write_new_json(str(path), result)  # never overwritten
    assert [p.name for p in path.parent.iterdir()] == ["r.json"]  # no temporary file left behind


def test_main_with_a_stand_in_binary(tmp_path):
    model = tmp_path / "m"
    model.mkdir()
    fake = tmp_path / "fake_nnis.py"
    fake.write_text("import sys\nprint(' '.join(sys.argv[1:]))\n")
    out = tmp_path / "r.json"
    code = process.main(["--model", str(model), "--prompt-ids", "1,2,3", "--result", str(out), "--nnis-bin", str(fake),
                         "--max-new-tokens", "5"])
    assert code == 0
    record = json.loads(out.read_text())
    assert record["status"] == "generated" and "--prompt-ids 1,2,3" in record["stdout"]["utf8"]
    assert "--max-new-tokens 5" in record["stdout"]["utf8"] and record["inputs"]["device_ordinal"] == 0
    assert process.main(["--model", str(model), "--prompt-ids", "1", "--result", str(out), "--nnis-bin", str(fake)]) == 2

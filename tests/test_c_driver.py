"""A C program written against the reference's names (tests/c_api/kfac_driver_main.c, the shape of
drivers/main_driver.c:62-305) compiles against include/*.h, links the two libraries and starts: the drop-in
boundary is plain C.  Without arguments the program exits before anything touches a device."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_reference_shaped_driver_compiles_links_and_starts(tmp_path):
    exe = str(tmp_path / "kfac_driver")
    lib_dir = os.path.join(ROOT, "fitre_amd")
    build = subprocess.run(["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"),
                            os.path.join(ROOT, "tests", "c_api", "kfac_driver_main.c"), "-o", exe, "-L", lib_dir,
                            "-lfitre_cnn", "-lfitre_hip", "-Wl,-rpath," + lib_dir], capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([exe], capture_output=True, text=True)
    assert run.returncode == 2 and "usage:" in run.stderr

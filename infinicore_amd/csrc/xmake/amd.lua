-- xmake targets for the AMD Instinct (HIP, gfx950) backend of InfiniRT / InfiniOP.
--
-- Drop this file into the reference tree as xmake/amd.lua and hook it up the way the other vendors
-- are (reference xmake.lua:221-237 for the option, :527-529 / :604-606 for the add_deps):
--
--   option("amd-gpu")  set_default(false)  set_showmenu(true)
--       set_description("Whether to compile implementations for AMD Instinct GPUs (HIP)")
--   option_end()
--   if has_config("amd-gpu") then
--       add_defines("ENABLE_AMD_API")
--       includes("xmake/amd.lua")
--   end
--   -- in target("infinirt"):  if has_config("amd-gpu") then add_deps("infinirt-amd") end
--   -- in target("infiniop"):  if has_config("amd-gpu") then add_deps("infiniop-amd") end
--
-- The sources are the ones under infinicore_amd/csrc of this repository, copied to the matching
-- places of the reference tree (src/infinirt/amd, src/infiniop/devices/amd,
-- src/infiniop/ops/paged_attention/amd, src/infiniop/ops/paged_attention_prefill/amd,
-- src/infiniop/ops/paged_caching/amd, src/infiniop/ops/kv_caching/amd, src/infiniop/ops/rope_paged_caching/amd).
-- xmake is not installed in the environment this file was written in; the Makefile next to it builds
-- the same objects with the same flags and is what the tests use.

local ROCM = os.getenv("ROCM_PATH") or "/opt/rocm"
local ARCH = os.getenv("INFINI_AMD_ARCH") or "gfx950"

toolchain("amd.hip.toolchain")
    set_toolset("cc", ROCM .. "/bin/hipcc")
    set_toolset("cxx", ROCM .. "/bin/hipcc")
    set_toolset("ld", ROCM .. "/bin/hipcc")
    set_toolset("sh", ROCM .. "/bin/hipcc")
    set_toolset("ar", "ar")
toolchain_end()

rule("amd.hip")
    set_extensions(".hip")
    on_build_file(function (target, sourcefile, opt)
        import("core.project.depend")
        local objectfile = target:objectfile(sourcefile)
        os.mkdir(path.directory(objectfile))
        local args = {
            "-x", "hip", "--offload-arch=" .. ARCH, "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
            "-D__HIP_PLATFORM_AMD__", "-DENABLE_AMD_API",
            -- keep fp32 arithmetic on the one-value-per-lane VALU forms
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
            "-Iinclude", "-Isrc", "-c", sourcefile, "-o", objectfile,
        }
        -- per-file flags given with add_files(..., {cxflags = ...})
        local fileconfig = target:fileconfig(sourcefile)
        if fileconfig and fileconfig.cxflags then
            for _, flag in ipairs(fileconfig.cxflags) do
                table.insert(args, #args - 3, flag)
            end
        end
        depend.on_changed(function ()
            os.vrunv(ROCM .. "/bin/hipcc", args)
        end, {files = sourcefile})
        table.insert(target:objectfiles(), objectfile)
    end)
rule_end()

target("infinirt-amd")
    set_kind("static")
    set_languages("cxx17")
    add_deps("infini-utils")
    on_install(function (target) end)
    set_toolchains("amd.hip.toolchain")
    add_defines("__HIP_PLATFORM_AMD__", "ENABLE_AMD_API")
    add_includedirs(ROCM .. "/include")
    add_linkdirs(ROCM .. "/lib")
    add_links("amdhip64")
    add_cxflags("-fPIC")
    add_files("../src/infinirt/amd/*.cc")
target_end()

target("infiniop-amd")
    set_kind("static")
    set_languages("cxx17")
    add_deps("infini-utils")
    on_install(function (target) end)
    set_toolchains("amd.hip.toolchain")
    add_rules("amd.hip")
    add_defines("__HIP_PLATFORM_AMD__", "ENABLE_AMD_API")
    add_includedirs(ROCM .. "/include")
    add_linkdirs(ROCM .. "/lib")
    add_links("amdhip64")
    add_cxflags("-fPIC")
    add_files("../src/infiniop/devices/amd/*.cc")
    add_files("../src/infiniop/ops/kv_caching/amd/*.hip")
    add_files("../src/infiniop/ops/rope_paged_caching/amd/*.hip")
    -- the scatter kernel gets its first 14 argument words in scalar registers at wavefront start
    add_files("../src/infiniop/ops/paged_caching/amd/*.hip", {cxflags = {"-mllvm", "-amdgpu-kernarg-preload-count=14"}})
    -- the attention kernels keep their matrix-instruction accumulators in ordinary vector registers
    add_files("../src/infiniop/ops/paged_attention_prefill/amd/*.hip", {cxflags = {"-mllvm", "-amdgpu-mfma-vgpr-form=1"}})
    -- decode also gets the first five argument words of its work-equalising kernels in scalar registers at wavefront start
    add_files("../src/infiniop/ops/paged_attention/amd/*.hip",
              {cxflags = {"-mllvm", "-amdgpu-mfma-vgpr-form=1", "-mllvm", "-amdgpu-kernarg-preload-count=5"}})
target_end()

from deplodock_amd.cli import main

main()
